# Julia host side of the launcher: lowers a reference-style Config / Transform / Epilogue to the
# plain structs of include/gemmkernels_hip.h and calls gk_matmul through ccall.
#
# It replaces the body of `matmul` in the reference (src/matmul.jl:7-44): everything above it
# (get_config, create_config, matmatmul!, mul!) keeps working on the lowered objects.  Julia is not
# available in the build image of this library, so this file has not been executed there; the
# tested host layer is the Python package next to it, which lowers the same structs field by field.
#
# Sizes that are not whole tiles: the reference's create_config puts such a product on Layout.ColMajor /
# RowMajor (src/matmul.jl:121-156).  The library runs it on the aligned kernel of the configuration's block
# shape all the same when A and B have 16-byte aligned columns, K is a multiple of 8 and M (N) is a multiple
# of 8 along the contiguous index of A (B); otherwise on its bounds-checked kernel, which exists for the
# 64 x 64 x 32 block only.  A create_config that wants the fast path for ragged sizes therefore keeps the
# reference's layout rule and picks a block shape with a compiled aligned instance (128 x 128 x 64 on 4 x 2
# warps, which is what the reference's heuristic arrives at for FP16 x FP16 -> FP32, is one).
module GemmKernelsHIP

using Libdl

const libgk = Ref{String}(joinpath(@__DIR__, "..", "..", "..", "lib", "libgemmkernels_hip.so"))

struct ConfigError <: Exception
    message::String
    status::Cint
end
Base.showerror(io::IO, e::ConfigError) = print(io, "ConfigError: ", e.message)

# ---- mirrors of the C structs (field order and types as in the header) ----
struct GkShape; M::Int32; N::Int32; K::Int32; end
struct GkOperator
    kind::Int32; M::Int32; N::Int32; K::Int32; mb::Int32; nb::Int32; kb::Int32
    compute_type::Int32; accum_type::Int32
end
struct GkLayout; kind::Int32; eltype::Int32; pad::Int32; reserved::Int32; ld::Int64; end
struct GkSwizzle; kind::Int32; param::Int32; end
struct GkGettDim
    nmodes::Int32
    extent::NTuple{4,Int32}
    stride0::NTuple{4,Int64}
    stride1::NTuple{4,Int64}
end
struct GkGett; m::GkGettDim; n::GkGettDim; k::GkGettDim; end
struct GkConfig
    matmul_shape::GkShape; block_shape::GkShape; warps_per_block::Int32
    mem_a_warp::GkShape; mem_a_thread::GkShape
    mem_b_warp::GkShape; mem_b_thread::GkShape
    mem_cd_warp::GkShape; mem_cd_thread::GkShape
    compute_warp::GkShape; compute_op_shape::GkShape
    global_a_layout::GkLayout; global_b_layout::GkLayout; global_c_layout::GkLayout; global_d_layout::GkLayout
    shared_a_layout::GkLayout; shared_b_layout::GkLayout; shared_c_layout::GkLayout; shared_d_layout::GkLayout
    op::GkOperator
    is_a_col_major::Int32; is_b_col_major::Int32
    cta_swizzle::GkSwizzle
    gett::GkGett
end
struct GkOp; kind::Int32; p0::Float32; p1::Float32; end
struct GkTransform; n_ops::Int32; ops::NTuple{4,GkOp}; end
struct GkTransforms; hook::NTuple{8,GkTransform}; end
struct GkEpilogue; kind::Int32; reserved::Int32; bias::Ptr{Cvoid}; end

# ---- enums of the header ----
const DTYPE = Dict(Float16 => 0, Float32 => 2, Float64 => 3)          # BFloat16 => 1 when BFloat16s.jl is loaded
const LAYOUT_KIND = Dict(:Zero => 0, :ColMajor => 1, :RowMajor => 2, :UnsafeAlignedColMajor => 3,
                         :UnsafeAlignedRowMajor => 4, :Diagonal => 5, :InterleavedColMajor => 6,
                         :InterleavedRowMajor => 7, :SplitColMajor => 8, :SplitRowMajor => 9, :GETT => 10)
const KERNEL_KIND = Dict(:matmul_singlestage => 0, :matmul_pipelined => 1, :matmul_pipelined_ng => 2, :matmul_split_k => 3)
const OP_KIND = Dict(:identity => 0, :scale => 1, :add => 2, :relu => 3, :neg => 4, :abs => 5, :clamp => 6, :square => 7)

shape(nt) = GkShape(get(nt, :M, 0), get(nt, :N, 0), get(nt, :K, 0))

"Layout type of the reference (e.g. `Layout.Padded{Layout.UnsafeAlignedColMajor{Float16}, 8}`) -> GkLayout"
function lower_layout(L::Type, ld::Integer = 0)
    pad = 0
    if nameof(L) == :Padded
        pad = L.parameters[2]
        L = L.parameters[1]
    end
    GkLayout(LAYOUT_KIND[nameof(L)], DTYPE[L.parameters[1]], pad, 0, ld)
end

"A closed description of an elementwise function: a vector of (op, p0, p1)."
struct OpList; ops::Vector{Tuple{Symbol,Float32,Float32}}; end
OpList() = OpList(Tuple{Symbol,Float32,Float32}[])
scale(s) = OpList([(:scale, Float32(s), 0f0)])
relu() = OpList([(:relu, 0f0, 0f0)])
lower(t::OpList) = GkTransform(length(t.ops),
    ntuple(i -> i <= length(t.ops) ? GkOp(OP_KIND[t.ops[i][1]], t.ops[i][2], t.ops[i][3]) : GkOp(0, 0f0, 0f0), 4))

function last_error()
    buf = Vector{UInt8}(undef, 1024)
    ccall((:gk_last_error, libgk[]), Csize_t, (Ptr{UInt8}, Csize_t), buf, length(buf))
    unsafe_string(pointer(buf))
end

"""
    matmul(conf::GkConfig, a, b, c, d; transforms, epilogue, kernel, stream)

`a`, `b`, `c`, `d` are device pointers (`Ptr{Cvoid}`, e.g. `pointer(::ROCArray)`); `transforms` is a
tuple of 8 `OpList`s in the keyword order of the reference launcher (src/matmul.jl:8-15).
"""
function matmul(conf::GkConfig, a, b, c, d;
                transforms::NTuple{8,OpList} = ntuple(_ -> OpList(), 8),
                epilogue::GkEpilogue = GkEpilogue(0, 0, C_NULL),
                kernel::Symbol = :matmul_singlestage, stream::Ptr{Cvoid} = C_NULL)
    tr = Ref(GkTransforms(map(lower, transforms)))
    ep = Ref(epilogue)
    cf = Ref(conf)
    rc = ccall((:gk_matmul, libgk[]), Cint,
               (Ref{GkConfig}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ref{GkTransforms}, Ref{GkEpilogue}, Int32, Ptr{Cvoid}),
               cf, a, b, c, d, tr, ep, KERNEL_KIND[kernel], stream)
    rc == 0 || throw(ConfigError(last_error(), rc))
    return d
end

"All ConfigError checks of the reference, on the host (src/config.jl:203-275, src/matmul.jl:28-41)."
function validate(conf::GkConfig, kernel::Symbol = :matmul_singlestage)
    rc = ccall((:gk_validate, libgk[]), Cint, (Ref{GkConfig}, Int32), Ref(conf), KERNEL_KIND[kernel])
    rc == 0 || throw(ConfigError(last_error(), rc))
    nothing
end

"`heuristic_block_shape` of the reference (src/config.jl:84-120), answered by the library."
function heuristic_block_shape(shared_a::Type, shared_b::Type, shared_c::Type, shared_d::Type)
    out = Ref(GkShape(0, 0, 0))
    rc = ccall((:gk_heuristic_block_shape, libgk[]), Cint,
               (Ref{GkLayout}, Ref{GkLayout}, Ref{GkLayout}, Ref{GkLayout}, Ref{GkShape}),
               Ref(lower_layout(shared_a)), Ref(lower_layout(shared_b)), Ref(lower_layout(shared_c)), Ref(lower_layout(shared_d)), out)
    rc == 0 || throw(ConfigError(last_error(), rc))
    (M = Int(out[].M), N = Int(out[].N), K = Int(out[].K))
end

"""
    specialize(conf::GkConfig, hooks; kernel = :matmul_pipelined) -> SpecializedKernel

A kernel compiled at run time for `conf` with its transform hooks inlined: the counterpart of the
reference's JIT-compiled kernel per `Config` with arbitrary functors (src/matmul.jl:38,
src/transform.jl:26-30).  `hooks` is a tuple of 8 entries in the keyword order of the reference launcher
(src/matmul.jl:8-15), each `nothing` (identity) or a C expression in the Float32 variable `x`, e.g.
`"x > 0.0f ? x : 0.01f * x"`.  The block shape of `conf` may be any tile the kernel template accepts.
"""
struct SpecializedKernel
    handle::Ptr{Cvoid}
    conf::GkConfig
end

function specialize(conf::GkConfig, hooks::NTuple{8,Union{Nothing,String}}; kernel::Symbol = :matmul_pipelined)
    strs = [h === nothing ? C_NULL : Base.unsafe_convert(Cstring, Base.cconvert(Cstring, h)) for h in hooks]
    handle = Ref{Ptr{Cvoid}}(C_NULL)
    GC.@preserve hooks begin
        check(ccall((:gk_rtc_compile, libgk[]), Cint, (Ref{GkConfig}, Ptr{Cstring}, Int32, Ref{Ptr{Cvoid}}),
                    Ref(conf), strs, KERNEL_KIND[kernel], handle))
    end
    SpecializedKernel(handle[], conf)
end

function kernel_name(k::SpecializedKernel)
    buf = Vector{UInt8}(undef, 256)
    check(ccall((:gk_rtc_kernel_name, libgk[]), Cint, (Ptr{Cvoid}, Ptr{UInt8}, Csize_t), k.handle, buf, length(buf)))
    unsafe_string(pointer(buf))
end

"Launch a specialised kernel; same operands, epilogue and stream as `matmul`."
function (k::SpecializedKernel)(a, b, c, d; epilogue::GkEpilogue = GkEpilogue(0, 0, C_NULL), stream::Ptr{Cvoid} = C_NULL)
    check(ccall((:gk_rtc_matmul, libgk[]), Cint,
                (Ptr{Cvoid}, Ref{GkConfig}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ref{GkEpilogue}, Ptr{Cvoid}),
                k.handle, Ref(k.conf), a, b, c, d, Ref(epilogue), stream))
    return d
end

# Device memory without AMDGPU.jl: the library's own thin wrappers over hipMalloc / hipMemcpy.
check(rc) = rc == 0 ? nothing : throw(ConfigError(last_error(), rc))
function dev_alloc(bytes::Integer)
    p = Ref{Ptr{Cvoid}}(C_NULL)
    check(ccall((:gk_dev_alloc, libgk[]), Cint, (Csize_t, Ref{Ptr{Cvoid}}), bytes, p))
    p[]
end
dev_free(p::Ptr{Cvoid}) = check(ccall((:gk_dev_free, libgk[]), Cint, (Ptr{Cvoid},), p))
function to_device(x::Array)
    p = dev_alloc(sizeof(x))
    check(ccall((:gk_copy_to_device, libgk[]), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t), p, x, sizeof(x)))
    p
end
function to_host!(x::Array, p::Ptr{Cvoid})
    check(ccall((:gk_copy_to_host, libgk[]), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t), x, p, sizeof(x)))
    x
end
synchronize() = check(ccall((:gk_synchronize, libgk[]), Cint, ()))

function __init__()
    sizes = (sizeof(GkConfig), sizeof(GkLayout), sizeof(GkOperator), sizeof(GkTransforms), sizeof(GkEpilogue), sizeof(GkGett))
    isfile(libgk[]) || return
    for (i, s) in enumerate(sizes)
        n = ccall((:gk_sizeof, libgk[]), Int32, (Int32,), i - 1)
        n == s || error("ABI mismatch for struct $(i - 1): library $n bytes, Julia mirror $s bytes")
    end
end

end # module
