# Julia host layer of libgemmkernels_hip.so: the reference's own API above the launcher -- Config, get_config,
# create_config, matmatmul!, mul! and the component modules Layout, Operator, Transform, Epilogue, CTASwizzle,
# Kernel (reference src/config.jl, src/matmul.jl, src/layout.jl, src/operator.jl, src/transform.jl,
# src/epilogue.jl, src/cta-swizzle.jl, src/kernel.jl) -- lowered to the plain structs of
# include/gemmkernels_hip.h and launched with ccall.  Everything below `matmul` (the kernels) is in the library.
#
# Julia is not available in the image this library is built and tested in, so this file has not been executed
# there; the tested host layer is the Python package next to it, which has the same structure function for
# function (gemmkernels/config.py, matmul.py, transform.py ...).  A CPU test checks this file's struct mirrors
# against the header field by field and that every name the integration notes use is defined here.
#
# Device arrays: anything with `pointer`, `size`, `strides` and `eltype` (an AMDGPU.jl ROCArray), or the
# `DeviceArray` of this module, which owns memory from the library's own gk_dev_alloc.
module GemmKernelsHIP

export Layout, Operator, Transform, Epilogue, CTASwizzle, Kernel, Config, ConfigError, get_config, create_config,
       matmul, matmatmul!, mul!, DeviceArray, to_device, to_host, BFloat16

const libgk = Ref{String}(joinpath(@__DIR__, "..", "..", "..", "lib", "libgemmkernels_hip.so"))
const WARP_SIZE = 64          # lanes of a wavefront: the reference's 32 (src/matmul.jl:24) is 64 on this hardware
const NUM_CUS = 256

struct ConfigError <: Exception          # reference src/config.jl:78-82
    message::String
    status::Cint
end
ConfigError(message::AbstractString) = ConfigError(String(message), Cint(10))
Base.showerror(io::IO, e::ConfigError) = print(io, "ConfigError: ", e.message)

"bfloat16 as an element-type tag and storage type (Julia's Base has none); BFloat16s.BFloat16 is accepted as well."
primitive type BFloat16 <: AbstractFloat 16 end

# ------------------------------------------------------------------------------------------------------------
# Mirrors of the C structs (field order and types as in the header; checked against gk_sizeof at load time)
# ------------------------------------------------------------------------------------------------------------
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
const DTYPE = Dict{Symbol,Int32}(:Float16 => 0, :BFloat16 => 1, :Float32 => 2, :Float64 => 3, :Int16 => 4, :Int32 => 5, :Int64 => 6)
const LAYOUT_KIND = Dict{Symbol,Int32}(:Zero => 0, :ColMajor => 1, :RowMajor => 2, :UnsafeAlignedColMajor => 3,
                                       :UnsafeAlignedRowMajor => 4, :Diagonal => 5, :InterleavedColMajor => 6,
                                       :InterleavedRowMajor => 7, :SplitColMajor => 8, :SplitRowMajor => 9, :GETT => 10)
const KERNEL_KIND = Dict{Symbol,Int32}(:matmul_singlestage => 0, :matmul_pipelined => 1, :matmul_pipelined_ng => 2, :matmul_split_k => 3)
const OP_KIND = Dict{Symbol,Int32}(:identity => 0, :scale => 1, :add => 2, :relu => 3, :neg => 4, :abs => 5, :clamp => 6, :square => 7)
const OPERATOR_KIND = Dict{Symbol,Int32}(:MFMAOp => 0, :WMMAOp => 0, :FPUOp => 1, :TropicalFPUOp => 2, :MFMAComplexOp => 3,
                                         :WMMAComplexOp => 3, :MFMADualOp => 4, :WMMADualOp => 4)
const SWIZZLE_KIND = Dict{Symbol,Int32}(:Identity => 0, :HorizontallyTiled => 1, :VerticallyTiled => 2, :LebesgueCurve => 3, :XCDAware => 4)
const EPILOGUE_KIND = Dict{Symbol,Int32}(:Default => 0, :Bias => 1, :BiasRow => 2)

"gk_dtype code of an element type (by name, so that BFloat16s.BFloat16 and this module's BFloat16 both work)"
function dtype_code(T::Type)
    name = nameof(T)
    haskey(DTYPE, name) || throw(ConfigError("element type $T has no counterpart in the library"))
    DTYPE[name]
end

shape(nt) = GkShape(get(nt, :M, 0), get(nt, :N, 0), get(nt, :K, 0))

check(rc) = rc == 0 ? nothing : throw(ConfigError(last_error(), rc))

function last_error()
    buf = Vector{UInt8}(undef, 2048)
    ccall((:gk_last_error, libgk[]), Csize_t, (Ptr{UInt8}, Csize_t), buf, length(buf))
    GC.@preserve buf unsafe_string(pointer(buf))
end

# ------------------------------------------------------------------------------------------------------------
# Layout (reference src/layout.jl): types only describe; the loads and stores they stand for are in the kernels
# ------------------------------------------------------------------------------------------------------------
module Layout
    abstract type LayoutBase{T} end
    struct Zero{T} <: LayoutBase{T} end                       # :82-89
    struct ColMajor{T} <: LayoutBase{T} end                   # :111-148
    struct RowMajor{T} <: LayoutBase{T} end                   # :156-184
    struct UnsafeAlignedColMajor{T} <: LayoutBase{T} end      # :192-219
    struct UnsafeAlignedRowMajor{T} <: LayoutBase{T} end      # :244-270
    struct Diagonal{T} <: LayoutBase{T} end                   # :225-236
    struct InterleavedColMajor{T} <: LayoutBase{T} end        # :276-302
    struct InterleavedRowMajor{T} <: LayoutBase{T} end        # :310-334
    struct SplitColMajor{T} <: LayoutBase{T} end              # :340-372
    struct SplitRowMajor{T} <: LayoutBase{T} end              # :380-411
    struct Padded{L,P} end                                    # :95-105

    # The helpers below read a layout type by its name and parameters, so they also take the layout types of
    # GemmKernels.jl itself (Layout.Padded{Layout.UnsafeAlignedColMajor{Float16}, 8} has the same shape there).
    base(L::Type) = nameof(L) == :Padded ? L.parameters[1] : L
    padding(L::Type) = nameof(L) == :Padded ? Int(L.parameters[2]) : 0
    eltype(L::Type) = base(L).parameters[1]                  # :75
    kind_name(L::Type) = nameof(base(L))

    is_row_major(L::Type) = kind_name(L) in (:RowMajor, :UnsafeAlignedRowMajor, :InterleavedRowMajor, :SplitRowMajor)
    is_aligned(L::Type) = kind_name(L) in (:UnsafeAlignedColMajor, :UnsafeAlignedRowMajor)
    is_checked(L::Type) = kind_name(L) in (:ColMajor, :RowMajor)

    "reference src/layout.jl:76, :113, :152, :194, :246, :342-345, :381-383"
    function physical_size(L::Type, logical_size)
        t = Tuple(logical_size)
        P = padding(L)
        k = kind_name(L)
        if k in (:RowMajor, :UnsafeAlignedRowMajor)
            return P > 0 ? (t[2] + P, t[1]) : t
        elseif k == :SplitRowMajor
            return P > 0 ? (t[2] + P, t[1], 2) : (t..., 2)
        elseif k == :SplitColMajor
            return (t[1] + P, t[2:end]..., 2)
        end
        (t[1] + P, t[2:end]...)
    end
end # module Layout

"Layout type (e.g. `Layout.Padded{Layout.UnsafeAlignedColMajor{Float16}, 8}`) and leading dimension -> GkLayout"
function lower_layout(L::Type, ld::Integer = 0)
    GkLayout(LAYOUT_KIND[Layout.kind_name(L)], dtype_code(Layout.eltype(L)), Layout.padding(L), 0, ld)
end

# ------------------------------------------------------------------------------------------------------------
# Operator (reference src/operator.jl)
# ------------------------------------------------------------------------------------------------------------
module Operator
    # the matrix-core operator: MFMAOp{32,32,16,CT,AT}; WMMAOp keeps the reference's name and shapes (:163-245)
    struct MFMAOp{M,N,K,CT,AT} end
    const WMMAOp = MFMAOp
    struct MFMAComplexOp{M,N,K,CT,AT} end                     # :251-314
    const WMMAComplexOp = MFMAComplexOp
    struct MFMADualOp{M,N,K,CT,AT} end                        # :320-372
    const WMMADualOp = MFMADualOp
    struct FPUOp{M,N,K,mb,nb,kb,CT,AT} end                    # :35-153; base shape mb * nb = 64 lanes here
    struct TropicalFPUOp{M,N,K,mb,nb,kb,CT,AT} end            # :134-137

    # read by name and parameters, so the operator types of GemmKernels.jl itself are taken as well
    is_fpu(O::Type) = nameof(O) in (:FPUOp, :TropicalFPUOp)
    is_mfma(O::Type) = nameof(O) in (:MFMAOp, :WMMAOp)
    shape(O::Type) = (M = Int(O.parameters[1]), N = Int(O.parameters[2]), K = Int(O.parameters[3]))      # :41, :165, :253, :322
    base_shape(O::Type) = is_fpu(O) ? merge(shape(O), (mb = Int(O.parameters[4]), nb = Int(O.parameters[5]), kb = Int(O.parameters[6]))) :
                                      merge(shape(O), (mb = 0, nb = 0, kb = 0))                          # :42
    compute_type(O::Type) = O.parameters[end - 1]
    accum_type(O::Type) = O.parameters[end]
end # module Operator

function lower_operator(O::Type)
    bs = Operator.base_shape(O)
    GkOperator(OPERATOR_KIND[nameof(O)], bs.M, bs.N, bs.K, bs.mb, bs.nb, bs.kb,
               dtype_code(Operator.compute_type(O)), dtype_code(Operator.accum_type(O)))
end

# ------------------------------------------------------------------------------------------------------------
# Transform (reference src/transform.jl:20-30).  A closure cannot cross a C ABI: Elementwise(f) calls f once on
# a symbolic value and records a short list of ops from the closed vocabulary (scale, add, relu, neg, abs, clamp,
# square).  `identity`, `x -> x * α`, `x -> max(x, 0)`, `x -> clamp(x, lo, hi)`, `x -> abs(x) + 1` ... are
# recognised; anything else raises ConfigError("unsupported transform").  Elementwise(expr = "...") carries a
# C expression in the Float32 variable x for a kernel specialised at run time instead.
# ------------------------------------------------------------------------------------------------------------
module Transform
    import ..ConfigError
    const MAX_OPS = 4

    "A closed description of an elementwise function: a vector of (op, p0, p1)."
    struct OpList
        ops::Vector{Tuple{Symbol,Float32,Float32}}
    end
    OpList() = OpList(Tuple{Symbol,Float32,Float32}[])

    "symbolic scalar that records the ops applied to it"
    struct Sym
        ops::Vector{Tuple{Symbol,Float32,Float32}}
    end
    Sym() = Sym(Tuple{Symbol,Float32,Float32}[])
    with(x::Sym, op::Symbol, p0 = 0, p1 = 0) = Sym(vcat(x.ops, [(op, Float32(p0), Float32(p1))]))
    unsupported() = throw(ConfigError("unsupported transform: only arithmetic with constants, max, min, clamp and abs can be lowered"))

    Base.:*(x::Sym, v::Real) = with(x, :scale, v)
    Base.:*(v::Real, x::Sym) = with(x, :scale, v)
    Base.:*(x::Sym, y::Sym) = x === y || x.ops == y.ops ? with(x, :square) : unsupported()
    Base.:/(x::Sym, v::Real) = with(x, :scale, 1 / v)
    Base.:+(x::Sym, v::Real) = with(x, :add, v)
    Base.:+(v::Real, x::Sym) = with(x, :add, v)
    Base.:-(x::Sym, v::Real) = with(x, :add, -v)
    Base.:-(v::Real, x::Sym) = with(with(x, :neg), :add, v)
    Base.:-(x::Sym) = with(x, :neg)
    Base.:+(x::Sym) = x
    Base.abs(x::Sym) = with(x, :abs)
    Base.:^(x::Sym, p::Integer) = p == 2 ? with(x, :square) : unsupported()
    Base.literal_pow(::typeof(^), x::Sym, ::Val{2}) = with(x, :square)
    Base.max(x::Sym, v::Real) = v == 0 ? with(x, :relu) : with(x, :clamp, v, Inf32)
    Base.max(v::Real, x::Sym) = max(x, v)
    Base.min(x::Sym, v::Real) = with(x, :clamp, -Inf32, v)
    Base.min(v::Real, x::Sym) = min(x, v)
    Base.clamp(x::Sym, lo::Real, hi::Real) = with(x, :clamp, lo, hi)
    Base.isless(::Sym, ::Real) = unsupported()          # data-dependent control flow cannot be lowered
    Base.isless(::Real, ::Sym) = unsupported()
    Base.:<(::Sym, ::Real) = unsupported()
    Base.:<(::Real, ::Sym) = unsupported()
    relu(x) = max(x, 0)
    square(x) = x * x

    struct Elementwise{F}                              # :20-24; Elementwise() is the identity
        func::F
        ops::OpList
        expr::Union{Nothing,String}
    end
    function Elementwise(f::F = identity; expr::Union{Nothing,String} = nothing) where {F}
        if expr !== nothing
            occursin("x", expr) || throw(ConfigError("unsupported transform: the expression does not depend on x"))
            return Elementwise{F}(f, OpList(), expr)
        end
        out = f(Sym())
        out isa Sym || throw(ConfigError("unsupported transform: the function does not depend on its argument"))
        ops = filter(op -> op[1] != :identity, out.ops)
        length(ops) <= MAX_OPS || throw(ConfigError("unsupported transform: more than $MAX_OPS elementwise ops in one hook"))
        Elementwise{F}(f, OpList(ops), nothing)
    end
    (t::Elementwise)(x, tile = nothing) = t.func.(x)    # host evaluation, :26
    is_identity(t::Elementwise) = isempty(t.ops.ops) && t.expr === nothing
end # module Transform

lower(t::Transform.OpList) = GkTransform(length(t.ops),
    ntuple(i -> i <= length(t.ops) ? GkOp(OP_KIND[t.ops[i][1]], t.ops[i][2], t.ops[i][3]) : GkOp(0, 0f0, 0f0), 4))

"A transform (this module's Transform.Elementwise, GemmKernels.jl's own -- anything with a `func` field -- or a plain function) -> GkTransform"
lower_transform(t::Transform.Elementwise) =
    t.expr === nothing ? lower(t.ops) : throw(ConfigError("expression transforms need a specialised kernel (specialize)"))
lower_transform(f::Function) = lower_transform(Transform.Elementwise(f))
lower_transform(::Nothing) = lower(Transform.OpList())
lower_transform(t) = hasproperty(t, :func) ? lower_transform(Transform.Elementwise(t.func)) : throw(ConfigError("unsupported transform"))

# ------------------------------------------------------------------------------------------------------------
# Epilogue (reference src/epilogue.jl)
# ------------------------------------------------------------------------------------------------------------
module Epilogue
    struct Default end                                        # :14-34
    "adds bias[j], one Float32 per COLUMN j of D, before the shared_to_global_d transform (:40-73)"
    struct Bias{B}
        bias_pointer::B
    end
    "adds bias[i], one value per ROW i of D; no counterpart in the reference"
    struct BiasRow{B}
        bias_pointer::B
    end
end # module Epilogue

"an epilogue object (by type name, so GemmKernels.jl's Epilogue.Default / Epilogue.Bias are taken as they are) -> GkEpilogue"
function lower_epilogue(e)
    name = nameof(typeof(e))
    haskey(EPILOGUE_KIND, name) || throw(ConfigError("unsupported epilogue $name"))
    GkEpilogue(EPILOGUE_KIND[name], 0, name == :Default ? C_NULL : devptr(e.bias_pointer))
end

# ------------------------------------------------------------------------------------------------------------
# CTASwizzle (reference src/cta-swizzle.jl); XCDAware{G} has no counterpart there: it undoes the round-robin deal
# of workgroups over the 8 XCDs and walks the tile grid in panels G tiles high
# ------------------------------------------------------------------------------------------------------------
module CTASwizzle
    struct Identity end                                       # :26-41
    struct HorizontallyTiled{N} end                           # :67-82
    struct VerticallyTiled{N} end                             # :102-117
    struct LebesgueCurve end                                  # :147-160
    struct XCDAware{N} end
    param(S::Type) = isempty(S.parameters) ? 0 : Int(S.parameters[1])
end # module CTASwizzle

lower_swizzle(S::Type) = GkSwizzle(SWIZZLE_KIND[nameof(S)], CTASwizzle.param(S))

const EMPTY_DIM = GkGettDim(0, ntuple(_ -> Int32(0), 4), ntuple(_ -> Int64(0), 4), ntuple(_ -> Int64(0), 4))
"the index-map block of a configuration without tensor-contraction layouts"
empty_gett() = GkGett(EMPTY_DIM, EMPTY_DIM, EMPTY_DIM)

"one GEMM dimension of a contraction from (extent, stride0, stride1) triples, fastest mode first"
function gett_dim(modes)
    length(modes) <= 4 || throw(ConfigError("at most 4 tensor modes per GEMM dimension"))
    pad(f, T) = ntuple(i -> i <= length(modes) ? T(f(modes[i])) : T(0), 4)
    GkGettDim(length(modes), pad(m -> m[1], Int32), pad(m -> m[2], Int64), pad(m -> m[3], Int64))
end

# ------------------------------------------------------------------------------------------------------------
# Kernel (reference src/kernel.jl): the three names are kept; matmul_split_k is an addition (K slices as separate
# workgroups of one launch, ordered reduction in a workspace)
# ------------------------------------------------------------------------------------------------------------
module Kernel
    function matmul_singlestage end                            # :10-129
    function matmul_pipelined end                              # :147-350
    function matmul_pipelined_ng end                           # :368-574
    function matmul_split_k end
end # module Kernel

# ------------------------------------------------------------------------------------------------------------
# Config and get_config (reference src/config.jl:3-41, :180-316), defaults re-derived for 64-lane waves, 160 KiB
# of LDS and the tile table compiled into the library
# ------------------------------------------------------------------------------------------------------------
struct Config
    matmul_shape; block_shape; warps_per_block::Int
    mem_a_warp; mem_a_thread; mem_b_warp; mem_b_thread; mem_cd_warp; mem_cd_thread
    compute_warp; compute_op_shape
    global_a_layout::Type; global_b_layout::Type; global_c_layout::Type; global_d_layout::Type
    shared_a_layout::Type; shared_b_layout::Type; shared_c_layout::Type; shared_d_layout::Type
    operator::Type
    is_a_col_major::Bool; is_b_col_major::Bool
    cta_swizzle::Type
    gett::GkGett
end

function Base.show(io::IO, conf::Config)                      # reference src/config.jl:43-76
    for name in fieldnames(Config)
        name == :gett && continue
        println(io, rpad(string(name, ":"), 20), getfield(conf, name))
    end
end

# block shape -> waves (M x N) of the instances compiled into the library
const MFMA_TILES = [((256, 256, 64), (2, 4)), ((256, 256, 32), (2, 4)), ((256, 128, 64), (2, 2)), ((128, 256, 64), (2, 2)),
                    ((128, 128, 32), (2, 2)), ((128, 128, 64), (2, 2)), ((64, 64, 64), (2, 2)), ((64, 64, 32), (2, 2))]
# throughput of a CU that has one tile at a time, relative to 256 x 256 x 64 on four waves, measured; a pair: a launch with
# at most one tile per CU, a launch with several (the small tiles are bound by latency when alone)
const MFMA_TILE_RATE = Dict((256, 256, 64) => (1.0, 1.0), (256, 256, 32) => (0.68, 0.68), (256, 128, 64) => (0.61, 0.70),
                            (128, 256, 64) => (0.62, 0.72), (128, 128, 32) => (0.415, 0.345), (128, 128, 64) => (0.39, 0.39),
                            (64, 64, 64) => (0.169, 0.169), (64, 64, 32) => (0.163, 0.13))
# tile times of a launch: whole rounds for the tiles of which a CU holds one at a time; two 128 x 128 tiles run side by side
# in 1.15 times the time of one; the time of 64 x 64 tiles grows by about a third of a tile time per further tile of a CU
function tile_rounds(t, tiles)
    per_cu = tiles / NUM_CUS
    t[1] * t[2] >= 128 * 256 && return Float64(cld(tiles, NUM_CUS))
    per_cu <= 1 && return 1.0
    t[1] * t[2] >= 128 * 128 && return 1.15 * cld(tiles, 2 * NUM_CUS)
    1.0 + 0.36 * (per_cu - 1.0)
end
# complex / dual tiles (complex elements): one real product of the real views of A and B (interleaved or planar),
# the same table for every transpose
const COMPLEX_PAIR_TILES = [((128, 128, 64), (2, 4)), ((64, 64, 64), (2, 2)), ((64, 64, 32), (2, 2)), ((32, 32, 32), (2, 2))]
complex_tiles(operator::Type, a_kmajor::Bool, b_kmajor::Bool; planar::Bool = false) = COMPLEX_PAIR_TILES
const FPU_TILES = [((64, 64, 32), (2, 2)), ((128, 128, 16), (2, 2)), ((32, 32, 32), (2, 2)), ((32, 32, 32), (1, 1))]

"reference src/config.jl:84-120, unchanged (the reference-compatible answer; the launch uses the tile table)"
function heuristic_block_shape(shared_a::Type, shared_b::Type, shared_c::Type, shared_d::Type)
    out = Ref(GkShape(0, 0, 0))
    check(ccall((:gk_heuristic_block_shape, libgk[]), Cint,
                (Ref{GkLayout}, Ref{GkLayout}, Ref{GkLayout}, Ref{GkLayout}, Ref{GkShape}),
                Ref(lower_layout(shared_a)), Ref(lower_layout(shared_b)), Ref(lower_layout(shared_c)), Ref(lower_layout(shared_d)), out))
    (M = Int(out[].M), N = Int(out[].N), K = Int(out[].K))
end

"reference src/config.jl:124-134"
function adjacent_elements(num, parent_size, is_col_major)
    p = Tuple(parent_size)
    t = is_col_major ? (min(num, p[1]), num ÷ min(num, p[1])) : (num ÷ min(num, p[2]), min(num, p[2]))
    NamedTuple{keys(parent_size)}(t)
end

"MI355X block shape: of the tiles of the table that fit, the one with the shortest estimated launch"
function default_block_shape(operator::Type, gemm_shape; tile_sized::Bool = true, a_kmajor::Bool = false, b_kmajor::Bool = true, planar::Bool = false)
    M, N, K = gemm_shape.M, gemm_shape.N, gemm_shape.K
    if Operator.is_fpu(operator)
        small = nameof(operator) == :FPUOp && Operator.compute_type(operator) == Float32 && Operator.accum_type(operator) == Float32 &&
                tile_sized && M % 32 == 0 && N % 32 == 0 && K % 32 == 0 && cld(M, 64) * cld(N, 64) < NUM_CUS ÷ 2
        return small ? (M = 32, N = 32, K = 32) : (M = 64, N = 64, K = 32)
    elseif !Operator.is_mfma(operator)
        fitting = [t for (t, _) in complex_tiles(operator, a_kmajor, b_kmajor; planar = planar) if M % t[1] == 0 && N % t[2] == 0 && K % t[3] == 0]
        for t in fitting
            (M ÷ t[1]) * (N ÷ t[2]) >= NUM_CUS && return (M = t[1], N = t[2], K = t[3])
        end
        t = isempty(fitting) ? (64, 64, 32) : fitting[end]
        return (M = t[1], N = t[2], K = t[3])
    end
    fitting = [t for (t, _) in MFMA_TILES if !tile_sized || (M % t[1] == 0 && N % t[2] == 0 && K % t[3] == 0)]
    isempty(fitting) && return (M = 64, N = 64, K = 32)
    function cost(t)
        tiles = cld(M, t[1]) * cld(N, t[2])
        rate = MFMA_TILE_RATE[t][tiles <= NUM_CUS ? 1 : 2]
        t == (64, 64, 32) && tiles <= NUM_CUS && K >= 2048 && (rate = 0.24)      # a lone workgroup on a long K: four stages in flight
        tile_rounds(t, tiles) * t[1] * t[2] / rate
    end
    best = fitting[argmin(map(cost, fitting))]
    (M = best[1], N = best[2], K = best[3])
end

# One wave per SIMD: 256 x 256 x 64 on four waves with 128 x 128 wave tiles, compiled for plain products without hooks
# (whole tiles, or any extents with an FP32 C / D) and with hooks of D in closed form.  The library runs the 2 x 4
# arrangement of the same block shape, with the same bits, for any other launch of such a configuration.
const SOLO_TILE = (256, 256, 64)
const SOLO_WAVES = (2, 2)
const SOLO_COMPLEX_TILE = (128, 128, 64)       # in complex elements

function default_waves(operator::Type, block_shape; a_kmajor::Bool = false, b_kmajor::Bool = true, planar::Bool = false, whole_tiles::Bool = false)
    key = (block_shape.M, block_shape.N, block_shape.K)
    Operator.is_mfma(operator) && key == SOLO_TILE && whole_tiles && return SOLO_WAVES
    # the tiles with a side of 192 (a caller's choice of block_shape): four waves in whole tiles, else the eight waves that
    # share the 192 side in pairs
    Operator.is_mfma(operator) && key in ((256, 192, 64), (192, 256, 64)) && return whole_tiles ? SOLO_WAVES : (key[1] == 256 ? (4, 2) : (2, 4))
    # ... and the complex / dual product on interleaved matrices of an 'N','N' launch, whose real tile is that tile
    # (planar matrices: every transpose)
    !Operator.is_fpu(operator) && !Operator.is_mfma(operator) && key == SOLO_COMPLEX_TILE && whole_tiles && (planar || (!a_kmajor && b_kmajor)) && return SOLO_WAVES
    table = Operator.is_fpu(operator) ? FPU_TILES : (Operator.is_mfma(operator) ? MFMA_TILES : complex_tiles(operator, a_kmajor, b_kmajor; planar = planar))
    for (t, w) in table
        t == key && return w
    end
    nothing
end

require_tile_sized_global(L::Type) = !(Layout.kind_name(L) == :Zero || Layout.is_checked(L))      # reference src/config.jl:175-178

"""
    get_config(; gemm_shape, operator, global_a_layout, global_c_layout, kwargs...)

reference src/config.jl:180-316 with the same keywords.  Every check of the reference is run by the library
(gk_validate) and raises ConfigError.
"""
function get_config(; gemm_shape, operator, global_a_layout, global_c_layout, kwargs...)
    params = Dict{Symbol,Any}(kwargs)
    global_b_layout = get(params, :global_b_layout, global_a_layout)
    global_d_layout = get(params, :global_d_layout, global_c_layout)
    padded(L) = Layout.kind_name(L) in (:Zero, :Diagonal) ? L : Layout.Padded{L,16 ÷ sizeof(Layout.eltype(L))}
    shared_a_layout = get(params, :shared_a_layout, padded(global_a_layout))
    shared_b_layout = get(params, :shared_b_layout, padded(global_b_layout))
    shared_c_layout = get(params, :shared_c_layout, global_c_layout)
    shared_d_layout = get(params, :shared_d_layout, global_d_layout)

    globals = (global_a_layout, global_b_layout, global_c_layout, global_d_layout)
    tile_sized = any(require_tile_sized_global, globals)
    a_kmajor = Layout.is_row_major(global_a_layout)             # 'T' A: stored K x M, k contiguous
    b_kmajor = !Layout.is_row_major(global_b_layout)            # 'N' B: stored K x N, k contiguous
    planar = Layout.kind_name(global_a_layout) in (:SplitColMajor, :SplitRowMajor)      # planar complex global matrices
    block_shape = get(params, :block_shape, default_block_shape(operator, gemm_shape; tile_sized = tile_sized, a_kmajor = a_kmajor, b_kmajor = b_kmajor, planar = planar))
    op_shape = Operator.shape(operator)

    whole_tiles = gemm_shape.M % block_shape.M == 0 && gemm_shape.N % block_shape.N == 0 && gemm_shape.K % block_shape.K == 0
    if Operator.is_mfma(operator) && !haskey(params, :gett)
        # (the plain product also where tiles stick out over the edges; the library runs the eight-wave arrangement
        # where C / D are not FP32)
        whole_tiles = whole_tiles || (gemm_shape.M >= 8 && gemm_shape.K >= 64)
    end
    waves = default_waves(operator, block_shape; a_kmajor = a_kmajor, b_kmajor = b_kmajor, planar = planar, whole_tiles = whole_tiles)
    if waves !== nothing
        warps_default = waves[1] * waves[2]
        compute_warp_default = (M = block_shape.M ÷ waves[1], N = block_shape.N ÷ waves[2], K = op_shape.K)
    else        # reference src/config.jl:216-229: 8 warps as 4 x 2 unless the block is too small for that
        warps_default = 8
        compute_warp_default = (M = block_shape.M ÷ 4, N = block_shape.N ÷ 2, K = op_shape.K)
        if block_shape.M ÷ op_shape.M < 4 || block_shape.N ÷ op_shape.N < 2
            compute_warp_default = (M = max(op_shape.M, block_shape.M ÷ 4), N = max(op_shape.N, block_shape.N ÷ 2), K = op_shape.K)
            warps_default = min(block_shape.M ÷ op_shape.M, 4) * min(block_shape.N ÷ op_shape.N, 2)
        end
    end
    warps_per_block = get(params, :warps_per_block, warps_default)
    compute_warp = get(params, :compute_warp, compute_warp_default)

    is_a_col_major = get(params, :is_a_col_major, true)
    is_b_col_major = get(params, :is_b_col_major, true)
    is_cd_col_major = get(params, :is_cd_col_major, true)

    # reference src/config.jl:240-260 with 64 lanes: 16 bytes per lane
    lanes = WARP_SIZE * max(1, warps_per_block)
    per_lane(L, elems) = max(1, min(16 ÷ sizeof(Layout.eltype(L)), elems ÷ lanes))
    n_a = per_lane(global_a_layout, block_shape.M * block_shape.K)
    n_b = per_lane(global_b_layout, block_shape.K * block_shape.N)
    n_c = per_lane(global_c_layout, block_shape.M * block_shape.N)
    mk = (M = block_shape.M, K = block_shape.K); kn = (K = block_shape.K, N = block_shape.N); mn = (M = block_shape.M, N = block_shape.N)
    mem_a_warp = get(params, :mem_a_warp, adjacent_elements(WARP_SIZE * n_a, mk, is_a_col_major))
    mem_b_warp = get(params, :mem_b_warp, adjacent_elements(WARP_SIZE * n_b, kn, is_b_col_major))
    mem_cd_warp = get(params, :mem_cd_warp, adjacent_elements(WARP_SIZE * n_c, mn, is_cd_col_major))
    mem_a_thread = get(params, :mem_a_thread, adjacent_elements(n_a, mk, is_a_col_major))
    mem_b_thread = get(params, :mem_b_thread, adjacent_elements(n_b, kn, is_b_col_major))
    mem_cd_thread = get(params, :mem_cd_thread, adjacent_elements(n_c, mn, is_cd_col_major))

    # reference src/config.jl:277-279 defaults to Identity; here the XCD-aware walk is the default
    n_tiles = cld(gemm_shape.M, block_shape.M) * cld(gemm_shape.N, block_shape.N)
    cta_swizzle = get(params, :cta_swizzle, CTASwizzle.XCDAware{n_tiles >= 4096 ? 16 : (n_tiles >= NUM_CUS ? 8 : 4)})

    conf = Config(gemm_shape, block_shape, warps_per_block, mem_a_warp, mem_a_thread, mem_b_warp, mem_b_thread,
                  mem_cd_warp, mem_cd_thread, compute_warp, op_shape,
                  global_a_layout, global_b_layout, global_c_layout, global_d_layout,
                  shared_a_layout, shared_b_layout, shared_c_layout, shared_d_layout,
                  operator, is_a_col_major, is_b_col_major, cta_swizzle, get(params, :gett, empty_gett()))
    validate(conf, get(params, :kernel, Kernel.matmul_singlestage))
    conf
end

"""
Config (reference src/config.jl:3-41) -> GkConfig, field by field; leading dimensions come from the arrays of the
call.  `conf` is this module's Config or GemmKernels.jl's own: the 23 fields have the same names, and their
values are read by name and type parameters.
"""
function lower(conf, lda::Integer = 0, ldb::Integer = 0, ldc::Integer = 0, ldd::Integer = 0)
    GkConfig(shape(conf.matmul_shape), shape(conf.block_shape), conf.warps_per_block,
             shape(conf.mem_a_warp), shape(conf.mem_a_thread), shape(conf.mem_b_warp), shape(conf.mem_b_thread),
             shape(conf.mem_cd_warp), shape(conf.mem_cd_thread), shape(conf.compute_warp), shape(conf.compute_op_shape),
             lower_layout(conf.global_a_layout, lda), lower_layout(conf.global_b_layout, ldb),
             lower_layout(conf.global_c_layout, ldc), lower_layout(conf.global_d_layout, ldd),
             lower_layout(conf.shared_a_layout), lower_layout(conf.shared_b_layout),
             lower_layout(conf.shared_c_layout), lower_layout(conf.shared_d_layout),
             lower_operator(conf.operator), conf.is_a_col_major, conf.is_b_col_major,
             lower_swizzle(conf.cta_swizzle), hasproperty(conf, :gett) ? conf.gett : empty_gett())
end

kernel_code(k) = KERNEL_KIND[nameof(k)]
kernel_code(k::Symbol) = KERNEL_KIND[k]

"All ConfigError checks of the reference, on the host (src/config.jl:203-275, src/matmul.jl:28-41)."
function validate(conf, kernel = Kernel.matmul_singlestage)
    check(ccall((:gk_validate, libgk[]), Cint, (Ref{GkConfig}, Int32), Ref(lower(conf)), kernel_code(kernel)))
end

"Kernel.shmem_size (reference src/kernel.jl:131-145, 352-366): LDS bytes of the instance the launch runs"
function shmem_size(conf, kernel = Kernel.matmul_singlestage)
    n = ccall((:gk_shmem_size, libgk[]), Int64, (Ref{GkConfig}, Int32), Ref(lower(conf)), kernel_code(kernel))
    n >= 0 || throw(ConfigError(last_error(), Cint(10)))
    Int(n)
end

"the reference's own formula for Kernel.shmem_size: max(size_c, size_a + size_b, size_d) over the shared layouts"
function reference_shmem_size(conf)
    n = ccall((:gk_reference_shmem_size, libgk[]), Int64, (Ref{GkConfig},), Ref(lower(conf)))
    n >= 0 || throw(ConfigError(last_error(), Cint(1)))
    Int(n)
end

"CTASwizzle.number_of_blocks (reference src/cta-swizzle.jl:28-31, 69-72, 104-107, 149-151)"
function number_of_blocks(conf)
    bx = Ref{Int32}(0); by = Ref{Int32}(0)
    check(ccall((:gk_number_of_blocks, libgk[]), Cint, (Ref{GkConfig}, Ref{Int32}, Ref{Int32}), Ref(lower(conf)), bx, by))
    (Int(bx[]), Int(by[]))
end

# ------------------------------------------------------------------------------------------------------------
# Device arrays
# ------------------------------------------------------------------------------------------------------------
"column-major device array over memory from the library's own allocator (for sessions without AMDGPU.jl)"
mutable struct DeviceArray{T,N}
    ptr::Ptr{Cvoid}
    dims::NTuple{N,Int}
end
Base.size(x::DeviceArray) = x.dims
Base.size(x::DeviceArray, i::Integer) = i <= length(x.dims) ? x.dims[i] : 1
Base.eltype(::DeviceArray{T}) where {T} = T
Base.strides(x::DeviceArray) = ntuple(i -> prod(x.dims[1:i-1]; init = 1), length(x.dims))
Base.stride(x::DeviceArray, i::Integer) = strides(x)[i]
Base.pointer(x::DeviceArray) = x.ptr
Base.ndims(::DeviceArray{T,N}) where {T,N} = N

function dev_alloc(bytes::Integer)
    p = Ref{Ptr{Cvoid}}(C_NULL)
    check(ccall((:gk_dev_alloc, libgk[]), Cint, (Csize_t, Ref{Ptr{Cvoid}}), bytes, p))
    p[]
end
dev_free(p::Ptr{Cvoid}) = check(ccall((:gk_dev_free, libgk[]), Cint, (Ptr{Cvoid},), p))
function DeviceArray{T}(dims::Integer...) where {T}
    x = DeviceArray{T,length(dims)}(dev_alloc(sizeof(T) * prod(dims)), map(Int, dims))
    finalizer(y -> dev_free(y.ptr), x)
end
function to_device(x::Array{T}) where {T}
    d = DeviceArray{T}(size(x)...)
    GC.@preserve x check(ccall((:gk_copy_to_device, libgk[]), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t), d.ptr, pointer(x), sizeof(x)))
    d
end
function to_host(d::DeviceArray{T}) where {T}
    x = Array{T}(undef, d.dims...)
    GC.@preserve x check(ccall((:gk_copy_to_host, libgk[]), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t), pointer(x), d.ptr, sizeof(x)))
    x
end
synchronize() = check(ccall((:gk_synchronize, libgk[]), Cint, ()))

"raw device address of an operand (a device array, a raw pointer, or nothing)"
devptr(x::DeviceArray) = x.ptr
devptr(p::Ptr) = Ptr{Cvoid}(p)
devptr(::Nothing) = C_NULL
devptr(x) = Ptr{Cvoid}(UInt(pointer(x)))            # ROCArray and friends

"leading dimension of a column-major device matrix, in elements (complex elements for Complex arrays)"
leading_dim(::Nothing) = 0
leading_dim(x) = ndims(x) >= 2 ? (size(x, 2) > 1 ? stride(x, 2) : max(size(x, 1), 1)) : 0

"the HIP stream launches go to: NULL (the default stream) unless the caller passes one (e.g. AMDGPU.stream().stream)"
current_stream() = C_NULL

# ------------------------------------------------------------------------------------------------------------
# matmul: the launcher (reference src/matmul.jl:7-44), same positional and keyword arguments
# ------------------------------------------------------------------------------------------------------------
const split_k_workspaces = Dict{Ptr{Cvoid},DeviceArray{UInt8,1}}()       # one zeroed workspace per stream, grown on demand

function split_k_workspace(cf::GkConfig, stream::Ptr{Cvoid})
    need = Ref{Csize_t}(0)
    check(ccall((:gk_split_k_workspace_size, libgk[]), Cint, (Ref{GkConfig}, Ref{Csize_t}), Ref(cf), need))
    need[] == 0 && return (C_NULL, Csize_t(0))
    ws = get(split_k_workspaces, stream, nothing)
    if ws === nothing || length(ws.dims) == 0 || ws.dims[1] < need[]
        ws = to_device(zeros(UInt8, max(Int(need[]), 1 << 20)))      # the arrival counters at its head must start at zero
        split_k_workspaces[stream] = ws
    end
    (ws.ptr, Csize_t(ws.dims[1]))
end

function matmul(conf, a, b, c, d;
                transform_global_to_shared_a = Transform.Elementwise(), transform_global_to_shared_b = Transform.Elementwise(),
                transform_global_to_shared_c = Transform.Elementwise(), transform_shared_to_global_d = Transform.Elementwise(),
                transform_shared_to_regs_a = Transform.Elementwise(), transform_shared_to_regs_b = Transform.Elementwise(),
                transform_shared_to_regs_c = Transform.Elementwise(), transform_regs_to_shared_d = Transform.Elementwise(),
                epilogue = Epilogue.Default(), kernel = Kernel.matmul_singlestage, stream::Ptr{Cvoid} = current_stream())
    hooks = (transform_global_to_shared_a, transform_global_to_shared_b, transform_global_to_shared_c, transform_shared_to_global_d,
             transform_shared_to_regs_a, transform_shared_to_regs_b, transform_shared_to_regs_c, transform_regs_to_shared_d)
    cf = lower(conf, leading_dim(a), leading_dim(b), leading_dim(c), leading_dim(d))
    tr = Ref(GkTransforms(map(lower_transform, hooks)))
    ep = Ref(lower_epilogue(epilogue))
    if kernel_code(kernel) == KERNEL_KIND[:matmul_split_k]
        ws, ws_bytes = split_k_workspace(cf, stream)
        check(ccall((:gk_matmul_split_k, libgk[]), Cint,
                    (Ref{GkConfig}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ref{GkTransforms}, Ref{GkEpilogue}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                    Ref(cf), devptr(a), devptr(b), devptr(c), devptr(d), tr, ep, ws, ws_bytes, stream))
    else
        check(ccall((:gk_matmul, libgk[]), Cint,
                    (Ref{GkConfig}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ref{GkTransforms}, Ref{GkEpilogue}, Int32, Ptr{Cvoid}),
                    Ref(cf), devptr(a), devptr(b), devptr(c), devptr(d), tr, ep, kernel_code(kernel), stream))
    end
    d
end

# ------------------------------------------------------------------------------------------------------------
# Kernels specialised at run time: arbitrary functors as C expressions in x, any tile the kernel template accepts
# (the counterpart of the reference's JIT-compiled kernel per Config, src/matmul.jl:38, src/transform.jl:26-30)
# ------------------------------------------------------------------------------------------------------------
struct SpecializedKernel
    handle::Ptr{Cvoid}
    conf::Config
end

function specialize(conf::Config, hooks::NTuple{8,Union{Nothing,String}}; kernel = Kernel.matmul_pipelined)
    strs = [h === nothing ? Cstring(C_NULL) : Base.unsafe_convert(Cstring, Base.cconvert(Cstring, h)) for h in hooks]
    handle = Ref{Ptr{Cvoid}}(C_NULL)
    GC.@preserve hooks strs begin
        check(ccall((:gk_rtc_compile, libgk[]), Cint, (Ref{GkConfig}, Ptr{Cstring}, Int32, Ref{Ptr{Cvoid}}),
                    Ref(lower(conf)), strs, kernel_code(kernel), handle))
    end
    SpecializedKernel(handle[], conf)
end

function kernel_name(k::SpecializedKernel)
    buf = Vector{UInt8}(undef, 256)
    check(ccall((:gk_rtc_kernel_name, libgk[]), Cint, (Ptr{Cvoid}, Ptr{UInt8}, Csize_t), k.handle, buf, length(buf)))
    GC.@preserve buf unsafe_string(pointer(buf))
end

"Launch a specialised kernel; same operands, epilogue and stream as `matmul`."
function (k::SpecializedKernel)(a, b, c, d; epilogue = Epilogue.Default(), stream::Ptr{Cvoid} = current_stream())
    cf = lower(k.conf, leading_dim(a), leading_dim(b), leading_dim(c), leading_dim(d))
    check(ccall((:gk_rtc_matmul, libgk[]), Cint,
                (Ptr{Cvoid}, Ref{GkConfig}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ref{GkEpilogue}, Ptr{Cvoid}),
                k.handle, Ref(cf), devptr(a), devptr(b), devptr(c), devptr(d), Ref(lower_epilogue(epilogue)), stream))
    d
end

# ------------------------------------------------------------------------------------------------------------
# BLAS-like entry points (reference src/matmul.jl:52-215)
# ------------------------------------------------------------------------------------------------------------
"reference src/matmul.jl:52-56: the pipelined kernel when both operands are aligned"
select_kernel(layout_a::Type, layout_b::Type) =
    Layout.is_aligned(layout_a) && Layout.is_aligned(layout_b) ? Kernel.matmul_pipelined : Kernel.matmul_singlestage

const configs = Dict{Any,Any}()          # reference src/matmul.jl:58-65 (a plain Dict there as well: not thread-safe)

get_cached_config(args...) = get!(() -> create_config(args...), configs, args)

"""
reference src/matmul.jl:66-183 with the operator and block-shape choices of this library.  `aligned_pointers`
says whether A, B and C start on 16-byte boundaries (the reference decides from the strides alone and traps
on the device for a misaligned view, src/layout.jl:22-25; here such an operand gets the bounds-checked layout).
"""
function create_config(A::Type, sizeA::Dims, stridesA::Dims, transA::Bool,
                       B::Type, sizeB::Dims, stridesB::Dims, transB::Bool,
                       C::Type, sizeC::Dims, stridesC::Dims,
                       alpha::Type, zeroAlpha::Bool, beta::Type, zeroBeta::Bool,
                       wmma::Union{Bool,Nothing} = nothing, aligned_pointers::NTuple{3,Bool} = (true, true, true))
    m = sizeA[transA ? 2 : 1]
    k = sizeA[transA ? 1 : 2]
    n = sizeB[transB ? 1 : 2]
    if m != sizeC[1] || n != sizeC[2] || k != sizeB[transB ? 2 : 1]
        throw(DimensionMismatch("Dimensions do not match"))
    end

    a_layout_base = transA ? Layout.RowMajor : Layout.ColMajor
    b_layout_base = transB ? Layout.RowMajor : Layout.ColMajor
    a_aligned_layout_base = transA ? Layout.UnsafeAlignedRowMajor : Layout.UnsafeAlignedColMajor
    b_aligned_layout_base = transB ? Layout.UnsafeAlignedRowMajor : Layout.UnsafeAlignedColMajor

    # the matrix cores for 16-bit inputs with Float32 accumulation (reference src/matmul.jl:85-91)
    compute_type = promote_type(A, B)
    sixteen_bit = nameof(compute_type) in (:Float16, :BFloat16)
    supported = sixteen_bit && A == B && (C == Float32 || C == compute_type)
    use_mfma = wmma === nothing ? supported : wmma

    shared_a_layout = Layout.Padded{a_aligned_layout_base{use_mfma ? compute_type : A},8}
    shared_b_layout = Layout.Padded{b_aligned_layout_base{use_mfma ? compute_type : B},8}
    shared_c_layout = zeroBeta ? Layout.Zero{C} : Layout.UnsafeAlignedColMajor{C}
    shared_d_layout = Layout.UnsafeAlignedColMajor{C}

    operator = use_mfma ? Operator.MFMAOp{32,32,16,compute_type,C == Float16 ? Float32 : C} :
                          Operator.FPUOp{8,8,1,8,8,1,compute_type,C}
    a_aligned = (stridesA[2] * sizeof(A)) % 16 == 0 && aligned_pointers[1]
    b_aligned = (stridesB[2] * sizeof(B)) % 16 == 0 && aligned_pointers[2]
    c_aligned = (stridesC[2] * sizeof(C)) % 16 == 0 && aligned_pointers[3]

    # reference src/matmul.jl:121-156: vector loads and stores need 16-byte aligned columns and whole tiles
    function layouts_for(bs)
        if zeroAlpha
            ga, gb = Layout.Zero{A}, Layout.Zero{B}
        else
            ga = a_aligned && m % bs.M == 0 && k % bs.K == 0 ? a_aligned_layout_base{A} : a_layout_base{A}
            gb = b_aligned && k % bs.K == 0 && n % bs.N == 0 ? b_aligned_layout_base{B} : b_layout_base{B}
        end
        cd_aligned = c_aligned && m % bs.M == 0 && n % bs.N == 0
        gc = zeroBeta ? Layout.Zero{C} : (cd_aligned ? Layout.UnsafeAlignedColMajor{C} : Layout.ColMajor{C})
        gd = cd_aligned ? Layout.UnsafeAlignedColMajor{C} : Layout.ColMajor{C}
        (ga, gb, gc, gd)
    end

    # The library runs a 16-bit product on bounds-checked layouts on its aligned kernels all the same (any address
    # and leading dimension, tiles over the edge, a partial last K tile) as long as A and B hold one whole chunk of
    # 8 elements along their contiguous index: then the tile is chosen among all tiles, not only those that divide
    # the sizes, and the operands it does not divide get the bounds-checked layouts, as the reference's rule says.
    edge_ok = use_mfma && !zeroAlpha && (transA ? k : m) >= 8 && (transB ? n : k) >= 8
    block_shape = default_block_shape(operator, (M = m, N = n, K = k); tile_sized = !edge_ok)
    ga, gb, gc, gd = layouts_for(block_shape)
    if !edge_ok && any(Layout.is_checked, (ga, gb, gc, gd))
        block_shape = (M = 64, N = 64, K = 32)          # the bounds-checked kernels have one tile shape
        ga, gb, gc, gd = layouts_for(block_shape)
    end

    conf = get_config(; gemm_shape = (M = m, N = n, K = k), block_shape = block_shape, operator = operator,
                      global_a_layout = ga, global_b_layout = gb, global_c_layout = gc, global_d_layout = gd,
                      shared_a_layout = shared_a_layout, shared_b_layout = shared_b_layout,
                      shared_c_layout = shared_c_layout, shared_d_layout = shared_d_layout,
                      is_a_col_major = !transA, is_b_col_major = !transB)
    (conf, compute_type, select_kernel(ga, gb))
end

is_aligned_16(x) = UInt(devptr(x)) % 16 == 0

"""
    matmatmul!(C, transA, transB, A, B, alpha, beta; wmma = nothing)

reference src/matmul.jl:185-204: C = alpha * op(A) * op(B) + beta * C, alpha applied to A in the compute type,
beta to C in eltype(C).  'T' is a plain transpose; an Adjoint is treated as one (no conjugation, :211-213).
"""
function matmatmul!(C, transA::Char, transB::Char, A, B, alpha::Number, beta::Number; wmma::Union{Bool,Nothing} = nothing)
    tA, tB = transA == 'T', transB == 'T'
    conf, compute_type, kernel = get_cached_config(
        eltype(A), size(A), strides(A), tA, eltype(B), size(B), strides(B), tB,
        eltype(C), size(C), strides(C), typeof(alpha), iszero(alpha), typeof(beta), iszero(beta), wmma,
        (is_aligned_16(A), is_aligned_16(B), is_aligned_16(C)))
    alpha_c = convert(compute_type === BFloat16 ? Float32 : compute_type, alpha)       # :196
    beta_c = convert(eltype(C) === BFloat16 ? Float32 : eltype(C), beta)               # :197
    for (name, v) in (("alpha", alpha_c), ("beta", beta_c))
        Float64(Float32(v)) == Float64(v) || throw(ConfigError("$name = $v is not representable in binary32, the parameter type of the transform hooks"))
    end
    ta = isone(alpha_c) ? Transform.Elementwise() : Transform.Elementwise(x -> x * Float32(alpha_c))
    tc = (isone(beta_c) || iszero(beta)) ? Transform.Elementwise() : Transform.Elementwise(x -> x * Float32(beta_c))
    if Operator.is_mfma(conf.operator)
        # few output tiles and a long K loop: K slices as workgroups of one launch (ordered sum: same bits every run)
        bs, ms = conf.block_shape, conf.matmul_shape
        if cld(ms.M, bs.M) * cld(ms.N, bs.N) <= 256 && ms.K >= 2048
            kernel = Kernel.matmul_split_k
        end
    end
    matmul(conf, A, B, C, C; transform_shared_to_regs_a = ta, transform_shared_to_regs_c = tc, kernel = kernel)
    C
end

"lazy transpose of a device matrix (LinearAlgebra's Transpose / Adjoint wrappers are unwrapped the same way)"
struct Transposed{T}
    parent::T
end
unwrap(x::Transposed) = (x.parent, 'T')
unwrap(x) = hasproperty(x, :parent) && nameof(typeof(x)) in (:Transpose, :Adjoint) ? (x.parent, 'T') : (x, 'N')

"reference src/matmul.jl:207-215 (without the undefined `info` keyword it forwards there)"
function mul!(C, A, B, alpha = true, beta = false)
    a, tA = unwrap(A)
    b, tB = unwrap(B)
    matmatmul!(C, tA, tB, a, b, alpha, beta)
end

function __init__()
    sizes = (sizeof(GkConfig), sizeof(GkLayout), sizeof(GkOperator), sizeof(GkTransforms), sizeof(GkEpilogue), sizeof(GkGett))
    isfile(libgk[]) || return
    for (i, s) in enumerate(sizes)
        n = ccall((:gk_sizeof, libgk[]), Int32, (Int32,), i - 1)
        n == s || error("ABI mismatch for struct $(i - 1): library $n bytes, Julia mirror $s bytes")
    end
end

end # module
