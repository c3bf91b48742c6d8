/*
 * gemmkernels_hip.h -- C ABI of libgemmkernels_hip.so: the tiled GEMM hot path of GemmKernels.jl
 * as hand-written HIP kernels for gfx950 (MI355X).
 *
 * The library replaces everything below the reference's low-level launcher
 *     GemmKernels.matmul(conf, a, b, c, d; transforms..., epilogue, kernel)   (reference src/matmul.jl:7-44)
 * i.e. the three device kernels of reference src/kernel.jl and the device-side components they
 * compose (src/layout.jl, src/operator.jl, src/transform.jl, src/epilogue.jl, src/cta-swizzle.jl).
 * The host language layer (Julia, or the Python mirror shipped with this library) keeps
 * get_config / create_config / matmatmul! / mul! and lowers its Config, Transform and Epilogue
 * objects to the plain structs below.
 *
 * Conventions
 *  - All pointers a, b, c, d and bias are DEVICE pointers owned by the caller.  The launchers never
 *    allocate or free device memory; the one kind of launch that needs a workspace (K-split) takes it
 *    from the caller.  d may alias c.
 *  - Everything is column-major like the reference: an 'N' operand A is M x K with leading
 *    dimension lda >= M (layout kinds *_COL_MAJOR), a 'T' operand is the K x M array of its
 *    transpose (layout kinds *_ROW_MAJOR), reference src/matmul.jl:79-83.
 *  - A "warp" is a 64-lane wavefront: a block has warps_per_block * 64 threads.
 *  - Every function returns a gk_status; 0 is success.  No exception or abort crosses the ABI.
 *    The message of the last failure on the calling thread is kept for gk_last_error().
 *  - gk_matmul is asynchronous on the given HIP stream (NULL = the default stream) and may be
 *    called from several host threads.
 */
#ifndef GEMMKERNELS_HIP_H
#define GEMMKERNELS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GK_VERSION 100
#define GK_MAX_OPS 4      /* elementwise ops per transform hook */
#define GK_MAX_MODES 4    /* tensor modes per GEMM dimension (GETT) */

/* Status codes.  Every ConfigError the reference throws before a launch has a code
 * (reference src/config.jl:203-275, src/matmul.jl:28-41); DimensionMismatch is src/matmul.jl:75-77. */
typedef enum gk_status {
  GK_OK = 0,
  GK_ERR_INVALID_ARGUMENT = 1,   /* NULL pointer, unknown enum value */
  GK_ERR_LDS = 2,                /* "Requested too much shared memory"            src/matmul.jl:28-31 */
  GK_ERR_STAGES = 3,             /* pipelined kernel with BLOCK_K < 2*OPERATOR_K  src/matmul.jl:34-36 */
  GK_ERR_THREADS = 4,            /* more threads than a block can hold            src/matmul.jl:41    */
  GK_ERR_BLOCK_SHAPE = 5,        /* block too small / block vs operator shape     src/config.jl:203-212 */
  GK_ERR_OP_SHAPE = 6,           /* operator shape rules                          src/config.jl:136-173 */
  GK_ERR_MEM_TILE = 7,           /* mem_*_warp too big for the block              src/config.jl:263-265 */
  GK_ERR_TILE_MULTIPLE = 8,      /* tile divisibility                             src/config.jl:268-275 */
  GK_ERR_ALIGNMENT = 9,          /* pointer / leading dimension not 16-byte aligned for an aligned layout (src/layout.jl:22-34) */
  GK_ERR_UNSUPPORTED = 10,       /* valid configuration with no compiled kernel instance */
  GK_ERR_DIMENSION_MISMATCH = 11,
  GK_ERR_HIP = 12                /* HIP runtime error at launch */
} gk_status;

typedef enum gk_dtype { GK_F16 = 0, GK_BF16 = 1, GK_F32 = 2, GK_F64 = 3, GK_I16 = 4, GK_I32 = 5, GK_I64 = 6 } gk_dtype;

/* Operators (reference src/operator.jl).  GK_OP_MFMA stands where WMMAOp stands in the reference
 * (:163-245) and runs v_mfma_f32_16x16x32_{f16,bf16} (the operator shape a configuration names --
 * 32 x 32 x 16, or the reference's 16 x 16 x 16 WMMA shapes -- sets the granularity of the wave tiles, the
 * instruction is the library's choice); GK_OP_MFMA_COMPLEX is WMMAComplexOp
 * (:251-314), GK_OP_MFMA_DUAL is WMMADualOp (:320-372), GK_OP_FPU is FPUOp and
 * GK_OP_FPU_TROPICAL is TropicalFPUOp (:35-153). */
typedef enum gk_operator_kind {
  GK_OP_MFMA = 0,
  GK_OP_FPU = 1,
  GK_OP_FPU_TROPICAL = 2,
  GK_OP_MFMA_COMPLEX = 3,
  GK_OP_MFMA_DUAL = 4
} gk_operator_kind;

typedef struct gk_operator {
  int32_t kind;                 /* gk_operator_kind */
  int32_t M, N, K;              /* operator shape */
  int32_t mb, nb, kb;           /* FPU base shape (mb * nb == 64 lanes, kb == 1); 0 for MFMA */
  int32_t compute_type;         /* gk_dtype of the multiplicands */
  int32_t accum_type;           /* gk_dtype of the accumulators */
} gk_operator;

/* Layouts (reference src/layout.jl). */
typedef enum gk_layout_kind {
  GK_LAYOUT_ZERO = 0,                   /* :82-89   loads zeros, stores nothing */
  GK_LAYOUT_COL_MAJOR = 1,              /* :111-148 bounds-checked, any size and alignment.  A real MFMA product on these
                                         * layouts whose A and B happen to have 16-byte aligned columns (pointer and leading
                                         * dimension), K a multiple of 8, and M (N) a multiple of 8 where that is the
                                         * contiguous index of A (B), runs on the aligned kernel of its block shape: tiles
                                         * over the edge clamp their loads and mask their stores, a partial last K tile is
                                         * zeroed beyond K.  Same results; decided
                                         * per launch, everything else runs on the bounds-checked kernel (64 x 64 x 32) */
  GK_LAYOUT_ROW_MAJOR = 2,              /* :156-184 */
  GK_LAYOUT_ALIGNED_COL_MAJOR = 3,      /* :192-219 UnsafeAlignedColMajor: 16-byte vectors, tile-sized */
  GK_LAYOUT_ALIGNED_ROW_MAJOR = 4,      /* :244-270 */
  GK_LAYOUT_DIAGONAL = 5,               /* :225-236 A given by its diagonal */
  GK_LAYOUT_INTERLEAVED_COL_MAJOR = 6,  /* :276-302 Complex{T}, re/im adjacent */
  GK_LAYOUT_INTERLEAVED_ROW_MAJOR = 7,  /* :310-334 */
  GK_LAYOUT_SPLIT_COL_MAJOR = 8,        /* :340-372 planar re/im.  The reference uses it in shared memory only; here it is
                                           also a global layout of the complex operator: the matrix is the real array
                                           (rows, cols, 2) in column-major order, i.e. the imaginary plane starts
                                           ld * cols elements after the real one, and ld counts elements of a plane */
  GK_LAYOUT_SPLIT_ROW_MAJOR = 9,        /* :380-411 (as a global layout: the planar array of the transpose) */
  GK_LAYOUT_GETT = 10                   /* tensor-contraction index map, see gk_gett */
} gk_layout_kind;

typedef struct gk_layout {
  int32_t kind;      /* gk_layout_kind */
  int32_t eltype;    /* gk_dtype (real part type for complex layouts) */
  int32_t pad;       /* Layout.Padded{L,P}: P elements added to the leading physical dimension (:95-105) */
  int32_t reserved;
  int64_t ld;        /* global layouts: leading dimension in elements (complex elements for interleaved) */
} gk_layout;

typedef struct gk_shape { int32_t M, N, K; } gk_shape;

/* CTA swizzles (reference src/cta-swizzle.jl): Identity :26-41, HorizontallyTiled :67-82,
 * VerticallyTiled :102-117, LebesgueCurve :147-160.  GK_SWIZZLE_XCD has no counterpart in the
 * reference: it first undoes the round-robin deal of workgroups over the 8 XCDs of the MI355X
 * (each XCD has its own L2) and then walks the tile grid in panels `param` tiles high. */
typedef enum gk_swizzle_kind {
  GK_SWIZZLE_IDENTITY = 0,
  GK_SWIZZLE_HORIZONTALLY_TILED = 1,
  GK_SWIZZLE_VERTICALLY_TILED = 2,
  GK_SWIZZLE_LEBESGUE = 3,
  GK_SWIZZLE_XCD = 4
} gk_swizzle_kind;

typedef struct gk_swizzle { int32_t kind; int32_t param; } gk_swizzle;

/* One GEMM dimension of a tensor contraction: the dimension's index is the mixed-radix number
 * whose digits (fastest first) are the indices of `nmodes` tensor modes.  stride0/stride1 are the
 * element strides of each mode in the two tensors that carry the dimension:
 *   m: stride0 in A, stride1 in C and D;   n: stride0 in B, stride1 in C and D;
 *   k: stride0 in A, stride1 in B. */
typedef struct gk_gett_dim {
  int32_t nmodes;
  int32_t extent[GK_MAX_MODES];
  int64_t stride0[GK_MAX_MODES];
  int64_t stride1[GK_MAX_MODES];
} gk_gett_dim;

typedef struct gk_gett { gk_gett_dim m, n, k; } gk_gett;

/* Mirror of the reference Config (src/config.jl:3-41), field for field. */
typedef struct gk_config {
  gk_shape matmul_shape;
  gk_shape block_shape;
  int32_t warps_per_block;
  gk_shape mem_a_warp, mem_a_thread;     /* M, K used */
  gk_shape mem_b_warp, mem_b_thread;     /* K, N used */
  gk_shape mem_cd_warp, mem_cd_thread;   /* M, N used */
  gk_shape compute_warp;
  gk_shape compute_op_shape;
  gk_layout global_a_layout, global_b_layout, global_c_layout, global_d_layout;
  gk_layout shared_a_layout, shared_b_layout, shared_c_layout, shared_d_layout;
  gk_operator op;
  int32_t is_a_col_major, is_b_col_major;
  gk_swizzle cta_swizzle;
  gk_gett gett;                          /* read when a global layout is GK_LAYOUT_GETT */
} gk_config;

/* Kernels (reference src/kernel.jl: matmul_singlestage :10-129, matmul_pipelined :147-350,
 * matmul_pipelined_ng :368-574).  GK_KERNEL_SPLIT_K has no counterpart in the reference: for
 * problems with too few output tiles to fill the 256 CUs (skinny M or N, long K) the K range is cut
 * into slices that run as separate workgroups of ONE launch.  Slice 0 starts from T_c(C), the others
 * from zero; every slice leaves its partial tile in a workspace and counts itself at the tile's arrival
 * counter; the last to arrive adds the partial tiles in slice order (so the bits of D do not depend on
 * the order of arrival and do not change from run to run), applies the D hooks and the bias and
 * stores D in its element type.  No workgroup waits for another.  It needs a workspace and therefore
 * has its own entry point, gk_matmul_split_k; gk_matmul refuses this kind.  Real MFMA operator
 * (aligned or bounds-checked layouts).  With enough tiles, or a tile that has no K-split instance, it
 * is the pipelined (bounds-checked layouts: the single-stage) kernel. */
typedef enum gk_kernel_kind {
  GK_KERNEL_SINGLESTAGE = 0,
  GK_KERNEL_PIPELINED = 1,
  GK_KERNEL_PIPELINED_NG = 2,
  GK_KERNEL_SPLIT_K = 3
} gk_kernel_kind;

/* Transform.Elementwise (reference src/transform.jl:20-30) as a closed vocabulary: a hook is a
 * list of up to GK_MAX_OPS ops applied in order.  Ops are evaluated in fp32 (fp64 for fp64 data),
 * one rounding per op, and the result is rounded to the destination type of the hook. */
typedef enum gk_op_kind {
  GK_T_IDENTITY = 0,
  GK_T_SCALE = 1,     /* x * p0 */
  GK_T_ADD = 2,       /* x + p0 */
  GK_T_RELU = 3,      /* max(x, 0) */
  GK_T_NEG = 4,
  GK_T_ABS = 5,
  GK_T_CLAMP = 6,     /* min(max(x, p0), p1) */
  GK_T_SQUARE = 7
} gk_op_kind;

typedef struct gk_op { int32_t kind; float p0, p1; } gk_op;
typedef struct gk_transform { int32_t n_ops; gk_op ops[GK_MAX_OPS]; } gk_transform;

/* The eight hooks, in the keyword order of the reference launcher (src/matmul.jl:8-15). */
typedef enum gk_hook {
  GK_HOOK_GLOBAL_TO_SHARED_A = 0,
  GK_HOOK_GLOBAL_TO_SHARED_B = 1,
  GK_HOOK_GLOBAL_TO_SHARED_C = 2,
  GK_HOOK_SHARED_TO_GLOBAL_D = 3,
  GK_HOOK_SHARED_TO_REGS_A = 4,
  GK_HOOK_SHARED_TO_REGS_B = 5,
  GK_HOOK_SHARED_TO_REGS_C = 6,
  GK_HOOK_REGS_TO_SHARED_D = 7
} gk_hook;

typedef struct gk_transforms { gk_transform hook[8]; } gk_transforms;

/* Epilogues (reference src/epilogue.jl): Default :14-34, Bias :40-73 (one fp32 value per COLUMN
 * of D, added before the shared_to_global_d transform).  GK_EPILOGUE_BIAS_ROW adds one value per
 * ROW instead and has no counterpart in the reference. */
typedef enum gk_epilogue_kind { GK_EPILOGUE_DEFAULT = 0, GK_EPILOGUE_BIAS = 1, GK_EPILOGUE_BIAS_ROW = 2 } gk_epilogue_kind;
typedef struct gk_epilogue { int32_t kind; int32_t reserved; const void* bias; } gk_epilogue;

/* ---- entry points ---- */

/* Library version (GK_VERSION of the build). */
int gk_version(void);

/* Copies the message of the calling thread's last failure into buf (NUL-terminated, truncated to
 * n); returns its full length.  Stands where the message of ConfigError stands (src/config.jl:78-82). */
size_t gk_last_error(char* buf, size_t n);

/* Short name of a status code. */
const char* gk_status_string(int status);

/* Device limits used by the checks.  lds_bytes / max_threads <= 0 restore "ask the device"
 * (160 KiB and 1024 when no device is present).  Lets the host-side checks run without a GPU;
 * stands where attribute(device(), MAX_SHARED_MEMORY_PER_BLOCK_OPTIN) stands (src/matmul.jl:28). */
int gk_set_device_limits(int64_t lds_bytes, int32_t max_threads);

/* All launch-time and config-time checks of the reference, on the host, nothing is launched:
 * src/config.jl:203-212 (block shape), :136-173 (operator), :263-265 (mem tiles), :268-275
 * (divisibility), src/matmul.jl:28-36 (LDS, stages), :41 (threads). */
int gk_validate(const gk_config* conf, int32_t kernel);

/* CTASwizzle.number_of_blocks (src/cta-swizzle.jl:28-31,69-72,104-107,149-151). */
int gk_number_of_blocks(const gk_config* conf, int32_t* blocks_x, int32_t* blocks_y);

/* CTASwizzle.cta_swizzle evaluated on the host with the code the kernels use (:33-41,74-82,
 * 109-117,153-160); block_x/block_y are 0-based; the outputs are element offsets of the tile. */
int gk_cta_swizzle(const gk_config* conf, int32_t block_x, int32_t block_y, int32_t* block_i, int32_t* block_j);

/* Kernel.shmem_size (src/kernel.jl:131-145,352-366,576-590): LDS bytes the chosen kernel
 * instance requests; negative on error. */
int64_t gk_shmem_size(const gk_config* conf, int32_t kernel);

/* The reference's own answer to Kernel.shmem_size (src/kernel.jl:131-145, 352-366), unchanged:
 * max(size_c, size_a + size_b, size_d) over the four SHARED layouts of the configuration, each tile in
 * its Layout.physical_size (padding on the leading dimension, two planes for Split layouts).  Host
 * arithmetic only; the kernels of this library size their LDS differently (gk_shmem_size).  Negative on error. */
int64_t gk_reference_shmem_size(const gk_config* conf);

/* Threads per block of the launch (src/matmul.jl:24, with 64-lane wavefronts). */
int32_t gk_threads_per_block(const gk_config* conf);

/* heuristic_block_shape (src/config.jl:84-120), the reference's own rule, unchanged: M and N double
 * in turn while a C / D tile in its shared layout fits 64 KiB, then K doubles while the A and B tiles
 * fit 64 KiB together.  Only kind, eltype and pad of the four shared layouts are read.  This is the
 * reference-compatible answer; gk_matmul itself runs the tiles compiled for the MI355X. */
int gk_heuristic_block_shape(const gk_layout* shared_a, const gk_layout* shared_b, const gk_layout* shared_c,
                             const gk_layout* shared_d, gk_shape* block_shape);

/* Name of the kernel instance gk_matmul would launch, for logs and profiles. */
int gk_kernel_name(const gk_config* conf, const gk_transforms* transforms, const gk_epilogue* epilogue,
                   int32_t kernel, char* buf, size_t n);

/* GemmKernels.matmul (src/matmul.jl:7-44).  transforms == NULL means all identity, epilogue ==
 * NULL means Epilogue.Default.  Enqueues one kernel on `stream` (a hipStream_t) and returns. */
int gk_matmul(const gk_config* conf, const void* a, const void* b, const void* c, void* d,
              const gk_transforms* transforms, const gk_epilogue* epilogue, int32_t kernel, void* stream);

/* The K-split kind of launch (GK_KERNEL_SPLIT_K above; no counterpart in the reference, whose launcher
 * src/matmul.jl:7-44 has one kernel per product).  gk_split_k_workspace_size gives an upper bound of
 * the workspace a launch of `conf` needs (0: it runs unsplit); gk_matmul_split_k is gk_matmul plus the
 * workspace: device memory owned by the caller, 16-byte aligned, ZEROED BEFORE ITS FIRST USE.  Its first
 * 2048 bytes hold the arrival counters of the output tiles -- a region of the same size for every product,
 * so that launches of different shapes find their counters in the same place -- which every launch leaves
 * at zero again: one workspace serves any number of launches of any products one after the other; launches
 * that overlap in time (two streams) need a workspace each.  A launch that faulted or was aborted may leave
 * counters behind: zero the first 2048 bytes again before the workspace is used after such a failure. */
int gk_split_k_workspace_size(const gk_config* conf, size_t* bytes);
int gk_matmul_split_k(const gk_config* conf, const void* a, const void* b, const void* c, void* d,
                      const gk_transforms* transforms, const gk_epilogue* epilogue, void* workspace,
                      size_t workspace_bytes, void* stream);

/* gk_matmul_split_k for callers that cannot allocate device memory.  No counterpart in the reference; it is
 * for code under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc.  Same
 * arguments and same results, bit for bit, as gk_matmul_split_k, without the workspace: the partial tiles
 * meet in a device array that is part of the library (gk_split_k_noalloc_capacity() bytes, 32 MiB, on every
 * GPU the library is used on, for the life of the process).  A launch that needs more is refused with
 * GK_ERR_INVALID_ARGUMENT and a message that names both sizes; nothing is allocated or freed by the call,
 * on the device or through any library.  All calls on one GPU share the array: calls that overlap in time
 * (two streams, two host threads) race on it and must be serialised by the caller.  The first call on a
 * device asks the runtime for the array's address, which may load the library's device code at that moment:
 * make that first call (any product will do) outside of a stream capture; every later call on that device
 * only launches the kernel. */
size_t gk_split_k_noalloc_capacity(void);
int gk_matmul_split_k_noalloc(const gk_config* conf, const void* a, const void* b, const void* c, void* d,
                              const gk_transforms* transforms, const gk_epilogue* epilogue, void* stream);

/* A measurement aid with no counterpart in the reference (its benchmarks quote fractions of a data-sheet peak): the
 * rate, in TFLOP/s, of a register-only loop of the MFMA instruction the GEMM kernels use (v_mfma_f32_16x16x32_f16,
 * one wave per SIMD, 64 accumulator blocks per wave, operands that change every 64 MFMAs), over `launches` launches
 * of `iterations` loop passes each on `stream`, timed with events.  With random_operands != 0 the operands are FP16
 * values spread over [-1, 1), otherwise zeros: under the power cap of the device the clock, and with it the rate,
 * depends on the data.  bench.py reports both next to the rate of the headline kernel. */
int gk_probe_matrix_rate(int32_t launches, int32_t iterations, int32_t random_operands, void* stream, double* tflops);

/* Kernels specialised at run time (hipRTC).  The reference compiles one kernel per Config type and
 * inlines arbitrary Julia functors at the eight transform hooks (src/matmul.jl:38,
 * src/transform.jl:20-30); gk_matmul offers a closed op vocabulary and a table of tiles instead.
 * gk_rtc_compile closes that gap for the real MFMA operator with aligned layouts: hooks[h] is NULL
 * (identity) or a C expression in the fp32 variable x, e.g. "x > 0.0f ? x : 0.01f * x", for hook h
 * in the order of gk_hook; block_shape / compute_warp may be any tile the kernel template accepts
 * (32x32 accumulator blocks, BLOCK_K of 16, 32, 64 or 128, at most 160 KiB of LDS).  Expressions are
 * evaluated in fp32 without contraction and the result is rounded to the hook's destination type,
 * like the op lists of gk_matmul.  Compiled kernels are cached by configuration, expressions and
 * device and live until the process ends.  gk_rtc_matmul runs the same checks as gk_matmul. */
typedef struct gk_rtc_kernel gk_rtc_kernel;
int gk_rtc_compile(const gk_config* conf, const char* const hooks[8], int32_t kernel, gk_rtc_kernel** out);
int gk_rtc_matmul(gk_rtc_kernel* kernel, const gk_config* conf, const void* a, const void* b, const void* c, void* d,
                  const gk_epilogue* epilogue, void* stream);
int gk_rtc_kernel_name(const gk_rtc_kernel* kernel, char* buf, size_t n);

/* Device memory for callers that have no GPU array package of their own (a Julia session without
 * AMDGPU.jl, a C test): thin wrappers over hipMalloc / hipFree / hipMemcpy / hipDeviceSynchronize on
 * the current device.  The reference relies on CUDA.jl's CuArray for this (src/matmul.jl:185-215,
 * configs/configs.jl:96-103); gk_matmul itself never allocates. */
int gk_dev_alloc(size_t bytes, void** ptr);
int gk_dev_free(void* ptr);
int gk_copy_to_device(void* dst_device, const void* src_host, size_t bytes);
int gk_copy_to_host(void* dst_host, const void* src_device, size_t bytes);
int gk_synchronize(void);

/* sizeof() of the ABI structs as compiled, so that a binding can check its own mirror:
 * 0 gk_config, 1 gk_layout, 2 gk_operator, 3 gk_transforms, 4 gk_epilogue, 5 gk_gett. */
int32_t gk_sizeof(int32_t which);

#ifdef __cplusplus
}
#endif
#endif /* GEMMKERNELS_HIP_H */
