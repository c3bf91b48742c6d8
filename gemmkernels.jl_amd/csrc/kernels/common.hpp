// Shared device/host definitions of the gfx950 GEMM kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gk {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef short short4v __attribute__((__vector_size__(4 * sizeof(short))));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef int int4v __attribute__((ext_vector_type(4)));
typedef int int2v __attribute__((ext_vector_type(2)));

#define GK_LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))
#define GK_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

constexpr int kWaveSize = 64;
constexpr int kNumCUs = 256;      // MI355X

// dtype codes (same values as gk_dtype of the C ABI)
enum : int { DT_F16 = 0, DT_BF16 = 1, DT_F32 = 2, DT_F64 = 3, DT_I16 = 4, DT_I32 = 5, DT_I64 = 6 };

// op codes (same values as gk_op_kind of the C ABI)
enum : int { T_IDENTITY = 0, T_SCALE = 1, T_ADD = 2, T_RELU = 3, T_NEG = 4, T_ABS = 5, T_CLAMP = 6, T_SQUARE = 7 };

// swizzle codes (same values as gk_swizzle_kind)
enum : int { SWZ_IDENTITY = 0, SWZ_HTILED = 1, SWZ_VTILED = 2, SWZ_LEBESGUE = 3, SWZ_XCD = 4 };

constexpr int kMaxOps = 4;
constexpr int kMaxModes = 4;

// One transform hook: a short list of elementwise ops.
struct OpList {
  int n;
  int kind[kMaxOps];
  float p0[kMaxOps];
  float p1[kMaxOps];
};

// Hook indices, keyword order of the reference launcher (reference src/matmul.jl:8-15).
enum : int { H_GL2SH_A = 0, H_GL2SH_B = 1, H_GL2SH_C = 2, H_SH2GL_D = 3, H_SH2RF_A = 4, H_SH2RF_B = 5, H_SH2RF_C = 6, H_RF2SH_D = 7 };

// One GEMM dimension of a tensor contraction (mixed-radix index -> two element offsets).
struct GettDim {
  int nmodes;
  int extent[kMaxModes];
  long long stride0[kMaxModes];
  long long stride1[kMaxModes];
  // division by extent[i] as a multiplication (see gett_div), filled by the host with gett_fill_division()
  unsigned magic[kMaxModes];
  int shift[kMaxModes];
};

// n / e for 0 <= n < 2^31 and a divisor known on the host: with s = ceil(log2 e), magic = floor(2^(31+s) / e) + 1
// fits in 32 bits and floor(n * magic / 2^(31+s)) is the quotient exactly (the error of the reciprocal, at most
// e / 2^(31+s) relative, stays below 1/e for every n < 2^31).  e = 1 is marked by magic = 0.
__host__ __device__ inline void gett_fill_division(GettDim& d) {
  for (int i = 0; i < kMaxModes; ++i) {
    d.magic[i] = 0;
    d.shift[i] = 0;
    const unsigned e = i < d.nmodes ? (unsigned)d.extent[i] : 1u;
    if (e <= 1) continue;
    int s = 0;
    while ((1ull << s) < e) ++s;
    d.magic[i] = (unsigned)(((1ull << (31 + s)) / e) + 1ull);
    d.shift[i] = s - 1;
  }
}
__host__ __device__ inline int gett_div(int n, unsigned magic, int shift) {
  if (magic == 0) return n;
  return (int)((unsigned)(((unsigned long long)(unsigned)n * magic) >> 32) >> shift);
}
// the two element offsets of index idx (< 2^31) of a GEMM dimension: a mixed-radix walk over its modes
__host__ __device__ inline void gett_offsets32(const GettDim& d, int idx, long long& off0, long long& off1) {
  off0 = 0; off1 = 0;
  for (int i = 0; i < d.nmodes; ++i) {
    const int q = gett_div(idx, d.magic[i], d.shift[i]);
    const int digit = idx - q * d.extent[i];
    idx = q;
    off0 += (long long)digit * d.stride0[i];
    off1 += (long long)digit * d.stride1[i];
  }
}
// The same walk written out over all kMaxModes modes, a mode beyond nmodes as one of extent 1: the table entries are then
// read at constant places of the kernel arguments, once for all the walks of a kernel, where the loop over nmodes reads
// them again, and waits for them, in every iteration of every walk.  It holds the tables in some sixty scalar registers
// meanwhile: for kernels that make few walks and have the registers to spare (the one-wave-per-SIMD contraction kernel).
__host__ __device__ inline void gett_offsets32_flat(const GettDim& d, int idx, long long& off0, long long& off1) {
  off0 = 0; off1 = 0;
#pragma unroll
  for (int i = 0; i < kMaxModes; ++i) {
    const bool on = i < d.nmodes;
    const unsigned magic = on ? d.magic[i] : 0u;
    const int q = magic == 0 ? idx : (int)((unsigned)(((unsigned long long)(unsigned)idx * magic) >> 32) >> d.shift[i]);
    const int digit = idx - q * (on ? d.extent[i] : 1);
    idx = q;
    off0 += (long long)digit * (on ? d.stride0[i] : 0ll);
    off1 += (long long)digit * (on ? d.stride1[i] : 0ll);
  }
}

__host__ __device__ inline void gett_offsets(const GettDim& d, long long idx, long long& off0, long long& off1) {
  off0 = 0; off1 = 0;
  for (int i = 0; i < d.nmodes; ++i) {
    long long e = d.extent[i];
    long long digit = idx % e;
    idx /= e;
    off0 += digit * d.stride0[i];
    off1 += digit * d.stride1[i];
  }
}

// Arguments common to every GEMM kernel of the library.
struct GemmArgs {
  const void* a;
  const void* b;
  const void* c;
  void* d;
  const float* bias;
  int M, N, K;
  long long lda, ldb, ldc, ldd;   // leading dimensions in elements
  int nbm, nbn;                   // tile grid
  int swz_kind, swz_param;
  int c_mode;                     // 0: C is Layout.Zero, 1: C is loaded
  int epi_kind;                   // 0 default, 1 bias per column, 2 bias per row
  int c_dtype, d_dtype;
  int a_kind, b_kind;             // gk_layout_kind of the global A / B layouts (diagonal, GETT ...)
  int cd_gett;                    // 1: C and D are addressed through gett.m / gett.n stride1
  OpList t[8];
  // set by the host when the two load hooks of A (resp. B) amount to one multiplication by a
  // constant that is exact in the operand's 16-bit type: done as a packed 16-bit multiply
  int fast_scale_a, fast_scale_b;
  float scale_a, scale_b;
  // a multiplication of A or B by a power of two commutes with every rounding of the sum: the host takes such
  // a hook out of the K loop, the accumulators start from acc_pre_scale * T_c(C) and are multiplied by
  // acc_post_scale = 1 / acc_pre_scale before the hooks of D (both 1 otherwise)
  float acc_pre_scale, acc_post_scale;
  GettDim gm, gn, gk;
  // How a K tile lies in the K modes of a contraction: it covers the modes below gk_mode whole (their extents
  // multiply to a divisor of BLOCK_K) and gk_step indices of mode gk_mode, whose extent gk_step divides.
  // (BLOCK_K divides the first K mode: gk_mode 0, gk_step BLOCK_K.)
  int gk_mode, gk_step;
  // 1: the first M mode and the first N mode are multiples of 32, so the 16 rows and the 4 columns of an accumulator
  // block follow each other in C / D with one stride and block origins need one walk per wave; 0: every lane walks
  int gett_fast;
  // K-split launches (all 0 otherwise): workgroup z of k_slices handles the k_steps tiles of K that start at
  // tile z * k_steps; slice 0 starts from C.  Every slice writes its partial tile to ws_partials and counts
  // itself in ws_counters[tile]; the last one to arrive adds the partial tiles in slice order, runs the
  // epilogue and puts the counter back to zero (see splitk_reduce).
  int k_steps, k_slices;
  void* ws_partials;
  unsigned* ws_counters;
  // planar complex operands (0 otherwise): distance in elements from the real plane of a matrix to
  // its imaginary plane
  long long plane_a, plane_b, plane_c, plane_d;
};

// ---------------------------------------------------------------------------------------------
// CTA swizzle: (blockIdx.x, blockIdx.y) -> tile coordinates.  Identity, HorizontallyTiled,
// VerticallyTiled and LebesgueCurve follow reference src/cta-swizzle.jl:33-41, 74-82, 109-117,
// 153-160.  SWZ_XCD is specific to the MI355X: workgroup n of a launch runs on XCD n % 8 and every
// XCD has a private L2, so consecutive ids are first regrouped per XCD and the tile grid is then
// walked in panels `param` tiles high, which makes the tiles that share an L2 share rows of A and
// columns of B.
// ---------------------------------------------------------------------------------------------
__host__ __device__ inline unsigned extract_even_bits(unsigned x) {
  x = x & 0x55555555u;
  x = (x | (x >> 1)) & 0x33333333u;
  x = (x | (x >> 2)) & 0x0F0F0F0Fu;
  x = (x | (x >> 4)) & 0x00FF00FFu;
  x = (x | (x >> 8)) & 0x0000FFFFu;
  return x;
}

__host__ __device__ inline void cta_swizzle(int kind, int param, int bx, int by, int nbm, int nbn, int& ti, int& tj) {
  switch (kind) {
    case SWZ_HTILED:
      ti = bx / param;
      tj = by * param + bx % param;
      break;
    case SWZ_VTILED:
      ti = bx * param + by % param;
      tj = by / param;
      break;
    case SWZ_LEBESGUE:
      ti = (int)extract_even_bits((unsigned)bx);
      tj = (int)extract_even_bits((unsigned)bx >> 1);
      break;
    case SWZ_XCD: {
      const int total = nbm * nbn;
      // ids x, x + 8, x + 16, ... run on XCD x: XCD x holds total / 8 of them, one more when x < total % 8;
      // the ids of one XCD become consecutive
      const int x = bx % 8, q = total / 8, rem = total % 8;
      const int r = x * q + (x < rem ? x : rem) + bx / 8;
      const int g = param > 0 ? param : 1;
      const int width = g * nbn;
      const int group = r / width;
      const int first = group * g;
      const int gsz = (nbm - first) < g ? (nbm - first) : g;
      const int in_group = r % width;
      ti = first + in_group % gsz;
      tj = in_group / gsz;
      break;
    }
    default:
      ti = bx;
      tj = by;
      break;
  }
}

__host__ __device__ inline void number_of_blocks(int kind, int param, int nbm_elems_M, int nbn_elems_N, int BM, int BN, int& gx, int& gy) {
  // cld() forms of reference src/cta-swizzle.jl:28-31, 69-72, 104-107, 149-151
  auto cld = [](long long a, long long b) { return (int)((a + b - 1) / b); };
  switch (kind) {
    case SWZ_HTILED:
      gx = cld((long long)nbm_elems_M * param, BM);
      gy = cld(nbn_elems_N, (long long)BN * param);
      break;
    case SWZ_VTILED:
      gx = cld(nbm_elems_M, (long long)BM * param);
      gy = cld((long long)nbn_elems_N * param, BN);
      break;
    case SWZ_LEBESGUE:
    case SWZ_XCD:
      gx = cld(nbm_elems_M, BM) * cld(nbn_elems_N, BN);
      gy = 1;
      break;
    default:
      gx = cld(nbm_elems_M, BM);
      gy = cld(nbn_elems_N, BN);
      break;
  }
}

// ---------------------------------------------------------------------------------------------
// Elementwise op lists.  One rounding per op, fp32 arithmetic, no fused multiply-add.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float apply_op(int kind, float p0, float p1, float x) {
  switch (kind) {
    case T_SCALE: return x * p0;
    case T_ADD: return x + p0;
    case T_RELU: return x > 0.0f ? x : 0.0f;
    case T_NEG: return -x;
    case T_ABS: return __builtin_fabsf(x);
    case T_CLAMP: return x < p0 ? p0 : (x > p1 ? p1 : x);
    case T_SQUARE: return x * x;
    default: return x;
  }
}

__device__ __forceinline__ float apply_list(const OpList& t, float x) {
  for (int i = 0; i < t.n; ++i) x = apply_op(t.kind[i], t.p0[i], t.p1[i], x);
  return x;
}

// One op of a list handed to `each` as an elementwise function: the (wave-uniform) switch on the op
// is paid once per call of `each`, which applies the function to as many registers as the caller
// holds (a fragment, or all accumulators of a lane).
template <typename Each>
__device__ __forceinline__ void dispatch_op(int kind, float p0, float p1, Each&& each) {
  switch (kind) {
    case T_SCALE:  each([=](float x) { return x * p0; }); break;
    case T_ADD:    each([=](float x) { return x + p0; }); break;
    case T_RELU:   each([=](float x) { return x > 0.0f ? x : 0.0f; }); break;
    case T_NEG:    each([=](float x) { return -x; }); break;
    case T_ABS:    each([=](float x) { return __builtin_fabsf(x); }); break;
    case T_CLAMP:  each([=](float x) { return x < p0 ? p0 : (x > p1 ? p1 : x); }); break;
    case T_SQUARE: each([=](float x) { return x * x; }); break;
    default: break;
  }
}

// Applies a list to an array of registers with the op switch outside the element loop.
template <int COUNT>
__device__ __forceinline__ void apply_list_regs(const OpList& t, float (&x)[COUNT]) {
  for (int i = 0; i < t.n; ++i)
    dispatch_op(t.kind[i], t.p0[i], t.p1[i], [&](auto f) {
#pragma unroll
      for (int e = 0; e < COUNT; ++e) x[e] = f(x[e]);
    });
}

// ---------------------------------------------------------------------------------------------
// Transform hooks.  The kernels compiled into the library interpret the op lists of the launch
// arguments.  A translation unit that defines GK_USER_HOOKS before including this header supplies
//   struct gk::UserHooks { static constexpr bool present[8];
//                          template <int H> static __device__ float apply(float x); };
// and every hook becomes inline code of the caller's choosing: that is how kernels specialised
// at run time carry arbitrary elementwise functions, like the functors the reference inlines
// through its JIT (src/transform.jl:20-30).
// ---------------------------------------------------------------------------------------------
template <int H>
__device__ __forceinline__ bool hook_present(const GemmArgs& args) {
#ifdef GK_USER_HOOKS
  (void)args;
  return UserHooks::present[H];
#else
  return args.t[H].n > 0;
#endif
}

template <int H, int COUNT>
__device__ __forceinline__ void hook_regs(const GemmArgs& args, float (&x)[COUNT]) {
#ifdef GK_USER_HOOKS
  (void)args;
  if constexpr (UserHooks::present[H]) {
#pragma unroll
    for (int e = 0; e < COUNT; ++e) x[e] = UserHooks::template apply<H>(x[e]);
  }
#else
  apply_list_regs<COUNT>(args.t[H], x);
#endif
}

// One element of C / D in the element type the layout names (accumulators are fp32; a 16-bit D gets
// one rounding, at the store).
__device__ __forceinline__ float load_cd(const void* base, int dtype, long long idx) {
  if (dtype == DT_F32) return ((const float*)base)[idx];
  if (dtype == DT_F16) return (float)((const _Float16*)base)[idx];
  return (float)((const __bf16*)base)[idx];
}
__device__ __forceinline__ void store_cd(void* base, int dtype, long long idx, float x) {
  if (dtype == DT_F32) ((float*)base)[idx] = x;
  else if (dtype == DT_F16) ((_Float16*)base)[idx] = (_Float16)x;
  else ((__bf16*)base)[idx] = (__bf16)x;
}

// ---------------------------------------------------------------------------------------------
// K-split launches: ordered reduction of the partial tiles of the K slices of one output tile.
// acc2 holds the partial tile of this workgroup (ROWS x COLS accumulator blocks per lane).  Returns
// false in every workgroup but the last to arrive at the tile; in that one acc2 comes back as
// partial(0) + partial(1) + ... + partial(k_slices - 1), added in this order whatever the order of arrival,
// so the result does not change from run to run.  The partial tiles lie in the workspace in the lane order
// of the accumulators: a store or load instruction of a wave moves 256 consecutive bytes.
//
// The workgroups of a tile run on different XCDs, whose L2 caches are not coherent with each other.  The
// partial tiles are therefore written and read with device-scope accesses (they go through to memory,
// whatever L2 the workgroup sits behind), a lane waits for its own stores to be acknowledged before the
// workgroup counts itself at the tile's arrival counter, and the workgroup that finds all others counted
// reads their tiles.  A device-wide release / acquire fence pair around the counter would do the same for
// ordinary stores and loads, but it writes back and invalidates the whole L2 of the XCD once per
// workgroup, which made the launch five times longer (measured: 70 us against 13 us for 4096 x 64 x 4096).
// No workgroup waits for another.
// ---------------------------------------------------------------------------------------------
template <int THREADS, int ROWS, int COLS, class V>
__device__ __forceinline__ bool splitk_reduce(V (&acc2)[ROWS][COLS], const GemmArgs& args, int tile_id, unsigned* lds_word) {
  constexpr int COUNT = ROWS * COLS;
  constexpr int NV = (int)(sizeof(V) / sizeof(float));   // floats per accumulator block and lane
  auto blk = [&](int i) -> V& { return acc2[i / COLS][i % COLS]; };
  const int S = args.k_slices, z = (int)blockIdx.z, tid = (int)threadIdx.x;
  constexpr size_t TILE_FLOATS = (size_t)COUNT * NV * THREADS;
  float* tile_ws = (float*)args.ws_partials + (size_t)tile_id * S * TILE_FLOATS;
  float* mine = tile_ws + (size_t)z * TILE_FLOATS;
#pragma unroll
  for (int i = 0; i < COUNT; ++i)
#pragma unroll
    for (int e = 0; e < NV; ++e)
      __hip_atomic_store(&mine[(size_t)(i * NV + e) * THREADS + tid], blk(i)[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // this lane's part of the tile has reached memory ...
  __syncthreads();                                     // ... and so has every other lane's, before the arrival is counted
  if (tid == 0) *lds_word = __hip_atomic_fetch_add(&args.ws_counters[tile_id], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  const unsigned before_me = *lds_word;
  if (before_me != (unsigned)(S - 1)) return false;
#pragma unroll
  for (int i = 0; i < COUNT; ++i)
#pragma unroll
    for (int e = 0; e < NV; ++e) blk(i)[e] = 0.0f;
  // The partial tiles of U slices travel together (one slice at a time the loop would pay the latency of the
  // memory behind the L2 once per slice); they are added in slice order all the same.
  constexpr int PER = COUNT * NV;                            // floats per lane and slice
  constexpr int U = PER >= 32 ? 1 : (PER >= 16 ? 3 : 4);     // at most 63 loads can be outstanding per wave
  for (int s0 = 0; s0 < S; s0 += U) {
    float x[U][PER];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // a slice beyond the last one re-reads the last (its values are not added)
      const float* part = tile_ws + (size_t)(s0 + u < S ? s0 + u : S - 1) * TILE_FLOATS;
#pragma unroll
      for (int q = 0; q < PER; ++q)
        x[u][q] = __hip_atomic_load(&part[(size_t)q * THREADS + tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (s0 + u < S) {
#pragma unroll
        for (int i = 0; i < COUNT; ++i)
#pragma unroll
          for (int e = 0; e < NV; ++e) blk(i)[e] += x[u][i * NV + e];
      }
  }
  // the next launch on this workspace finds the counter at zero
  if (tid == 0) __hip_atomic_store(&args.ws_counters[tile_id], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return true;
}

// waits and barriers placed by hand around the LDS-DMA pipeline
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void wait_lgkmcnt0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void block_barrier() { asm volatile("s_barrier" ::: "memory"); }

// Which of the C / D paths of a one-wave-per-SIMD instance (MfmaGemmConfig::SOLO) a launch takes (16-byte accesses where the pointers and the leading
// dimensions allow them).
// (path 4: C on its way during the first K tiles, for products of at least kSoloStreamTiles K tiles; `stream_ok`: the instance has that path;
// path 5: C spread over more K tiles, kSoloSpreadBlocks of the wave tile's `blocks` accumulator blocks per K tile, for products of
// at least `spread_tiles` = solo_spread_tiles(blocks) K tiles; 0: the instance has no such path)
constexpr int kSoloStreamTiles = 11;
constexpr int kSoloSpreadBlocks = 2;
constexpr int solo_spread_tiles(int blocks) { return blocks / kSoloSpreadBlocks + 3; }
// (path 6: 4 for an FP16 C and an FP16 D that take 8-byte accesses; `half_cd_ok`: the instance has it)
inline int solo_cd_path(const GemmArgs& args, bool stream_ok = false, int block_k = 64, int spread_tiles = 0, bool half_cd_ok = false) {
  const bool d_wide = args.d_dtype == DT_F32 && ((((uintptr_t)args.d) | ((uintptr_t)args.ldd << 2)) & 15u) == 0;
  const bool c_wide = args.c_dtype == DT_F32 && ((((uintptr_t)args.c) | ((uintptr_t)args.ldc << 2)) & 15u) == 0;
  if (half_cd_ok && stream_ok && args.c_mode != 0 && args.d_dtype == DT_F16 && args.c_dtype == DT_F16 &&
      ((((uintptr_t)args.d) | ((uintptr_t)args.ldd << 1) | ((uintptr_t)args.c) | ((uintptr_t)args.ldc << 1)) & 7u) == 0 &&
      args.K / block_k >= kSoloStreamTiles)
    return 6;
  if (d_wide && args.c_mode != 0 && c_wide) {
    if (stream_ok && spread_tiles > 0 && args.K / block_k >= spread_tiles) return 5;
    return (stream_ok && args.K / block_k >= kSoloStreamTiles) ? 4 : 1;
  }
  if (d_wide && args.c_mode == 0) return 2;
  return 0;
}

}  // namespace gk
