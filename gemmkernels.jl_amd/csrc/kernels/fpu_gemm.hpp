// Tiled GEMM on the vector ALUs: stands where Operator.FPUOp / TropicalFPUOp stand in the
// reference (src/operator.jl:35-153) together with the kernels that drive them
// (src/kernel.jl:10-129, 147-350).
//
// Every output element is one fp32 accumulator updated by a scalar fused multiply-add per k, in
// ascending k, exactly like FPUOp.mma (src/operator.jl:139-153), so results are bit-identical to
// a sequential fmaf loop on the host.  A wave is an 8 x 8 grid of lanes (the reference's base
// shape mb x nb = 32 lanes becomes 64 here); a lane owns TM x TN outputs in 4-wide chunks so that
// LDS reads and D stores are 16-byte accesses.  Tiles go global -> registers -> LDS with the next
// tile's global loads in flight during the FMAs of the current one.  With CHECKED the loads and
// stores are per element and bounds-checked (reference Layout.ColMajor / RowMajor,
// src/layout.jl:117-184: out-of-range loads give 0, out-of-range stores are dropped), so any
// problem size and any leading dimension works.
#pragma once
#include "common.hpp"

namespace gk {

template <typename T> struct FpuIn;
template <> struct FpuIn<float> {
  static constexpr int DT = DT_F32;
  __device__ static __forceinline__ float to_float(float x) { return x; }
  __device__ static __forceinline__ float round(float x) { return x; }
};
template <> struct FpuIn<_Float16> {
  static constexpr int DT = DT_F16;
  __device__ static __forceinline__ float to_float(_Float16 x) { return (float)x; }
  __device__ static __forceinline__ float round(float x) { return (float)(_Float16)x; }
};

template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, typename TIN_, bool A_KMAJOR_, bool B_KMAJOR_, bool CHECKED_, bool TROPICAL_>
struct FpuGemmConfig {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr bool A_KMAJOR = A_KMAJOR_, B_KMAJOR = B_KMAJOR_, CHECKED = CHECKED_, TROPICAL = TROPICAL_;
  typedef TIN_ TIN;
  static constexpr int THREADS = WAVES_M * WAVES_N * kWaveSize;
  static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static constexpr int TM = WTM / 8, TN = WTN / 8;          // outputs per lane
  static constexpr int CM = TM / 4, CN = TN / 4;            // 4-wide chunks per lane
  static constexpr int PAD = 4;
  static constexpr int LDA_S = BM + PAD, LDB_S = BN + PAD;  // LDS row pitch (floats), rows are k
  static constexpr int LDS_BYTES = (BK * LDA_S + BK * LDB_S) * 4;
  static constexpr int A_CHUNKS = BM * BK / 4, B_CHUNKS = BN * BK / 4;
  static constexpr int A_PER_THREAD = A_CHUNKS / THREADS, B_PER_THREAD = B_CHUNKS / THREADS;
  static_assert(TM % 4 == 0 && TN % 4 == 0, "a lane owns whole 4-wide chunks");
  static_assert(A_CHUNKS % THREADS == 0 && B_CHUNKS % THREADS == 0, "tile loads divide evenly over the threads");
};

// Loads the 4 elements of chunk `chunk` of an R x BK operand tile: rows r0.. of the operand,
// k from k0.  MAJOR_K: memory is contiguous along k.  Out-of-range elements read as 0.
template <class Cfg, int R, bool KMAJOR>
__device__ __forceinline__ void load_chunk(const typename Cfg::TIN* __restrict__ base, long long ld, int r0, int k0, int chunk,
                                           int r_limit, int k_limit, bool zero, float (&out)[4], int& r_local, int& k_local) {
  typedef typename Cfg::TIN TIN;
  if (KMAJOR) {
    constexpr int CPR = Cfg::BK / 4;          // chunks per row
    r_local = chunk / CPR;
    k_local = (chunk % CPR) * 4;
  } else {
    constexpr int CPK = R / 4;                // chunks per k
    k_local = chunk / CPK;
    r_local = (chunk % CPK) * 4;
  }
  const int r = r0 + r_local, k = k0 + k_local;
  if (zero) {          // Layout.Zero: nothing is read (alpha == 0, reference src/matmul.jl:127-130)
#pragma unroll
    for (int e = 0; e < 4; ++e) out[e] = 0.0f;
  } else if (!Cfg::CHECKED) {
    const TIN* p = base + (KMAJOR ? (long long)r * ld + k : (long long)k * ld + r);
    typedef TIN vec4 __attribute__((ext_vector_type(4)));
    const vec4 v = *(const vec4*)p;
#pragma unroll
    for (int e = 0; e < 4; ++e) out[e] = FpuIn<TIN>::to_float(v[e]);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int rr = KMAJOR ? r : r + e, kk = KMAJOR ? k + e : k;
      // padding: 0 for the ordinary product; -inf along k for the tropical one so that max() ignores it
      float x = (Cfg::TROPICAL && kk >= k_limit) ? -__builtin_inff() : 0.0f;
      if (rr < r_limit && kk < k_limit) x = FpuIn<TIN>::to_float(base[KMAJOR ? (long long)rr * ld + kk : (long long)kk * ld + rr]);
      out[e] = x;
    }
  }
}

template <class Cfg>
__global__ void __launch_bounds__(Cfg::THREADS) fpu_gemm_kernel(const GemmArgs args) {
  typedef typename Cfg::TIN TIN;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, TM = Cfg::TM, TN = Cfg::TN;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float* As = (float*)smem;                       // [BK][LDA_S], rows are k
  float* Bs = As + BK * Cfg::LDA_S;               // [BK][LDB_S]

  int ti, tj;
  cta_swizzle(args.swz_kind, args.swz_param, (int)blockIdx.x, (int)blockIdx.y, args.nbm, args.nbn, ti, tj);
  if (ti >= args.nbm || tj >= args.nbn) return;
  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave % Cfg::WAVES_M, wn = wave / Cfg::WAVES_M;
  const int ly = lane & 7, lx = lane >> 3;
  const int m0 = ti * BM, n0 = tj * BN;
  const TIN* A = (const TIN*)args.a;
  const TIN* B = (const TIN*)args.b;
  const bool zero_ab = (args.a_kind == 0 /* Layout.Zero */);
  const bool xf_a = args.t[H_GL2SH_A].n > 0 || args.t[H_SH2RF_A].n > 0;
  const bool xf_b = args.t[H_GL2SH_B].n > 0 || args.t[H_SH2RF_B].n > 0;

  // accumulators: acc[i][j] is row wm*WTM + (i/4)*32 + 4*ly + i%4, column wn*WTN + (j/4)*32 + 4*lx + j%4
  float acc[TM][TN];
  auto row_of = [&](int i) { return m0 + wm * Cfg::WTM + (i / 4) * 32 + 4 * ly + (i % 4); };
  auto col_of = [&](int j) { return n0 + wn * Cfg::WTN + (j / 4) * 32 + 4 * lx + (j % 4); };
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      float c = 0.0f;
      if (args.c_mode != 0) {
        const int r = row_of(i), cc = col_of(j);
        if (!Cfg::CHECKED || (r < args.M && cc < args.N)) c = ((const float*)args.c)[r + (long long)cc * args.ldc];
        c = apply_list(args.t[H_GL2SH_C], c);
        c = apply_list(args.t[H_SH2RF_C], c);
      }
      acc[i][j] = c;
    }

  float ra[Cfg::A_PER_THREAD][4], rb[Cfg::B_PER_THREAD][4];
  int ar[Cfg::A_PER_THREAD], ak[Cfg::A_PER_THREAD], br[Cfg::B_PER_THREAD], bk[Cfg::B_PER_THREAD];

  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < Cfg::A_PER_THREAD; ++i) {
      load_chunk<Cfg, BM, Cfg::A_KMAJOR>(A, args.lda, m0, k0, tid + i * Cfg::THREADS, args.M, args.K, zero_ab, ra[i], ar[i], ak[i]);
    }
#pragma unroll
    for (int i = 0; i < Cfg::B_PER_THREAD; ++i) {
      load_chunk<Cfg, BN, Cfg::B_KMAJOR>(B, args.ldb, n0, k0, tid + i * Cfg::THREADS, args.N, args.K, zero_ab, rb[i], br[i], bk[i]);
    }
  };
  // transforms of the two load hooks, each rounded to the element type of its destination
  auto xform = [&](float (&v)[4], const OpList& t0, const OpList& t1) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float x = v[e];
      if (t0.n > 0) x = FpuIn<TIN>::round(apply_list(t0, x));
      if (t1.n > 0) x = FpuIn<TIN>::round(apply_list(t1, x));
      v[e] = x;
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < Cfg::A_PER_THREAD; ++i) {
      if (xf_a) xform(ra[i], args.t[H_GL2SH_A], args.t[H_SH2RF_A]);
      if (Cfg::A_KMAJOR) {
#pragma unroll
        for (int e = 0; e < 4; ++e) As[(ak[i] + e) * Cfg::LDA_S + ar[i]] = ra[i][e];
      } else {
        *(float4v*)&As[ak[i] * Cfg::LDA_S + ar[i]] = (float4v){ra[i][0], ra[i][1], ra[i][2], ra[i][3]};
      }
    }
#pragma unroll
    for (int i = 0; i < Cfg::B_PER_THREAD; ++i) {
      if (xf_b) xform(rb[i], args.t[H_GL2SH_B], args.t[H_SH2RF_B]);
      if (Cfg::B_KMAJOR) {
#pragma unroll
        for (int e = 0; e < 4; ++e) Bs[(bk[i] + e) * Cfg::LDB_S + br[i]] = rb[i][e];
      } else {
        *(float4v*)&Bs[bk[i] * Cfg::LDB_S + br[i]] = (float4v){rb[i][0], rb[i][1], rb[i][2], rb[i][3]};
      }
    }
  };

  const int KT = (args.K + BK - 1) / BK;
  fetch(0);
  for (int kt = 0; kt < KT; ++kt) {
    __syncthreads();          // everyone is done reading the previous tile
    stash();
    __syncthreads();
    if (kt + 1 < KT) fetch((kt + 1) * BK);
    const float* ap = As + wm * Cfg::WTM + 4 * ly;
    const float* bp = Bs + wn * Cfg::WTN + 4 * lx;
#pragma unroll 4
    for (int k = 0; k < BK; ++k) {
      float a[TM], b[TN];
#pragma unroll
      for (int c = 0; c < Cfg::CM; ++c) {
        const float4v v = *(const float4v*)&ap[k * Cfg::LDA_S + c * 32];
        a[4 * c] = v[0]; a[4 * c + 1] = v[1]; a[4 * c + 2] = v[2]; a[4 * c + 3] = v[3];
      }
#pragma unroll
      for (int c = 0; c < Cfg::CN; ++c) {
        const float4v v = *(const float4v*)&bp[k * Cfg::LDB_S + c * 32];
        b[4 * c] = v[0]; b[4 * c + 1] = v[1]; b[4 * c + 2] = v[2]; b[4 * c + 3] = v[3];
      }
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          if (Cfg::TROPICAL) {
            const float s = a[i] + b[j];
            acc[i][j] = s > acc[i][j] ? s : acc[i][j];
          } else {
            acc[i][j] = __builtin_fmaf(a[i], b[j], acc[i][j]);
          }
        }
    }
  }

  // epilogue: transform, bias, transform, store (4 consecutive rows per 16-byte store)
  float* D = (float*)args.d;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int cc = col_of(j);
#pragma unroll
    for (int c = 0; c < Cfg::CM; ++c) {
      float x[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = apply_list(args.t[H_RF2SH_D], acc[4 * c + e][j]);
        if (args.epi_kind == 1) v = v + args.bias[Cfg::CHECKED ? (cc < args.N ? cc : 0) : cc];
        else if (args.epi_kind == 2) { const int r = row_of(4 * c + e); v = v + args.bias[Cfg::CHECKED ? (r < args.M ? r : 0) : r]; }
        x[e] = apply_list(args.t[H_SH2GL_D], v);
      }
      const int r = row_of(4 * c);
      if (!Cfg::CHECKED) {
        *(float4v*)&D[r + (long long)cc * args.ldd] = (float4v){x[0], x[1], x[2], x[3]};
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (r + e < args.M && cc < args.N) D[r + e + (long long)cc * args.ldd] = x[e];
      }
    }
  }
}

}  // namespace gk
