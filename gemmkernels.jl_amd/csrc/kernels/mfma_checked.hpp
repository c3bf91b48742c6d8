// Bounds-checked MFMA GEMM for operands of any size, alignment and leading dimension: stands where
// Kernel.matmul_singlestage with the Layout.ColMajor / RowMajor layouts stands in the reference
// (src/kernel.jl:10-129, src/layout.jl:117-184).  Elements are loaded one by one (out-of-range
// reads give 0), written to LDS in the K-major swizzled tile layout of the fast kernel, and the
// same fragment reader and MFMA sequence consume them; out-of-range stores are dropped.  One LDS
// stage: load, barrier, compute, barrier.  Slow by design, like the reference's checked layouts.
#pragma once
#include "mfma_gemm.hpp"

namespace gk {

template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, bool A_KMAJOR_, bool B_KMAJOR_, typename T_>
struct MfmaCheckedConfig {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr bool A_KMAJOR = A_KMAJOR_, B_KMAJOR = B_KMAJOR_;
  typedef T_ T;
  static constexpr int NWAVES = WAVES_M * WAVES_N, THREADS = NWAVES * kWaveSize;
  static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N, FM = WTM / 32, FN = WTN / 32, KSTEPS = BK / 16;
  typedef OperandGeom<BM, BK, OPK_KMAJOR, false> GA;     // both LDS tiles are K-major whatever the memory order
  typedef OperandGeom<BN, BK, OPK_KMAJOR, false> GB;
  static constexpr int LDS_BYTES = GA::BYTES + GB::BYTES;
  static constexpr int A_PER_THREAD = BM * BK / THREADS, B_PER_THREAD = BN * BK / THREADS;
  static_assert((BM * BK) % THREADS == 0 && (BN * BK) % THREADS == 0, "tile loads divide evenly over the threads");
};

template <class Cfg>
__global__ void __launch_bounds__(Cfg::THREADS) mfma_gemm_checked_kernel(const GemmArgs args) {
  typedef typename Cfg::T T;
  typedef typename Cfg::GA GA;
  typedef typename Cfg::GB GB;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, FM = Cfg::FM, FN = Cfg::FN;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  char* sa = smem;
  char* sb = smem + GA::BYTES;

  int ti, tj;
  cta_swizzle(args.swz_kind, args.swz_param, (int)blockIdx.x, (int)blockIdx.y, args.nbm, args.nbn, ti, tj);
  if (ti >= args.nbm || tj >= args.nbn) return;
  const int tid = (int)threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % Cfg::WAVES_M, wn = wave / Cfg::WAVES_M;
  const int m0 = ti * BM, n0 = tj * BN;
  const T* A = (const T*)args.a;
  const T* B = (const T*)args.b;
  const bool zero_ab = (args.a_kind == 0 /* Layout.Zero */);
  const bool xf_a = args.t[H_GL2SH_A].n > 0 || args.t[H_SH2RF_A].n > 0;
  const bool xf_b = args.t[H_GL2SH_B].n > 0 || args.t[H_SH2RF_B].n > 0;

  float16v acc[FM][FN];
  const int mrow = m0 + wm * Cfg::WTM + (lane & 31);
  const int ncol = n0 + wn * Cfg::WTN + 4 * (lane >> 5);
#pragma unroll
  for (int fi = 0; fi < FM; ++fi)
#pragma unroll
    for (int fj = 0; fj < FN; ++fj)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float c = 0.0f;
        const int r = mrow + 32 * fi, cc = ncol + 32 * fj + 8 * (v / 4) + (v % 4);
        if (args.c_mode != 0) {
          if (r < args.M && cc < args.N) c = load_cd(args.c, args.c_dtype, r + (long long)cc * args.ldc);
          c = apply_list(args.t[H_GL2SH_C], c);
          c = apply_list(args.t[H_SH2RF_C], c);
        }
        acc[fi][fj][v] = c;
      }

  // element e of a tile: K-major memory walks k fastest, M-major memory walks the row fastest, so
  // that consecutive threads touch consecutive addresses
  auto load_tile = [&](const T* base, long long ld, bool kmajor, int R, int r0, int r_limit, int k0, char* dst, int per_thread,
                       bool xf, const OpList& t0, const OpList& t1, int cpr_shift_rows) {
    (void)cpr_shift_rows;
    for (int i = 0; i < per_thread; ++i) {
      const int e = tid + i * Cfg::THREADS;
      int r, k;
      if (kmajor) { r = e / BK; k = e % BK; } else { k = e / R; r = e % R; }
      T x = (T)0.0f;
      const int gr = r0 + r, gk_ = k0 + k;
      if (!zero_ab && gr < r_limit && gk_ < args.K) x = base[kmajor ? (long long)gr * ld + gk_ : (long long)gk_ * ld + gr];
      if (xf) {
        float f = (float)x;
        if (t0.n > 0) f = (float)(T)apply_list(t0, f);
        if (t1.n > 0) f = (float)(T)apply_list(t1, f);
        x = (T)f;
      }
      constexpr int CPR = BK / 8;
      const int c = k >> 3;
      const int swz = (r / OperandGeom<64, BK, OPK_KMAJOR, false>::RP256) & (CPR - 1);
      *(T*)(dst + 16 * (r * CPR + (c ^ swz)) + (k & 7) * 2) = x;
    }
  };

  typedef FragReader<BM, BK, OPK_KMAJOR, false, FM> RA;
  typedef FragReader<BN, BK, OPK_KMAJOR, false, FN> RB;
  RA ra;
  RB rb;
  ra.init(wm * Cfg::WTM, lane);
  rb.init(wn * Cfg::WTN, lane);
  const unsigned lds_base = (unsigned)(uintptr_t)GK_LDS_PTR(char, smem);
  ra.set_stage(lds_base);
  rb.set_stage(lds_base + GA::BYTES);

  const int KT = (args.K + BK - 1) / BK;
  for (int kt = 0; kt < KT; ++kt) {
    load_tile(A, args.lda, Cfg::A_KMAJOR, BM, m0, args.M, kt * BK, sa, Cfg::A_PER_THREAD, xf_a, args.t[H_GL2SH_A], args.t[H_SH2RF_A], 0);
    load_tile(B, args.ldb, Cfg::B_KMAJOR, BN, n0, args.N, kt * BK, sb, Cfg::B_PER_THREAD, xf_b, args.t[H_GL2SH_B], args.t[H_SH2RF_B], 0);
    __syncthreads();
    static_for<0, Cfg::KSTEPS>([&](auto ks_c) {
      constexpr int ks = decltype(ks_c)::value;
      typename RA::Raw fa[FM];
      typename RB::Raw fb[FN];
      load_frags<ks>(ra, rb, fa, fb);
      wait_lgkmcnt<0>();
      int4v va[FM], vb[FN];
#pragma unroll
      for (int fi = 0; fi < FM; ++fi) { RA::pin_raw(fa[fi]); va[fi] = RA::finish(fa[fi]); }
#pragma unroll
      for (int fj = 0; fj < FN; ++fj) { RB::pin_raw(fb[fj]); vb[fj] = RB::finish(fb[fj]); }
#pragma unroll
      for (int fi = 0; fi < FM; ++fi)
#pragma unroll
        for (int fj = 0; fj < FN; ++fj) acc[fi][fj] = Mfma<T>::run(vb[fj], va[fi], acc[fi][fj]);
    });
    __syncthreads();
  }

#pragma unroll
  for (int fi = 0; fi < FM; ++fi)
#pragma unroll
    for (int fj = 0; fj < FN; ++fj)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int r = mrow + 32 * fi, cc = ncol + 32 * fj + 8 * (v / 4) + (v % 4);
        float x = apply_list(args.t[H_RF2SH_D], acc[fi][fj][v]);
        if (args.epi_kind == 1) x = x + args.bias[cc < args.N ? cc : 0];
        else if (args.epi_kind == 2) x = x + args.bias[r < args.M ? r : 0];
        x = apply_list(args.t[H_SH2GL_D], x);
        if (r < args.M && cc < args.N) store_cd(args.d, args.d_dtype, r + (long long)cc * args.ldd, x);
      }
}

}  // namespace gk
