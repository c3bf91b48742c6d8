// Bounds-checked MFMA GEMM for operands of any size, alignment and leading dimension: stands where
// Kernel.matmul_singlestage with the Layout.ColMajor / RowMajor layouts stands in the reference
// (src/kernel.jl:10-129, src/layout.jl:117-184).  Elements are loaded one by one (out-of-range
// reads give 0), written to LDS in the K-major swizzled tile layout of the fast kernel, and the
// same fragment reader and MFMA sequence consume them; out-of-range stores are dropped.  One LDS
// stage; the element loads of the next four tiles are in flight (in registers) while the current
// one is multiplied.  Scalar accesses make it several times slower than the aligned kernels, like the
// reference's checked layouts.
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
  typedef OperandGeom<BM, BK, OPK_KMAJOR> GA;     // both LDS tiles are K-major whatever the memory order
  typedef OperandGeom<BN, BK, OPK_KMAJOR> GB;
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
        if (args.c_mode != 0 && blockIdx.z == 0) {       // K-split launches: the first slice starts from C
          if (r < args.M && cc < args.N) c = load_cd(args.c, args.c_dtype, r + (long long)cc * args.ldc);
          c = apply_list(args.t[H_GL2SH_C], c);
          c = apply_list(args.t[H_SH2RF_C], c);
          c = c * args.acc_pre_scale;          // 1 unless the host folded a power-of-two scale of A or B
        }
        acc[fi][fj][v] = c;
      }

  // element e of a tile: K-major memory walks k fastest, M-major memory walks the row fastest, so
  // that consecutive threads touch consecutive addresses.  fetch() only issues the loads of a tile
  // (all of them before anything waits); stash() runs the hooks and writes the tile to LDS.
  auto coords = [&](auto kmajor_c, auto rows_c, int i, int& r, int& k) __attribute__((always_inline)) {
    constexpr bool KMAJOR = decltype(kmajor_c)::value;
    constexpr int R = decltype(rows_c)::value;
    const int e = tid + i * Cfg::THREADS;
    if (KMAJOR) { r = e / BK; k = e % BK; } else { k = e / R; r = e % R; }
  };
  auto fetch = [&](const T* base, long long ld, auto kmajor_c, auto rows_c, int r0, int r_limit, int k0, auto& regs) __attribute__((always_inline)) {
    constexpr bool KMAJOR = decltype(kmajor_c)::value;
    constexpr int PER = decltype(rows_c)::value * BK / Cfg::THREADS;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      int r, k;
      coords(kmajor_c, rows_c, i, r, k);
      const int gr = r0 + r, gk_ = k0 + k;
      T x = (T)0.0f;
      if (!zero_ab && gr < r_limit && gk_ < args.K) x = base[KMAJOR ? (long long)gr * ld + gk_ : (long long)gk_ * ld + gr];
      regs[i] = x;
    }
  };
  auto stash = [&](auto kmajor_c, auto rows_c, const auto& regs, char* dst, bool xf, auto h0_c, auto h1_c) __attribute__((always_inline)) {
    const OpList& t0 = args.t[decltype(h0_c)::value];
    const OpList& t1 = args.t[decltype(h1_c)::value];
    constexpr int PER = decltype(rows_c)::value * BK / Cfg::THREADS;
    T vals[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) vals[i] = regs[i];
    if (xf) {
      // each of the two hooks is evaluated in fp32 and rounded to the operand's type; the dispatch on the
      // op runs once per list, not once per element
      float f[PER];
#pragma unroll
      for (int i = 0; i < PER; ++i) f[i] = (float)vals[i];
      if (t0.n > 0) {
        apply_list_regs<PER>(t0, f);
#pragma unroll
        for (int i = 0; i < PER; ++i) f[i] = (float)(T)f[i];
      }
      if (t1.n > 0) {
        apply_list_regs<PER>(t1, f);
#pragma unroll
        for (int i = 0; i < PER; ++i) f[i] = (float)(T)f[i];
      }
#pragma unroll
      for (int i = 0; i < PER; ++i) vals[i] = (T)f[i];
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      int r, k;
      coords(kmajor_c, rows_c, i, r, k);
      const T x = vals[i];
      constexpr int CPR = BK / 8;
      const int c = k >> 3;
      const int swz = (r / OperandGeom<64, BK, OPK_KMAJOR>::RP256) & (CPR - 1);
      *(T*)(dst + 16 * (r * CPR + (c ^ swz)) + (k & 7) * 2) = x;
    }
  };
  typedef std::integral_constant<bool, Cfg::A_KMAJOR> AKM;
  typedef std::integral_constant<bool, Cfg::B_KMAJOR> BKM;
  typedef std::integral_constant<int, BM> RowsA;
  typedef std::integral_constant<int, BN> RowsB;
  // tiles in flight: a workgroup at the rim of a cut-up product runs alone on its CU and its K loop is
  // as long as the memory latency times the number of tiles divided by this depth
  constexpr int DEPTH = 4;
  T ga[DEPTH][Cfg::A_PER_THREAD], gb[DEPTH][Cfg::B_PER_THREAD];

  typedef FragReader<BM, BK, OPK_KMAJOR, FM> RA;
  typedef FragReader<BN, BK, OPK_KMAJOR, FN> RB;
  RA ra;
  RB rb;
  ra.init(wm * Cfg::WTM, lane);
  rb.init(wn * Cfg::WTN, lane);
  const unsigned lds_base = (unsigned)(uintptr_t)GK_LDS_PTR(char, smem);
  ra.set_stage(lds_base);
  rb.set_stage(lds_base + GA::BYTES);

  // K tiles of this workgroup: all of them, or (k_steps > 0) the slice blockIdx.z of a K-split launch
  int kt_first = 0, KT = (args.K + BK - 1) / BK;
  if (args.k_steps > 0) {
    kt_first = (int)blockIdx.z * args.k_steps;
    KT = KT < kt_first + args.k_steps ? KT : kt_first + args.k_steps;
    if (kt_first >= KT) return;       // the whole workgroup leaves together, before any barrier
  }
  static_for<0, DEPTH>([&](auto j_c) __attribute__((always_inline)) {
    constexpr int j = decltype(j_c)::value;
    if (kt_first + j < KT) {
      fetch(A, args.lda, AKM{}, RowsA{}, m0, args.M, (kt_first + j) * BK, ga[j]);
      fetch(B, args.ldb, BKM{}, RowsB{}, n0, args.N, (kt_first + j) * BK, gb[j]);
    }
  });
  for (int kt0 = kt_first; kt0 < KT; kt0 += DEPTH)
  static_for<0, DEPTH>([&](auto j_c) __attribute__((always_inline)) {
    constexpr int j = decltype(j_c)::value;       // register buffer of tile kt
    const int kt = kt0 + j;
    if (kt < KT) {
    stash(AKM{}, RowsA{}, ga[j], sa, xf_a, std::integral_constant<int, H_GL2SH_A>{}, std::integral_constant<int, H_SH2RF_A>{});
    stash(BKM{}, RowsB{}, gb[j], sb, xf_b, std::integral_constant<int, H_GL2SH_B>{}, std::integral_constant<int, H_SH2RF_B>{});
    __syncthreads();
    if (kt + DEPTH < KT) {     // its buffer is free again: tile kt + DEPTH starts to travel
      fetch(A, args.lda, AKM{}, RowsA{}, m0, args.M, (kt + DEPTH) * BK, ga[j]);
      fetch(B, args.ldb, BKM{}, RowsB{}, n0, args.N, (kt + DEPTH) * BK, gb[j]);
    }
    static_for<0, Cfg::KSTEPS>([&](auto ks_c) {
      constexpr int ks = decltype(ks_c)::value;
      typename RA::Raw fa[FM];
      typename RB::Raw fb[FN];
      load_frags<ks>(ra, rb, fa, fb);
      wait_lgkmcnt<0>();
      int4v va[FM], vb[FN];
#pragma unroll
      for (int fi = 0; fi < FM; ++fi) { RA::pin_raw(fa[fi]); va[fi] = RA::finish(fa[fi], lane); }
#pragma unroll
      for (int fj = 0; fj < FN; ++fj) { RB::pin_raw(fb[fj]); vb[fj] = RB::finish(fb[fj], lane); }
#pragma unroll
      for (int fi = 0; fi < FM; ++fi)
#pragma unroll
        for (int fj = 0; fj < FN; ++fj) acc[fi][fj] = Mfma<T>::run(vb[fj], va[fi], acc[fi][fj]);
    });
    __syncthreads();
    }
  });

  // K-split launches: the partial tiles of the slices meet in the workspace, the last workgroup to arrive
  // sums them in slice order and stores D (the loop above ends with a barrier: LDS is free)
  if (args.k_slices > 1 && !splitk_reduce<Cfg::THREADS>(acc, args, ti + tj * args.nbm, (unsigned*)smem)) return;

#pragma unroll
  for (int fi = 0; fi < FM; ++fi)
#pragma unroll
    for (int fj = 0; fj < FN; ++fj)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int r = mrow + 32 * fi, cc = ncol + 32 * fj + 8 * (v / 4) + (v % 4);
        float x = apply_list(args.t[H_RF2SH_D], acc[fi][fj][v] * args.acc_post_scale);
        if (args.epi_kind == 1) x = x + args.bias[cc < args.N ? cc : 0];
        else if (args.epi_kind == 2) x = x + args.bias[r < args.M ? r : 0];
        x = apply_list(args.t[H_SH2GL_D], x);
        if (r < args.M && cc < args.N) {
          store_cd(args.d, args.d_dtype, r + (long long)cc * args.ldd, x);
        }
      }
}

}  // namespace gk
