// Tiled GEMM on the vector ALUs: stands where Operator.FPUOp / TropicalFPUOp stand in the
// reference (src/operator.jl:35-153) together with the kernels that drive them
// (src/kernel.jl:10-129, 147-350).
//
// Every output element is one accumulator updated by a scalar fused multiply-add per k, in
// ascending k, exactly like FPUOp.mma (src/operator.jl:139-153), so results are bit-identical to
// a sequential fma loop on the host.  The accumulator type TACC is the element type of C and D and
// the multiplicands are converted to it before the fma, which is what Julia's promotion makes of
// fma(a::CT, b::CT, c::AT) for the type triples the reference runs (configs/configs.jl:489-497):
// Float16 -> Float32, Float32 -> Float32, Float32 -> Float64, Float64 -> Float64 and Int16 / Int32 /
// Int64 with wrap-around.  A wave is a LANES_M x LANES_N grid of lanes (the reference's base shape
// OPERATOR_M_BASE x OPERATOR_N_BASE, src/operator.jl:58-61: 32 lanes there, 64 here; 8 x 8 unless a
// configuration asks for another grid); a lane owns TM x TN outputs in chunks of up to 4 so that LDS
// reads and D stores are vector accesses.  Tiles go global -> registers -> LDS with the next tile's global
// loads in flight during the fmas of the current one.  With CHECKED the loads and stores are per
// element and bounds-checked (reference Layout.ColMajor / RowMajor, src/layout.jl:117-184:
// out-of-range loads give 0, out-of-range stores are dropped), so any problem size and any leading
// dimension works.
#pragma once
#include "common.hpp"
#include <type_traits>

namespace gk {

// dtype code of an element type
template <typename T> struct DtypeOf;
template <> struct DtypeOf<_Float16> { static constexpr int DT = DT_F16; };
template <> struct DtypeOf<float> { static constexpr int DT = DT_F32; };
template <> struct DtypeOf<double> { static constexpr int DT = DT_F64; };
template <> struct DtypeOf<short> { static constexpr int DT = DT_I16; };
template <> struct DtypeOf<int> { static constexpr int DT = DT_I32; };
template <> struct DtypeOf<long long> { static constexpr int DT = DT_I64; };

// The type a transform of a T-typed value is evaluated in (one rounding per op): fp32 for the
// 16- and 32-bit floats, fp64 for fp64, the integer type itself for integers.
template <typename T> struct ArithOf { typedef T type; };
template <> struct ArithOf<_Float16> { typedef float type; };

// One elementwise op in arithmetic type X.  The fp32 forms are those of apply_op; integers wrap.
template <typename X>
__device__ __forceinline__ X apply_op_t(int kind, float p0, float p1, X x) {
  if constexpr (std::is_same<X, float>::value) {
    return apply_op(kind, p0, p1, x);
  } else if constexpr (std::is_floating_point<X>::value) {
    const X q0 = (X)p0, q1 = (X)p1;
    switch (kind) {
      case T_SCALE: return x * q0;
      case T_ADD: return x + q0;
      case T_RELU: return x > (X)0 ? x : (X)0;
      case T_NEG: return -x;
      case T_ABS: return x < (X)0 ? -x : x;
      case T_CLAMP: return x < q0 ? q0 : (x > q1 ? q1 : x);
      case T_SQUARE: return x * x;
      default: return x;
    }
  } else {
    typedef typename std::make_unsigned<X>::type U;
    const X q0 = (X)p0, q1 = (X)p1;
    switch (kind) {
      case T_SCALE: return (X)((U)x * (U)q0);
      case T_ADD: return (X)((U)x + (U)q0);
      case T_RELU: return x > 0 ? x : (X)0;
      case T_NEG: return (X)((U)0 - (U)x);
      case T_ABS: return x < 0 ? (X)((U)0 - (U)x) : x;
      case T_CLAMP: return x < q0 ? q0 : (x > q1 ? q1 : x);
      case T_SQUARE: return (X)((U)x * (U)x);
      default: return x;
    }
  }
}

// A list applied to COUNT values at once.  The loop over the slots of the list is unrolled (with constant indices
// the launch arguments stay in the kernel-argument segment; a run-time index makes the compiler copy the whole
// argument block to scratch memory once the kernel is large, and every later access to it then goes to memory)
// and the switch on the op is paid once per slot, not once per value.
template <typename X, int COUNT>
__device__ __forceinline__ void apply_list_regs_t(const OpList& t, X (&x)[COUNT]) {
#pragma unroll
  for (int i = 0; i < kMaxOps; ++i)
    if (i < t.n) {
      const float p0 = t.p0[i], p1 = t.p1[i];
      auto each = [&](auto kind_c) __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < COUNT; ++e) x[e] = apply_op_t<X>(decltype(kind_c)::value, p0, p1, x[e]);
      };
      switch (t.kind[i]) {
        case T_SCALE: each(std::integral_constant<int, T_SCALE>{}); break;
        case T_ADD: each(std::integral_constant<int, T_ADD>{}); break;
        case T_RELU: each(std::integral_constant<int, T_RELU>{}); break;
        case T_NEG: each(std::integral_constant<int, T_NEG>{}); break;
        case T_ABS: each(std::integral_constant<int, T_ABS>{}); break;
        case T_CLAMP: each(std::integral_constant<int, T_CLAMP>{}); break;
        case T_SQUARE: each(std::integral_constant<int, T_SQUARE>{}); break;
        default: break;
      }
    }
}

// acc <- a * b + acc with one rounding (floats) or wrap-around (integers): operator_fma of FPUOp
template <typename TACC>
__device__ __forceinline__ TACC fpu_fma(TACC a, TACC b, TACC c) {
  if constexpr (std::is_same<TACC, float>::value) return __builtin_fmaf(a, b, c);
  else if constexpr (std::is_same<TACC, double>::value) return __builtin_fma(a, b, c);
  else {
    typedef typename std::make_unsigned<TACC>::type U;
    return (TACC)((U)a * (U)b + (U)c);
  }
}

template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, typename TIN_, bool A_KMAJOR_, bool B_KMAJOR_, bool CHECKED_,
          bool TROPICAL_, typename TACC_ = float, bool FUSED_ = true, int LANES_M_ = 8>
struct FpuGemmConfig {
  // the lane grid of a wave: lane l stands at row l % LANES_M, column l / LANES_M of it (reference src/operator.jl:61)
  static constexpr int LANES_M = LANES_M_, LANES_N = kWaveSize / LANES_M_;
  static_assert(LANES_M_ > 0 && kWaveSize % LANES_M_ == 0, "the lane grid is LANES_M x (64 / LANES_M)");
  // FUSED: the kernel carries the eight transform hooks and the bias; without, none of that code exists
  static constexpr bool FUSED = FUSED_;
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr bool A_KMAJOR = A_KMAJOR_, B_KMAJOR = B_KMAJOR_, CHECKED = CHECKED_, TROPICAL = TROPICAL_;
  typedef TIN_ TIN;
  typedef TACC_ TACC;
  static constexpr int THREADS = WAVES_M * WAVES_N * kWaveSize;
  static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static constexpr int TM = WTM / LANES_M, TN = WTN / LANES_N;          // outputs per lane
  // a lane's outputs come in chunks of consecutive rows (columns), 4 wide, or fewer where a lane owns fewer
  static constexpr int CWM = TM < 4 ? TM : 4, CWN = TN < 4 ? TN : 4;
  static constexpr int CM = TM / CWM, CN = TN / CWN;        // chunks per lane
  static constexpr int PAD = 4;
  static constexpr int LDA_S = BM + PAD, LDB_S = BN + PAD;  // LDS row pitch (elements of TACC), rows are k
  static constexpr int LDS_BYTES = (BK * LDA_S + BK * LDB_S) * (int)sizeof(TACC);
  static constexpr int A_CHUNKS = BM * BK / 4, B_CHUNKS = BN * BK / 4;
  static constexpr int A_PER_THREAD = A_CHUNKS / THREADS, B_PER_THREAD = B_CHUNKS / THREADS;
  // K tiles whose global loads are in flight (in registers) while the current one is multiplied: the fma chain
  // of a tile is shorter than the memory latency, so one tile ahead left every tile waiting for its loads
  // (256^3 on 16 workgroups: 19.4 us with one tile in flight)
  // -- four tiles without hooks, two with; the bounds-checked and the 64-bit kernels stay with one (their
  // per-element loads and wide registers make deeper buffers expensive to compile and to hold)
  static constexpr int DEPTH = (CHECKED_ || sizeof(TIN_) > 4) ? 1 : (FUSED_ ? 2 : 4);
  static_assert(WTM % LANES_M == 0 && WTN % LANES_N == 0 && TM >= 1 && TN >= 1 && TM % CWM == 0 && TN % CWN == 0,
                "the lane grid divides the wave tile and a lane owns whole chunks");
  static_assert(LANES_M_ != 8 || (TM >= 2 && TN >= 2), "8 x 8 lanes: a lane owns whole chunks of 2 or 4 outputs");
  static_assert(A_CHUNKS % THREADS == 0 && B_CHUNKS % THREADS == 0, "tile loads divide evenly over the threads");
  static_assert(!TROPICAL || std::is_same<TACC, float>::value, "the max-plus product is compiled for fp32");
};

// Loads the 4 elements of chunk `chunk` of an R x BK operand tile: rows r0.. of the operand,
// k from k0.  MAJOR_K: memory is contiguous along k.  Out-of-range elements read as 0.  The values
// stay in the operand's own type until the load hooks have run.
template <class Cfg, int R, bool KMAJOR>
__device__ __forceinline__ void load_chunk(const typename Cfg::TIN* __restrict__ base, long long ld, int r0, int k0, int chunk,
                                           int r_limit, int k_limit, bool zero, typename Cfg::TIN (&out)[4], bool (&pad_k)[4],
                                           int& r_local, int& k_local) {
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
#pragma unroll
  for (int e = 0; e < 4; ++e) pad_k[e] = false;
  if (zero) {          // Layout.Zero: nothing is read (alpha == 0, reference src/matmul.jl:127-130)
#pragma unroll
    for (int e = 0; e < 4; ++e) out[e] = (TIN)0;
  } else if (!Cfg::CHECKED) {
    const TIN* p = base + (KMAJOR ? (long long)r * ld + k : (long long)k * ld + r);
    typedef TIN vec4 __attribute__((ext_vector_type(4)));
    const vec4 v = *(const vec4*)p;
#pragma unroll
    for (int e = 0; e < 4; ++e) out[e] = v[e];
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int rr = KMAJOR ? r : r + e, kk = KMAJOR ? k + e : k;
      TIN x = (TIN)0;
      pad_k[e] = kk >= k_limit;     // the tropical product pads k with -inf so that max() ignores it
      if (rr < r_limit && kk < k_limit) x = base[KMAJOR ? (long long)rr * ld + kk : (long long)kk * ld + rr];
      out[e] = x;
    }
  }
}

template <int I, int N, class F>
__device__ __forceinline__ void fpu_static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    fpu_static_for<I + 1, N>(f);
  }
}

template <class Cfg>
__global__ void __launch_bounds__(Cfg::THREADS) fpu_gemm_kernel(const GemmArgs args) {
  typedef typename Cfg::TIN TIN;
  typedef typename Cfg::TACC TACC;
  typedef typename ArithOf<TIN>::type TAR;       // arithmetic type of the A / B hooks
  typedef TACC acc4 __attribute__((ext_vector_type(4)));
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, TM = Cfg::TM, TN = Cfg::TN;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  TACC* As = (TACC*)smem;                         // [BK][LDA_S], rows are k
  TACC* Bs = As + BK * Cfg::LDA_S;                // [BK][LDB_S]

  int ti, tj;
  cta_swizzle(args.swz_kind, args.swz_param, (int)blockIdx.x, (int)blockIdx.y, args.nbm, args.nbn, ti, tj);
  if (ti >= args.nbm || tj >= args.nbn) return;
  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave % Cfg::WAVES_M, wn = wave / Cfg::WAVES_M;
  const int ly = lane % Cfg::LANES_M, lx = lane / Cfg::LANES_M;
  const int m0 = ti * BM, n0 = tj * BN;
  const TIN* A = (const TIN*)args.a;
  const TIN* B = (const TIN*)args.b;
  const TACC* C = (const TACC*)args.c;
  const bool zero_ab = (args.a_kind == 0 /* Layout.Zero */);
  const bool xf_a = Cfg::FUSED && (args.t[H_GL2SH_A].n > 0 || args.t[H_SH2RF_A].n > 0);
  const bool xf_b = Cfg::FUSED && (args.t[H_GL2SH_B].n > 0 || args.t[H_SH2RF_B].n > 0);

  // accumulators: acc[i][j] is row wm*WTM + (i/CW)*LANES_M*CW + CW*ly + i%CW (CW = 4, or fewer), columns likewise with lx
  constexpr int CWM = Cfg::CWM, CWN = Cfg::CWN;
  typedef TACC accm __attribute__((ext_vector_type(CWM)));
  typedef TACC accn __attribute__((ext_vector_type(CWN)));
  TACC acc[TM][TN];
  auto row_of = [&](int i) { return m0 + wm * Cfg::WTM + (i / CWM) * Cfg::LANES_M * CWM + CWM * ly + (i % CWM); };
  auto col_of = [&](int j) { return n0 + wn * Cfg::WTN + (j / CWN) * Cfg::LANES_N * CWN + CWN * lx + (j % CWN); };
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      TACC c = (TACC)0;
      if (args.c_mode != 0) {
        const int r = row_of(i), cc = col_of(j);
        if (!Cfg::CHECKED || (r < args.M && cc < args.N)) c = C[r + (long long)cc * args.ldc];
      }
      acc[i][j] = c;
    }
  // one hook over all accumulators of the lane
  [[maybe_unused]] auto hook_acc = [&](const OpList& t) __attribute__((always_inline)) {
    TACC flat[TM * TN];
#pragma unroll
    for (int q = 0; q < TM * TN; ++q) flat[q] = acc[q % TM][q / TM];
    apply_list_regs_t<TACC, TM * TN>(t, flat);
#pragma unroll
    for (int q = 0; q < TM * TN; ++q) acc[q % TM][q / TM] = flat[q];
  };
  if constexpr (Cfg::FUSED) {
    if (args.c_mode != 0) {
      hook_acc(args.t[H_GL2SH_C]);
      hook_acc(args.t[H_SH2RF_C]);
    }
  }

  constexpr int DEPTH = Cfg::DEPTH;
  TIN ra[DEPTH][Cfg::A_PER_THREAD][4], rb[DEPTH][Cfg::B_PER_THREAD][4];
  bool pa[DEPTH][Cfg::A_PER_THREAD][4], pb[DEPTH][Cfg::B_PER_THREAD][4];
  int ar[Cfg::A_PER_THREAD], ak[Cfg::A_PER_THREAD], br[Cfg::B_PER_THREAD], bk[Cfg::B_PER_THREAD];   // the same for every tile

  auto fetch = [&](int k0, auto slot_c) __attribute__((always_inline)) {
    constexpr int S = decltype(slot_c)::value;
#pragma unroll
    for (int i = 0; i < Cfg::A_PER_THREAD; ++i) {
      load_chunk<Cfg, BM, Cfg::A_KMAJOR>(A, args.lda, m0, k0, tid + i * Cfg::THREADS, args.M, args.K, zero_ab, ra[S][i], pa[S][i], ar[i], ak[i]);
    }
#pragma unroll
    for (int i = 0; i < Cfg::B_PER_THREAD; ++i) {
      load_chunk<Cfg, BN, Cfg::B_KMAJOR>(B, args.ldb, n0, k0, tid + i * Cfg::THREADS, args.N, args.K, zero_ab, rb[S][i], pb[S][i], br[i], bk[i]);
    }
  };
  // the two load hooks, each rounded to the element type of its destination (the operand's own
  // type), then the conversion to the accumulator type for the fma
  auto prepare = [&](const TIN (&v)[4], const bool (&pad)[4], bool xf, const OpList& t0, const OpList& t1, TACC (&out)[4]) {
    TIN x[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) x[e] = v[e];
    if constexpr (Cfg::FUSED) {
      if (xf) {
        TAR y[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = (TAR)x[e];
        if (t0.n > 0) {
          apply_list_regs_t<TAR, 4>(t0, y);
#pragma unroll
          for (int e = 0; e < 4; ++e) y[e] = (TAR)(TIN)y[e];       // rounded to the operand's type between the hooks
        }
        if (t1.n > 0) apply_list_regs_t<TAR, 4>(t1, y);
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = (TIN)y[e];
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      TACC y = (TACC)x[e];
      if constexpr (Cfg::TROPICAL && Cfg::CHECKED) {
        if (pad[e]) y = -__builtin_inff();
      }
      out[e] = y;
    }
  };
  auto stash = [&](auto slot_c) __attribute__((always_inline)) {
    constexpr int S = decltype(slot_c)::value;
#pragma unroll
    for (int i = 0; i < Cfg::A_PER_THREAD; ++i) {
      TACC v[4];
      prepare(ra[S][i], pa[S][i], xf_a, args.t[H_GL2SH_A], args.t[H_SH2RF_A], v);
      if (Cfg::A_KMAJOR) {
#pragma unroll
        for (int e = 0; e < 4; ++e) As[(ak[i] + e) * Cfg::LDA_S + ar[i]] = v[e];
      } else {
        *(acc4*)&As[ak[i] * Cfg::LDA_S + ar[i]] = (acc4){v[0], v[1], v[2], v[3]};
      }
    }
#pragma unroll
    for (int i = 0; i < Cfg::B_PER_THREAD; ++i) {
      TACC v[4];
      prepare(rb[S][i], pb[S][i], xf_b, args.t[H_GL2SH_B], args.t[H_SH2RF_B], v);
      if (Cfg::B_KMAJOR) {
#pragma unroll
        for (int e = 0; e < 4; ++e) Bs[(bk[i] + e) * Cfg::LDB_S + br[i]] = v[e];
      } else {
        *(acc4*)&Bs[bk[i] * Cfg::LDB_S + br[i]] = (acc4){v[0], v[1], v[2], v[3]};
      }
    }
  };

  const int KT = (args.K + BK - 1) / BK;
  fpu_static_for<0, DEPTH>([&](auto slot_c) __attribute__((always_inline)) {
    constexpr int S = decltype(slot_c)::value;
    if (S < KT) fetch(S * BK, slot_c);
  });
  for (int kt0 = 0; kt0 < KT; kt0 += DEPTH)
  fpu_static_for<0, DEPTH>([&](auto slot_c) __attribute__((always_inline)) {
    constexpr int S = decltype(slot_c)::value;       // register buffer of tile kt
    const int kt = kt0 + S;
    if (kt < KT) {
    __syncthreads();          // everyone is done reading the previous tile
    stash(slot_c);
    __syncthreads();
    if (kt + DEPTH < KT) fetch((kt + DEPTH) * BK, slot_c);      // its buffer is free again
    const TACC* ap = As + wm * Cfg::WTM + CWM * ly;
    const TACC* bp = Bs + wn * Cfg::WTN + CWN * lx;
#pragma unroll 4
    for (int k = 0; k < BK; ++k) {
      TACC a[TM], b[TN];
#pragma unroll
      for (int c = 0; c < Cfg::CM; ++c) {
        const accm v = *(const accm*)&ap[k * Cfg::LDA_S + c * Cfg::LANES_M * CWM];
#pragma unroll
        for (int e = 0; e < CWM; ++e) a[CWM * c + e] = v[e];
      }
#pragma unroll
      for (int c = 0; c < Cfg::CN; ++c) {
        const accn v = *(const accn*)&bp[k * Cfg::LDB_S + c * Cfg::LANES_N * CWN];
#pragma unroll
        for (int e = 0; e < CWN; ++e) b[CWN * c + e] = v[e];
      }
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          if constexpr (Cfg::TROPICAL) {
            const TACC s = a[i] + b[j];
            acc[i][j] = s > acc[i][j] ? s : acc[i][j];
          } else {
            acc[i][j] = fpu_fma<TACC>(a[i], b[j], acc[i][j]);
          }
        }
    }
    }
  });

  // epilogue: transform, bias, transform, store (a chunk of consecutive rows per vector store); the bias of
  // Epilogue.Bias is fp32 (reference src/epilogue.jl:44-52) and only offered with fp32 accumulators
  TACC* D = (TACC*)args.d;
  if constexpr (Cfg::FUSED) {
    hook_acc(args.t[H_RF2SH_D]);
    if constexpr (std::is_same<TACC, float>::value) {
      if (args.epi_kind == 1) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int cc = col_of(j);
          const float bv = args.bias[Cfg::CHECKED ? (cc < args.N ? cc : 0) : cc];
#pragma unroll
          for (int i = 0; i < TM; ++i) acc[i][j] = acc[i][j] + bv;
        }
      } else if (args.epi_kind == 2) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const int r = row_of(i);
          const float bv = args.bias[Cfg::CHECKED ? (r < args.M ? r : 0) : r];
#pragma unroll
          for (int j = 0; j < TN; ++j) acc[i][j] = acc[i][j] + bv;
        }
      }
    }
    hook_acc(args.t[H_SH2GL_D]);
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int cc = col_of(j);
#pragma unroll
    for (int c = 0; c < Cfg::CM; ++c) {
      const int r = row_of(CWM * c);
      if (!Cfg::CHECKED) {
        accm v;
#pragma unroll
        for (int e = 0; e < CWM; ++e) v[e] = acc[CWM * c + e][j];
        *(accm*)&D[r + (long long)cc * args.ldd] = v;
      } else {
#pragma unroll
        for (int e = 0; e < CWM; ++e)
          if (r + e < args.M && cc < args.N) D[r + e + (long long)cc * args.ldd] = acc[CWM * c + e][j];
      }
    }
  }
}

}  // namespace gk
