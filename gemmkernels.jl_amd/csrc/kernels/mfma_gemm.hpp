// Tiled GEMM on the CDNA4 matrix cores: D = epilogue(T_d(sum_k T_a(A) * T_b(B) + T_c(C))).
//
// Stands where Kernel.matmul_pipelined stands in the reference (src/kernel.jl:147-350) with
// Operator.WMMAOp (src/operator.jl:163-245) and the UnsafeAligned{Col,Row}Major layouts
// (src/layout.jl:192-219, 244-270), re-designed for gfx950:
//
//  * one v_mfma_f32_16x16x32 per 16x16x32 product (v_mfma_f32_32x32x16 where MI = 32 is asked for),
//    64-lane waves, accumulators stay in registers from the C load to the D store (the reference
//    round-trips them through LDS);
//  * A and B tiles travel global -> LDS with global_load_lds_dwordx4 (no register staging),
//    STAGES tiles deep, one s_barrier per K step;
//  * LDS tiles are XOR-swizzled in 16-byte chunks so that both the DMA writes and the fragment
//    reads are bank-conflict free (64 banks x 4 B, conflicts are resolved per 32-lane half);
//  * operands whose K index is contiguous in memory ("K-major": A of a 'T' GEMM, B of an 'N'
//    GEMM) are read with ds_read_b128, the others ("M-major") with the transposing
//    ds_read_b64_tr_b16, so all four transposes run at the same speed;
//  * the MFMA is issued with swapped operands (B fragment first) so that 16 (32) consecutive lanes
//    own consecutive rows m of D and write 64 (128) contiguous bytes of a column of D; the blocks
//    of a wave tile are walked so that the two halves of a 128-byte line follow each other.
#pragma once
#include "common.hpp"
#include <type_traits>

namespace gk {

// ----------------------------------------------------------------------------------------------
// Operand tiles in LDS.  R is the number of MFMA rows of the block tile in the operand's own
// dimension (m or n), BK the number of 16-bit k-values per K step.
//   OPK_KMAJOR: LDS row = tile row, 16-byte chunk c = k / 8            (memory contiguous along k)
//   OPK_MMAJOR: LDS row = k,        16-byte chunk c = row / 8          (memory contiguous along m / n)
//   OPK_KSPLIT: interleaved complex data contiguous along k, for the FIX_PAIR products: LDS row = complex row index
//               (R/2 of them), 16-byte chunk c = complex k / 4.  A lane reads the 32 bytes (8 complex k) of its
//               complex row once and makes two fragments of them, the real parts for fragment f and the imaginary
//               parts for fragment f + F/2
// ----------------------------------------------------------------------------------------------
enum : int { OPK_KMAJOR = 0, OPK_MMAJOR = 1, OPK_KSPLIT = 4 };
constexpr bool opk_complex_k(int kind) { return kind == OPK_KSPLIT; }
// FIX_PAIR / FIX_PAIR_DUAL: complex (dual-number) product on interleaved matrices as ONE real product of the
// matrices seen as real ones (2M x 2N x K: it holds re*re, re*im, im*re, im*im of every element of D, the four
// products of WMMAComplexOp.mma, reference src/operator.jl:307-311; dual numbers :366-369 use three of them).
// An interleaved matrix whose contiguous index is m (or n) is a real matrix with twice the rows, row 2m the real and
// row 2m+1 the imaginary parts, and the K loop of the real kernel runs on it unchanged (K counts complex k): the two
// parts of a row of A then sit in the lanes 2i, 2i+1, those of a column of B in the accumulator values 2j, 2j+1.
// One whose contiguous index is k is read as OPK_KSPLIT: the two parts sit in the row (column) blocks f and f + F/2.
// The four products are combined once, before the epilogue.
// FIX_PLANAR: the same for planar (split re / im) matrices, whose planes are plain real matrices: the real view of A
// is [A_re; A_im] stacked along m and that of B [B_re, B_im] side by side along n.  The tile rows (columns) are
// dealt out so that every wave holds both parts of its complex rows (columns): the upper half of the row blocks of
// a wave tile comes from A_re, the lower half from the same rows of A_im, the left half of the column blocks from
// B_re and the right half from B_im.  The four real products of an element of D then lie in four accumulator
// blocks of one lane and are combined without any exchange.
enum : int { FIX_NONE = 0, FIX_PLANAR = 3, FIX_PAIR = 4, FIX_PAIR_DUAL = 5 };

template <int R, int BK, int KIND>
struct OperandGeom {
  static constexpr int LDS_ROWS = KIND == OPK_KMAJOR ? R : (opk_complex_k(KIND) ? R / 2 : BK);
  static constexpr int ROW_BYTES = KIND == OPK_KMAJOR ? BK * 2 : (opk_complex_k(KIND) ? BK * 4 : R * 2);
  static constexpr int CPR = ROW_BYTES / 16;                   // 16-byte chunks per LDS row
  static constexpr int BYTES = LDS_ROWS * ROW_BYTES;
  static constexpr int NDMA = BYTES / 1024;                    // wave-wide 16 B/lane DMA instructions per tile
  static constexpr int RP256 = (256 / ROW_BYTES) > 1 ? (256 / ROW_BYTES) : 1;   // LDS rows per 256 B
  // K-major: XOR the chunk index with the row (per 256 B) so that 32 consecutive rows at one chunk
  // index spread evenly over the 16 chunk slots of the 64 banks.
  __device__ static __forceinline__ int swz_k(int row) { return (row / RP256) & (CPR - 1); }
  // OPK_KSPLIT: the 16 lanes of a read take one 16-byte chunk each from 16 consecutive complex rows, first the
  // chunk 2g of every row, then the chunk 2g + 1.  The XOR below sends the 16 rows to the 16 chunk slots of the
  // bank period for either chunk: eight rows in a row differ in the upper bits, a row and the one eight rows
  // further trade the two chunks of a pair.
  __device__ static __forceinline__ int swz_kp(int row) {
    const int q = row / RP256;
    return ((q & (CPR / 2 - 1)) << 1) | ((q / (CPR / 2)) & 1);
  }
  // M-major: XOR the 64-byte group index with k so that 4 consecutive k rows at one group land in
  // 4 different 64-byte slots of the 256-byte bank period.
  // Rows of 384 bytes (192 elements): consecutive k rows are already 128 bytes apart in the bank period, so
  // the XOR moves rows k + 2, k + 3 by one group (and stays inside the six groups of such a row).
  static constexpr int GROUPS = CPR / 4;
  static constexpr bool ROW_384 = KIND == OPK_MMAJOR && (ROW_BYTES % 256) == 128;
  static constexpr int GMASK = ROW_384 ? 1 : ((GROUPS - 1) < 3 ? (GROUPS - 1) : 3);
  __device__ static __forceinline__ int swz_m(int k) { return ROW_384 ? ((k >> 1) & 1) : ((k / RP256) & GMASK); }
  // ... and the two 32-byte halves of a 64-byte group trade places on every other block of 8 k rows, so
  // that the 16-lane groups of a transposing read for 16-row fragments (k, k + 8, ...) use both halves
  static_assert(KIND == OPK_MMAJOR || (CPR & (CPR - 1)) == 0, "chunks per row must be a power of two");
  static_assert(KIND != OPK_MMAJOR || ROW_384 || (GROUPS & (GROUPS - 1)) == 0, "M-major rows: a power of two of 64-byte groups, or 384 bytes");
  static_assert(!ROW_384 || GROUPS % 2 == 0, "the group XOR of 384-byte rows pairs groups");
  static_assert(KIND != OPK_MMAJOR || CPR >= 4, "M-major tiles need at least 32 rows");
  static_assert(BYTES % 1024 == 0, "tile must be a whole number of DMA instructions");
};

// Where lane `lane` of DMA instruction q reads: LDS row `row` of the tile and the first of its 8
// consecutive 16-bit elements `col` inside that row's span of memory (swizzle undone).  The data
// lands at LDS chunk position q*64 + lane.
template <class G, int KIND>
__device__ __forceinline__ void dma_lane_coords(int q, int lane, int& row, int& col) {
  const int p = q * 64 + lane;
  row = p / G::CPR;
  const int cs = p % G::CPR;
  if (KIND == OPK_KMAJOR) col = (cs ^ G::swz_k(row)) * 8;
  else if (opk_complex_k(KIND)) col = (cs ^ G::swz_kp(row)) * 8;
  else col = (((cs >> 2) ^ G::swz_m(row)) * 4 + ((cs & 3) ^ (((row >> 3) & 1) << 1))) * 8;
}

// A pointer that is the same in every lane, as one pair of scalar registers that the compiler does not look into.
__device__ __forceinline__ void pin_scalar(const char*& p) {
  const unsigned long long x = (unsigned long long)p;
  int lo = __builtin_amdgcn_readfirstlane((int)(unsigned)x), hi = __builtin_amdgcn_readfirstlane((int)(unsigned)(x >> 32));
  asm volatile("" : "+s"(lo), "+s"(hi));
  p = (const char*)(((unsigned long long)(unsigned)hi << 32) | (unsigned)lo);
}

// Tensor-contraction index maps: walks the K index of a contraction tile by tile.  A tile covers the K modes below
// `mode` whole and `step` indices of mode `mode` (see GemmArgs::gk_mode); the modes above are the digits of a counter.
struct KWalker {
  int d0, d1, d2;           // digits of the K modes 0 .. 2 at the first k of the tile (modes below `mode` stay 0)
  long long oa, ob;         // element offsets of the tile's first k in A and in B, kept up to date by advance()
  // copies of the mode table, held in scalar registers for the whole K loop: read from the kernel arguments inside the
  // loop they would be scalar loads, and the wait for a scalar load also waits for every LDS read in flight.  Only
  // additions are left in the loop: step_a / step_b move the offsets by one tile along `mode`, wrap_a[i] / wrap_b[i]
  // are what a carry out of mode i adds (one stride of mode i + 1 minus the whole extent of mode i).
  int nmodes, mode, step, e0, e1, e2;
  long long step_a, step_b, wa0, wa1, wa2, wb0, wb1, wb2;
  // (the values are the same in every lane; readfirstlane says so to the compiler where it has loaded the kernel
  // arguments with vector instructions)
  __device__ __forceinline__ static void keep(int& x) { x = __builtin_amdgcn_readfirstlane(x); asm volatile("" : "+s"(x)); }
  __device__ __forceinline__ static void keep(long long& x) {
    int lo = __builtin_amdgcn_readfirstlane((int)(unsigned)(unsigned long long)x), hi = __builtin_amdgcn_readfirstlane((int)((unsigned long long)x >> 32));
    asm volatile("" : "+s"(lo), "+s"(hi));
    x = (long long)(((unsigned long long)(unsigned)hi << 32) | (unsigned)lo);
  }
  __device__ __forceinline__ void init(const GettDim& gk, int mode_, int step_) {
    d0 = d1 = d2 = 0;
    oa = ob = 0;
    nmodes = gk.nmodes; mode = mode_; step = step_;
    e0 = gk.extent[0]; e1 = gk.extent[1]; e2 = gk.extent[2];
    step_a = (long long)step_ * gk.stride0[mode_];
    step_b = (long long)step_ * gk.stride1[mode_];
    wa0 = gk.stride0[1] - (long long)e0 * gk.stride0[0]; wb0 = gk.stride1[1] - (long long)e0 * gk.stride1[0];
    wa1 = gk.stride0[2] - (long long)e1 * gk.stride0[1]; wb1 = gk.stride1[2] - (long long)e1 * gk.stride1[1];
    wa2 = gk.stride0[3] - (long long)e2 * gk.stride0[2]; wb2 = gk.stride1[3] - (long long)e2 * gk.stride1[2];
    keep(nmodes); keep(mode); keep(step); keep(e0); keep(e1); keep(e2);
    keep(step_a); keep(step_b); keep(wa0); keep(wa1); keep(wa2); keep(wb0); keep(wb1); keep(wb2);
  }
  __device__ __forceinline__ void advance() {
    // the digit of `mode` moves on by step; a digit that reaches its extent goes back to 0 and carries (the digit
    // of the last mode never wraps inside K and is not kept)
    if (mode == 0) d0 += step; else if (mode == 1) d1 += step; else if (mode == 2) d2 += step;
    oa += step_a; ob += step_b;
    if (nmodes > 1 && d0 >= e0) { d0 = 0; ++d1; oa += wa0; ob += wb0; }
    if (nmodes > 2 && d1 >= e1) { d1 = 0; ++d2; oa += wa1; ob += wb1; }
    if (nmodes > 3 && d2 >= e2) { d2 = 0; oa += wa2; ob += wb2; }
  }
  // element offsets of the tile's first k in A and in B
  __device__ __forceinline__ long long offset_a() const { return oa; }
  __device__ __forceinline__ long long offset_b() const { return ob; }
};
// element offset of k-value k (< BLOCK_K) of a tile from the tile's first k: digits of the modes the tile covers whole,
// the rest along mode `mode`
__device__ __forceinline__ long long gett_k_local(const GettDim& gk, int mode, int k, const long long* stride) {
  long long o = 0;
  for (int i = 0; i < mode; ++i) {
    const int q = gett_div(k, gk.magic[i], gk.shift[i]);
    o += (long long)(k - q * gk.extent[i]) * stride[i];
    k = q;
  }
  return o + (long long)k * stride[mode];
}
// (the same modulo 2^32 and written out over all modes like gett_offsets32_flat: a mode below `mode` gives a digit, mode
// `mode` takes what is left of k, the modes above it nothing)
__device__ __forceinline__ unsigned gett_k_local_flat(const GettDim& gk, int mode, int k, const long long* stride) {
  unsigned o = 0;
#pragma unroll
  for (int i = 0; i < kMaxModes; ++i) {
    const bool whole = i < mode;
    const unsigned magic = whole ? gk.magic[i] : 0u;
    const int q = magic == 0 ? k : (int)((unsigned)(((unsigned long long)(unsigned)k * magic) >> 32) >> gk.shift[i]);
    const int digit = k - q * (whole ? gk.extent[i] : 0);          // (mode `mode`: q = k, the digit is k itself)
    k = whole ? q : 0;
    o += (unsigned)digit * (unsigned)(unsigned long long)stride[i];
  }
  return o;
}

// Makes every later use of x depend on the point where pin() stands (no instruction is emitted).
__device__ __forceinline__ void pin(int4v& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void pin(int2v& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void pin(int& x) { asm volatile("" : "+v"(x)); }

template <int N>
__device__ __forceinline__ void wait_lgkmcnt() {
  asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N < 15 ? N : 15) : "memory");
}

// Fragment of MI MFMA rows x 512/MI k-values: lane l receives the 8 k-values 8*(l/MI)..+7 of row
// row0 + l%MI, which is the operand layout of v_mfma_f32_16x16x32 (MI = 16) and of
// v_mfma_f32_32x32x16 (MI = 32).
//
// The reads are issued from inline assembly: the compiler would otherwise make every
// transposing LDS read wait for all outstanding global->LDS DMA (it cannot tell the stages
// apart), which serialises the pipeline.  Their completion is therefore tracked by hand:
// read() only issues, the registers it names (Raw) must not be looked at before
// wait_lgkmcnt<N>() + pin_raw(), and finish() turns them into the MFMA operand afterwards.
template <int R, int BK, int KIND, int F, int MI = 32>
struct FragReader {
  typedef OperandGeom<R, BK, KIND> G;
  // MI = 32: fragments of 32 rows x 16 k (v_mfma_f32_32x32x16); MI = 16: 16 rows x 32 k (v_mfma_f32_16x16x32),
  // lane l holds the 8 k-values 8*(l/MI)..+7 of row l%MI in both cases
  static constexpr int KSTEP_K = MI == 32 ? 16 : 32;
  static constexpr int KSTEPS = BK / KSTEP_K;
  // M-major, 16-row fragments: fragments 2j and 2j+1 are the two 32-byte halves of one 64-byte group, so one
  // address serves both (the odd one is the even one with bit 5 flipped)
  static constexpr bool PAIRED = KIND == OPK_MMAJOR && MI == 16 && F % 2 == 0;
  static constexpr int NBASE = KIND == OPK_KMAJOR ? KSTEPS : (opk_complex_k(KIND) ? 2 * KSTEPS : (PAIRED ? F / 2 : F));
  static constexpr int OPS = KIND == OPK_KMAJOR ? 1 : 2;   // LDS instructions per fragment that is read
  static constexpr int NREAD = KIND == OPK_KSPLIT ? F / 2 : F;   // fragments that are read (OPK_KSPLIT: each read serves two)
  static constexpr int FRAG_ROWS = MI;       // tile rows (complex rows for OPK_KSPLIT) per fragment
  struct Raw {
    int4v q;          // OPK_KMAJOR; OPK_KSPLIT: complex k 0..3 of the lane's eight
    int4v q1;         // OPK_KSPLIT: complex k 4..7
    int2v lo, hi;     // OPK_MMAJOR
  };
  unsigned cur[NBASE];                          // lane-dependent byte addresses inside the tile of the current stage
  unsigned stage_addr;                          // LDS address of that tile (wave-uniform)

  // row0: first MFMA row of the wave inside the block tile (multiple of 32)
  __device__ __forceinline__ void init(int row0, int lane) {
    if (KIND == OPK_KMAJOR) {
      const int row = row0 + (lane % MI);
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        const int c = ks * (KSTEP_K / 8) + (lane / MI);
        cur[ks < NBASE ? ks : 0] = 16u * (unsigned)(row * G::CPR + (c ^ G::swz_k(row)));
      }
    } else if (opk_complex_k(KIND)) {
      // the wave's rows are complex rows row0 / 2 ..., 16 per fragment, for both parts.  The lane's eight k-slots of a
      // k-step are the complex k 8*(lane/MI) .. +7 of its row: chunks 2*(lane/MI) and the next one, each with an
      // address of its own (the swizzle may have traded their places)
      const int row = (row0 >> 1) + (lane % MI);
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        const int c = ks * (KSTEP_K / 4) + 2 * (lane / MI);
        cur[2 * ks] = 16u * (unsigned)(row * G::CPR + (c ^ G::swz_kp(row)));
        cur[2 * ks + 1] = 16u * (unsigned)(row * G::CPR + ((c + 1) ^ G::swz_kp(row)));
      }
    } else {
      const int i = lane & 15;
      const int k = 8 * (lane / MI) + (i >> 2);
      const int m = (MI == 32 ? (lane & 16) : 0) + 4 * (i & 3);          // offset inside the fragment
#pragma unroll
      for (int fi = 0; fi < F; fi += (PAIRED ? 2 : 1)) {
        const int rowf = row0 + fi * MI;                 // first row of the fragment inside the block tile
        const int mm = (rowf & 31) + m;                  // offset inside the 32-row (64-byte) group
        const int g = (rowf >> 5) ^ G::swz_m(k);
        const int c = ((mm >> 3) & 3) ^ (((k >> 3) & 1) << 1);
        cur[(PAIRED ? fi / 2 : fi) < NBASE ? (PAIRED ? fi / 2 : fi) : 0] = (unsigned)(k * G::ROW_BYTES + g * 64 + c * 16 + (mm & 4) * 2);
      }
    }
    stage_addr = 0;
  }
  __device__ __forceinline__ void set_stage(unsigned tile_lds_addr) {
    const unsigned delta = tile_lds_addr - stage_addr;     // one register per address: the offsets move with the stage
#pragma unroll
    for (int i = 0; i < NBASE; ++i) cur[i] += delta;
    stage_addr = tile_lds_addr;
  }
  // SYNC: the wait for the data is part of the same assembly statement, so that the registers are
  // valid wherever the compiler may look at them (kernels that spill registers use this form: a
  // spill store between an asynchronous read and its wait would save stale values)
  template <int FI, int KS, bool SYNC = false>
  __device__ __forceinline__ void read(Raw& r) const {
    if constexpr (SYNC && KIND == OPK_KMAJOR) {
      asm volatile("ds_read_b128 %0, %1 offset:%2\n\ts_waitcnt lgkmcnt(0)" : "=&v"(r.q) : "v"(cur[KS < NBASE ? KS : 0]), "n"(FI * FRAG_ROWS * G::ROW_BYTES) : "memory");
      return;
    } else if constexpr (SYNC && opk_complex_k(KIND)) {
      asm volatile("ds_read_b128 %0, %2 offset:%4\n\tds_read_b128 %1, %3 offset:%4\n\ts_waitcnt lgkmcnt(0)"
                   : "=&v"(r.q), "=&v"(r.q1)
                   : "v"(cur[2 * KS]), "v"(cur[2 * KS + 1]), "n"(FI * FRAG_ROWS * G::ROW_BYTES) : "memory");
      return;
    } else if constexpr (SYNC && KIND == OPK_MMAJOR) {
      asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4\n\ts_waitcnt lgkmcnt(0)"
                   : "=&v"(r.lo), "=&v"(r.hi)
                   : "v"(mmajor_addr<FI>()), "n"((KS * KSTEP_K) * G::ROW_BYTES), "n"((KS * KSTEP_K + 4) * G::ROW_BYTES) : "memory");
      return;
    }
    if (KIND == OPK_KMAJOR) {
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r.q) : "v"(cur[KS < NBASE ? KS : 0]), "n"(FI * FRAG_ROWS * G::ROW_BYTES) : "memory");
    } else if (opk_complex_k(KIND)) {
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r.q) : "v"(cur[2 * KS]), "n"(FI * FRAG_ROWS * G::ROW_BYTES) : "memory");
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r.q1) : "v"(cur[2 * KS + 1]), "n"(FI * FRAG_ROWS * G::ROW_BYTES) : "memory");
    } else {
      asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r.lo) : "v"(mmajor_addr<FI>()), "n"((KS * KSTEP_K) * G::ROW_BYTES) : "memory");
      asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r.hi) : "v"(mmajor_addr<FI>()), "n"((KS * KSTEP_K + 4) * G::ROW_BYTES) : "memory");
    }
  }
  // one LDS instruction of read<FI, KS>: H < OPS
  template <int FI, int KS, int H>
  __device__ __forceinline__ void read_op(Raw& r) const {
    if constexpr (opk_complex_k(KIND)) {
      if constexpr (H == 0) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r.q) : "v"(cur[2 * KS]), "n"(FI * FRAG_ROWS * G::ROW_BYTES) : "memory");
      else asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r.q1) : "v"(cur[2 * KS + 1]), "n"(FI * FRAG_ROWS * G::ROW_BYTES) : "memory");
    } else if constexpr (KIND == OPK_KMAJOR) {
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r.q) : "v"(cur[KS < NBASE ? KS : 0]), "n"(FI * FRAG_ROWS * G::ROW_BYTES) : "memory");
    } else if constexpr (H == 0) {
      asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r.lo) : "v"(mmajor_addr<FI>()), "n"((KS * KSTEP_K) * G::ROW_BYTES) : "memory");
    } else {
      asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r.hi) : "v"(mmajor_addr<FI>()), "n"((KS * KSTEP_K + 4) * G::ROW_BYTES) : "memory");
    }
  }
  template <int FI>
  __device__ __forceinline__ unsigned mmajor_addr() const {
    if constexpr (PAIRED) return (FI & 1) ? (cur[FI / 2] ^ 32u) : cur[FI / 2];
    else return cur[FI < NBASE ? FI : 0];
  }
  __device__ static __forceinline__ void pin_raw(Raw& r) {
    if (KIND == OPK_KMAJOR) pin(r.q);
    else if (opk_complex_k(KIND)) { pin(r.q); pin(r.q1); }
    else { pin(r.lo); pin(r.hi); }
  }
  // imag: OPK_KSPLIT, the fragment of imaginary parts is asked for
  __device__ static __forceinline__ int4v finish(const Raw& r, [[maybe_unused]] int lane, [[maybe_unused]] bool imag = false) {
    if (KIND == OPK_KMAJOR) return r.q;
    int4v v;
    if (opk_complex_k(KIND)) {
      // one part of the lane's eight complex k: the low (real) or the high (imaginary) halves of the eight words
      const unsigned sel = imag ? 0x07060302u : 0x05040100u;
      v[0] = (int)__builtin_amdgcn_perm((unsigned)r.q[1], (unsigned)r.q[0], sel);
      v[1] = (int)__builtin_amdgcn_perm((unsigned)r.q[3], (unsigned)r.q[2], sel);
      v[2] = (int)__builtin_amdgcn_perm((unsigned)r.q1[1], (unsigned)r.q1[0], sel);
      v[3] = (int)__builtin_amdgcn_perm((unsigned)r.q1[3], (unsigned)r.q1[2], sel);
      return v;
    }
    v[0] = r.lo[0]; v[1] = r.lo[1]; v[2] = r.hi[0]; v[3] = r.hi[1];
    return v;
  }
  // puts a (transformed) operand back into the registers of its fragment
  __device__ static __forceinline__ void store(Raw& r, int4v v) {
    if (KIND == OPK_KMAJOR) r.q = v;
    else { r.lo[0] = v[0]; r.lo[1] = v[1]; r.hi[0] = v[2]; r.hi[1] = v[3]; }
  }
  static_assert(KIND != OPK_MMAJOR || (KSTEPS * KSTEP_K + 4) * G::ROW_BYTES < 65536, "LDS immediate offset is 16 bits");
  static_assert((KIND != OPK_KMAJOR && !opk_complex_k(KIND)) || NREAD * FRAG_ROWS * G::ROW_BYTES <= 65536, "LDS immediate offset is 16 bits");
  static_assert(!opk_complex_k(KIND) || (MI == 16 && G::RP256 * G::CPR == 16), "complex fragments: 16-row blocks; the swizzle has a period of 16 rows, so every fragment of a wave shares the addresses of the first");
  static_assert(KIND != OPK_KSPLIT || F % 2 == 0, "the fragments of real and of imaginary parts come in pairs");
  static_assert(MI == 32 || MI == 16, "fragments of 32 or 16 rows");
};

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

template <int KS, bool SYNC = false, class RA, class RB, int FM, int FN>
__device__ __forceinline__ void load_frags(const RA& ra, const RB& rb, typename RA::Raw (&fa)[FM], typename RB::Raw (&fb)[FN]) {
  static_for<0, RA::NREAD>([&](auto fi) { ra.template read<decltype(fi)::value, KS, SYNC>(fa[decltype(fi)::value]); });
  static_for<0, RB::NREAD>([&](auto fj) { rb.template read<decltype(fj)::value, KS, SYNC>(fb[decltype(fj)::value]); });
}

template <typename T, int MI = 32> struct Mfma;
template <> struct Mfma<_Float16, 32> {
  typedef float16v Acc;
  __device__ static __forceinline__ float16v run(int4v a, int4v b, float16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), c, 0, 0, 0);
  }
};
template <> struct Mfma<__bf16, 32> {
  typedef float16v Acc;
  __device__ static __forceinline__ float16v run(int4v a, int4v b, float16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
// 16x16x32: the same flop per operand byte; on U[-1,1) data the matrix cores hold a 14 % higher clock
// with it under the power limit (register-only loop: 1.98 against 1.74 PFLOP/s)
template <> struct Mfma<_Float16, 16> {
  typedef float4v Acc;
  __device__ static __forceinline__ float4v run(int4v a, int4v b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), c, 0, 0, 0);
  }
  // ... on the accumulator block in the accumulation registers a[R : R + 3], named in the instruction text: kernels that
  // manage the accumulation registers themselves (see CPATH 4 of mfma_gemm_kernel).  FIRST: the block starts from zero.
  template <int R, bool FIRST>
  __device__ static __forceinline__ void run_fixed(int4v a, int4v b) {
    if constexpr (FIRST) asm volatile("v_mfma_f32_16x16x32_f16 a[%2:%3], %0, %1, 0" :: "v"(a), "v"(b), "n"(R), "n"(R + 3));
    else asm volatile("v_mfma_f32_16x16x32_f16 a[%2:%3], %0, %1, a[%2:%3]" :: "v"(a), "v"(b), "n"(R), "n"(R + 3));
  }
};
template <> struct Mfma<__bf16, 16> {
  typedef float4v Acc;
  __device__ static __forceinline__ float4v run(int4v a, int4v b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  template <int R, bool FIRST>
  __device__ static __forceinline__ void run_fixed(int4v a, int4v b) {
    if constexpr (FIRST) asm volatile("v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, 0" :: "v"(a), "v"(b), "n"(R), "n"(R + 3));
    else asm volatile("v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, a[%2:%3]" :: "v"(a), "v"(b), "n"(R), "n"(R + 3));
  }
};

// fp32 op list on the 8 packed 16-bit values of a fragment, rounded back to T.  gl2sh then
// sh2rf: the value is rounded to T after each hook like the LDS copy and the fragment of the
// reference (src/kernel.jl:224-236, 311-319).
template <typename T, int H0, int H1>
__device__ __forceinline__ int4v transform_fragment(int4v f, const GemmArgs& args) {
  typedef T vec8 __attribute__((ext_vector_type(8)));
  vec8 v = __builtin_bit_cast(vec8, f);
  float x[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = (float)v[e];
  if (hook_present<H0>(args)) {
    hook_regs<H0, 8>(args, x);
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = (float)(T)x[e];
  }
  if (hook_present<H1>(args)) hook_regs<H1, 8>(args, x);
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = (T)x[e];
  return __builtin_bit_cast(int4v, v);
}

// One multiplication by a constant that is exact in FP16: the FP16 product rounded to nearest even
// is the fp32 product (exact, 22 significant bits) rounded to FP16, so the packed FP16 multiply
// gives the same bits as the generic path at a quarter of the instructions.
__device__ __forceinline__ int4v scale_fragment_f16(int4v f, float scale) {
  half8 v = __builtin_bit_cast(half8, f);
  const _Float16 s = (_Float16)scale;
  v = v * s;
  return __builtin_bit_cast(int4v, v);
}

#ifndef GK_FORCE_SYNC_FRAGS
#define GK_FORCE_SYNC_FRAGS 0     // set by the run-time compiler for a tile that turned out to spill registers
#endif

template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, int STAGES_, int A_KIND_, int B_KIND_, typename T_, int FUSE_,
          bool GETT_ = false, int FIX_ = FIX_NONE, bool SPLITK_ = false, int MI_ = 32>
struct MfmaGemmConfig {
  static constexpr int MI = MI_;                         // rows of an MFMA block: 32 (32x32x16) or 16 (16x16x32)
  static constexpr int KSTEP_K = MI_ == 32 ? 16 : 32;    // k-values per MFMA
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, STAGES = STAGES_;
  static constexpr int A_KIND = A_KIND_, B_KIND = B_KIND_, FIX = FIX_;
  // 0: no transform and no bias; 1: C / D hooks, bias and at most one exact 16-bit scale on A and on B
  // (a packed multiply per fragment); 2: arbitrary op lists on A and B as well (evaluated in fp32 per
  // element inside the K loop: complete, and markedly slower); 3: C / D hooks and bias only, the K loop of
  // level 0 (also what a power-of-two scale of A or B runs on: the host folds it into the accumulators);
  // 4 (one-wave-per-SIMD instances only): level 3 narrowed to what the host can name in closed form -- no hook on C, at
  // most one op in each hook of D, a bias, a folded scale when there is no C -- which needs no op list walked on the device
  static constexpr int FUSE = FUSE_;
  static constexpr bool FUSED = FUSE_ != 0;
  static constexpr bool FUSED_AB_GENERIC = FUSE_ == 2;
  // the generic A / B hooks, and wave tiles of more than eight 32x32 blocks (256 accumulator registers),
  // need so many registers that the kernel spills: their fragment reads wait for their data inside the
  // assembly statement that issues them (see FragReader::read)
  // One wave per SIMD: four waves with wave tiles of 64 16x16 blocks (all 256 accumulation registers), two LDS stages.
  // The K loop of these instances is written out instruction slot by instruction slot (see the SOLO loop).
  // (64 accumulator blocks: all 256 accumulation registers; 48 for the tiles with a side of 192)
  static constexpr int SOLO_BLOCKS = (BM_ / WAVES_M_ / 16) * (BN_ / WAVES_N_ / 16);
  static constexpr bool SOLO = MI_ == 16 && WAVES_M_ * WAVES_N_ == 4 && (SOLO_BLOCKS == 64 || (SOLO_BLOCKS == 48 && FIX_ == FIX_NONE && !GETT_)) && STAGES_ == 2 &&
                               (BK_ / 32) % 2 == 0 && !SPLITK_ && (GK_FORCE_SYNC_FRAGS == 0) &&
                               ((FIX_ == FIX_NONE && (FUSE_ == 0 || FUSE_ == 4) && A_KIND_ != OPK_KSPLIT && B_KIND_ != OPK_KSPLIT) ||
                                // ... and the complex / dual real-view product of an 'N','N' launch (A contiguous along m, B along k)
                                ((FIX_ == FIX_PAIR || FIX_ == FIX_PAIR_DUAL) && FUSE_ == 0 && !GETT_ && A_KIND_ == OPK_MMAJOR && B_KIND_ == OPK_KSPLIT) ||
                                // ... and the complex product on planar matrices, whose planes are plain real operands
                                (FIX_ == FIX_PLANAR && FUSE_ == 0 && !GETT_ && A_KIND_ != OPK_KSPLIT && B_KIND_ != OPK_KSPLIT));
  // plain real products may have a last tile row / column that sticks out over M / N and a last, partial K
  // tile (the host asks for it only with 16-byte aligned columns, M or N a multiple of 8 where that index is
  // the contiguous one of A or B, and K a multiple of 8): loads are clamped, the C load and the D store
  // masked, the part of the last K tile beyond K zeroed in LDS
  // (the K-split instances take tiles over M and N, not a partial K tile)
  static constexpr bool RAGGED_OK = !GETT_ && FIX_ == FIX_NONE && !SOLO;
  static constexpr bool RAGGED_K_OK = RAGGED_OK && !SPLITK_;
  static constexpr bool SYNC_FRAGS = FUSE_ == 2 || (!SOLO && (BM_ / WAVES_M_ / 32) * (BN_ / WAVES_N_ / 32) > 8) || (GK_FORCE_SYNC_FRAGS != 0);
  static constexpr bool PLANAR = (FIX_ == FIX_PLANAR);
  static constexpr bool PAIR = (FIX_ == FIX_PAIR || FIX_ == FIX_PAIR_DUAL);     // complex / dual product as one real product (see FIX_PAIR)
  static constexpr bool COMPLEX = FIX_ != FIX_NONE;                             // C / D hold complex numbers
  // where the two parts of a complex column of B meet in the accumulators: in neighbouring values of a lane
  // (COLS_LANE: B seen as a real matrix with twice the columns) or in the column blocks fj and fj + FN / 2
  // (COLS_FRAG: planar B, or interleaved B contiguous along k read as OPK_KSPLIT)
  static constexpr bool COLS_FRAG = PLANAR || (PAIR && B_KIND_ == OPK_KSPLIT);
  static constexpr bool COLS_LANE = PAIR && !COLS_FRAG;
  // ... and the two parts of a complex row of A: in neighbouring lanes (ROWS_LANE: A seen as a real matrix with twice
  // the rows) or in the row blocks fi and fi + FM / 2 (ROWS_FRAG: planar A, or interleaved A contiguous along k)
  static constexpr bool ROWS_FRAG = PLANAR || (PAIR && A_KIND_ == OPK_KSPLIT);
  static constexpr bool ROWS_LANE = PAIR && !ROWS_FRAG;
  static constexpr bool GETT = GETT_;   // operands addressed through tensor-contraction index maps
  // K-split instances: a workgroup handles one slice of K (blockIdx.z); the slices of a tile meet in a
  // workspace and the last to arrive sums them in slice order and stores D (splitk_reduce).  A variant of
  // its own so that the plain kernels carry none of it.
  static constexpr bool SPLITK = SPLITK_;
  // 16-row blocks: a k-step of 32 holds twice the fragments of a 16-wide one, so the A fragments are read
  // and consumed in two halves (rows fi < FM/2, then the rest) with the reads of one half in flight under
  // the MFMAs of the other: 32 registers fewer than two whole buffers, and never more than 12 LDS reads
  // outstanding (the wait counter holds 15)
  static constexpr bool SPLIT_A = MI_ == 16 && ((BM_ / WAVES_M_ / MI_) % 2 == 0);
  static constexpr bool PREFETCH = !SPLIT_A && (STAGES_ >= 3) && ((BK_ / KSTEP_K) % 2 == 0);   // cross-step fragment prefetch
  // The DMA instructions of a tile are issued a few per k-step instead of all at once: a wave whose
  // DMA instruction waits for room in the memory pipeline cannot issue its MFMAs either, and a burst
  // from every wave right after the barrier makes all of them wait together (measured on 4096^3:
  // 3031 -> 2903 shader clocks per 64 of K for 256x256x64, 2985 -> 2767 for 256x256x32 with four stages).
  static constexpr bool SPREAD = true;
  typedef T_ T;
  static constexpr int NWAVES = WAVES_M * WAVES_N;
  static constexpr int THREADS = NWAVES * kWaveSize;
  static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;   // wave tile
  static constexpr int FM = WTM / MI, FN = WTN / MI;             // MI x MI accumulator blocks per wave
  static constexpr int KSTEPS = BK / KSTEP_K;
  typedef OperandGeom<BM, BK, A_KIND> GA;
  typedef OperandGeom<BN, BK, B_KIND> GB;
  static constexpr int STAGE_BYTES = GA::BYTES + GB::BYTES;
  // Contractions on the one-wave-per-SIMD arrangement keep the element offsets of every K tile in A and in B in a table
  // behind the LDS stages (two 64-bit offsets per tile, filled before the loop): walking the K modes tile by tile takes
  // some sixty scalar instructions and a dozen branches, which a lone wave on a SIMD cannot hide.
  static constexpr int KTABLE_BYTES = (SOLO && GETT_) ? 16 * 1024 : 0;     // 1024 K tiles
  static constexpr int KTABLE_TILES = KTABLE_BYTES / 16;
  // ... and, behind it, the walks over the M and N modes for every row and column of the tile, made once per row by one
  // lane each: offsets in A and in B (4 bytes per row), of k inside a tile (4 bytes per k, A and B), and in C / D (8 bytes)
  static constexpr int ROWTAB_BYTES = (SOLO && GETT_) ? (BM_ + BN_ + 2 * BK_) * 4 + (BM_ + BN_) * 8 : 0;
  static constexpr int LDS_BYTES = STAGE_BYTES * STAGES + KTABLE_BYTES + ROWTAB_BYTES;
  static constexpr int DMA_A = (GA::NDMA + NWAVES - 1) / NWAVES;   // per wave, per tile
  static constexpr int DMA_B = (GB::NDMA + NWAVES - 1) / NWAVES;
  static constexpr int DMA_PER_TILE = DMA_A + DMA_B;
  static_assert(GA::NDMA % NWAVES == 0 && GB::NDMA % NWAVES == 0, "every wave issues the same number of DMA instructions");
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tiles are multiples of 32 x 32 (two 16-row blocks share a 64-byte group of an M-major tile)");
  static_assert(BK_ % KSTEP_K == 0, "BLOCK_K is a whole number of MFMA k-steps");
  static_assert(STAGES >= 2, "at least two LDS stages");
  static_assert((STAGES - 2) * DMA_PER_TILE <= 63, "vmcnt is a 6-bit counter");
  static_assert(FM * FN > 0, "empty wave tile");
  static_assert(!GETT || FIX == FIX_NONE, "contractions are real");
  static_assert(!SPLITK || (!GETT && FIX == FIX_NONE), "K-split instances are plain real GEMMs");
  static_assert(!PLANAR || (MI_ == 16 && !opk_complex_k(A_KIND_) && !opk_complex_k(B_KIND_)), "planar complex: 16-row blocks on plain real planes");
  static_assert(!COMPLEX || FUSE_ == 0 || FUSE_ == 3, "complex products take hooks on C and D only");
  static_assert(!PAIR || (MI_ == 16 && A_KIND_ != OPK_KMAJOR && B_KIND_ != OPK_KMAJOR),
                "complex-pair products: 16-row blocks on the real view of the operands");
  static_assert(A_KIND_ != OPK_KSPLIT || SPLIT_A, "the real and the imaginary fragments of A are the two halves in which A is consumed");
  static_assert(PAIR || (!opk_complex_k(A_KIND_) && !opk_complex_k(B_KIND_)), "OPK_KSPLIT belongs to the complex-pair products");
};

// CPATH (Cfg::SOLO only; 0 elsewhere): how C comes in and D goes out.  1: FP32 C and D with 16-byte accesses, straight into
// and out of the accumulation registers; 2: no C, D as in 1; 3: as 1 and 2 for products whose extents are not whole numbers of
// tiles (FP32 C / D at any 4-byte alignment: edge tiles leave out what lies outside D, a partial last K tile runs behind the loop);
// 4: as 1 for products of at least kSoloStreamTiles K tiles, with C on its way while the matrix cores run: the accumulators start
// at zero, the C tile arrives one block column per K tile in registers of its own during the first K tiles and is added to the
// accumulators there (so the sum is (products of the first K tiles) + C + (the rest), where path 1 starts from C);
// 5: as 4 with C spread thinner, kSoloSpreadBlocks blocks per K tile, for products with that many K tiles (solo_spread_tiles):
// the loads of C share the path of the tile DMA, which has little to spare per K tile (4096^3: 105.5 us on path 4, 102.8 on 5);
// 6: as 4 for an FP16 C and an FP16 D (8 bytes per lane and block; C is widened where it is added, D rounded once where it is
// stored; 4096^3: 107.2 us on path 0, 102.5 on 6; spread as on path 5 it took 103.7: the widening costs vector-ALU slots in
// every K tile that adds);
// 0: anything else.  One kernel per path, chosen by the host
// (solo_cd_path): where the paths met in one kernel, the register allocator gave the accumulators different registers
// on each and shuffled 250 of them in front of the K loop.
template <class Cfg, int CPATH = 0>
__global__ void __launch_bounds__(Cfg::THREADS) mfma_gemm_kernel(const GemmArgs args) {
  static_assert(CPATH == 0 || Cfg::SOLO, "the C / D paths belong to the one-wave-per-SIMD instances");
  typedef typename Cfg::T T;
  typedef typename Cfg::GA GA;
  typedef typename Cfg::GB GB;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, STAGES = Cfg::STAGES;
  constexpr int FM = Cfg::FM, FN = Cfg::FN, NWAVES = Cfg::NWAVES;
  constexpr int DMA_A = Cfg::DMA_A, DMA_B = Cfg::DMA_B, DPT = Cfg::DMA_PER_TILE;
  // tiles that stick out over the edges of the operands and a partial last K tile: the instances compiled for them
  // (Cfg::RAGGED_OK) and path 3 of the one-wave-per-SIMD instances
  constexpr bool RAGGED = Cfg::RAGGED_OK || (Cfg::SOLO && CPATH == 3);
  constexpr bool RAGGED_K = Cfg::RAGGED_K_OK || (Cfg::SOLO && CPATH == 3);
  static_assert(CPATH != 3 || (!Cfg::GETT && Cfg::FIX == FIX_NONE && Cfg::FUSE == 0), "path 3 is compiled for plain real products");
  constexpr bool STREAM_C = CPATH >= 4 && CPATH <= 6;
  constexpr bool HALF_CD = CPATH == 6;                      // FP16 C and D on a streamed path (8 bytes per lane and block)
  constexpr int CDB = HALF_CD ? 2 : 4;                      // bytes per element of C and D there
  static_assert(!STREAM_C || (!Cfg::GETT && Cfg::FIX == FIX_NONE && Cfg::FUSE == 0), "paths 4 to 6 are compiled for plain real products");

  extern __shared__ __attribute__((aligned(1024))) char smem[];

  int ti, tj;
  cta_swizzle(args.swz_kind, args.swz_param, (int)blockIdx.x, (int)blockIdx.y, args.nbm, args.nbn, ti, tj);
  if (ti >= args.nbm || tj >= args.nbn) return;   // whole block leaves together

  const int lane = (int)threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int wm = wave % Cfg::WAVES_M, wn = wave / Cfg::WAVES_M;
  const int m0 = ti * BM, n0 = tj * BN;

  // --- global tile origins (bytes) and the per-lane DMA offsets, fixed for the whole K loop ---
  const char* ga;
  const char* gb;
  long long a_step = 0, b_step = 0;
  unsigned offa[DMA_A], offb[DMA_B];
  // Which 1 KiB chunk of a tile DMA instruction i of this wave fetches: chunk wave + i * NWAVES, or (GROUPED, the
  // one-wave-per-SIMD instances) four consecutive chunks per group of four instructions, so that a group shares one LDS
  // base in M0 and its instructions differ in their immediate offset, which the hardware adds to the LDS address and to
  // the global address alike (the K loop then writes M0 four times per tile instead of sixteen).  The lane offsets are
  // lowered by the immediate and raised by kDmaBias, which keeps them non-negative; the tile pointers ga / gb stand
  // kDmaBias bytes in front of the tile.
  constexpr bool GROUPED = Cfg::SOLO;
  constexpr int kDmaBias = GROUPED ? 3072 : 0;
  auto dma_group_chunk = [&](int i, int ndma) __attribute__((always_inline)) {      // first chunk of the group of instruction i
    if constexpr (!GROUPED) return wave + i * NWAVES;
    else { const int g4 = i & ~3, gs = (ndma - g4) < 4 ? (ndma - g4) : 4; return g4 * NWAVES + wave * gs; }
  };
  auto dma_chunk = [&](int i, int ndma) __attribute__((always_inline)) { return dma_group_chunk(i, ndma) + (GROUPED ? (i & 3) : 0); };
  [[maybe_unused]] KWalker walk;
  if constexpr (Cfg::GETT) walk.init(args.gk, args.gk_mode, args.gk_step);
  if constexpr (!Cfg::GETT) {
    // tile origin and K step in 16-bit elements (lda / ldb are in 16-bit elements as well; an
    // interleaved complex matrix counts two per complex number)
    const int m0g = Cfg::PLANAR ? m0 / 2 : m0;   // first row of the tile in the stored matrix
    const int n0g = Cfg::PLANAR ? n0 / 2 : n0;
    const long long a_org = Cfg::A_KIND == OPK_KMAJOR ? (long long)m0g * args.lda
                          : (opk_complex_k(Cfg::A_KIND) ? (long long)(m0 / 2) * args.lda : (long long)m0g);
    const long long b_org = Cfg::B_KIND == OPK_KMAJOR ? (long long)n0g * args.ldb
                          : (opk_complex_k(Cfg::B_KIND) ? (long long)(n0 / 2) * args.ldb : (long long)n0g);
    ga = (const char*)args.a + a_org * 2;
    gb = (const char*)args.b + b_org * 2;
    // planar complex: tile row (column) r belongs to wave row r / WT; the first half of a wave's rows are complex rows
    // of the real plane, the second half the same complex rows of the imaginary plane
    [[maybe_unused]] auto planar_index = [](int r, int wt, bool& imag) {
      const int w = r / wt, in = r % wt;
      imag = in >= wt / 2;
      return w * (wt / 2) + (in % (wt / 2));
    };
    a_step = (Cfg::A_KIND == OPK_KMAJOR ? (long long)BK : (opk_complex_k(Cfg::A_KIND) ? 2ll * BK : (long long)GA::LDS_ROWS * args.lda)) * 2;
    b_step = (Cfg::B_KIND == OPK_KMAJOR ? (long long)BK : (opk_complex_k(Cfg::B_KIND) ? 2ll * BK : (long long)GB::LDS_ROWS * args.ldb)) * 2;
#pragma unroll
    for (int i = 0; i < DMA_A; ++i) {
      int row, col;
      dma_lane_coords<GA, Cfg::A_KIND>(dma_chunk(i, DMA_A), lane, row, col);
      if constexpr (Cfg::PLANAR) {
        int& m = Cfg::A_KIND == OPK_KMAJOR ? row : col;
        bool imag;
        m = planar_index(m, Cfg::WTM, imag);
        offa[i] = (unsigned)(((long long)row * args.lda + col + (imag ? args.plane_a : 0ll)) * 2);
      } else {
        if constexpr (RAGGED) {
          // a tile that sticks out over the last row of A: chunks beyond it re-read the last valid chunk
          // (their products land in rows of the tile that are never stored)
          int& m = Cfg::A_KIND == OPK_KMAJOR ? row : col;
          const int last = Cfg::A_KIND == OPK_KMAJOR ? args.M - m0 - 1 : ((args.M - m0 - 1) >> 3) << 3;   // the row, or the chunk, of the last valid row
          m = m > last ? last : m;
        }
        offa[i] = (unsigned)(((long long)row * args.lda + col) * 2);
      }
    }
#pragma unroll
    for (int i = 0; i < DMA_B; ++i) {
      int row, col;
      dma_lane_coords<GB, Cfg::B_KIND>(dma_chunk(i, DMA_B), lane, row, col);
      if constexpr (RAGGED) {
        int& n = Cfg::B_KIND == OPK_KMAJOR ? row : col;
        const int last = Cfg::B_KIND == OPK_KMAJOR ? args.N - n0 - 1 : ((args.N - n0 - 1) >> 3) << 3;
        n = n > last ? last : n;
      }
      [[maybe_unused]] bool imag = false;
      if constexpr (Cfg::PLANAR) {
        int& n = Cfg::B_KIND == OPK_KMAJOR ? row : col;
        n = planar_index(n, Cfg::WTN, imag);
      }
      offb[i] = (unsigned)(((long long)row * args.ldb + col + ((Cfg::PLANAR && imag) ? args.plane_b : 0ll)) * 2);
    }
  } else {
    // element (m, k) of A lives at offM(m) + offK(k): the row part is a mixed-radix walk over the M
    // modes (done once per lane), the k part inside a tile is linear in the first K mode
    ga = (const char*)args.a;
    gb = (const char*)args.b;
    if constexpr (Cfg::SOLO) {
      // One walk over the M modes per row of the tile and one over the N modes per column, each by one lane of the
      // workgroup, into tables in LDS; the lanes then look up the rows and columns of their DMA chunks (and, before the K
      // loop, of their blocks of C / D).  Every lane walking the tables for its own sixteen chunks and sixteen block
      // origins was thirty-two walks with integer divisions in front of the first DMA and the first MFMA.
      static_assert(BM == Cfg::THREADS && BN == Cfg::THREADS && BK <= Cfg::THREADS, "one row, one column and at most one k per lane");
      unsigned* tab_a = (unsigned*)(smem + Cfg::STAGE_BYTES * STAGES + Cfg::KTABLE_BYTES);
      unsigned* tab_b = tab_a + BM;
      unsigned* tab_ka = tab_b + BN;
      unsigned* tab_kb = tab_ka + BK;
      long long* tab_dm = (long long*)(tab_kb + BK);
      long long* tab_dn = tab_dm + BM;
      const int t = (int)threadIdx.x;
      long long o0, o1;
      gett_offsets32_flat(args.gm, m0 + t, o0, o1);
      tab_a[t] = (unsigned)(unsigned long long)o0;
      tab_dm[t] = o1;
      gett_offsets32_flat(args.gn, n0 + t, o0, o1);
      tab_b[t] = (unsigned)(unsigned long long)o0;
      tab_dn[t] = o1;
      if (t < BK) {
        tab_ka[t] = gett_k_local_flat(args.gk, args.gk_mode, t, args.gk.stride0);
        tab_kb[t] = gett_k_local_flat(args.gk, args.gk_mode, t, args.gk.stride1);
      }
      __syncthreads();
#pragma unroll
      for (int i = 0; i < DMA_A; ++i) {
        int row, col;
        dma_lane_coords<GA, Cfg::A_KIND>(dma_chunk(i, DMA_A), lane, row, col);
        const int r = Cfg::A_KIND == OPK_KMAJOR ? row : col, k = Cfg::A_KIND == OPK_KMAJOR ? col : row;
        offa[i] = (tab_a[r] + tab_ka[k]) * 2u;
      }
#pragma unroll
      for (int i = 0; i < DMA_B; ++i) {
        int row, col;
        dma_lane_coords<GB, Cfg::B_KIND>(dma_chunk(i, DMA_B), lane, row, col);
        const int r = Cfg::B_KIND == OPK_KMAJOR ? row : col, k = Cfg::B_KIND == OPK_KMAJOR ? col : row;
        offb[i] = (tab_b[r] + tab_kb[k]) * 2u;
      }
    } else {
#pragma unroll
    for (int i = 0; i < DMA_A; ++i) {
      int row, col;
      dma_lane_coords<GA, Cfg::A_KIND>(dma_chunk(i, DMA_A), lane, row, col);
      const int r = Cfg::A_KIND == OPK_KMAJOR ? row : col, k = Cfg::A_KIND == OPK_KMAJOR ? col : row;
      long long o0, o1;
      gett_offsets32(args.gm, m0 + r, o0, o1);
      offa[i] = (unsigned)((o0 + gett_k_local(args.gk, args.gk_mode, k, args.gk.stride0)) * 2);
    }
#pragma unroll
    for (int i = 0; i < DMA_B; ++i) {
      int row, col;
      dma_lane_coords<GB, Cfg::B_KIND>(dma_chunk(i, DMA_B), lane, row, col);
      const int r = Cfg::B_KIND == OPK_KMAJOR ? row : col, k = Cfg::B_KIND == OPK_KMAJOR ? col : row;
      long long o0, o1;
      gett_offsets32(args.gn, n0 + r, o0, o1);
      offb[i] = (unsigned)((o0 + gett_k_local(args.gk, args.gk_mode, k, args.gk.stride1)) * 2);
    }
    }
  }

  if constexpr (GROUPED) {
#pragma unroll
    for (int i = 0; i < DMA_A; ++i) offa[i] += (unsigned)(kDmaBias - (i & 3) * 1024);
#pragma unroll
    for (int i = 0; i < DMA_B; ++i) offb[i] += (unsigned)(kDmaBias - (i & 3) * 1024);
    ga -= kDmaBias;
    gb -= kDmaBias;
  }

  auto issue_tile = [&](int stage) {
    char* sa = smem + stage * Cfg::STAGE_BYTES;
    char* sb = sa + GA::BYTES;
    const char* pa = ga;
    const char* pb = gb;
    if constexpr (Cfg::GETT) {
      pa = ga + walk.offset_a() * 2;
      pb = gb + walk.offset_b() * 2;
      walk.advance();
    }
    static_for<0, DMA_A>([&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      __builtin_amdgcn_global_load_lds(GK_GLOBAL_PTR(pa + offa[i]), GK_LDS_PTR(void, sa + dma_group_chunk(i, DMA_A) * 1024), 16, GROUPED ? (i & 3) * 1024 : 0, 0);
    });
    static_for<0, DMA_B>([&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      __builtin_amdgcn_global_load_lds(GK_GLOBAL_PTR(pb + offb[i]), GK_LDS_PTR(void, sb + dma_group_chunk(i, DMA_B) * 1024), 16, GROUPED ? (i & 3) * 1024 : 0, 0);
    });
    if constexpr (!Cfg::GETT) {
      ga += a_step;
      gb += b_step;
    }
  };

  [[maybe_unused]] const char* part_a = nullptr;
  [[maybe_unused]] const char* part_b = nullptr;
  // part P of NP of the same DMA (Cfg::SPREAD); the tile pointers move on with the last part
  auto issue_part = [&](auto p_c, auto np_c, int stage) __attribute__((always_inline)) {
    constexpr int P = decltype(p_c)::value, NP = decltype(np_c)::value;
    char* sa = smem + stage * Cfg::STAGE_BYTES;
    char* sb = sa + GA::BYTES;
    if constexpr (Cfg::GETT && P == 0) {
      // tile base of the tensor walk, the same for every part of this tile
      part_a = ga + walk.offset_a() * 2;
      part_b = gb + walk.offset_b() * 2;
      walk.advance();
    }
    const char* pa = Cfg::GETT ? part_a : ga;
    const char* pb = Cfg::GETT ? part_b : gb;
    // (the offsets pass through an empty assembly statement: their widening to 64 bits then stays next to the DMA
    // instruction, which takes the tile pointer from scalar registers and the 32-bit offset from the lane, instead of
    // being hoisted out of the loop as sixteen register pairs and a 64-bit addition per instruction)
    static_for<0, DMA_A>([&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      if constexpr ((i % NP) == P) {
        asm volatile("" : "+v"(offa[i]));
        __builtin_amdgcn_global_load_lds(GK_GLOBAL_PTR(pa + offa[i]), GK_LDS_PTR(void, sa + dma_group_chunk(i, DMA_A) * 1024), 16, GROUPED ? (i & 3) * 1024 : 0, 0);
      }
    });
    static_for<0, DMA_B>([&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      if constexpr (((DMA_A + i) % NP) == P) {
        asm volatile("" : "+v"(offb[i]));
        __builtin_amdgcn_global_load_lds(GK_GLOBAL_PTR(pb + offb[i]), GK_LDS_PTR(void, sb + dma_group_chunk(i, DMA_B) * 1024), 16, GROUPED ? (i & 3) * 1024 : 0, 0);
      }
    });
    if constexpr (P == NP - 1 && !Cfg::GETT) {
      ga += a_step;
      gb += b_step;
    }
  };

  // K tiles of this workgroup: all of them, or one slice of a K-split launch
  int KT = args.K / BK;
  // The last K tile runs outside the pipeline (after the loop) when it is a partial one, and also when it is whole
  // but a 16-byte chunk of this workgroup's tiles straddles the last row of an operand whose rows are contiguous in
  // memory (M, or N, not a multiple of 8): in the last k such a chunk would read past the end of the operand.
  [[maybe_unused]] int tail_k = 0;
  if constexpr (RAGGED_K) {
    tail_k = args.K - KT * BK;
    const bool straddle = (Cfg::A_KIND == OPK_MMAJOR && (args.M & 7) != 0 && m0 + BM > args.M) ||
                          (Cfg::B_KIND == OPK_MMAJOR && (args.N & 7) != 0 && n0 + BN > args.N);
    if (tail_k == 0 && straddle && KT > 0) { KT -= 1; tail_k = BK; }
  }
  if constexpr (Cfg::SPLITK) {
    const int kt0 = (int)blockIdx.z * args.k_steps;
    KT = (KT - kt0) < args.k_steps ? (KT - kt0) : args.k_steps;
    if (KT <= 0) return;       // the whole workgroup leaves together, before any barrier
    ga += (long long)kt0 * a_step;
    gb += (long long)kt0 * b_step;
  }

  // (SOLO: the loop leaves ga / gb at the last tile it fetched, so the tile behind the loop is kept here)
  [[maybe_unused]] const char* ga_tail = ga + kDmaBias;
  [[maybe_unused]] const char* gb_tail = gb + kDmaBias;
  if constexpr (Cfg::SOLO && RAGGED_K) {
    ga_tail += (long long)KT * a_step;
    gb_tail += (long long)KT * b_step;
  }

  // --- prologue: start the first STAGES-1 tiles on their way ---
#pragma unroll
  for (int s = 0; s < (Cfg::SOLO ? STAGES : STAGES - 1); ++s)
    if (s < KT) issue_tile(s);      // (SOLO: both stages are free and the loop issues tile kt + 2 from tile kt)
  if constexpr (Cfg::SOLO && Cfg::GETT) {
    // where K tile t starts in A and in B: the pointers that the DMA of the tile takes as its scalar base (published by the
    // barrier in front of the K loop)
    long long* table = (long long*)(smem + Cfg::STAGE_BYTES * STAGES);
    for (int t = (int)threadIdx.x; t < KT; t += Cfg::THREADS) {
      long long oa, ob;
      gett_offsets32(args.gk, t * BK, oa, ob);
      table[2 * t] = (long long)(ga + oa * 2);
      table[2 * t + 1] = (long long)(gb + ob * 2);
    }
  }

  // --- accumulators: C tile (two transforms) or zeros -------------------------------------------
  // 32x32 blocks: lane l owns row m = 32*fi + l%32 and columns n = 32*fj + 8*(v/4) + 4*(l/32) + v%4, v < 16;
  // 16x16 blocks: row m = 16*fi + l%16 and columns n = 16*fj + 4*(l/16) + v, v < 4
  constexpr int MI = Cfg::MI;
  constexpr int NV = MI == 32 ? 16 : 4;                       // accumulator values per lane and block
  typedef typename Mfma<T, MI>::Acc AccV;
  auto vcol = [](int v) { return MI == 32 ? 8 * (v / 4) + (v % 4) : v; };   // column of value v inside a block, from the lane's first
  // complex-pair products: a lane's four values of a block are two complex columns x the two parts of B; C is
  // loaded into, and D stored from, the values 0 and 2 (one per complex column), see pair_combine
  constexpr int NVO = Cfg::COLS_LANE ? 2 : NV;                // values per lane and block that C / D see
  constexpr int CB = Cfg::COLS_LANE ? MI / 2 : MI;            // columns of C / D per block
  auto slot = [](int v) { return Cfg::COLS_LANE ? 2 * v : v; };
  // COLS_FRAG: C / D see the left half of the column blocks (the right half holds the products with the imaginary
  // parts of B until they are combined).  Planar complex: row block fi is complex rows of the real plane for
  // fi < FM / 2, of the imaginary plane above
  constexpr int FNO = Cfg::COLS_FRAG ? FN / 2 : FN;
  constexpr int FMH = Cfg::ROWS_FRAG ? FM / 2 : FM;
  AccV acc[FM][FN];
  const int mrow = Cfg::ROWS_FRAG ? (m0 + wm * Cfg::WTM) / 2 + (lane % MI) : m0 + wm * Cfg::WTM + (lane % MI);   // ROWS_FRAG: a complex row
  const int ncol = Cfg::COLS_LANE ? (n0 + wn * Cfg::WTN) / 2 + 2 * (lane / MI)
                 : (Cfg::COLS_FRAG ? (n0 + wn * Cfg::WTN) / 2 + 4 * (lane / MI) : n0 + wn * Cfg::WTN + 4 * (lane / MI));
  // complex C / D: row block fi of this lane holds imaginary parts (interleaved: the odd lanes, whatever fi; planar:
  // the lower half of the row blocks)
  [[maybe_unused]] auto imag_rows = [&](int fi) { return Cfg::ROWS_FRAG ? fi >= FMH : (Cfg::COMPLEX && (lane & 1) != 0); };
  // element offset of the lane's first element of accumulator block (fi, fj) in C / D, and the
  // stride between its consecutive columns.
  // contractions: offset of the lane's row of row block fi (gett_om) and of the first of its four columns of
  // column block fj (gett_on) in C / D; filled before the C load and again before the D store (not kept across
  // the K loop)
  [[maybe_unused]] long long gett_om[Cfg::GETT ? FM : 1], gett_on[Cfg::GETT ? FN : 1];
  [[maybe_unused]] auto gett_origins = [&]() __attribute__((always_inline)) {
    if constexpr (Cfg::GETT) {
      long long t0;
      if (args.gett_fast) {
        // whole 32-wide blocks inside the first M mode and the first N mode: one walk per block origin (the same
        // for every lane of the wave), the lane's own row and first column follow with the strides of those modes
        const long long lane_m = (long long)(lane % MI) * args.gm.stride1[0], lane_n = (long long)(4 * (lane / MI)) * args.gn.stride1[0];
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) {
          if (MI == 16 && (fi & 1)) gett_om[fi] = gett_om[fi - 1] + 16 * args.gm.stride1[0];
          else { gett_offsets32(args.gm, m0 + wm * Cfg::WTM + MI * fi, t0, gett_om[fi]); gett_om[fi] += lane_m; }
        }
#pragma unroll
        for (int fj = 0; fj < FN; ++fj) {
          if (MI == 16 && (fj & 1)) gett_on[fj] = gett_on[fj - 1] + 16 * args.gn.stride1[0];
          else { gett_offsets32(args.gn, n0 + wn * Cfg::WTN + MI * fj, t0, gett_on[fj]); gett_on[fj] += lane_n; }
        }
      } else {
        // any extents: every lane walks the modes for its own row of each block and for the first of its four
        // columns (which lie inside the first N mode: its extent is a multiple of 4)
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) gett_offsets32(args.gm, m0 + wm * Cfg::WTM + MI * fi + (lane % MI), t0, gett_om[fi]);
#pragma unroll
        for (int fj = 0; fj < FN; ++fj) gett_offsets32(args.gn, n0 + wn * Cfg::WTN + MI * fj + 4 * (lane / MI), t0, gett_on[fj]);
      }
    }
  };
  auto cd_offset = [&](int fi, int fj, long long ld, [[maybe_unused]] long long plane) -> long long {
    if constexpr (Cfg::PLANAR) {
      return (long long)(mrow + MI * (fi % FMH)) + (long long)(ncol + MI * fj) * ld + (fi >= FMH ? plane : 0ll);
    } else if constexpr (Cfg::ROWS_FRAG) {
      // interleaved C / D seen as a real matrix: complex row m is its rows 2m (real part) and 2m + 1
      return 2ll * (mrow + MI * (fi % FMH)) + (fi >= FMH ? 1 : 0) + (long long)(ncol + CB * fj) * ld;
    } else if constexpr (!Cfg::GETT) {
      return (long long)(mrow + MI * fi) + (long long)(ncol + CB * fj) * ld;
    } else {
      return gett_om[fi] + gett_on[fj];
    }
  };
  auto cd_nstride = [&](long long ld) -> long long {
    if constexpr (!Cfg::GETT) return ld; else return args.gn.stride1[0];
  };
  // One hook over the accumulators of column block fj (FM blocks): the dispatch on the op is paid once per
  // op and column block, not once per 16x16 block.  (Over all accumulators at once the cases of the
  // dispatch meet in more registers than a lane has.)
  [[maybe_unused]] auto hook_col = [&](auto h_c, int fj) __attribute__((always_inline)) {
    constexpr int H = decltype(h_c)::value;
    auto each = [&](auto f) __attribute__((always_inline)) {
#pragma unroll
      for (int fi = 0; fi < FM; ++fi)
#pragma unroll
        for (int v = 0; v < NVO; ++v) acc[fi][fj][slot(v)] = f(acc[fi][fj][slot(v)]);
    };
#ifdef GK_USER_HOOKS
    if constexpr (UserHooks::present[H]) each([](float x) { return UserHooks::template apply<H>(x); });
#else
    const OpList& t = args.t[H];
    for (int i = 0; i < t.n; ++i) {
      if constexpr (Cfg::COMPLEX) {
        // z + p0 with a real p0 leaves the imaginary part as it is (the host admits the ops that act on the
        // two parts independently, and this one)
        if (t.kind[i] == T_ADD) {
          const float p0 = t.p0[i];
#pragma unroll
          for (int fi = 0; fi < FM; ++fi)
#pragma unroll
            for (int v = 0; v < NVO; ++v) acc[fi][fj][slot(v)] = imag_rows(fi) ? acc[fi][fj][slot(v)] : acc[fi][fj][slot(v)] + p0;
          continue;
        }
      }
      dispatch_op(t.kind[i], t.p0[i], t.p1[i], each);
    }
#endif
  };
  [[maybe_unused]] const bool ragged = Cfg::RAGGED_OK && (m0 + BM > args.M || n0 + BN > args.N);   // wave-uniform
  // K-split launches: the first slice of K starts from C, the others from zero
  const bool load_c = args.c_mode != 0 && (!Cfg::SPLITK || blockIdx.z == 0);
  // SOLO: the A fragment is the first MFMA operand, so a lane owns the rows 4 * (lane / 16) .. + 3 of column lane % 16 of
  // a block: 16 contiguous bytes of a column-major FP32 C / D.  The loads go straight into the accumulation registers.
  // (complex products: rows of the real view -- a lane's four rows are two complex numbers -- and complex columns, of which
  // the block columns fj and fj + FN / 2 hold the products with the real and with the imaginary parts of B)
  constexpr int SFN = Cfg::COLS_FRAG ? FN / 2 : FN;          // block columns that C / D see
  // (planar complex: complex rows, of which the row blocks fi and fi + FM / 2 hold the products of the real and of the
  // imaginary plane of A; C / D keep real parts in one plane and imaginary parts in the other)
  constexpr int SFM = Cfg::PLANAR ? FM / 2 : FM;
  [[maybe_unused]] const int solo_row = (Cfg::PLANAR ? (m0 + wm * Cfg::WTM) / 2 : m0 + wm * Cfg::WTM) + 4 * (lane / MI);
  [[maybe_unused]] const int solo_col = (Cfg::COLS_FRAG ? (n0 + wn * Cfg::WTN) / 2 : n0 + wn * Cfg::WTN) + (lane % MI);
  // Element offset of the lane's first row of block (fi, fj) in C / D.  Contractions: the lane walks the M modes for its
  // first row of every row block (the other three follow in the first M mode, whose stride in C / D is 1 and whose extent
  // is a multiple of 4: the host runs these instances on nothing else) and the N modes for its column of every block column.
  [[maybe_unused]] long long solo_om[Cfg::GETT ? FM : 1], solo_on[Cfg::GETT ? FN : 1];
  [[maybe_unused]] float bcol_early[Cfg::FUSE == 4 ? FN : 1], brow_early[Cfg::FUSE == 4 ? FM * 4 : 1];      // the lane's bias values (see below)
  [[maybe_unused]] auto solo_origins = [&](int row, int col) __attribute__((always_inline)) {
    if constexpr (Cfg::GETT) {
      // (from the tables of the tile's rows and columns, see the DMA offsets)
      const long long* tab_dm = (const long long*)(smem + Cfg::STAGE_BYTES * STAGES + Cfg::KTABLE_BYTES + (BM + BN + 2 * BK) * 4);
      const long long* tab_dn = tab_dm + BM;
#pragma unroll
      for (int fi = 0; fi < FM; ++fi) solo_om[fi] = tab_dm[row - m0 + MI * fi];
#pragma unroll
      for (int fj = 0; fj < FN; ++fj) solo_on[fj] = tab_dn[col - n0 + MI * fj];
    }
  };
  [[maybe_unused]] auto solo_off = [&](int row, int col, int fi, int fj, long long ld, [[maybe_unused]] long long plane) -> long long {
    if constexpr (Cfg::GETT) return solo_om[fi] + solo_on[fj];
    else if constexpr (Cfg::PLANAR) return (long long)(row + MI * (fi % SFM)) + (long long)(col + MI * fj) * ld + (fi >= SFM ? plane : 0ll);
    else return (long long)(row + MI * fi) + (long long)(col + MI * fj) * ld;
  };
  if constexpr (Cfg::SOLO) {
    static_assert(!Cfg::GETT || CPATH != 0, "contractions run the four waves with 16-byte C / D accesses only");
    // (contractions: the walks over the modes -- integer divisions, sixteen per lane -- run here, while the first tiles are
    // on their way, and their results stay in registers over the K loop; behind the loop they stood between the last MFMA
    // and the first store)
    if (Cfg::GETT || (load_c && !STREAM_C)) solo_origins(solo_row, solo_col);
    // (hooks of D in closed form: the lane's bias values -- its column of every block column, or its rows of every row block --
    // are fetched here, behind the DMA of the first tiles, and wait in registers; fetched behind the K loop their latency
    // stood in front of the first store)
    if constexpr (Cfg::FUSE == 4) {
#pragma unroll
      for (int j = 0; j < FN; ++j) bcol_early[j] = args.epi_kind == 1 ? args.bias[solo_col + MI * j] : 0.0f;
#pragma unroll
      for (int fi = 0; fi < FM; ++fi)
#pragma unroll
        for (int v = 0; v < 4; ++v) brow_early[4 * fi + v] = args.epi_kind == 2 ? args.bias[solo_row + MI * fi + v] : 0.0f;
    }
    if constexpr (CPATH == 3) {
      // FP32 C with 16-byte accesses (at any 4-byte alignment), tiles over the edge included: rows and columns outside are
      // read from the last ones inside, and what is accumulated on them is never stored
      if (load_c) {
#pragma unroll
        for (int fj = 0; fj < FN; ++fj)
#pragma unroll
          for (int fi = 0; fi < FM; ++fi) {
            int r = solo_row + MI * fi, cc = solo_col + MI * fj;
            r = r < args.M - 4 ? r : args.M - 4;
            cc = cc < args.N - 1 ? cc : args.N - 1;
            const float* cp = (const float*)args.c + ((long long)r + (long long)cc * args.ldc);
            asm volatile("global_load_dwordx4 %0, %1, off" : "=a"(acc[fi][fj]) : "v"(cp) : "memory");
          }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const int m4 = args.M & 3;
        if (m4 != 0) {
          // M not in fours: the lane whose four rows reach over the last row was loaded 4 - m4 rows early (the clamp
          // above); its rows inside C are the last m4 values of what arrived
#pragma unroll
          for (int fj = 0; fj < FN; ++fj)
#pragma unroll
            for (int fi = 0; fi < FM; ++fi) {
              const int r = solo_row + MI * fi;
              asm volatile("" : "+a"(acc[fi][fj]));         // (one block at a time)
              if (r < args.M && r + 4 > args.M) {
                const AccV t = acc[fi][fj];
                AccV o = t;
                o[0] = m4 == 3 ? t[1] : (m4 == 2 ? t[2] : t[3]);
                o[1] = m4 == 3 ? t[2] : t[3];
                o[2] = t[3];
                acc[fi][fj] = o;
              }
              asm volatile("" : "+a"(acc[fi][fj]));
            }
        }
      } else {
#pragma unroll
        for (int fi = 0; fi < FM; ++fi)
#pragma unroll
          for (int fj = 0; fj < FN; ++fj) acc[fi][fj] = AccV{};
      }
#pragma unroll
      for (int fj = 0; fj < FN; ++fj)
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) asm volatile("" : "+a"(acc[fi][fj]));
    } else if constexpr (STREAM_C) {
      // (the accumulators start from zero in the first k-step and C comes in during the first K tiles, see the K loop)
    } else if constexpr (CPATH == 2) {
      // (no C: zeroed in place, in the accumulation registers)
#pragma unroll
      for (int fi = 0; fi < FM; ++fi)
#pragma unroll
        for (int fj = 0; fj < FN; ++fj) {
          acc[fi][fj] = AccV{};
          asm volatile("" : "+a"(acc[fi][fj]));
        }
    } else if constexpr (CPATH == 1) {
#pragma unroll
      for (int fj = 0; fj < SFN; ++fj)
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) {
          const float* cp = (const float*)args.c + solo_off(solo_row, solo_col, fi, fj, args.ldc, args.plane_c);
          asm volatile("global_load_dwordx4 %0, %1, off" : "=a"(acc[fi][fj]) : "v"(cp) : "memory");
        }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
      for (int fj = 0; fj < SFN; ++fj)
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) asm volatile("" : "+a"(acc[fi][fj]));
    } else if (load_c && args.c_dtype == DT_F32 && ((((uintptr_t)args.c) | ((uintptr_t)args.ldc << 2)) & 15u) == 0) {
      // (FP32 C next to a D that is not: 16-byte loads through ordinary registers)
#pragma unroll
      for (int fj = 0; fj < SFN; ++fj)
#pragma unroll
        for (int fi = 0; fi < FM; ++fi)
          acc[fi][fj] = *(const float4v*)((const float*)args.c + solo_off(solo_row, solo_col, fi, fj, args.ldc, args.plane_c));
    } else if (load_c && args.c_dtype != DT_F32 && ((((uintptr_t)args.c) | ((uintptr_t)args.ldc << 1)) & 7u) == 0) {
      // 16-bit C: the lane's four rows are 8 contiguous bytes
#pragma unroll
      for (int fj = 0; fj < SFN; ++fj)
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) {
          const long long off = solo_off(solo_row, solo_col, fi, fj, args.ldc, args.plane_c);
          const int2v raw = *(const int2v*)((const char*)args.c + off * 2);
          if (args.c_dtype == DT_F16) {
            typedef _Float16 half4 __attribute__((ext_vector_type(4)));
            const half4 h = __builtin_bit_cast(half4, raw);
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[fi][fj][v] = (float)h[v];
          } else {
            acc[fi][fj][0] = __builtin_bit_cast(float, raw[0] << 16);
            acc[fi][fj][1] = __builtin_bit_cast(float, (int)((unsigned)raw[0] & 0xFFFF0000u));
            acc[fi][fj][2] = __builtin_bit_cast(float, raw[1] << 16);
            acc[fi][fj][3] = __builtin_bit_cast(float, (int)((unsigned)raw[1] & 0xFFFF0000u));
          }
        }
    } else if (load_c) {
#pragma unroll
      for (int fj = 0; fj < SFN; ++fj)
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) {
          const long long off = solo_off(solo_row, solo_col, fi, fj, args.ldc, args.plane_c);
#pragma unroll
          for (int v = 0; v < 4; ++v) acc[fi][fj][v] = load_cd(args.c, args.c_dtype, off + v);
        }
    } else {
#pragma unroll
      for (int fi = 0; fi < FM; ++fi)
#pragma unroll
        for (int fj = 0; fj < FN; ++fj) {
          acc[fi][fj] = AccV{};
          asm volatile("" : "+a"(acc[fi][fj]));     // (zeroed in place, in the accumulation registers)
        }
    }
    if constexpr (Cfg::COLS_FRAG) {
      // the products with the imaginary parts of B start from zero (C came in through the block columns of the real parts)
      if (load_c) {
#pragma unroll
        for (int fi = 0; fi < FM; ++fi)
#pragma unroll
          for (int fj = SFN; fj < FN; ++fj) {
            acc[fi][fj] = AccV{};
            asm volatile("" : "+a"(acc[fi][fj]));
          }
      }
    }
  } else
  if (Cfg::RAGGED_OK && ragged && load_c) {
    // tile over the edge: element by element, out-of-range elements start from zero
#pragma unroll
    for (int fj = 0; fj < FN; ++fj)
#pragma unroll
      for (int fi = 0; fi < FM; ++fi)
#pragma unroll
        for (int v = 0; v < NV; ++v) {
          const int r = mrow + MI * fi, cc = ncol + MI * fj + vcol(v);
          acc[fi][fj][v] = (r < args.M && cc < args.N) ? load_cd(args.c, args.c_dtype, r + (long long)cc * args.ldc) : 0.0f;
        }
    if (Cfg::FUSED) {
#pragma unroll
      for (int fj = 0; fj < FN; ++fj) {
        hook_col(std::integral_constant<int, H_GL2SH_C>{}, fj);
        hook_col(std::integral_constant<int, H_SH2RF_C>{}, fj);
      }
    }
  } else if (load_c) {
    gett_origins();
    // column blocks outermost: with 16-row blocks the two halves of a 128-byte line of C / D belong to
    // neighbouring row blocks, which are then read (and, below, written) right after each other
    if constexpr (Cfg::COLS_FRAG) {
#pragma unroll
      for (int fj = FNO; fj < FN; ++fj)
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) acc[fi][fj] = AccV{};     // the products with the imaginary parts of B start from zero
    }
#pragma unroll
    for (int fj = 0; fj < FNO; ++fj)
#pragma unroll
      for (int fi = 0; fi < FM; ++fi) {
        const long long off = cd_offset(fi, fj, args.ldc, args.plane_c);
        const long long ns = cd_nstride(args.ldc);
        if constexpr (Cfg::COLS_LANE) acc[fi][fj] = AccV{};      // the values between the complex columns start from zero
        if (args.c_dtype == DT_F32) {
          const float* cp = (const float*)args.c + off;
#pragma unroll
          for (int v = 0; v < NVO; ++v) acc[fi][fj][slot(v)] = cp[(long long)vcol(v) * ns];
        } else if (args.c_dtype == DT_F16) {
          const _Float16* cp = (const _Float16*)args.c + off;
#pragma unroll
          for (int v = 0; v < NVO; ++v) acc[fi][fj][slot(v)] = (float)cp[(long long)vcol(v) * ns];
        } else {
          const __bf16* cp = (const __bf16*)args.c + off;
#pragma unroll
          for (int v = 0; v < NVO; ++v) acc[fi][fj][slot(v)] = (float)cp[(long long)vcol(v) * ns];
        }
      }
    if (Cfg::FUSED) {
#pragma unroll
      for (int fj = 0; fj < FNO; ++fj) {
        hook_col(std::integral_constant<int, H_GL2SH_C>{}, fj);
        hook_col(std::integral_constant<int, H_SH2RF_C>{}, fj);
      }
    }
  } else {
#pragma unroll
    for (int fi = 0; fi < FM; ++fi)
#pragma unroll
      for (int fj = 0; fj < FN; ++fj)
#pragma unroll
        for (int v = 0; v < NV; ++v) acc[fi][fj][v] = 0.0f;
  }

  // a power-of-two scale of A or B that the host has folded into the accumulators (see GemmArgs)
  [[maybe_unused]] auto scale_acc = [&](float f) __attribute__((always_inline)) {
#pragma unroll
    for (int fi = 0; fi < FM; ++fi)
#pragma unroll
      for (int fj = 0; fj < FN; ++fj)
#pragma unroll
        for (int v = 0; v < NV; ++v) acc[fi][fj][v] = acc[fi][fj][v] * f;
  };
  if constexpr (Cfg::FUSED && !Cfg::SOLO) {
    if (load_c && args.acc_pre_scale != 1.0f) scale_acc(args.acc_pre_scale);
  }

  const bool xf_a = Cfg::FUSED && Cfg::FUSE != 3 && (hook_present<H_GL2SH_A>(args) || hook_present<H_SH2RF_A>(args));
  const bool xf_b = Cfg::FUSED && Cfg::FUSE != 3 && (hook_present<H_GL2SH_B>(args) || hook_present<H_SH2RF_B>(args));
  // kept in registers for the whole K loop: a scalar load inside the loop would make the compiler
  // wait for lgkmcnt(0), which also drains the LDS reads that are meant to stay in flight
  const bool fast_a = std::is_same<T, _Float16>::value && args.fast_scale_a != 0;
  const bool fast_b = std::is_same<T, _Float16>::value && args.fast_scale_b != 0;
  const float scale_a = args.scale_a, scale_b = args.scale_b;

  typedef FragReader<BM, BK, Cfg::A_KIND, FM, MI> RA;
  typedef FragReader<BN, BK, Cfg::B_KIND, FN, MI> RB;
  RA ra;
  RB rb;
  ra.init(wm * Cfg::WTM, lane);
  rb.init(wn * Cfg::WTN, lane);
  const unsigned lds_base = (unsigned)(uintptr_t)GK_LDS_PTR(char, smem);

  // --- main loop ------------------------------------------------------------------------------
  // Fragments are double-buffered: the LDS reads of the next k-step are in flight while the MFMAs
  // of the current one run.  LDS reads complete in order, so "at most NEXT outstanding" means that
  // the current set has arrived.
  typename RA::Raw fa[2][FM];
  typename RB::Raw fb[2][FN];
  constexpr int FRAG_OPS = RA::NREAD * RA::OPS + RB::NREAD * RB::OPS;

  // The whole K loop is a generic lambda whose MODE says at compile time what happens to the fragments
  // (bits 0 / 1: A / B multiplied by an FP16 factor): a flag tested inside the loop costs a branch around
  // every group of MFMAs.  MODE -1 reads the flags at run time (kernels without hooks, where they fold
  // away, and the generic functor kernels).
  auto k_loop = [&](auto mode_c) __attribute__((always_inline)) {
  constexpr int MODE = decltype(mode_c)::value;
  // the B fragments of a k-step, made once for both halves of A; the imaginary fragments of A
  [[maybe_unused]] int4v vb_keep[(Cfg::B_KIND == OPK_KSPLIT || Cfg::A_KIND == OPK_KSPLIT) ? FN : 1];
  [[maybe_unused]] int4v va_keep[Cfg::A_KIND == OPK_KSPLIT ? FM / 2 : 1];
  // runs after the wait that covers the reads of buffer ks & 1
  // With Cfg::SPLIT_A the A fragments live in two half buffers fa[h][0 .. FM/2) and `half_c` says which half
  // (rows fi = h * FM/2 + i) this call multiplies; otherwise fa[ks & 1] holds all FM fragments and half_c is -1.
  auto compute = [&](auto ks_c, auto half_c) {
    constexpr int ks = decltype(ks_c)::value;
    constexpr int half = decltype(half_c)::value;
    constexpr int NA = half < 0 ? FM : FM / 2;             // A fragments of this call
    constexpr int FI0 = half < 0 ? 0 : half * (FM / 2);     // the accumulator row block of the first one
    constexpr bool B_BOTH = Cfg::B_KIND == OPK_KSPLIT;      // (an OPK_KSPLIT A has its own loop below)
    constexpr int ABUF = half < 0 ? (ks & 1) : half;
    int4v va[NA], vb[FN];
#pragma unroll
    for (int fi = 0; fi < NA; ++fi) {
      RA::pin_raw(fa[ABUF][fi]);
      va[fi] = RA::finish(fa[ABUF][fi], lane);
    }
    if constexpr (B_BOTH && half == 1) {
      // the fragments of B were made by the call for the first half of A
#pragma unroll
      for (int fj = 0; fj < FN; ++fj) vb[fj] = vb_keep[fj];
    } else {
#pragma unroll
      for (int fj = 0; fj < FN; ++fj) {
        if (fj < RB::NREAD) RB::pin_raw(fb[ks & 1][fj]);
        vb[fj] = RB::finish(fb[ks & 1][fj % RB::NREAD], lane, fj >= RB::NREAD);
        if constexpr (B_BOTH && half == 0) vb_keep[fj] = vb[fj];
      }
    }
    if constexpr (MODE >= 0) {
      // A is scaled one fragment ahead of the MFMAs that use it: in this order the compiler lets part of
      // the multiplications issue in the shadow of MFMAs (with all of them written up front the loop is 5 %
      // slower; pinning a finer interleaving with scheduling barriers is slower still).  B is scaled once
      // per k-step: the call for the second half of A finds it scaled.
      if constexpr ((MODE & 2) != 0 && half <= 0) {
#pragma unroll
        for (int fj = 0; fj < FN; ++fj) {
          vb[fj] = scale_fragment_f16(vb[fj], scale_b);
          if constexpr (half == 0) RB::store(fb[ks & 1][fj], vb[fj]);
        }
      }
      if constexpr ((MODE & 1) != 0) va[0] = scale_fragment_f16(va[0], scale_a);
#pragma unroll
      for (int fi = 0; fi < NA; ++fi) {
#pragma unroll
        for (int fj = 0; fj < FN; ++fj) acc[FI0 + fi][fj] = Mfma<T, MI>::run(vb[fj], va[fi], acc[FI0 + fi][fj]);
        if constexpr ((MODE & 1) != 0) {
          if (fi + 1 < NA) va[fi + 1] = scale_fragment_f16(va[fi + 1], scale_a);
        }
      }
      return;
    } else if (Cfg::FUSED) {
      if (xf_a) {
        if (fast_a) {
#pragma unroll
          for (int fi = 0; fi < NA; ++fi) va[fi] = scale_fragment_f16(va[fi], scale_a);
        } else if constexpr (Cfg::FUSED_AB_GENERIC) {
#pragma unroll
          for (int fi = 0; fi < NA; ++fi) va[fi] = transform_fragment<T, H_GL2SH_A, H_SH2RF_A>(va[fi], args);
        }
      }
      if (xf_b) {
        if (fast_b) {
#pragma unroll
          for (int fj = 0; fj < FN; ++fj) vb[fj] = scale_fragment_f16(vb[fj], scale_b);
        } else if constexpr (Cfg::FUSED_AB_GENERIC) {
#pragma unroll
          for (int fj = 0; fj < FN; ++fj) vb[fj] = transform_fragment<T, H_GL2SH_B, H_SH2RF_B>(vb[fj], args);
        }
      }
    }
#pragma unroll
    for (int fi = 0; fi < NA; ++fi)
#pragma unroll
      for (int fj = 0; fj < FN; ++fj) {
        acc[FI0 + fi][fj] = Mfma<T, MI>::run(vb[fj], va[fi], acc[FI0 + fi][fj]);
      }
    if constexpr (B_BOTH && half == 0) {
      // the four byte permutes that make fragment fj + 1 of B issue in the shadow of the MFMA on fragment fj
      // (left to itself the compiler puts all sixteen in front of the first MFMA)
      __builtin_amdgcn_sched_group_barrier(0x2, 4, 0);
#pragma unroll
      for (int fj = 1; fj < FN; ++fj) {
        __builtin_amdgcn_sched_group_barrier(0x8, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x2, 4, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x8, NA * FN - (FN - 1), 0);
    }
  };
  // The last K tile of a product whose K is not a whole number of tiles (or that has a chunk over the end of an operand,
  // see tail_k): fetched into the first stage from gta / gtb with clamped coordinates and repaired there, outside the pipeline.
  [[maybe_unused]] auto fetch_tail_tile = [&](auto gta, auto gtb) __attribute__((always_inline)) {
    block_barrier();                                     // every wave is done with the stages of the loop
    char* sa = smem;
    char* sb = sa + GA::BYTES;
    // per chunk: elements it was fetched too far back (0 .. 7), leading elements that keep their value (0 .. 8)
    int shift_a[DMA_A], keep_a[DMA_A], shift_b[DMA_B], keep_b[DMA_B];
    auto fetch = [&](auto kind_c, auto geom, int q, const char* g, long long ld, int rows_valid, char* dst, int& shift, int& keep)
        __attribute__((always_inline)) {
      constexpr int KIND = decltype(kind_c)::value;
      typedef decltype(geom) G;
      int row, col;
      dma_lane_coords<G, KIND>(q, lane, row, col);
      int& r = KIND == OPK_KMAJOR ? row : col;           // index along M (A) or N (B), from the tile origin
      int& k = KIND == OPK_KMAJOR ? col : row;
      const int last_r = KIND == OPK_KMAJOR ? rows_valid - 1 : ((rows_valid - 1) >> 3) << 3;
      r = r > last_r ? last_r : r;
      keep = 8;
      if (KIND == OPK_KMAJOR) {                          // the chunk runs along k
        if (k >= tail_k) { keep = 0; k = ((tail_k - 1) >> 3) << 3; }
        else if (k + 8 > tail_k) keep = tail_k - k;
      } else if (k >= tail_k) { keep = 0; k = tail_k - 1; }
      long long e = (long long)row * ld + col;
      // one past the last element of the operand, counted from the tile origin
      const long long end = KIND == OPK_KMAJOR ? (long long)(rows_valid - 1) * ld + tail_k : (long long)(tail_k - 1) * ld + rows_valid;
      shift = 0;
      if (e + 8 > end) { shift = (int)(e + 8 - end); e -= shift; }
      __builtin_amdgcn_global_load_lds(GK_GLOBAL_PTR(g + e * 2), GK_LDS_PTR(void, dst + q * 1024), 16, 0, 0);
    };
#pragma unroll
    for (int i = 0; i < DMA_A; ++i)
      fetch(std::integral_constant<int, Cfg::A_KIND>{}, GA{}, wave + i * NWAVES, gta, args.lda, args.M - m0, sa, shift_a[i], keep_a[i]);
#pragma unroll
    for (int i = 0; i < DMA_B; ++i)
      fetch(std::integral_constant<int, Cfg::B_KIND>{}, GB{}, wave + i * NWAVES, gtb, args.ldb, args.N - n0, sb, shift_b[i], keep_b[i]);
    wait_vmcnt<0>();                                     // this lane's own slots have landed
    auto repair = [&](char* slot, int shift, int keep) __attribute__((always_inline)) {
      if (shift == 0 && keep == 8) return;
      short8v v = *(const short8v*)slot, out;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        short x = 0;
#pragma unroll
        for (int f = 0; f < 8; ++f) x = (f == e + shift) ? v[f] : x;      // element e was fetched into place e + shift
        out[e] = e < keep ? x : (short)0;
      }
      *(short8v*)slot = out;
    };
#pragma unroll
    for (int i = 0; i < DMA_A; ++i) repair(sa + (wave + i * NWAVES) * 1024 + lane * 16, shift_a[i], keep_a[i]);
#pragma unroll
    for (int i = 0; i < DMA_B; ++i) repair(sb + (wave + i * NWAVES) * 1024 + lane * 16, shift_b[i], keep_b[i]);
    __syncthreads();                                     // waits for the LDS writes as well
    ra.set_stage(lds_base);
    rb.set_stage(lds_base + GA::BYTES);
  };
  typedef std::integral_constant<int, -1> Whole;

  if constexpr (Cfg::SOLO) {
    constexpr int KS = Cfg::KSTEPS;
    constexpr int NM = FM * FN;                       // MFMAs per k-step
    constexpr int NOPA = RA::NREAD * RA::OPS, NOPS = NOPA + RB::NREAD * RB::OPS;    // LDS instructions of the fragment reads of a k-step
    // One side instruction behind an MFMA: a wave issues at most one instruction every four clocks, an MFMA keeps the
    // matrix core busy for sixteen, and with a single wave on the SIMD every further instruction between two MFMAs
    // is time in which the matrix core idles.  A DMA instruction (with its LDS address in M0) goes behind every GD-th
    // MFMA of the k-step that follows the barrier, an LDS read behind every other MFMA.
    constexpr int GD = (4 * (DPT - 1) < NM) ? 4 : 3, RSP = 1;
    static_assert(GD * (DPT - 1) < NM, "the DMA of a tile is issued in the k-step behind the barrier that frees its stage");
    static_assert(NOPS * RSP <= NM, "the fragment reads fit the MFMAs of a k-step");
    // DMA instruction I of the tile that ga / gb stand at
    auto dma_one = [&](auto i_c, int stage) __attribute__((always_inline)) {
      constexpr int I = decltype(i_c)::value;
      char* sa = smem + stage * Cfg::STAGE_BYTES;
      char* sb = sa + GA::BYTES;
      // (the offset passes through an empty assembly statement so that its widening to 64 bits stays next to the DMA
      // instruction, which then takes the tile pointer from scalar registers and the 32-bit offset from the lane)
      unsigned& o = I < DMA_A ? offa[I < DMA_A ? I : 0] : offb[I < DMA_A ? 0 : I - DMA_A];
      asm volatile("" : "+v"(o));
      if constexpr (I < DMA_A) __builtin_amdgcn_global_load_lds(GK_GLOBAL_PTR((Cfg::GETT ? part_a : ga) + o), GK_LDS_PTR(void, sa + dma_group_chunk(I, DMA_A) * 1024), 16, GROUPED ? (I & 3) * 1024 : 0, 0);
      else __builtin_amdgcn_global_load_lds(GK_GLOBAL_PTR((Cfg::GETT ? part_b : gb) + o), GK_LDS_PTR(void, sb + dma_group_chunk(I - DMA_A, DMA_B) * 1024), 16, GROUPED ? ((I - DMA_A) & 3) * 1024 : 0, 0);
    };
    // LDS instruction R of the fragment reads of k-step KS2 (of the stage the readers stand at), into buffer KS2 & 1
    // (into buffer BUF)
    auto read_op = [&](auto r_c, auto ks2_c, auto buf_c) __attribute__((always_inline)) {
      constexpr int R = decltype(r_c)::value, KS2 = decltype(ks2_c)::value, BUF = decltype(buf_c)::value;
      if constexpr (R < NOPA) ra.template read_op<R / RA::OPS, KS2, R % RA::OPS>(fa[BUF][R / RA::OPS]);
      else rb.template read_op<(R - NOPA) / RB::OPS, KS2, (R - NOPA) % RB::OPS>(fb[BUF][(R - NOPA) / RB::OPS]);
    };
    // The MFMAs of k-step ks.  The fragments of k-step (ks + 1) % KS -- of this tile, or of the next one when ks is the
    // last k-step -- are read in the slots behind the first MFMAs.  DMA: the k-step also issues the DMA of a tile.
    // Path 4: the kernel manages the accumulation registers itself.  Block (fi, fj) of the wave tile lives in a[R : R + 3],
    // R = 4 * (fj * FM + fi), and every instruction that touches it -- MFMA, the moves below, the store of D -- names these
    // registers in its text; the compiler never sees them (they are listed as clobbered once, so that the kernel is given
    // the whole register file).  The accumulators start from zero (the MFMAs of the very first k-step take the constant 0 as
    // their third operand) and C comes in while the matrix cores run, block column by block column (group G = block
    // column G: FM blocks, 16 contiguous bytes per lane and block).  K tile G fetches group G in its first k-step, behind the
    // fragment reads, into one of two sets of FM * 4 registers; these loads are younger than the DMA of the next tile, so
    // the wait in front of the barrier lets them stay in flight (memory reads return in order) and the wait of K tile G + 1
    // covers them; the last k-step of K tile G + 1 adds the group to the accumulators: an accumulation register is read,
    // added to and written back by the vector ALU, two values per MFMA slot, starting four slots behind the MFMA of the block
    // (a block whose turn would reach the end of the k-step takes the first slots instead, before its MFMA and a dozen slots
    // after the one of the k-step before): the matrix core has long delivered the block and does not need it again for fifty
    // slots.  So the sum is (products of the first K tiles) + C + (the rest), where the other paths start from C.
    // (a group: CBLK consecutive blocks of a block column, FM of them on path 4; group G holds blocks G * CBLK ... of the
    // wave tile in the order of their registers, block b = fj * FM + fi)
    constexpr int CBLK = (CPATH == 4 || CPATH == 6) ? FM : kSoloSpreadBlocks;
    constexpr int CGROUPS = STREAM_C ? NM / CBLK : 0;
    static_assert(FM % CBLK == 0, "a group of C lies in one block column");
    static_assert((CPATH != 4 && CPATH != 6) || CGROUPS + 3 <= kSoloStreamTiles, "the K tiles that bring C in are written out in front of the loop, the last two behind it");
    static_assert(CPATH != 5 || CGROUPS + 3 == solo_spread_tiles(NM), "the host sends products with enough K tiles");
    static_assert(!STREAM_C || KS >= 2, "the loads of C go into the first k-step of a tile, the additions into the last");
    [[maybe_unused]] float4v cland[(STREAM_C && !HALF_CD) ? 2 : 1][(STREAM_C && !HALF_CD) ? CBLK : 1];
    [[maybe_unused]] int2v cland16[HALF_CD ? 2 : 1][HALF_CD ? CBLK : 1];        // four FP16 values of C per lane and block
    [[maybe_unused]] float ctmp[4][4];                 // values on their way from an accumulation register and back (see c_add_step)
    [[maybe_unused]] unsigned c_voff = 0;              // byte offset of the lane's four rows of block (0, 0) from the wave tile's origin in C
    [[maybe_unused]] const char* c_tile = nullptr;     // the wave tile's origin in C (the same in every lane)
    [[maybe_unused]] long long c_col16 = 0;            // bytes from a block column to the next
    if constexpr (STREAM_C) {
      c_voff = (unsigned)((4 * (lane / MI) + (long long)(lane % MI) * args.ldc) * CDB);
      c_tile = (const char*)args.c + ((long long)(m0 + wm * Cfg::WTM) + (long long)(n0 + wn * Cfg::WTN) * args.ldc) * CDB;
      c_col16 = (long long)args.ldc * (MI * CDB);
      asm volatile("" ::: "a255");           // (the highest one: the kernel is given all 256)
    }
    // the load of block (J, G)
    [[maybe_unused]] auto c_load = [&](auto g_c, auto j_c) __attribute__((always_inline)) {
      constexpr int G = decltype(g_c)::value, J = decltype(j_c)::value;
      constexpr int B = G * CBLK + J, FI = B % FM, FJ = B / FM;
      const char* base = c_tile + c_col16 * FJ;
      const unsigned vo = c_voff;             // (named here: an operand of an assembly statement does not capture by itself)
      if constexpr (HALF_CD) {
        int2v& dst = cland16[G & 1][J];
        asm volatile("global_load_dwordx2 %0, %1, %2 offset:%3" : "=v"(dst) : "v"(vo), "s"(base), "n"(FI * MI * 2) : "memory");
      } else {
        float4v& dst = cland[G & 1][J];
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(dst) : "v"(vo), "s"(base), "n"(FI * MI * 4) : "memory");
      }
    };
    // Step Q (0 .. 5) of the addition of block (J, G): two accumulation registers read, two values added, two registers
    // written back
    // (T: the set of temporaries.  The additions of two blocks overlap in time when their slots do: blocks two rows apart
    // never do, a block that takes the first slots of the k-step may meet any of the first rows and has sets of its own)
    [[maybe_unused]] auto c_add_step = [&](auto g_c, auto j_c, auto q_c, auto t_c) __attribute__((always_inline)) {
      constexpr int G = decltype(g_c)::value, J = decltype(j_c)::value, Q = decltype(q_c)::value, T = decltype(t_c)::value;
      constexpr int R = 4 * (G * CBLK + J), E = 2 * (Q & 1);
      float& t0 = ctmp[T][E];
      float& t1 = ctmp[T][E + 1];
      if constexpr (Q == 0) {
        if constexpr (HALF_CD) asm volatile("" : "+v"(cland16[G & 1][J]));
        else asm volatile("" : "+v"(cland[G & 1][J]));
      }
      if constexpr (Q < 2) {
        asm volatile("v_accvgpr_read_b32 %0, a[%2]\n\tv_accvgpr_read_b32 %1, a[%3]" : "=v"(t0), "=v"(t1) : "n"(R + E), "n"(R + E + 1));
      } else if constexpr (Q < 4) {
        if constexpr (HALF_CD) {
          // (values E and E + 1 are the two halves of a register; FP16 widens exactly)
          const unsigned w = (unsigned)cland16[G & 1][J][E / 2];
          t0 = t0 + (float)__builtin_bit_cast(_Float16, (unsigned short)(w & 0xffffu));
          t1 = t1 + (float)__builtin_bit_cast(_Float16, (unsigned short)(w >> 16));
        } else {
          t0 = t0 + cland[G & 1][J][E];
          t1 = t1 + cland[G & 1][J][E + 1];
        }
      } else {
        asm volatile("v_accvgpr_write_b32 a[%2], %0\n\tv_accvgpr_write_b32 a[%3], %1" :: "v"(t0), "v"(t1), "n"(R + E), "n"(R + E + 1));
      }
    };
    // Contractions: the table entry of K tile kt + 2 (where the tile starts in A and in B) is read from LDS in a slot of the
    // last k-step of tile kt - 1, has arrived when the first k-step of tile kt starts, and becomes the tile pointers of the
    // DMA in two MFMA slots of that k-step, behind the fragment reads (in front of the k-step that issues the DMA the two
    // pairs of v_readfirstlane and the scalar additions behind them stood between two MFMAs: some hundred clocks per K tile
    // in which the matrix core had nothing to do).
    [[maybe_unused]] int4v ktab;                              // a table entry on its way from LDS
    [[maybe_unused]] int gett_next_entry = 0;                 // which one the next DMA k-step asks for
    [[maybe_unused]] auto gett_read_entry = [&](int t) __attribute__((always_inline)) {
      const unsigned addr = lds_base + (unsigned)(Cfg::STAGE_BYTES * STAGES) + 16u * (unsigned)t;
      asm volatile("ds_read_b128 %0, %1" : "=v"(ktab) : "v"(addr) : "memory");
    };
    [[maybe_unused]] auto gett_pointer_a = [&]() __attribute__((always_inline)) {
      asm volatile("" : "+v"(ktab));
      // (one pair of scalar registers, opaque to the compiler: the DMA instructions take it as their scalar base next to the
      // lane's 32-bit offset)
      part_a = (const char*)(((unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane(ktab[1]) << 32) | (unsigned)__builtin_amdgcn_readfirstlane(ktab[0]));
      pin_scalar(part_a);
    };
    [[maybe_unused]] auto gett_pointer_b = [&]() __attribute__((always_inline)) {
      asm volatile("" : "+v"(ktab));
      part_b = (const char*)(((unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane(ktab[3]) << 32) | (unsigned)__builtin_amdgcn_readfirstlane(ktab[2]));
      pin_scalar(part_b);
    };
    // What the read addresses move by when the readers go on to the next stage.  The additions (one per address register)
    // stand in MFMA slots of the last k-step but one of a tile, behind its fragment reads, which are the last that use the
    // old addresses; between the barrier and the first MFMA of the last k-step they were six to eight instructions with
    // the matrix core idle (4096^3: 1.2-1.5 us).
    [[maybe_unused]] unsigned stage_step = 0;
    // PAR: the fragment buffer that the MFMAs of this k-step read (the reads go into the other one)
    // RD: the k-step reads the fragments of the next one
    auto phase = [&](auto ks_c, auto dma_c, int dma_stage, auto lg_c, auto ag_c, auto first_c, auto par_c, auto rd_c) __attribute__((always_inline)) {
      constexpr int ks = decltype(ks_c)::value;
      constexpr int PAR = decltype(par_c)::value;
      constexpr bool RD = decltype(rd_c)::value;
      constexpr bool DMA = decltype(dma_c)::value;
      constexpr int LG = decltype(lg_c)::value, AG = decltype(ag_c)::value;     // groups of C to fetch / to add in this k-step (-1: none)
      [[maybe_unused]] constexpr bool FIRST = decltype(first_c)::value;         // path 4: the accumulators start from zero here
      constexpr int NKS = (ks + 1) % KS;
      int4v va[FM], vb[FN];
      __builtin_amdgcn_sched_barrier(0);       // no MFMA of the k-step before moves behind the waits in front of this one
#pragma unroll
      for (int fi = 0; fi < FM; ++fi) { RA::pin_raw(fa[PAR][fi]); va[fi] = RA::finish(fa[PAR][fi], lane); }
      // B read as OPK_KSPLIT: a fragment of real parts (block column fj) and one of imaginary parts (fj + FN / 2) are made
      // of each set of registers read, four byte permutes each, right before the MFMAs that use them first: the block
      // columns are the outer loop there
      constexpr bool B_BOTH = Cfg::B_KIND == OPK_KSPLIT;
      if constexpr (!B_BOTH) {
#pragma unroll
        for (int fj = 0; fj < FN; ++fj) { RB::pin_raw(fb[PAR][fj]); vb[fj] = RB::finish(fb[PAR][fj], lane); }
      } else {
#pragma unroll
        for (int fj = 0; fj < RB::NREAD; ++fj) RB::pin_raw(fb[PAR][fj]);
      }
      static_for<0, NM>([&](auto i_c) {
        constexpr int i = decltype(i_c)::value;
        constexpr int o_ = B_BOTH ? i / FM : i / FN, q_ = B_BOTH ? ((o_ & 1) ? FM - 1 - (i % FM) : i % FM) : ((o_ & 1) ? FN - 1 - (i % FN) : i % FN);
        constexpr int fi = B_BOTH ? q_ : o_, fj = B_BOTH ? o_ : q_;
        if constexpr (B_BOTH && (i % FM) == 0) vb[fj] = RB::finish(fb[PAR][fj % RB::NREAD], lane, fj >= RB::NREAD);
        if constexpr (STREAM_C) Mfma<T, MI>::template run_fixed<4 * (fj * FM + fi), FIRST>(va[fi], vb[fj]);
        else acc[fi][fj] = Mfma<T, MI>::run(va[fi], vb[fj], acc[fi][fj]);
        // (the scheduling barriers keep every instruction in the slot it is written in)
        if constexpr (DMA && i % GD == 0 && i / GD < DPT) {
          __builtin_amdgcn_sched_barrier(0);
          dma_one(std::integral_constant<int, i / GD>{}, dma_stage);
          __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (RD && (i % RSP) == 0 && i / RSP < NOPS) {
          __builtin_amdgcn_sched_barrier(0);
          read_op(std::integral_constant<int, i / RSP>{}, std::integral_constant<int, NKS>{}, std::integral_constant<int, (PAR ^ 1)>{});
          __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (!DMA && ks == KS - 2 && RD) {
          // (odd distances from the last fragment read: the loads of C and the tile pointers of a contraction take even ones
          // and the distances 1 and 5)
          constexpr int NBA = RA::NBASE, NBB = RB::NBASE, S0 = NOPS * RSP + 7;
          constexpr int SSTEP = (S0 + 2 * (NBA + NBB - 1) < NM) ? 2 : 1;
          static_assert(S0 + SSTEP * (NBA + NBB - 1) < NM, "the address updates fit behind the fragment reads");
          if constexpr (i >= S0 && (i - S0) % SSTEP == 0 && (i - S0) / SSTEP < NBA + NBB) {
            constexpr int J = (i - S0) / SSTEP;
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (J < NBA) ra.cur[J] += stage_step; else rb.cur[J - NBA] += stage_step;
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        if constexpr (Cfg::GETT && DMA && RD) {
          if constexpr (i == NOPS * RSP + 1) { __builtin_amdgcn_sched_barrier(0); gett_read_entry(gett_next_entry); __builtin_amdgcn_sched_barrier(0); }
        }
        if constexpr (Cfg::GETT && !DMA && ks == 0 && RD) {
          static_assert(!Cfg::GETT || NOPS * RSP + 6 < NM, "the slots of the tile pointers lie behind the fragment reads");
          if constexpr (i == NOPS * RSP + 1) { __builtin_amdgcn_sched_barrier(0); gett_pointer_a(); __builtin_amdgcn_sched_barrier(0); }
          if constexpr (i == NOPS * RSP + 5) { __builtin_amdgcn_sched_barrier(0); gett_pointer_b(); __builtin_amdgcn_sched_barrier(0); }
        }
        if constexpr (STREAM_C && !B_BOTH) {
          constexpr int LSLOT0 = NOPS * RSP + 2;                   // (behind the fragment reads)
          constexpr int LSTEP = (LSLOT0 + 4 * (CBLK - 1) < NM) ? 4 : (LSLOT0 + 3 * (CBLK - 1) < NM) ? 3 : 2;
          static_assert(LG < 0 || LSLOT0 + LSTEP * (CBLK - 1) < NM, "the loads of a group of C fit the k-step");
          if constexpr (LG >= 0 && i >= LSLOT0 && (i - LSLOT0) % LSTEP == 0 && (i - LSLOT0) / LSTEP < CBLK) {
            __builtin_amdgcn_sched_barrier(0);
            c_load(lg_c, std::integral_constant<int, (i - LSLOT0) / LSTEP>{});
            __builtin_amdgcn_sched_barrier(0);
          }
          if constexpr (AG >= 0) {
            static_for<0, CBLK * 6>([&](auto u_c) {
              constexpr int u = decltype(u_c)::value, j = u / 6, q = u % 6;
              constexpr int b = AG * CBLK + j, bi = b % FM, bj = b / FM;
              constexpr int p = bi * FN + ((bi & 1) ? FN - 1 - bj : bj);     // the MFMA of block (bi, bj) in this k-step
              constexpr bool early = !(p + 9 < NM);
              constexpr int s0 = early ? p + 4 - NM + 8 : p + 4;
              // (the two halves of a step trade places so that a value is read, added and written two slots apart)
              constexpr int at = s0 + (q / 2) * 2 + (q & 1);
              if constexpr (at == i) {
                __builtin_amdgcn_sched_barrier(0);
                c_add_step(ag_c, std::integral_constant<int, j>{}, std::integral_constant<int, q>{}, std::integral_constant<int, (bi & 1) + (early ? 2 : 0)>{});
                __builtin_amdgcn_sched_barrier(0);
              }
            });
          }
        }
      });
    };
    typedef std::integral_constant<bool, true> Yes;
    typedef std::integral_constant<bool, false> No;
    typedef std::integral_constant<int, -1> NoGroup;
    // tiles 0 and 1 were issued before the C load.  From here on ga / gb stand at the tile that the next DMA fetches:
    // tile kt + 2 in step kt.  The last two tiles have nothing left to fetch and are written out behind the loop without
    // the DMA (a branch around every DMA instruction would cost more issue slots than the instruction; fetching the last
    // tile again into a stage nobody reads, as an earlier version did, costs the memory pipeline two tiles' worth of time).
    if (KT > 1) wait_vmcnt<DPT>(); else wait_vmcnt<0>();
    block_barrier();
    ra.set_stage(lds_base);
    rb.set_stage(lds_base + GA::BYTES);
    if constexpr (Cfg::GETT) gett_read_entry(2 < KT ? 2 : KT - 1);      // (the table is published by the barrier above)
    static_for<0, NOPS>([&](auto r_c) { read_op(r_c, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}); });
    // DMA: the tile fetches tile kt + 2; LAST: there is no tile kt + 1 (nothing to wait for, nothing to read ahead)
    // PEND: loads of C, younger than the DMA of tile kt + 1, that stay in flight over the wait for that tile
    auto tile_body = [&](int kt, auto lg_c, auto ag_c, auto first_c, auto dma_c, auto last_c, auto pend_c) __attribute__((always_inline)) {
      constexpr bool LAST = decltype(last_c)::value;
      static_for<0, KS>([&](auto ks_c) {
        constexpr int ks = decltype(ks_c)::value;
        __builtin_amdgcn_sched_barrier(0);
        wait_lgkmcnt<0>();                              // the fragments of this k-step have arrived
        if constexpr (ks == KS - 1) {
          if constexpr (!LAST) {
            // tile kt+1 has landed (its DMA was issued a k-step or more ago); behind the barrier it is visible to all
            // waves, and all are done reading tile kt: its stage takes tile kt+2
            // (the loads of C that this tile has issued stay in flight: memory reads return in order, and they are younger than the DMA)
            wait_vmcnt<decltype(pend_c)::value>();
            block_barrier();
            // (the readers' addresses moved on to the stage of tile kt + 1 in the k-step before, see stage_step)
          }
          // contractions: the table entry of the tile that the DMA k-step of the next tile fetches (tile kt + 3, or the last
          // tile once more) is read in a slot of this k-step and arrives with the fragments that it reads
          if constexpr (Cfg::GETT) gett_next_entry = kt + 3 < KT ? kt + 3 : KT - 1;
          phase(ks_c, dma_c, kt & 1, NoGroup{}, ag_c, No{}, std::integral_constant<int, (ks & 1)>{}, std::integral_constant<bool, !LAST>{});
          if constexpr (decltype(dma_c)::value) { ga += a_step; gb += b_step; }
        } else {
          if constexpr (ks == KS - 2) stage_step = ((kt + 1) & 1) ? (unsigned)Cfg::STAGE_BYTES : 0u - (unsigned)Cfg::STAGE_BYTES;
          if constexpr (ks == 0) phase(ks_c, No{}, 0, lg_c, NoGroup{}, first_c, std::integral_constant<int, 0>{}, Yes{});
          else phase(ks_c, No{}, 0, NoGroup{}, NoGroup{}, No{}, std::integral_constant<int, (ks & 1)>{}, Yes{});
          if constexpr (ks == KS - 2) { ra.stage_addr += stage_step; rb.stage_addr += stage_step; }
        }
      });
    };
    if constexpr (STREAM_C) {
      // the first K tiles, written out: tile t fetches group t of C and adds group t - 1 (the host sends products of at
      // least kSoloStreamTiles K tiles here) ...
      typedef std::integral_constant<int, 0> Pend0;
      static_for<0, CGROUPS + 1>([&](auto t_c) {
        constexpr int t = decltype(t_c)::value;
        constexpr int LGT = t < CGROUPS ? t : -1;
        tile_body(t, std::integral_constant<int, LGT>{}, std::integral_constant<int, t - 1>{}, std::integral_constant<bool, t == 0>{}, Yes{}, No{},
                  std::integral_constant<int, (LGT >= 0 ? CBLK : 0)>{});
      });
      for (int kt = CGROUPS + 1; kt < KT - 2; ++kt) tile_body(kt, NoGroup{}, NoGroup{}, No{}, Yes{}, No{}, Pend0{});
      // ... and the last two, which have nothing left to fetch
      tile_body(KT - 2, NoGroup{}, NoGroup{}, No{}, No{}, No{}, Pend0{});
      tile_body(KT - 1, NoGroup{}, NoGroup{}, No{}, No{}, Yes{}, Pend0{});
    } else {
      typedef std::integral_constant<int, 0> Pend0;
      for (int kt = 0; kt < KT - 2; ++kt) tile_body(kt, NoGroup{}, NoGroup{}, No{}, Yes{}, No{}, Pend0{});
      if (KT >= 2) tile_body(KT - 2, NoGroup{}, NoGroup{}, No{}, No{}, No{}, Pend0{});
      if (KT >= 1) tile_body(KT - 1, NoGroup{}, NoGroup{}, No{}, No{}, Yes{}, Pend0{});
    }
    wait_vmcnt<0>();     // (the last DMA of the loop may still be on its way; so are reads
    wait_lgkmcnt<0>();   // of fragments)
    // (path 4 issues its MFMAs from assembly statements, which the compiler does not see: the results of the last ones must
    // have left the matrix core before anything else reads their registers)
    if constexpr (STREAM_C) asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    if constexpr (RAGGED_K) {
      // the last, partial K tile, outside the schedule of the loop: the k-steps that hold valid values
      if (tail_k > 0) {
        stage_step = 0;                                  // (the k-steps below read one stage)
        fetch_tail_tile(ga_tail, gb_tail);
        static_for<0, KS>([&](auto ks_c) {
          constexpr int ks = decltype(ks_c)::value;
          if (ks * Cfg::KSTEP_K < tail_k) {
            static_for<0, NOPS>([&](auto r_c) { read_op(r_c, ks_c, std::integral_constant<int, (ks & 1)>{}); });
            wait_lgkmcnt<0>();
            phase(ks_c, No{}, 0, NoGroup{}, NoGroup{}, No{}, std::integral_constant<int, (ks & 1)>{}, Yes{});        // (what it reads ahead for the next k-step is read again there, or never used)
            wait_lgkmcnt<0>();
          }
        });
      }
    }
  } else if constexpr (!Cfg::PREFETCH) {
    // Two LDS stages: the DMA of tile kt+1 runs while tile kt is consumed; the first fragments of a
    // tile are read after the barrier that publishes it.
    for (int kt = 0; kt < KT; ++kt) {
      // tile kt has landed once at most the DMA of the STAGES-2 younger tiles is outstanding
      if (kt + STAGES - 2 < KT) wait_vmcnt<(STAGES - 2) * DPT>(); else wait_vmcnt<0>();
      block_barrier();   // every wave's share of tile kt is in LDS; every wave is done with tile kt-1
      const unsigned stage_addr = lds_base + (unsigned)(kt % STAGES) * Cfg::STAGE_BYTES;
      ra.set_stage(stage_addr);
      rb.set_stage(stage_addr + GA::BYTES);
      const bool issue = (kt + STAGES - 1 < KT);
      if constexpr (Cfg::SPLIT_A) {
        constexpr int HF = FM / 2;
        constexpr int OPS_AH = HF * RA::OPS, OPS_B = RB::NREAD * RB::OPS;
        // reads of A half H of k-step KS into fa[H], of B of k-step KS into fb[KS & 1]
        auto load_a_half = [&](auto ks2_c, auto h_c) __attribute__((always_inline)) {
          constexpr int KS2 = decltype(ks2_c)::value, H = decltype(h_c)::value;
          static_for<0, HF>([&](auto i_c) {
            constexpr int I = decltype(i_c)::value;
            ra.template read<H * HF + I, KS2, Cfg::SYNC_FRAGS>(fa[H][I]);
          });
        };
        auto load_b = [&](auto ks2_c) __attribute__((always_inline)) {
          constexpr int KS2 = decltype(ks2_c)::value;
          static_for<0, RB::NREAD>([&](auto j_c) {
            constexpr int J = decltype(j_c)::value;
            rb.template read<J, KS2, Cfg::SYNC_FRAGS>(fb[KS2 & 1][J]);
          });
        };
        if constexpr (Cfg::A_KIND == OPK_KSPLIT) {
          // One set of reads per k-step serves both halves: once it has arrived, the real and the imaginary fragments
          // of A (and the fragments of B) are made from it and kept, which frees the registers of the reads for those
          // of the next k-step; they are in flight under the MFMAs of both halves.  One buffer each for A and B.
          auto load_both = [&](auto ks2_c) __attribute__((always_inline)) {
            constexpr int KS2 = decltype(ks2_c)::value;
            static_for<0, HF>([&](auto i_c) {
              constexpr int I = decltype(i_c)::value;
              ra.template read<I, KS2, Cfg::SYNC_FRAGS>(fa[0][I]);
            });
            static_for<0, RB::NREAD>([&](auto j_c) {
              constexpr int J = decltype(j_c)::value;
              rb.template read<J, KS2, Cfg::SYNC_FRAGS>(fb[0][J]);
            });
          };
          load_both(std::integral_constant<int, 0>{});
          static_for<0, 2 * Cfg::KSTEPS>([&](auto u_c) {
            constexpr int u = decltype(u_c)::value;
            constexpr int ks = u / 2, h = u % 2;
            if (issue) issue_part(u_c, std::integral_constant<int, 2 * Cfg::KSTEPS>{}, (kt + STAGES - 1) % STAGES);
            if constexpr (h == 0) {
              wait_lgkmcnt<0>();                          // the reads of this k-step have arrived
              // Program order = the order the instructions should issue in (the scheduling groups below pin it): the
              // byte permutes that make a fragment stand right before the MFMAs that first need it, those of the
              // imaginary fragments of A (needed by the second half) between the MFMA groups of the first half, so
              // that all but the first eight run in the shadow of MFMAs; the reads of the next k-step follow the
              // last permute (they reuse the registers the permutes read) and have the whole second half to land.
              constexpr bool B_BOTH = Cfg::B_KIND == OPK_KSPLIT;
              int4v va[HF];
#pragma unroll
              for (int i = 0; i < HF; ++i) RA::pin_raw(fa[0][i]);
#pragma unroll
              for (int fj = 0; fj < RB::NREAD; ++fj) RB::pin_raw(fb[0][fj]);
              va[0] = RA::finish(fa[0][0], lane, false);
#pragma unroll
              for (int fj = 0; fj < FN; ++fj) {
                vb_keep[fj] = RB::finish(fb[0][fj % RB::NREAD], lane, fj >= RB::NREAD);
                acc[0][fj] = Mfma<T, MI>::run(vb_keep[fj], va[0], acc[0][fj]);
              }
#pragma unroll
              for (int i = 1; i < HF; ++i) {
                va[i] = RA::finish(fa[0][i], lane, false);
                va_keep[i - 1] = RA::finish(fa[0][i - 1], lane, true);
                pin(va_keep[i - 1]);          // made here, not where the second half uses it
#pragma unroll
                for (int fj = 0; fj < FN; ++fj) acc[i][fj] = Mfma<T, MI>::run(vb_keep[fj], va[i], acc[i][fj]);
              }
              va_keep[HF - 1] = RA::finish(fa[0][HF - 1], lane, true);
              pin(va_keep[HF - 1]);
              if constexpr (B_BOTH) {
                __builtin_amdgcn_sched_group_barrier(0x2, 8, 0);
                __builtin_amdgcn_sched_group_barrier(0x8, 1, 0);
#pragma unroll
                for (int fj = 1; fj < FN; ++fj) {
                  __builtin_amdgcn_sched_group_barrier(0x2, 4, 0);
                  __builtin_amdgcn_sched_group_barrier(0x8, 1, 0);
                }
              } else {
                __builtin_amdgcn_sched_group_barrier(0x2, 4, 0);
                __builtin_amdgcn_sched_group_barrier(0x8, FN, 0);
              }
#pragma unroll
              for (int i = 1; i < HF; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x2, 8, 0);
                __builtin_amdgcn_sched_group_barrier(0x8, FN, 0);
              }
              __builtin_amdgcn_sched_group_barrier(0x2, 4, 0);
              if constexpr (ks + 1 < Cfg::KSTEPS) load_both(std::integral_constant<int, ks + 1>{});
            } else {
#pragma unroll
              for (int i = 0; i < HF; ++i)
#pragma unroll
                for (int fj = 0; fj < FN; ++fj) acc[HF + i][fj] = Mfma<T, MI>::run(vb_keep[fj], va_keep[i], acc[HF + i][fj]);
            }
          });
          // (the last reads of the stage were waited for before its last MFMAs: complete before the next barrier)
          continue;
        }
        load_a_half(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
        load_b(std::integral_constant<int, 0>{});
        static_for<0, 2 * Cfg::KSTEPS>([&](auto u_c) {
          constexpr int u = decltype(u_c)::value;
          constexpr int ks = u / 2, h = u % 2;
          if (issue) issue_part(u_c, std::integral_constant<int, 2 * Cfg::KSTEPS>{}, (kt + STAGES - 1) % STAGES);
          if constexpr (h == 0) {
            load_a_half(std::integral_constant<int, ks>{}, std::integral_constant<int, 1>{});
            wait_lgkmcnt<OPS_AH>();                     // half 0 and B of this k-step have arrived
          } else if constexpr (ks + 1 < Cfg::KSTEPS) {
            load_a_half(std::integral_constant<int, ks + 1>{}, std::integral_constant<int, 0>{});
            load_b(std::integral_constant<int, ks + 1>{});
            wait_lgkmcnt<OPS_AH + OPS_B>();             // half 1 of this k-step has arrived
          } else {
            wait_lgkmcnt<0>();                          // all LDS reads of this stage are complete before the next barrier
          }
          compute(std::integral_constant<int, ks>{}, std::integral_constant<int, h>{});
        });
        continue;
      }
      load_frags<0, Cfg::SYNC_FRAGS>(ra, rb, fa[0], fb[0]);
      if constexpr (!Cfg::SPREAD) {
        if (issue) issue_tile((kt + STAGES - 1) % STAGES);
      }
      static_for<0, Cfg::KSTEPS>([&](auto ks_c) {
        constexpr int ks = decltype(ks_c)::value;
        constexpr bool more = (ks + 1 < Cfg::KSTEPS);
        if constexpr (Cfg::SPREAD) {
          if (issue) issue_part(ks_c, std::integral_constant<int, Cfg::KSTEPS>{}, (kt + STAGES - 1) % STAGES);
        }
        if constexpr (more) load_frags<ks + 1, Cfg::SYNC_FRAGS>(ra, rb, fa[(ks + 1) & 1], fb[(ks + 1) & 1]);
        wait_lgkmcnt<more ? FRAG_OPS : 0>();
        compute(ks_c, Whole{});
      });
      // the last wait above was lgkmcnt(0): all LDS reads of this stage are complete before the
      // next barrier lets a DMA overwrite it
    }
  } else {
    // Three or more LDS stages: the barrier of step kt publishes tile kt+1, so the first fragments
    // of tile kt+1 are read at the end of step kt and the MFMAs of a step start right after its
    // barrier, with neither the LDS latency nor the DMA issue in the way.
    static_assert(!Cfg::PREFETCH || (Cfg::KSTEPS % 2 == 0), "fragment buffers alternate per k-step");
    if (STAGES - 1 <= KT) wait_vmcnt<(STAGES - 2) * DPT>(); else wait_vmcnt<0>();
    block_barrier();
    ra.set_stage(lds_base);
    rb.set_stage(lds_base + GA::BYTES);
    load_frags<0, Cfg::SYNC_FRAGS>(ra, rb, fa[0], fb[0]);
    for (int kt = 0; kt < KT; ++kt) {
      // tiles <= kt+1 have landed once at most the STAGES-3 younger tiles are outstanding
      if (kt + STAGES - 2 < KT) wait_vmcnt<(STAGES - 3) * DPT>(); else wait_vmcnt<0>();
      block_barrier();   // tile kt+1 is visible; every wave is done reading tile kt-1
      const bool issue = (kt + STAGES - 1 < KT);
      const bool last = (kt + 1 >= KT);
      static_for<0, Cfg::KSTEPS>([&](auto ks_c) {
        constexpr int ks = decltype(ks_c)::value;
        if constexpr (ks + 1 < Cfg::KSTEPS) {
          load_frags<ks + 1, Cfg::SYNC_FRAGS>(ra, rb, fa[(ks + 1) & 1], fb[(ks + 1) & 1]);
          wait_lgkmcnt<FRAG_OPS>();
          if constexpr (ks == 0 && !Cfg::SPREAD) {
            if (issue) issue_tile((kt + STAGES - 1) % STAGES);
          }
        } else {
          if (!last) {
            const unsigned stage_addr = lds_base + (unsigned)((kt + 1) % STAGES) * Cfg::STAGE_BYTES;
            ra.set_stage(stage_addr);
            rb.set_stage(stage_addr + GA::BYTES);
            load_frags<0, Cfg::SYNC_FRAGS>(ra, rb, fa[0], fb[0]);
            wait_lgkmcnt<FRAG_OPS>();
          } else {
            wait_lgkmcnt<0>();
          }
        }
        if constexpr (Cfg::SPREAD) {
          if (issue) issue_part(ks_c, std::integral_constant<int, Cfg::KSTEPS>{}, (kt + STAGES - 1) % STAGES);
        }
        compute(ks_c, Whole{});
      });
    }
  }
  if constexpr (Cfg::RAGGED_K_OK) {
    // --- the last K tile, when it is partial or has a chunk over the end of an operand (see tail_k above) ---------
    // Outside the pipeline: every lane fetches its 16-byte chunks with coordinates clamped to valid ones -- a chunk
    // that would reach past the last element of the operand is fetched from 1 .. 7 elements further back -- and
    // then repairs its own chunks in LDS: shifted into place, values whose k is beyond K set to zero.  Then the
    // k-steps that hold valid values are multiplied.  ga / gb stand at this tile: every earlier tile has been issued.
    if (tail_k > 0) {
      fetch_tail_tile(ga, gb);
      static_for<0, Cfg::KSTEPS>([&](auto ks_c) {
        constexpr int ks = decltype(ks_c)::value;
        if (ks * Cfg::KSTEP_K < tail_k) {
          if constexpr (Cfg::SPLIT_A) {
            constexpr int HF = FM / 2;
            static_for<0, 2>([&](auto h_c) {
              constexpr int H = decltype(h_c)::value;
              static_for<0, HF>([&](auto i_c) {
                constexpr int I = decltype(i_c)::value;
                ra.template read<H * HF + I, ks, true>(fa[H][I]);
              });
              if constexpr (H == 0) {
                static_for<0, RB::NREAD>([&](auto j_c) {
                  constexpr int J = decltype(j_c)::value;
                  rb.template read<J, ks, true>(fb[ks & 1][J]);
                });
              }
              compute(ks_c, h_c);
            });
          } else {
            load_frags<ks, true>(ra, rb, fa[ks & 1], fb[ks & 1]);
            compute(ks_c, Whole{});
          }
        }
      });
    }
  }
  };   // k_loop
  if constexpr (Cfg::FUSE == 1) {
    // FP16 operands whose hooks are at most one multiplication by a factor that is exact in FP16 (the host
    // passes 1 for an operand without one): both multiplications always run.  Separate copies of the loop
    // per combination cost more than the multiplications save (the accumulators of the copies meet in
    // registers the compiler then has to spill).
    k_loop(std::integral_constant<int, 3>{});
  } else {
    k_loop(std::integral_constant<int, -1>{});
  }

  if constexpr (Cfg::SPLITK) {
    // every slice of K leaves its partial tile in the workspace; the last one to arrive adds them up in slice
    // order and goes on to the epilogue, the others are done
    if (args.k_slices > 1) {
      block_barrier();         // every wave is done with the LDS tiles: the first word now carries the arrival count
      if (!splitk_reduce<Cfg::THREADS>(acc, args, ti + tj * args.nbm, (unsigned*)smem)) return;
    }
  }

  if constexpr (Cfg::FUSED && !Cfg::SOLO) {      // (SOLO: in its own epilogue)
    if (args.acc_post_scale != 1.0f) scale_acc(args.acc_post_scale);
  }

  if constexpr (Cfg::ROWS_LANE && Cfg::COLS_FRAG && !Cfg::SOLO) {
    // As below, with the products of the imaginary parts of B in the column blocks fj + FN / 2: lane 2i holds
    // re A * re B in block fj and re A * im B in block fj + FN / 2, lane 2i+1 im A * re B and im A * im B.
#pragma unroll
    for (int fi = 0; fi < FM; ++fi)
#pragma unroll
      for (int fj = 0; fj < FNO; ++fj)
#pragma unroll
        for (int v = 0; v < NV; ++v) {
          const float own = acc[fi][fj][v];
          const float mine = acc[fi][fj + FNO][v];
          const float other = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, mine), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
          acc[fi][fj][v] = (lane & 1) ? own + other : (Cfg::FIX == FIX_PAIR_DUAL ? own : own - other);
        }
  }
  if constexpr (Cfg::ROWS_LANE && Cfg::COLS_LANE && !Cfg::SOLO) {
    // The four real products of a complex element of D = (re A + i im A)(re B + i im B): lane 2i holds, for
    // each of its two complex columns, re A * re B (value 0 / 2) and re A * im B (value 1 / 3), lane 2i+1
    // im A * re B and im A * im B.  The neighbours trade their odd values: lane 2i becomes the real part
    // re*re - im*im, lane 2i+1 the imaginary part im*re + re*im (dual numbers: re*re, and du*re + re*du), left in
    // the values 0 and 2 -- the row of the real view of D that the lane already stands for.  C came in through
    // the same values.
#pragma unroll
    for (int fi = 0; fi < FM; ++fi)
#pragma unroll
      for (int fj = 0; fj < FN; ++fj)
#pragma unroll
        for (int v = 0; v < 2; ++v) {
          const float own = acc[fi][fj][2 * v];
          // (the value goes through a scalar first: a bit cast applied to the vector element itself is
          // compiled as a cast of the whole vector, of which element 0 is then taken)
          const float mine = acc[fi][fj][2 * v + 1];
          const float other = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, mine), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
          acc[fi][fj][2 * v] = (lane & 1) ? own + other : (Cfg::FIX == FIX_PAIR_DUAL ? own : own - other);
        }
  }

  if constexpr (Cfg::ROWS_FRAG && Cfg::COLS_FRAG && !Cfg::SOLO) {
    // The four real products of the elements of D lie in four blocks of the lane: (row blocks of re A | im A) x
    // (column blocks of re B | im B).  Real part re*re - im*im into the upper left block, imaginary part
    // im*re + re*im into the lower left one (dual numbers: re*re, and du*re + re*du); C came in through the same two.
#pragma unroll
    for (int fi = 0; fi < FMH; ++fi)
#pragma unroll
      for (int fj = 0; fj < FNO; ++fj) {
        if constexpr (Cfg::FIX != FIX_PAIR_DUAL) acc[fi][fj] = acc[fi][fj] - acc[fi + FMH][fj + FNO];
        acc[fi + FMH][fj] = acc[fi + FMH][fj] + acc[fi][fj + FNO];
      }
  }
  if constexpr (Cfg::ROWS_FRAG && Cfg::COLS_LANE && !Cfg::SOLO) {
    // re A | im A in the row blocks fi | fi + FM / 2, re B | im B in the values 2v | 2v + 1 of a block
#pragma unroll
    for (int fi = 0; fi < FMH; ++fi)
#pragma unroll
      for (int fj = 0; fj < FN; ++fj)
#pragma unroll
        for (int v = 0; v < 2; ++v) {
          const float rr = acc[fi][fj][2 * v], ri = acc[fi][fj][2 * v + 1], ir = acc[fi + FMH][fj][2 * v], ii = acc[fi + FMH][fj][2 * v + 1];
          acc[fi][fj][2 * v] = Cfg::FIX == FIX_PAIR_DUAL ? rr : rr - ii;
          acc[fi + FMH][fj][2 * v] = ir + ri;
        }
  }

  if constexpr (Cfg::SOLO) {
    // (the lane number is asked for again: nothing of the store addresses is then kept in registers across the K loop)
    int lane_e = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    asm volatile("" : "+v"(lane_e));
    const int solo_row = (Cfg::PLANAR ? (m0 + wm * Cfg::WTM) / 2 : m0 + wm * Cfg::WTM) + 4 * (lane_e / MI);
    const int solo_col = (Cfg::COLS_FRAG ? (n0 + wn * Cfg::WTN) / 2 : n0 + wn * Cfg::WTN) + (lane_e % MI);      // (as before the K loop)
    if constexpr (!Cfg::GETT) solo_origins(solo_row, solo_col);
    if constexpr (Cfg::PLANAR) {
      // (row blocks of re A | im A) x (block columns of re B | im B): real part re*re - im*im into the upper left block,
      // imaginary part im*re + re*im into the lower left one; C came in through the same two
#pragma unroll
      for (int fj = 0; fj < SFN; ++fj)
#pragma unroll
        for (int fi = 0; fi < SFM; ++fi) {
          asm volatile("" : "+a"(acc[fi][fj]));
          asm volatile("" : "+a"(acc[fi + SFM][fj + SFN]));
          acc[fi][fj] = acc[fi][fj] - acc[fi + SFM][fj + SFN];
          asm volatile("" : "+a"(acc[fi][fj]));
          asm volatile("" : "+a"(acc[fi + SFM][fj]));
          asm volatile("" : "+a"(acc[fi][fj + SFN]));
          acc[fi + SFM][fj] = acc[fi + SFM][fj] + acc[fi][fj + SFN];
          asm volatile("" : "+a"(acc[fi + SFM][fj]));
        }
    }
    if constexpr (Cfg::PAIR) {
      // The four real products of two complex elements of D in one lane: its rows 0 .. 3 of block (fi, fj) are
      // re A re B, im A re B of complex row m and of m + 1, those of block (fi, fj + FN / 2) re A im B, im A im B.
      // Real part re*re - im*im, imaginary part im*re + re*im (dual numbers: re*re, and du*re + re*du), left where
      // the real view of D has them: values 0 .. 3 of block (fi, fj).  C came in through the same values.
#pragma unroll
      for (int fj = 0; fj < SFN; ++fj)
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) {
          asm volatile("" : "+a"(acc[fi][fj]));
          asm volatile("" : "+a"(acc[fi][fj + SFN]));
          const AccV a = acc[fi][fj], b = acc[fi][fj + SFN];
          AccV o;
          o[0] = Cfg::FIX == FIX_PAIR_DUAL ? a[0] : a[0] - b[1];
          o[1] = a[1] + b[0];
          o[2] = Cfg::FIX == FIX_PAIR_DUAL ? a[2] : a[2] - b[3];
          o[3] = a[3] + b[2];
          acc[fi][fj] = o;
          asm volatile("" : "+a"(acc[fi][fj]));
        }
    }
    if constexpr (Cfg::FUSE == 4) {
      // D = op1(op0(s * acc) + bias): one block column at a time leaves the accumulation registers (32 values per lane),
      // is transformed and stored; the switch on an op is paid once per block column
      const int k0 = args.t[H_RF2SH_D].n > 0 ? args.t[H_RF2SH_D].kind[0] : (int)T_IDENTITY;
      const int k1 = args.t[H_SH2GL_D].n > 0 ? args.t[H_SH2GL_D].kind[0] : (int)T_IDENTITY;
      const float p00 = args.t[H_RF2SH_D].p0[0], p01 = args.t[H_RF2SH_D].p1[0], p10 = args.t[H_SH2GL_D].p0[0], p11 = args.t[H_SH2GL_D].p1[0];
      const float post = args.acc_post_scale;
      const int epi = args.epi_kind;
      const bool d_wide = args.d_dtype == DT_F32 && ((((uintptr_t)args.d) | ((uintptr_t)args.ldd << 2)) & 15u) == 0;
      [[maybe_unused]] const unsigned fused_voff = (unsigned)((4 * (lane_e / MI) + (long long)(lane_e % MI) * args.ldd) * 4);
      [[maybe_unused]] const char* fused_tile = (const char*)args.d + ((long long)(m0 + wm * Cfg::WTM) + (long long)(n0 + wn * Cfg::WTN) * args.ldd) * 4;
      [[maybe_unused]] const long long fused_col16 = (long long)args.ldd * (MI * 4);
      // the lane's bias values: its column of every block column, or its rows of every row block
      float bcol[FN], brow[FM * 4];
#pragma unroll
      for (int j = 0; j < FN; ++j) bcol[j] = bcol_early[j];        // (fetched in front of the K loop)
#pragma unroll
      for (int e = 0; e < FM * 4; ++e) brow[e] = brow_early[e];
      static_for<0, SFN>([&](auto fj_c) __attribute__((always_inline)) {
        constexpr int fj = decltype(fj_c)::value;
        float x[FM * 4];
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) {
          asm volatile("" : "+a"(acc[fi][fj]));
#pragma unroll
          for (int v = 0; v < 4; ++v) x[4 * fi + v] = acc[fi][fj][v] * post;
        }
        dispatch_op(k0, p00, p01, [&](auto f) __attribute__((always_inline)) {
#pragma unroll
          for (int e = 0; e < FM * 4; ++e) x[e] = f(x[e]);
        });
        if (epi == 1) {            // one bias value per column of D
#pragma unroll
          for (int e = 0; e < FM * 4; ++e) x[e] = x[e] + bcol[fj];
        } else if (epi == 2) {     // one bias value per row of D
#pragma unroll
          for (int e = 0; e < FM * 4; ++e) x[e] = x[e] + brow[e];
        }
        dispatch_op(k1, p10, p11, [&](auto f) __attribute__((always_inline)) {
#pragma unroll
          for (int e = 0; e < FM * 4; ++e) x[e] = f(x[e]);
        });
        static_for<0, FM>([&](auto fi_c) __attribute__((always_inline)) {
          constexpr int fi = decltype(fi_c)::value;
          const long long off = solo_off(solo_row, solo_col, fi, fj, args.ldd, args.plane_d);
          if (d_wide) {
            float4v o;
#pragma unroll
            for (int v = 0; v < 4; ++v) o[v] = x[4 * fi + v];
            if constexpr (!Cfg::GETT && !Cfg::PLANAR && !Cfg::COLS_FRAG) {
              // (the block column's origin in D from scalar registers, the lane's offset in it from a vector register, the row
              // block as an immediate: no address arithmetic per store, as on path 4)
              const unsigned vo = fused_voff;
              const char* sb = fused_tile + fused_col16 * fj;
              // (the wait states behind the store: a store of more than 8 bytes per lane reads its data registers over several
              // clocks, and the vector ALU must not write one of them meanwhile; the compiler inserts these for its own
              // stores and does not know that this statement is one -- without them the first value of a block came out
              // wrong in a quarter of the lanes whenever the next instruction reused its register)
              asm volatile("global_store_dwordx4 %0, %1, %2 offset:%3 sc0 sc1\n\ts_nop 1" :: "v"(vo), "v"(o), "s"(sb), "n"(fi * MI * 4) : "memory");
            } else {
              float* dp = (float*)args.d + off;
              asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" :: "v"(dp), "v"(o) : "memory");       // (write-through, see path 4)
            }
          } else {
#pragma unroll
            for (int v = 0; v < 4; ++v) store_cd(args.d, args.d_dtype, off + v, x[4 * fi + v]);
          }
        });
      });
      return;
    }
    if constexpr (CPATH == 3) {
      // (what lies outside D is left out: columns, groups of four rows, and the last rows of the group that reaches over
      // the last row of a D whose M is not in fours)
#pragma unroll
      for (int fj = 0; fj < FN; ++fj)
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) {
          const int r = solo_row + MI * fi, cc = solo_col + MI * fj;
          if (r < args.M && cc < args.N) {
            float* dp = (float*)args.d + ((long long)r + (long long)cc * args.ldd);
            if (r + 4 <= args.M) {
              asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" :: "v"(dp), "a"(acc[fi][fj]) : "memory");
            } else {
              const int left = args.M - r;     // 1 .. 3
              asm volatile("global_store_dword %0, %1, off" :: "v"(dp), "a"(acc[fi][fj][0]) : "memory");
              if (left > 1) asm volatile("global_store_dword %0, %1, off offset:4" :: "v"(dp), "a"(acc[fi][fj][1]) : "memory");
              if (left > 2) asm volatile("global_store_dword %0, %1, off offset:8" :: "v"(dp), "a"(acc[fi][fj][2]) : "memory");
            }
          }
        }
    } else if constexpr (STREAM_C) {
      // from the accumulation registers the kernel manages itself: the wave tile's origin in D from scalar registers, the
      // lane's offset in it from a vector register, the row block as an immediate.  The stores write through to memory
      // (sc0 sc1): D is not read again by this launch, and what stays dirty in the L2s has to be written back after the
      // last wave has ended, before the launch counts as complete (a kernel that only stores such tiles: 11.3 us from
      // launch to launch with plain stores, 10.1 us with these; the GEMM gains about one microsecond)
      const unsigned d_voff = (unsigned)((4 * (lane_e / MI) + (long long)(lane_e % MI) * args.ldd) * CDB);
      const char* d_tile = (const char*)args.d + ((long long)(m0 + wm * Cfg::WTM) + (long long)(n0 + wn * Cfg::WTN) * args.ldd) * CDB;
      const long long d_col16 = (long long)args.ldd * (MI * CDB);
      static_for<0, FN>([&](auto fj_c) {
        constexpr int fj = decltype(fj_c)::value;
        const char* base = d_tile + d_col16 * fj;
        static_for<0, FM>([&](auto fi_c) {
          constexpr int fi = decltype(fi_c)::value;
          constexpr int R = 4 * (fj * FM + fi);
          const unsigned vo = d_voff;             // (named here: an operand of an assembly statement does not capture by itself)
          const char* sb = base;
          if constexpr (HALF_CD) {
            // one rounding per value (to nearest even, as the conversion of the other paths), two values per register
            float x0, x1, x2, x3;
            asm volatile("v_accvgpr_read_b32 %0, a[%4]\n\tv_accvgpr_read_b32 %1, a[%5]\n\tv_accvgpr_read_b32 %2, a[%6]\n\tv_accvgpr_read_b32 %3, a[%7]"
                         : "=v"(x0), "=v"(x1), "=v"(x2), "=v"(x3) : "n"(R), "n"(R + 1), "n"(R + 2), "n"(R + 3));
            int2v out;
            out[0] = (int)((unsigned)__builtin_bit_cast(unsigned short, (_Float16)x0) | ((unsigned)__builtin_bit_cast(unsigned short, (_Float16)x1) << 16));
            out[1] = (int)((unsigned)__builtin_bit_cast(unsigned short, (_Float16)x2) | ((unsigned)__builtin_bit_cast(unsigned short, (_Float16)x3) << 16));
            asm volatile("global_store_dwordx2 %0, %1, %2 offset:%3 sc0 sc1" :: "v"(vo), "v"(out), "s"(sb), "n"(fi * MI * 2) : "memory");
          } else {
            asm volatile("global_store_dwordx4 %0, a[%2:%3], %1 offset:%4 sc0 sc1" :: "v"(vo), "s"(sb), "n"(R), "n"(R + 3), "n"(fi * MI * 4) : "memory");
          }
        });
      });
    } else if constexpr (CPATH != 0 && !Cfg::GETT && !Cfg::PLANAR) {
      // (as on path 4: the block column's origin in D from scalar registers, the lane's offset in it from a vector register,
      // the row block as an immediate; write-through)
      const unsigned d_voff = (unsigned)((4 * (lane_e / MI) + (long long)(lane_e % MI) * args.ldd) * 4);
      const int col0 = Cfg::COLS_FRAG ? (n0 + wn * Cfg::WTN) / 2 : n0 + wn * Cfg::WTN;      // (as solo_col)
      const char* d_tile = (const char*)args.d + ((long long)(m0 + wm * Cfg::WTM) + (long long)col0 * args.ldd) * 4;
      const long long d_col16 = (long long)args.ldd * (MI * 4);
      static_for<0, SFN>([&](auto fj_c) __attribute__((always_inline)) {
        constexpr int fj = decltype(fj_c)::value;
        const char* base = d_tile + d_col16 * fj;
        static_for<0, FM>([&](auto fi_c) __attribute__((always_inline)) {
          constexpr int fi = decltype(fi_c)::value;
          const unsigned vo = d_voff;             // (named here: an operand of an assembly statement does not capture by itself)
          const char* sb = base;
          AccV& blk = acc[fi][fj];
          asm volatile("global_store_dwordx4 %0, %1, %2 offset:%3 sc0 sc1" :: "v"(vo), "a"(blk), "s"(sb), "n"(fi * MI * 4) : "memory");
        });
      });
    } else if constexpr (CPATH != 0) {
#pragma unroll
      for (int fj = 0; fj < SFN; ++fj)
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) {
          float* dp = (float*)args.d + solo_off(solo_row, solo_col, fi, fj, args.ldd, args.plane_d);
          asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" :: "v"(dp), "a"(acc[fi][fj]) : "memory");       // (write-through, see path 4)
        }
    } else if (args.d_dtype == DT_F32 && ((((uintptr_t)args.d) | ((uintptr_t)args.ldd << 2)) & 15u) == 0) {
      // (FP32 D next to a C that is not)
#pragma unroll
      for (int fj = 0; fj < SFN; ++fj)
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) {
          asm volatile("" : "+a"(acc[fi][fj]));
          *(float4v*)((float*)args.d + solo_off(solo_row, solo_col, fi, fj, args.ldd, args.plane_d)) = acc[fi][fj];
        }
    } else if (args.d_dtype != DT_F32 && ((((uintptr_t)args.d) | ((uintptr_t)args.ldd << 1)) & 7u) == 0) {
      // 16-bit D: one rounding per value, 8 contiguous bytes per lane and block
#pragma unroll
      for (int fj = 0; fj < SFN; ++fj)
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) {
          asm volatile("" : "+a"(acc[fi][fj]));
          const long long off = solo_off(solo_row, solo_col, fi, fj, args.ldd, args.plane_d);
          unsigned short b[4];
#pragma unroll
          for (int v = 0; v < 4; ++v)
            b[v] = args.d_dtype == DT_F16 ? __builtin_bit_cast(unsigned short, (_Float16)acc[fi][fj][v]) : __builtin_bit_cast(unsigned short, (__bf16)acc[fi][fj][v]);
          int2v out;
          out[0] = (int)((unsigned)b[0] | ((unsigned)b[1] << 16));
          out[1] = (int)((unsigned)b[2] | ((unsigned)b[3] << 16));
          *(int2v*)((char*)args.d + off * 2) = out;
        }
    } else {
#pragma unroll
      for (int fj = 0; fj < SFN; ++fj)
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) {
          asm volatile("" : "+a"(acc[fi][fj]));      // (stays where it is until this branch is taken)
          const long long off = solo_off(solo_row, solo_col, fi, fj, args.ldd, args.plane_d);
#pragma unroll
          for (int v = 0; v < 4; ++v) store_cd(args.d, args.d_dtype, off + v, acc[fi][fj][v]);
        }
    }
    return;
  }
  // --- epilogue: regs -> (transform, bias, transform) -> global ------------------------------------
  gett_origins();
#pragma unroll
  for (int fj = 0; fj < FNO; ++fj) {
    if (Cfg::FUSED) {
      hook_col(std::integral_constant<int, H_RF2SH_D>{}, fj);
      if (args.epi_kind == 1) {          // one bias value per column of D
        // (a real bias value goes to the real part of a complex D)
        float bv[NVO];
#pragma unroll
        for (int v = 0; v < NVO; ++v) {
          const int cc = ncol + CB * fj + vcol(v);
          bv[v] = args.bias[(Cfg::RAGGED_OK && cc >= args.N) ? 0 : cc];      // columns over the edge are not stored
        }
#pragma unroll
        for (int fi = 0; fi < FM; ++fi)
#pragma unroll
          for (int v = 0; v < NVO; ++v) acc[fi][fj][slot(v)] = imag_rows(fi) ? acc[fi][fj][slot(v)] : acc[fi][fj][slot(v)] + bv[v];
      } else if (args.epi_kind == 2) {   // one bias value per row of D
#pragma unroll
        for (int fi = 0; fi < FM; ++fi) {
          const int r = Cfg::ROWS_FRAG ? mrow + MI * (fi % FMH) : (Cfg::COMPLEX ? (mrow + MI * fi) >> 1 : mrow + MI * fi);
          const float bv = args.bias[(Cfg::RAGGED_OK && r >= args.M) ? 0 : r];
#pragma unroll
          for (int v = 0; v < NVO; ++v) acc[fi][fj][slot(v)] = imag_rows(fi) ? acc[fi][fj][slot(v)] : acc[fi][fj][slot(v)] + bv;
        }
      }
      hook_col(std::integral_constant<int, H_SH2GL_D>{}, fj);
    }
#pragma unroll
    for (int fi = 0; fi < FM; ++fi) {
      const long long off = cd_offset(fi, fj, args.ldd, args.plane_d);
      const long long ns = cd_nstride(args.ldd);
      float x[NV];
#pragma unroll
      for (int v = 0; v < NVO; ++v) x[v] = acc[fi][fj][slot(v)];
      // the accumulator is rounded once, to the element type of D
      if constexpr (Cfg::RAGGED_OK) {
        if (ragged) {       // tile over the edge: element by element, out-of-range elements are dropped
#pragma unroll
          for (int v = 0; v < NV; ++v) {
            const int r = mrow + MI * fi, cc = ncol + MI * fj + vcol(v);
            if (r < args.M && cc < args.N) store_cd(args.d, args.d_dtype, r + (long long)cc * args.ldd, x[v]);
          }
          continue;
        }
      }
      if (args.d_dtype == DT_F32) {
        float* dp = (float*)args.d + off;
#pragma unroll
        for (int v = 0; v < NVO; ++v) dp[(long long)vcol(v) * ns] = x[v];
      } else if (args.d_dtype == DT_F16) {
        _Float16* dp = (_Float16*)args.d + off;
#pragma unroll
        for (int v = 0; v < NVO; ++v) dp[(long long)vcol(v) * ns] = (_Float16)x[v];
      } else {
        __bf16* dp = (__bf16*)args.d + off;
#pragma unroll
        for (int v = 0; v < NVO; ++v) dp[(long long)vcol(v) * ns] = (__bf16)x[v];
      }
    }
  }
}

}  // namespace gk
