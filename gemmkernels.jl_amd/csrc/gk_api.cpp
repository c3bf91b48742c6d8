// C ABI of libgemmkernels_hip.so: host-side checks, kernel-instance selection and launch.
// See include/gemmkernels_hip.h for the contract and the reference lines each entry replaces.
#include "gemmkernels_hip.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <string>

#include "gk_internal.hpp"
#include "kernels/common.hpp"
#include "kernels/registry.hpp"

namespace {
thread_local std::string g_last_error;
}

namespace gk_internal {

int fail(int code, const char* fmt, ...) {
  char buf[2048];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

}  // namespace gk_internal

namespace {

using gk_internal::fail;

std::atomic<long long> g_lds_override{0};
std::atomic<int> g_threads_override{0};

void device_limits(long long* lds, int* threads) {
  long long l = g_lds_override.load();
  int t = g_threads_override.load();
  if (l <= 0 || t <= 0) {
    int dev = 0, v = 0;
    long long ql = 160 * 1024;
    int qt = 1024;
    if (hipGetDevice(&dev) == hipSuccess) {
      if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) == hipSuccess && v > 0) ql = v;
      if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxThreadsPerBlock, dev) == hipSuccess && v > 0) qt = v;
    } else {
      (void)hipGetLastError();   // no device: keep the MI355X defaults
    }
    if (l <= 0) l = ql;
    if (t <= 0) t = qt;
  }
  *lds = l;
  *threads = t;
}

bool is_checked_layout(int kind) { return kind == GK_LAYOUT_COL_MAJOR || kind == GK_LAYOUT_ROW_MAJOR; }
bool is_row_major(int kind) {
  return kind == GK_LAYOUT_ROW_MAJOR || kind == GK_LAYOUT_ALIGNED_ROW_MAJOR || kind == GK_LAYOUT_INTERLEAVED_ROW_MAJOR ||
         kind == GK_LAYOUT_SPLIT_ROW_MAJOR;
}
bool is_split_layout(int kind) { return kind == GK_LAYOUT_SPLIT_COL_MAJOR || kind == GK_LAYOUT_SPLIT_ROW_MAJOR; }
// reference src/config.jl:175-178
bool require_tile_sized_global(int kind) { return !(kind == GK_LAYOUT_ZERO || is_checked_layout(kind)); }

bool valid_layout_kind(int k) { return k >= GK_LAYOUT_ZERO && k <= GK_LAYOUT_GETT; }

int dtype_size(int dt) {
  switch (dt) {
    case GK_F16: case GK_BF16: case GK_I16: return 2;
    case GK_F32: case GK_I32: return 4;
    case GK_F64: case GK_I64: return 8;
    default: return 0;
  }
}

bool is_mfma_kind(int k) { return k == GK_OP_MFMA || k == GK_OP_MFMA_COMPLEX || k == GK_OP_MFMA_DUAL; }
bool is_fpu_kind(int k) { return k == GK_OP_FPU || k == GK_OP_FPU_TROPICAL; }

bool transforms_present(const gk_transforms* t) {
  if (!t) return false;
  for (int h = 0; h < 8; ++h)
    if (t->hook[h].n_ops > 0) return true;
  return false;
}

// Bounds-checked layouts (Layout.ColMajor / RowMajor, reference src/layout.jl:117-184) promise nothing about
// size or alignment, and the aligned kernel of the configuration's block shape runs them all the same: its
// 16-byte global -> LDS transfers take any 2-byte aligned address; tiles that stick out over M or N clamp
// their loads and mask their C loads and D stores; the last K tile, when it is partial or has a 16-byte chunk
// that reaches over the last row of an operand (M, N or K not a multiple of 8), is fetched outside the
// pipeline and repaired in LDS.  What it needs is at least one whole chunk along the contiguous index of A
// and of B (else the bounds-checked kernel runs).  Decided from the configuration alone.
bool ragged_fast_path(const gk_config* c) {
  if (c->op.kind != GK_OP_MFMA) return false;
  const gk_layout& la = c->global_a_layout; const gk_layout& lb = c->global_b_layout;
  const gk_layout& lc = c->global_c_layout; const gk_layout& ld = c->global_d_layout;
  auto plain = [](int k) { return k == GK_LAYOUT_COL_MAJOR || k == GK_LAYOUT_ROW_MAJOR || k == GK_LAYOUT_ALIGNED_COL_MAJOR || k == GK_LAYOUT_ALIGNED_ROW_MAJOR; };
  if (!plain(la.kind) || !plain(lb.kind)) return false;
  if (ld.kind != GK_LAYOUT_COL_MAJOR && ld.kind != GK_LAYOUT_ALIGNED_COL_MAJOR) return false;
  if (lc.kind != GK_LAYOUT_ZERO && lc.kind != GK_LAYOUT_COL_MAJOR && lc.kind != GK_LAYOUT_ALIGNED_COL_MAJOR) return false;
  if (!(is_checked_layout(la.kind) || is_checked_layout(lb.kind) || is_checked_layout(lc.kind) || is_checked_layout(ld.kind))) return false;
  if ((la.eltype != GK_F16 && la.eltype != GK_BF16) || lb.eltype != la.eltype) return false;
  const long long M = c->matmul_shape.M, N = c->matmul_shape.N, K = c->matmul_shape.K;
  const bool a_row = is_row_major(la.kind), b_row = is_row_major(lb.kind);
  // a chunk is 8 elements along the contiguous index: k for a row-major ('T') A and a column-major ('N') B
  if ((a_row ? K : M) < 8 || (b_row ? N : K) < 8) return false;
  return true;
}

// The aligned kernel has to take the last K tile out of its pipeline (see ragged_fast_path): the instances that
// cannot (K-split) must not run such a product.
bool needs_tail_tile(const gk_config* c) {
  const bool a_row = is_row_major(c->global_a_layout.kind), b_row = is_row_major(c->global_b_layout.kind);
  return (c->matmul_shape.K % c->block_shape.K) != 0 || (!a_row && (c->matmul_shape.M % 8) != 0) || (b_row && (c->matmul_shape.N % 8) != 0);
}

// A multiplication of A (or B) by +-2^e commutes with every rounding of the sum as long as the scaled operand stays
// inside the normal range of its 16-bit type: sum_k (s a) b + c = s (sum_k a b + c / s), bit for bit.  For the
// matrix-core operators (real, complex and dual: s is real, so it acts on both parts of a number) such a hook -- a scale
// by +-2^e, or a negation -- therefore leaves the K loop: the accumulators start from T_c(C) / s and are multiplied by s
// before the hooks of D.  Outside that range the two forms differ: the reference (and the in-loop form) rounds s * a to
// the operand's type, so s = 2^20 turns finite FP16 values into Inf and s = 2^-20 flushes them into the subnormal range,
// where the folded form returns the exact product.  The fold is therefore limited to |e| <= 4 (operands up to 4095 in
// magnitude and down to 2^-10 keep every bit under the largest folded factor, 16); other powers of two run in the K loop
// like any other scale.  Returns the transforms that remain (`storage` when something was folded) and the factor s.
const gk_transforms* fold_pow2_scales(const gk_config* c, const gk_transforms* t, gk_transforms* storage, float* post) {
  *post = 1.0f;
  const bool matrix_core = c->op.kind == GK_OP_MFMA || c->op.kind == GK_OP_MFMA_COMPLEX || c->op.kind == GK_OP_MFMA_DUAL;
  if (!t || !matrix_core || c->global_a_layout.kind == GK_LAYOUT_DIAGONAL) return t;
  float factor = 1.0f;
  bool folded = false;
  gk_transforms out = *t;
  const int pairs[2][2] = {{GK_HOOK_GLOBAL_TO_SHARED_A, GK_HOOK_SHARED_TO_REGS_A}, {GK_HOOK_GLOBAL_TO_SHARED_B, GK_HOOK_SHARED_TO_REGS_B}};
  for (const auto& pr : pairs) {
    int n = 0;
    const gk_op* one = nullptr;
    for (int h : pr) {
      const gk_transform& tr = t->hook[h];
      if (tr.n_ops < 0 || tr.n_ops > GK_MAX_OPS) return t;        // malformed: left to the checks
      for (int i = 0; i < tr.n_ops; ++i)
        if (tr.ops[i].kind != GK_T_IDENTITY) { ++n; one = &tr.ops[i]; }
    }
    if (n != 1 || (one->kind != GK_T_SCALE && one->kind != GK_T_NEG)) continue;
    const float s = one->kind == GK_T_NEG ? -1.0f : one->p0;
    int e = 0;
    const float m = frexpf(s, &e);
    if (!(m == 0.5f || m == -0.5f) || e - 1 < -4 || e - 1 > 4) continue;   // +-2^(e-1), |e - 1| <= 4
    factor *= s;
    out.hook[pr[0]].n_ops = 0;
    out.hook[pr[1]].n_ops = 0;
    folded = true;
  }
  if (!folded) return t;
  *storage = out;
  *post = factor;
  return storage;
}

// Builds the run-time key of the kernel instance for a configuration.
// allow_ragged_fast = false: bounds-checked layouts run on the bounds-checked kernel whatever their alignment.
int make_key_as_configured(const gk_config* c, const gk_transforms* t, const gk_epilogue* e, gk::InstanceKey* key, bool allow_ragged_fast) {
  memset(key, 0, sizeof(*key));
  const int ak = c->global_a_layout.kind, bk = c->global_b_layout.kind;
  const int ck = c->global_c_layout.kind, dk = c->global_d_layout.kind;
  const bool any_gett = ak == GK_LAYOUT_GETT || bk == GK_LAYOUT_GETT || ck == GK_LAYOUT_GETT || dk == GK_LAYOUT_GETT;
  const bool any_checked = is_checked_layout(ak) || is_checked_layout(bk) || is_checked_layout(ck) || is_checked_layout(dk);
  switch (c->op.kind) {
    case GK_OP_MFMA:
      if (ak == GK_LAYOUT_DIAGONAL) key->family = gk::FAMILY_DIAGONAL;
      else if (any_gett) key->family = gk::FAMILY_GETT;
      else if (any_checked && !(allow_ragged_fast && ragged_fast_path(c))) key->family = gk::FAMILY_MFMA_CHECKED;
      else key->family = gk::FAMILY_MFMA;
      break;
    case GK_OP_FPU:
    case GK_OP_FPU_TROPICAL:
      key->family = gk::FAMILY_FPU;
      key->variant = ((c->op.kind == GK_OP_FPU_TROPICAL) ? 1 : 0) + (any_checked ? 2 : 0);
      if (c->op.mb != 8 && c->op.mb > 0) {          // another lane grid than 8 x 8: log2(OPERATOR_M_BASE) + 1 from bit 4 on
        int lg = 0;
        while ((1 << lg) < c->op.mb) ++lg;
        key->variant += (lg + 1) << 4;
      }
      break;
    case GK_OP_MFMA_COMPLEX:
    case GK_OP_MFMA_DUAL:
      key->family = gk::FAMILY_COMPLEX;
      key->variant = (c->op.kind == GK_OP_MFMA_DUAL) ? 1 : (is_split_layout(ak) ? 2 : 0);
      break;
    default:
      return fail(GK_ERR_INVALID_ARGUMENT, "unknown operator kind %d", c->op.kind);
  }
  key->BM = c->block_shape.M;
  key->BN = c->block_shape.N;
  key->BK = c->block_shape.K;
  if (c->compute_warp.M <= 0 || c->compute_warp.N <= 0) return fail(GK_ERR_INVALID_ARGUMENT, "compute_warp must be positive");
  key->waves_m = c->block_shape.M / c->compute_warp.M;
  key->waves_n = c->block_shape.N / c->compute_warp.N;
  key->a_kmajor = is_row_major(ak) ? 1 : 0;    // 'T' A: stored K x M, K contiguous
  key->b_kmajor = is_row_major(bk) ? 0 : 1;    // 'N' B: stored K x N, K contiguous
  if (key->family == gk::FAMILY_GETT) {
    // the contiguous tensor mode decides which LDS tile layout an operand gets
    key->a_kmajor = (c->gett.k.stride0[0] == 1) ? 1 : 0;
    key->b_kmajor = (c->gett.k.stride1[0] == 1) ? 1 : 0;
    key->variant = 1;
  }
  key->dtype = c->global_a_layout.eltype;
  key->acc_dtype = c->global_d_layout.eltype;
  gk_transforms folded_storage;
  float post = 1.0f;
  t = fold_pow2_scales(c, t, &folded_storage, &post);      // power-of-two scales of A / B do not run in the K loop
  key->fused = (transforms_present(t) || post != 1.0f || (e && e->kind != GK_EPILOGUE_DEFAULT)) ? 1 : 0;
  const bool mfma_family = key->family == gk::FAMILY_MFMA || key->family == gk::FAMILY_GETT || key->family == gk::FAMILY_COMPLEX;
  auto ab_hooks = [&]() {
    if (!t) return false;
    const int hooks[4] = {GK_HOOK_GLOBAL_TO_SHARED_A, GK_HOOK_SHARED_TO_REGS_A, GK_HOOK_GLOBAL_TO_SHARED_B, GK_HOOK_SHARED_TO_REGS_B};
    for (int h : hooks)
      for (int i = 0; i < t->hook[h].n_ops && i < GK_MAX_OPS; ++i)
        if (t->hook[h].ops[i].kind != GK_T_IDENTITY) return true;
    return false;
  };
  if (key->fused && mfma_family && !ab_hooks()) {
    key->fused = 3;          // hooks of C and D and the bias only: the K loop of the plain kernel
    return GK_OK;
  }
  if (key->fused && t && (key->family == gk::FAMILY_MFMA || key->family == gk::FAMILY_GETT)) {
    // level 1 covers A / B hooks that are one exact 16-bit scale (or nothing); anything else needs
    // the generic per-element path of level 2
    auto simple = [&](int h0, int h1) {
      const gk_transform& a0 = t->hook[h0];
      const gk_transform& a1 = t->hook[h1];
      int n = 0;
      const gk_op* one = nullptr;
      for (int i = 0; i < a0.n_ops && i < GK_MAX_OPS; ++i) if (a0.ops[i].kind != GK_T_IDENTITY) { ++n; one = &a0.ops[i]; }
      for (int i = 0; i < a1.n_ops && i < GK_MAX_OPS; ++i) if (a1.ops[i].kind != GK_T_IDENTITY) { ++n; one = &a1.ops[i]; }
      if (n == 0) return true;
      if (n != 1 || one->kind != GK_T_SCALE || c->global_a_layout.eltype != GK_F16) return false;
      return (float)(_Float16)one->p0 == one->p0;
    };
    if (!simple(GK_HOOK_GLOBAL_TO_SHARED_A, GK_HOOK_SHARED_TO_REGS_A) || !simple(GK_HOOK_GLOBAL_TO_SHARED_B, GK_HOOK_SHARED_TO_REGS_B))
      key->fused = 2;
    if (c->global_a_layout.eltype != GK_F16) key->fused = 2;   // level 1 is compiled for FP16 only
  }
  if (key->fused && !t && c->global_a_layout.eltype != GK_F16 && (key->family == gk::FAMILY_MFMA || key->family == gk::FAMILY_GETT))
    key->fused = 2;
  return GK_OK;
}

// The arrangement of four waves with 128 x 128 wave tiles (one wave per SIMD, see Cfg::SOLO) is compiled for plain
// products without hooks or bias whose extents are whole numbers of tiles, and for plain products without hooks of any extents
// (tiles over the edges, a partial last K tile: path 3 of the kernel, which moves an FP32 C / D 16 bytes at a time).  Any other launch of such a configuration runs the
// eight-wave arrangement of the same block shape, which gives the same bits (the order of the k-steps and of the
// products inside them does not depend on how the tile is dealt out to waves).
bool wide_tile(const gk::InstanceKey& key) {
  return key.BK == 64 && ((key.BM == 256 && key.BN == 192) || (key.BM == 192 && key.BN == 256));
}
void wide_tile_on_eight_waves(gk::InstanceKey* key) {
  key->waves_m = key->BM == 256 ? 4 : 2;
  key->waves_n = key->BM == 256 ? 2 : 4;
}

int make_key(const gk_config* c, const gk_transforms* t, const gk_epilogue* e, gk::InstanceKey* key, bool allow_ragged_fast = true) {
  const int rc = make_key_as_configured(c, t, e, key, allow_ragged_fast);
  if (rc != GK_OK) return rc;
  const bool plain = key->family == gk::FAMILY_MFMA, contraction = key->family == gk::FAMILY_GETT;
  if ((plain || contraction) && key->BM == 256 && key->BN == 256 && key->BK == 64 && key->waves_m == 2 && key->waves_n == 2) {
    const bool whole = c->matmul_shape.M % 256 == 0 && c->matmul_shape.N % 256 == 0 && c->matmul_shape.K % 64 == 0;
    bool ok = whole;
    if (!whole && plain && key->fused == 0) {
      const bool no_c = c->global_c_layout.kind == GK_LAYOUT_ZERO;
      ok = c->matmul_shape.M >= 8 && c->matmul_shape.K >= 64 && c->global_d_layout.eltype == GK_F32 && (no_c || c->global_c_layout.eltype == GK_F32);
    }
    if (key->fused == 3 && plain) {
      // hooks of C and D and a bias: the four waves take what has a closed form (fuse level 4 of the kernel): no hook on
      // C, at most one op in each hook of D, and a power-of-two scale of A or B folded into the accumulators only where
      // there is no C to scale the other way
      gk_transforms folded_storage;
      float post = 1.0f;
      const gk_transforms* tf = fold_pow2_scales(c, t, &folded_storage, &post);
      auto real_ops = [&](int h) {
        int n = 0;
        if (tf) for (int i = 0; i < tf->hook[h].n_ops && i < GK_MAX_OPS; ++i) if (tf->hook[h].ops[i].kind != GK_T_IDENTITY) ++n;
        return n;
      };
      const bool closed = real_ops(GK_HOOK_GLOBAL_TO_SHARED_C) == 0 && real_ops(GK_HOOK_SHARED_TO_REGS_C) == 0 &&
                          real_ops(GK_HOOK_REGS_TO_SHARED_D) <= 1 && real_ops(GK_HOOK_SHARED_TO_GLOBAL_D) <= 1 &&
                          (post == 1.0f || c->global_c_layout.kind == GK_LAYOUT_ZERO);
      if (closed) key->fused = 4; else ok = false;
    } else if (key->fused != 0) {
      ok = false;
    }
    if (contraction) {
      // contractions: four consecutive m of a lane are 16 contiguous, aligned bytes of an FP32 C / D
      const gk_gett_dim& gm = c->gett.m; const gk_gett_dim& gn = c->gett.n;
      ok = ok && c->global_d_layout.eltype == GK_F32 && (c->global_c_layout.kind == GK_LAYOUT_ZERO || c->global_c_layout.eltype == GK_F32);
      ok = ok && gm.nmodes >= 1 && gm.stride1[0] == 1 && gm.extent[0] % 4 == 0;
      ok = ok && c->matmul_shape.K / 64 <= 1024;          // the K tiles the offset table of these instances holds (KTABLE_TILES)
      for (int i = 1; i < gm.nmodes && i < GK_MAX_MODES; ++i) ok = ok && gm.stride1[i] % 4 == 0;
      for (int i = 0; i < gn.nmodes && i < GK_MAX_MODES; ++i) ok = ok && gn.stride1[i] % 4 == 0;
    }
    if (!ok) {
      key->waves_n = 4;
      if (key->fused == 4) key->fused = 3;
    }
  }
  // ... for the tiles with a side of 192 (wave tiles of 128 x 96 or 96 x 128): plain products without hooks or bias
  // in whole tiles; any other launch runs the eight waves that have the 192 side to themselves in pairs
  if ((plain || key->family == gk::FAMILY_MFMA_CHECKED) && wide_tile(*key) && key->waves_m == 2 && key->waves_n == 2) {
    const bool whole = c->matmul_shape.M % key->BM == 0 && c->matmul_shape.N % key->BN == 0 && c->matmul_shape.K % 64 == 0;
    if (!(plain && whole && key->fused == 0 && key->variant == 0)) wide_tile_on_eight_waves(key);
  }
  // ... and for the complex / dual product on interleaved matrices of an 'N','N' launch (real tile 256 x 256 x 64)
  // (planar matrices, variant 2: every transpose, the planes being plain real operands)
  // (the bounds-checked kernel has no such arrangement)
  if (key->family == gk::FAMILY_MFMA_CHECKED && key->BM == 256 && key->BN == 256 && key->BK == 64 && key->waves_m == 2 && key->waves_n == 2)
    key->waves_n = 4;
  if (key->family == gk::FAMILY_COMPLEX && key->BM == 128 && key->BN == 128 && key->BK == 64 && key->waves_m == 2 && key->waves_n == 2) {
    const bool ok = c->matmul_shape.M % 128 == 0 && c->matmul_shape.N % 128 == 0 && c->matmul_shape.K % 64 == 0 && key->fused == 0 &&
                    (key->variant == 2 || (key->a_kmajor == 0 && key->b_kmajor == 1));
    if (!ok) key->waves_n = 4;
  }
  return GK_OK;
}

bool gett_k_tiling(const gk_gett_dim& k, int bk, int* mode, int* prod, int* step);

void make_args(const gk_config* c, const void* a, const void* b, const void* cc, void* d, const gk_transforms* t,
               const gk_epilogue* e, gk::GemmArgs* args) {
  memset(args, 0, sizeof(*args));
  args->a = a; args->b = b; args->c = cc; args->d = d;
  args->bias = e ? (const float*)e->bias : nullptr;
  args->M = c->matmul_shape.M; args->N = c->matmul_shape.N; args->K = c->matmul_shape.K;
  const bool a_row = is_row_major(c->global_a_layout.kind), b_row = is_row_major(c->global_b_layout.kind);
  args->lda = c->global_a_layout.ld > 0 ? c->global_a_layout.ld : (a_row ? args->K : args->M);
  args->ldb = c->global_b_layout.ld > 0 ? c->global_b_layout.ld : (b_row ? args->N : args->K);
  args->ldc = c->global_c_layout.ld > 0 ? c->global_c_layout.ld : args->M;
  args->ldd = c->global_d_layout.ld > 0 ? c->global_d_layout.ld : args->M;
  args->nbm = (args->M + c->block_shape.M - 1) / c->block_shape.M;
  args->nbn = (args->N + c->block_shape.N - 1) / c->block_shape.N;
  if (c->op.kind == GK_OP_MFMA_COMPLEX || c->op.kind == GK_OP_MFMA_DUAL) {
    // complex operands seen as real matrices: the real views of A (both parts of every row) and of B (both parts of
    // every column) meet in one real product of 2M x 2N x K; the leading dimensions of interleaved matrices count
    // real elements
    args->M *= 2;
    args->N *= 2;
    if (is_split_layout(c->global_a_layout.kind)) {
      // planar operands: a matrix is the real array (rows, cols, 2) in column-major order, so the
      // imaginary plane starts ld * cols elements after the real one
      args->plane_a = args->lda * (a_row ? c->matmul_shape.M : c->matmul_shape.K);
      args->plane_b = args->ldb * (b_row ? c->matmul_shape.K : c->matmul_shape.N);
      args->plane_c = args->ldc * c->matmul_shape.N;
      args->plane_d = args->ldd * c->matmul_shape.N;
    } else {
      args->lda *= 2; args->ldb *= 2; args->ldc *= 2; args->ldd *= 2;
    }
  }
  args->swz_kind = c->cta_swizzle.kind;
  args->swz_param = c->cta_swizzle.param;
  args->c_mode = (c->global_c_layout.kind == GK_LAYOUT_ZERO) ? 0 : 1;
  args->epi_kind = e ? e->kind : 0;
  args->c_dtype = c->global_c_layout.eltype;
  args->d_dtype = c->global_d_layout.eltype;
  args->a_kind = c->global_a_layout.kind;
  args->b_kind = c->global_b_layout.kind;
  args->cd_gett = (c->global_d_layout.kind == GK_LAYOUT_GETT) ? 1 : 0;
  gk_transforms folded_storage;
  float post = 1.0f;
  t = fold_pow2_scales(c, t, &folded_storage, &post);
  args->acc_post_scale = post;
  args->acc_pre_scale = 1.0f / post;       // exact: post is a power of two
  if (t) {
    for (int h = 0; h < 8; ++h) {
      const gk_transform& src = t->hook[h];
      gk::OpList& dst = args->t[h];
      int n = src.n_ops < 0 ? 0 : (src.n_ops > GK_MAX_OPS ? GK_MAX_OPS : src.n_ops);
      int out = 0;
      for (int i = 0; i < n; ++i) {
        if (src.ops[i].kind == GK_T_IDENTITY) continue;
        dst.kind[out] = src.ops[i].kind;
        dst.p0[out] = src.ops[i].p0;
        dst.p1[out] = src.ops[i].p1;
        ++out;
      }
      dst.n = out;
    }
  }
  // one exact FP16 scale over the two load hooks of an operand -> packed multiply in the kernel
  auto single_scale = [&](int h0, int h1, int* fast, float* scale) {
    const gk::OpList& a0 = args->t[h0];
    const gk::OpList& a1 = args->t[h1];
    *fast = 0;
    *scale = 1.0f;
    if (a0.n + a1.n != 1) return;
    const gk::OpList& one = a0.n ? a0 : a1;
    if (one.kind[0] != GK_T_SCALE) return;
    const float v = one.p0[0];
    if ((float)(_Float16)v != v) return;
    *fast = 1;
    *scale = v;
  };
  single_scale(GK_HOOK_GLOBAL_TO_SHARED_A, GK_HOOK_SHARED_TO_REGS_A, &args->fast_scale_a, &args->scale_a);
  single_scale(GK_HOOK_GLOBAL_TO_SHARED_B, GK_HOOK_SHARED_TO_REGS_B, &args->fast_scale_b, &args->scale_b);
  auto copy_dim = [](const gk_gett_dim& s, gk::GettDim& d) {
    d.nmodes = s.nmodes;
    for (int i = 0; i < GK_MAX_MODES; ++i) {
      d.extent[i] = s.extent[i];
      d.stride0[i] = s.stride0[i];
      d.stride1[i] = s.stride1[i];
    }
  };
  copy_dim(c->gett.m, args->gm);
  copy_dim(c->gett.n, args->gn);
  copy_dim(c->gett.k, args->gk);
  gk::gett_fill_division(args->gm);
  gk::gett_fill_division(args->gn);
  gk::gett_fill_division(args->gk);
  args->gk_mode = 0; args->gk_step = c->block_shape.K;
  if (c->global_a_layout.kind == GK_LAYOUT_GETT) {
    int prod = 1;
    gett_k_tiling(c->gett.k, c->block_shape.K, &args->gk_mode, &prod, &args->gk_step);     // validated before
    args->gett_fast = (c->gett.m.extent[0] % 32 == 0 && c->gett.n.extent[0] % 32 == 0) ? 1 : 0;
  }
}

gk::FamilyFn family_fn(const gk::InstanceKey& key) {
  switch (key.family) {
    case gk::FAMILY_MFMA:
      if (wide_tile(key) && key.waves_m == 2 && key.waves_n == 2) {
        // the tiles with a side of 192 on four waves are compiled in translation units of their own
        if (key.a_kmajor) return key.b_kmajor ? (key.BM == 256 ? gk::family_mfma_wide_tn : gk::family_mfma_wide_tn_192x256) : gk::family_mfma_wide_tt;
        return key.b_kmajor ? gk::family_mfma_wide_nn : gk::family_mfma_wide_nt;
      }
      [[fallthrough]];
    case gk::FAMILY_GETT:
      if (key.a_kmajor) return key.b_kmajor ? gk::family_mfma_tn : gk::family_mfma_tt;
      return key.b_kmajor ? gk::family_mfma_nn : gk::family_mfma_nt;
    case gk::FAMILY_FPU:
      return gk::family_fpu;
    case gk::FAMILY_DIAGONAL:
      return gk::family_diagonal;
    case gk::FAMILY_COMPLEX:
      return gk::family_complex;
    case gk::FAMILY_MFMA_CHECKED:
      return gk::family_mfma_checked;
    default:
      return nullptr;
  }
}

int find_instance(const gk_config* c, const gk_transforms* t, const gk_epilogue* e, gk::InstanceKey* key, gk::InstanceInfo* info,
                  bool allow_ragged_fast = true) {
  int rc = make_key(c, t, e, key, allow_ragged_fast);
  if (rc != GK_OK) return rc;
  gk::FamilyFn fn = family_fn(*key);
  gk::GemmArgs dummy;
  memset(&dummy, 0, sizeof(dummy));
  dummy.M = c->matmul_shape.M; dummy.N = c->matmul_shape.N; dummy.K = c->matmul_shape.K;     // (instances that depend on the extents: tiles over the edges)
  hipError_t err = hipSuccess;
  if (key->family == gk::FAMILY_MFMA && allow_ragged_fast && ragged_fast_path(c) && (!fn || !fn(*key, dummy, dim3(1), nullptr, 0, info, &err))) {
    // no aligned instance of this tile: the bounds-checked kernel after all
    rc = make_key(c, t, e, key, false);
    if (rc != GK_OK) return rc;
    fn = family_fn(*key);
  }
  if (!fn || !fn(*key, dummy, dim3(1), nullptr, 0, info, &err)) {
    return fail(GK_ERR_UNSUPPORTED,
                "no compiled kernel instance for operator %d, block (%d, %d, %d), warps %d x %d, A/B layouts %d/%d, eltype %d",
                c->op.kind, key->BM, key->BN, key->BK, key->waves_m, key->waves_n, c->global_a_layout.kind,
                c->global_b_layout.kind, key->dtype);
  }
  return GK_OK;
}

// Tensor-contraction index maps: what the GETT loader assumes about the mode tables.
// How a K tile of bk indices lies in the K modes: it covers modes 0 .. *mode - 1 whole (extents multiplying to *prod)
// and *step indices of mode *mode.  False when no such split exists (bk does not divide evenly into the modes).
bool gett_k_tiling(const gk_gett_dim& k, int bk, int* mode, int* prod, int* step) {
  long long p = 1;
  for (int j = 0; j < k.nmodes && j < GK_MAX_MODES; ++j) {
    if (p <= 0 || bk % p != 0) return false;
    const long long need = bk / p;            // indices of mode j that a tile takes
    if (need <= k.extent[j]) {
      if (k.extent[j] % need != 0) return false;
      *mode = j; *prod = (int)p; *step = (int)need;
      return true;
    }
    p *= k.extent[j];                         // mode j lies inside the tile whole
  }
  return false;
}

// Number of leading modes of `d` (strides `stride`) that are packed densely and whose extents multiply to a multiple
// of 8, so that 8 consecutive indices of the GEMM dimension are 8 consecutive elements in memory (a 16-byte vector);
// 0 when there is no such prefix.
int gett_dense_prefix(const gk_gett_dim& d, const int64_t* stride) {
  long long p = 1;
  for (int i = 0; i < d.nmodes && i < GK_MAX_MODES; ++i) {
    if (stride[i] != p) return 0;
    p *= d.extent[i];
    if (p % 8 == 0) return i + 1;
  }
  return 0;
}

int validate_gett(const gk_config* c) {
  const gk_gett& g = c->gett;
  if (c->op.kind != GK_OP_MFMA) return fail(GK_ERR_UNSUPPORTED, "tensor-contraction layouts need the MFMA operator");
  if (c->global_a_layout.kind != GK_LAYOUT_GETT || c->global_b_layout.kind != GK_LAYOUT_GETT ||
      c->global_d_layout.kind != GK_LAYOUT_GETT ||
      (c->global_c_layout.kind != GK_LAYOUT_GETT && c->global_c_layout.kind != GK_LAYOUT_ZERO))
    return fail(GK_ERR_UNSUPPORTED, "a tensor contraction needs GETT layouts for A, B and D (C: GETT or Zero)");
  const gk_gett_dim* dims[3] = {&g.m, &g.n, &g.k};
  const int want[3] = {c->matmul_shape.M, c->matmul_shape.N, c->matmul_shape.K};
  const char* names[3] = {"M", "N", "K"};
  long long span[3] = {0, 0, 0};   // largest element offset in A, B, D
  for (int d = 0; d < 3; ++d) {
    if (dims[d]->nmodes < 1 || dims[d]->nmodes > GK_MAX_MODES) return fail(GK_ERR_INVALID_ARGUMENT, "%s needs 1..%d tensor modes", names[d], GK_MAX_MODES);
    long long prod = 1;
    for (int i = 0; i < dims[d]->nmodes; ++i) {
      if (dims[d]->extent[i] <= 0) return fail(GK_ERR_INVALID_ARGUMENT, "mode extents must be positive");
      prod *= dims[d]->extent[i];
      const long long e1 = dims[d]->extent[i] - 1;
      if (d == 0) { span[0] += e1 * dims[d]->stride0[i]; span[2] += e1 * dims[d]->stride1[i]; }
      if (d == 1) { span[1] += e1 * dims[d]->stride0[i]; span[2] += e1 * dims[d]->stride1[i]; }
      if (d == 2) { span[0] += e1 * dims[d]->stride0[i]; span[1] += e1 * dims[d]->stride1[i]; }
    }
    if (prod != want[d]) return fail(GK_ERR_DIMENSION_MISMATCH, "the extents of the %s modes multiply to %lld, matmul_shape.%s is %d", names[d], prod, names[d], want[d]);
  }
  if (span[0] * 2 >= (1ll << 31) || span[1] * 2 >= (1ll << 31)) return fail(GK_ERR_UNSUPPORTED, "tensor too large for 32-bit tile offsets");
  // a K tile is a whole number of leading K modes times a slab of the next one (BLOCK_K dividing the first K mode is
  // the simplest case)
  int kmode = 0, kprod = 1, kstep = 0;
  if (!gett_k_tiling(g.k, c->block_shape.K, &kmode, &kprod, &kstep))
    return fail(GK_ERR_TILE_MULTIPLE, "BLOCK_K = %d does not tile the K modes: it must divide the extent %d of the first K mode, or be a whole number "
                                      "of leading K modes times a divisor of the next one", c->block_shape.K, g.k.extent[0]);
  // a lane's four columns of C / D follow each other with the stride of the first N mode
  if (g.n.extent[0] % 4 != 0)
    return fail(GK_ERR_TILE_MULTIPLE, "the first N mode must have an extent that is a multiple of 4, got %d", g.n.extent[0]);
  // 16-byte vectors: each operand has 8 consecutive elements along its leading M (N) modes or along its leading K
  // modes (modes packed densely, extents multiplying to a multiple of 8), and every stride outside that run keeps the
  // alignment
  const bool a_k = g.k.stride0[0] == 1, b_k = g.k.stride1[0] == 1;
  const int a_run = a_k ? gett_dense_prefix(g.k, g.k.stride0) : gett_dense_prefix(g.m, g.m.stride0);
  const int b_run = b_k ? gett_dense_prefix(g.k, g.k.stride1) : gett_dense_prefix(g.n, g.n.stride0);
  if (a_run == 0) return fail(GK_ERR_ALIGNMENT, "A needs 8 consecutive elements along its leading M modes or its leading K modes (densely packed modes whose extents multiply to a multiple of 8)");
  if (b_run == 0) return fail(GK_ERR_ALIGNMENT, "B needs 8 consecutive elements along its leading N modes or its leading K modes (densely packed modes whose extents multiply to a multiple of 8)");
  for (int i = 0; i < g.m.nmodes; ++i) if (!(!a_k && i < a_run) && g.m.stride0[i] % 8 != 0) return fail(GK_ERR_ALIGNMENT, "stride of M mode %d of A is not a multiple of 16 bytes", i);
  for (int i = 0; i < g.k.nmodes; ++i) if (!(a_k && i < a_run) && g.k.stride0[i] % 8 != 0) return fail(GK_ERR_ALIGNMENT, "stride of K mode %d of A is not a multiple of 16 bytes", i);
  for (int i = 0; i < g.n.nmodes; ++i) if (!(!b_k && i < b_run) && g.n.stride0[i] % 8 != 0) return fail(GK_ERR_ALIGNMENT, "stride of N mode %d of B is not a multiple of 16 bytes", i);
  for (int i = 0; i < g.k.nmodes; ++i) if (!(b_k && i < b_run) && g.k.stride1[i] % 8 != 0) return fail(GK_ERR_ALIGNMENT, "stride of K mode %d of B is not a multiple of 16 bytes", i);
  return GK_OK;
}

// All checks that need no pointers; reference src/config.jl:203-275 then src/matmul.jl:28-41.
int validate_config(const gk_config* c, int kernel, const gk_transforms* t, const gk_epilogue* e, gk::InstanceKey* key,
                    gk::InstanceInfo* info, const gk::InstanceInfo* custom = nullptr, bool allow_ragged_fast = true) {
  if (!c) return fail(GK_ERR_INVALID_ARGUMENT, "config is NULL");
  const gk_shape& g = c->matmul_shape;
  const gk_shape& b = c->block_shape;
  const gk_operator& op = c->op;
  if (g.M <= 0 || g.N <= 0 || g.K <= 0) return fail(GK_ERR_DIMENSION_MISMATCH, "matmul_shape must be positive, got (%d, %d, %d)", g.M, g.N, g.K);
  if (b.M <= 0 || b.N <= 0 || b.K <= 0) return fail(GK_ERR_BLOCK_SHAPE, "block_shape must be positive");
  if (kernel < GK_KERNEL_SINGLESTAGE || kernel > GK_KERNEL_SPLIT_K) return fail(GK_ERR_INVALID_ARGUMENT, "unknown kernel kind %d", kernel);
  const gk_layout* layouts[8] = {&c->global_a_layout, &c->global_b_layout, &c->global_c_layout, &c->global_d_layout,
                                 &c->shared_a_layout, &c->shared_b_layout, &c->shared_c_layout, &c->shared_d_layout};
  for (const gk_layout* l : layouts)
    if (!valid_layout_kind(l->kind)) return fail(GK_ERR_INVALID_ARGUMENT, "unknown layout kind %d", l->kind);
  if (c->cta_swizzle.kind < GK_SWIZZLE_IDENTITY || c->cta_swizzle.kind > GK_SWIZZLE_XCD)
    return fail(GK_ERR_INVALID_ARGUMENT, "unknown CTA swizzle kind %d", c->cta_swizzle.kind);
  if ((c->cta_swizzle.kind == GK_SWIZZLE_HORIZONTALLY_TILED || c->cta_swizzle.kind == GK_SWIZZLE_VERTICALLY_TILED) && c->cta_swizzle.param <= 0)
    return fail(GK_ERR_INVALID_ARGUMENT, "tiled CTA swizzles need a positive tile size");

  if (t) {
    for (int h = 0; h < 8; ++h) {
      if (t->hook[h].n_ops < 0 || t->hook[h].n_ops > GK_MAX_OPS)
        return fail(GK_ERR_INVALID_ARGUMENT, "hook %d carries %d ops, a hook holds 0..%d", h, t->hook[h].n_ops, GK_MAX_OPS);
      for (int i = 0; i < t->hook[h].n_ops; ++i)
        if (t->hook[h].ops[i].kind < GK_T_IDENTITY || t->hook[h].ops[i].kind > GK_T_SQUARE)
          return fail(GK_ERR_INVALID_ARGUMENT, "unknown elementwise op %d in hook %d", t->hook[h].ops[i].kind, h);
    }
  }
  if (e && (e->kind < GK_EPILOGUE_DEFAULT || e->kind > GK_EPILOGUE_BIAS_ROW)) return fail(GK_ERR_INVALID_ARGUMENT, "unknown epilogue kind %d", e->kind);

  // src/config.jl:203-205
  if ((long long)b.M * b.K < 128 || (long long)b.K * b.N < 128 || b.K < 8)
    return fail(GK_ERR_BLOCK_SHAPE,
                "The block shape is too small. The dimensions of the block shape must adhere to the following constraints: "
                "BLOCK_M * BLOCK_K >= 128, BLOCK_K * BLOCK_N >= 128, BLOCK_K >= 8.");
  // src/config.jl:209-212
  if (b.M < 2 * op.M || b.N < 2 * op.N || b.K < op.K)
    return fail(GK_ERR_BLOCK_SHAPE,
                "There is a mismatch between the block shape and the operator shape. Their dimensions must adhere to the "
                "following constraints: BLOCK_M >= 2 * OPERATOR_M, BLOCK_N >= 2 * OPERATOR_N, BLOCK_K >= OPERATOR_K.");
  // src/config.jl:136-173, with 64-lane wavefronts
  if (is_fpu_kind(op.kind)) {
    if (op.M * op.N < gk::kWaveSize)
      return fail(GK_ERR_OP_SHAPE, "The operator shape is too small. The dimensions of the operator shape must adhere to the following constraint: OPERATOR_M * OPERATOR_N >= 64.");
    if (op.mb * op.nb != gk::kWaveSize)
      return fail(GK_ERR_OP_SHAPE, "The base FPU operator shape should adhere to the following constraint: OPERATOR_M_BASE * OPERATOR_N_BASE = 64.");
    if (op.kb != 1)
      return fail(GK_ERR_OP_SHAPE, "The base FPU operator shape should adhere to the following constraint: OPERATOR_K_BASE = 1.");
    if (op.M % op.mb != 0 || op.N % op.nb != 0 || op.K % op.kb != 0)
      return fail(GK_ERR_OP_SHAPE, "The operator shape should adhere to the following constraint: OPERATOR_M, OPERATOR_N, OPERATOR_K are multiples of OPERATOR_M_BASE, OPERATOR_N_BASE, OPERATOR_K_BASE, respectively.");
    // The base shape says how the lanes of a wave are laid over a block of outputs; the operator shape, how many
    // outputs a lane owns.  Neither changes a result (every output is one fma chain in ascending k).  The
    // vector-ALU kernels own their outputs in chunks of up to 4 whatever the operator shape says.  The square 8 x 8
    // lane grid is compiled for every tile, element type and layout; the other grids of the reference's sweep
    // (configs/configs.jl:545-550, doubled for 64 lanes: 1 x 64, 2 x 32, 4 x 16, 16 x 4, 32 x 2, 64 x 1) for Float32 on
    // aligned layouts and the 128 x 128 x 16 tile, whose 64 x 64 wave tiles every grid divides.  Anything else is
    // refused rather than silently run on another grid.
    if (op.mb != 8 || op.nb != 8) {
      if ((op.mb & (op.mb - 1)) != 0)
        return fail(GK_ERR_OP_SHAPE, "OPERATOR_M_BASE must be a power of two, got %d.", op.mb);
      const bool f32 = c->global_a_layout.eltype == GK_F32 && c->global_b_layout.eltype == GK_F32 && c->global_d_layout.eltype == GK_F32;
      auto aligned = [](int k) { return k == GK_LAYOUT_ALIGNED_COL_MAJOR || k == GK_LAYOUT_ALIGNED_ROW_MAJOR; };
      const bool lay = aligned(c->global_a_layout.kind) && aligned(c->global_b_layout.kind) && c->global_d_layout.kind == GK_LAYOUT_ALIGNED_COL_MAJOR &&
                       (c->global_c_layout.kind == GK_LAYOUT_ALIGNED_COL_MAJOR || c->global_c_layout.kind == GK_LAYOUT_ZERO);
      if (op.kind != GK_OP_FPU || !f32 || !lay || b.M != 128 || b.N != 128 || b.K != 16 || c->compute_warp.M != 64 || c->compute_warp.N != 64)
        return fail(GK_ERR_OP_SHAPE, "The base shape OPERATOR_M_BASE x OPERATOR_N_BASE = %d x %d (a wave as a %d x %d grid of lanes) is compiled for FPUOp on Float32 "
                                     "with aligned layouts, block shape 128 x 128 x 16 and 64 x 64 wave tiles; every other configuration runs 8 x 8.",
                    op.mb, op.nb, op.mb, op.nb);
    }
  } else if (is_mfma_kind(op.kind)) {
    const bool native = (op.M == 32 && op.N == 32 && op.K == 16);
    const bool wmma_compat = (op.K == 16) && ((op.M == 16 && op.N == 16) || (op.M == 8 && op.N == 32) || (op.M == 32 && op.N == 8));
    if (!native && !wmma_compat) return fail(GK_ERR_OP_SHAPE, "Unsupported MFMA Operator shape (M = %d, N = %d, K = %d)!", op.M, op.N, op.K);
  } else {
    return fail(GK_ERR_INVALID_ARGUMENT, "unknown operator kind %d", op.kind);
  }
  if (c->warps_per_block <= 0) return fail(GK_ERR_INVALID_ARGUMENT, "warps_per_block must be positive");
  // src/config.jl:263-265
  const long long w = c->warps_per_block;
  if ((long long)c->mem_a_warp.M * c->mem_a_warp.K * w > (long long)b.M * b.K)
    return fail(GK_ERR_MEM_TILE, "mem_a_warp is too big for the selected block shape: need at least one iteration in the memory copy loop!");
  if ((long long)c->mem_b_warp.K * c->mem_b_warp.N * w > (long long)b.K * b.N)
    return fail(GK_ERR_MEM_TILE, "mem_b_warp is too big for the selected block shape: need at least one iteration in the memory copy loop!");
  if ((long long)c->mem_cd_warp.M * c->mem_cd_warp.N * w > (long long)b.M * b.N)
    return fail(GK_ERR_MEM_TILE, "mem_cd_warp is too big for the selected block shape: need at least one iteration in the memory copy loop!");
  // src/config.jl:268-275
  const gk_shape& cw = c->compute_warp;
  const gk_shape& os = c->compute_op_shape;
  if (cw.M <= 0 || cw.N <= 0 || cw.K <= 0 || os.M <= 0 || os.N <= 0 || os.K <= 0) return fail(GK_ERR_INVALID_ARGUMENT, "compute_warp and compute_op_shape must be positive");
  if (b.M % cw.M || b.N % cw.N || b.K % cw.K) return fail(GK_ERR_TILE_MULTIPLE, "block_shape must be a multiple of compute_warp!");
  if (cw.M % os.M || cw.N % os.N || cw.K % os.K) return fail(GK_ERR_TILE_MULTIPLE, "compute_warp must be a multiple of op_shape!");
  if (require_tile_sized_global(c->global_a_layout.kind) && (g.M % b.M || g.K % b.K))
    return fail(GK_ERR_TILE_MULTIPLE, "gemm_shape.MK must be a multiple of block_shape.MK!");
  if (require_tile_sized_global(c->global_b_layout.kind) && (g.K % b.K || g.N % b.N))
    return fail(GK_ERR_TILE_MULTIPLE, "gemm_shape.KN must be a multiple of block_shape.KN!");
  if (require_tile_sized_global(c->global_c_layout.kind) && (g.M % b.M || g.N % b.N))
    return fail(GK_ERR_TILE_MULTIPLE, "gemm_shape.MN must be a multiple of block_shape.MN!");
  if (require_tile_sized_global(c->global_d_layout.kind) && (g.M % b.M || g.N % b.N))
    return fail(GK_ERR_TILE_MULTIPLE, "gemm_shape.MN must be a multiple of block_shape.MN!");

  if (c->global_a_layout.kind == GK_LAYOUT_GETT || c->global_b_layout.kind == GK_LAYOUT_GETT ||
      c->global_c_layout.kind == GK_LAYOUT_GETT || c->global_d_layout.kind == GK_LAYOUT_GETT) {
    int rc_g = validate_gett(c);
    if (rc_g != GK_OK) return rc_g;
  }

  if (op.kind == GK_OP_MFMA_COMPLEX || op.kind == GK_OP_MFMA_DUAL) {
    auto inter = [](int k) { return k == GK_LAYOUT_INTERLEAVED_COL_MAJOR || k == GK_LAYOUT_INTERLEAVED_ROW_MAJOR; };
    const bool all_inter = inter(c->global_a_layout.kind) && inter(c->global_b_layout.kind) &&
                           c->global_d_layout.kind == GK_LAYOUT_INTERLEAVED_COL_MAJOR &&
                           (c->global_c_layout.kind == GK_LAYOUT_INTERLEAVED_COL_MAJOR || c->global_c_layout.kind == GK_LAYOUT_ZERO);
    // planar global matrices (re plane, then im plane) are an addition for the complex operator
    const bool all_split = op.kind == GK_OP_MFMA_COMPLEX && is_split_layout(c->global_a_layout.kind) &&
                           is_split_layout(c->global_b_layout.kind) && c->global_d_layout.kind == GK_LAYOUT_SPLIT_COL_MAJOR &&
                           (c->global_c_layout.kind == GK_LAYOUT_SPLIT_COL_MAJOR || c->global_c_layout.kind == GK_LAYOUT_ZERO);
    if (!all_inter && !all_split)
      return fail(GK_ERR_UNSUPPORTED, "complex and dual operators need Interleaved layouts for A and B and InterleavedColMajor for C and D "
                                      "(the complex operator also takes Split layouts for all of them)");
    // Hooks see complex numbers (src/kernel.jl:167-187, 337-347 hand tiles of the layout's element type to the
    // transform).  The hooks of C and D take the ops whose result on a complex number is the op on its two parts,
    // x * p0 and -x, and x + p0, which acts on the real part; max / abs / clamp have no complex counterpart of the
    // same type.  A bias value is real and goes to the real part.
    if (t) {
      // (on A and B: what folds into the accumulators -- one scale by +-2^e, |e| <= 4, or one negation per operand: a real
      // factor acts on both parts of a number and commutes with the product; see fold_pow2_scales)
      gk_transforms folded_storage;
      float post = 1.0f;
      const gk_transforms* rest = fold_pow2_scales(c, t, &folded_storage, &post);
      const int ab_hooks[4] = {GK_HOOK_GLOBAL_TO_SHARED_A, GK_HOOK_SHARED_TO_REGS_A, GK_HOOK_GLOBAL_TO_SHARED_B, GK_HOOK_SHARED_TO_REGS_B};
      for (int h : ab_hooks)
        for (int i = 0; i < rest->hook[h].n_ops && i < GK_MAX_OPS; ++i)
          if (rest->hook[h].ops[i].kind != GK_T_IDENTITY)
            return fail(GK_ERR_UNSUPPORTED, "the complex and dual operators take transforms on C and D, and on A and B one scale by a power of two "
                                            "between 1/16 and 16 or one negation each (anything else would have to run inside their K loop)");
      for (int h = 0; h < 8; ++h)
        for (int i = 0; i < t->hook[h].n_ops && i < GK_MAX_OPS; ++i) {
          const int k = t->hook[h].ops[i].kind;
          if (k != GK_T_IDENTITY && k != GK_T_SCALE && k != GK_T_ADD && k != GK_T_NEG)
            return fail(GK_ERR_UNSUPPORTED, "transform op %d is not defined on complex numbers (scale, add and neg are)", k);
        }
    }
  }
  if (c->global_a_layout.kind == GK_LAYOUT_DIAGONAL) {
    if (g.M != g.K) return fail(GK_ERR_DIMENSION_MISMATCH, "Diagonal only supports a square A matrix (M == K)");
    const int bkind = c->global_b_layout.kind;
    if ((bkind != GK_LAYOUT_ALIGNED_COL_MAJOR && bkind != GK_LAYOUT_ALIGNED_ROW_MAJOR) ||
        c->global_d_layout.kind != GK_LAYOUT_ALIGNED_COL_MAJOR ||
        (c->global_c_layout.kind != GK_LAYOUT_ALIGNED_COL_MAJOR && c->global_c_layout.kind != GK_LAYOUT_ZERO))
      return fail(GK_ERR_UNSUPPORTED, "a diagonal A needs aligned layouts for B, C and D");
    if (t) {
      // off-diagonal zeros of A are never materialised: the A hooks must map 0 to 0
      const int hooks[2] = {GK_HOOK_GLOBAL_TO_SHARED_A, GK_HOOK_SHARED_TO_REGS_A};
      for (int h : hooks)
        for (int i = 0; i < t->hook[h].n_ops && i < GK_MAX_OPS; ++i) {
          const gk_op& o = t->hook[h].ops[i];
          if (o.kind == GK_T_ADD && o.p0 != 0.0f) return fail(GK_ERR_UNSUPPORTED, "a transform of a diagonal A must keep zero at zero");
          if (o.kind == GK_T_CLAMP && (o.p0 > 0.0f || o.p1 < 0.0f)) return fail(GK_ERR_UNSUPPORTED, "a transform of a diagonal A must keep zero at zero");
        }
    }
  }

  // element types of C and D: fp32 everywhere; the real MFMA kernels also read and write 16-bit
  // matrices (fp32 accumulation, one rounding at the store; the reference's F16 -> F16 WMMA
  // configuration, configs/configs.jl:574)
  if (is_fpu_kind(op.kind)) {
    // the vector-ALU kernels accumulate in the element type of C and D; the pairs (A and B, C and D)
    // are those the reference runs FPUOp with (configs/configs.jl:489-497)
    const int ab = c->global_a_layout.eltype, cd = c->global_d_layout.eltype;
    if (c->global_b_layout.eltype != ab) return fail(GK_ERR_UNSUPPORTED, "A and B must have the same element type");
    const bool pair_ok = (ab == GK_F16 && cd == GK_F32) || (ab == GK_F32 && (cd == GK_F32 || cd == GK_F64)) ||
                         (ab == GK_F64 && cd == GK_F64) || (ab == GK_I16 && cd == GK_I16) || (ab == GK_I32 && cd == GK_I32) ||
                         (ab == GK_I64 && cd == GK_I64);
    if (!pair_ok) return fail(GK_ERR_UNSUPPORTED, "element types %d (A, B) and %d (D) are not a pair the vector-ALU operator is compiled for", ab, cd);
    if (c->global_c_layout.kind != GK_LAYOUT_ZERO && c->global_c_layout.eltype != cd)
      return fail(GK_ERR_UNSUPPORTED, "C and D must have the same element type");
    if (op.kind == GK_OP_FPU_TROPICAL && cd != GK_F32) return fail(GK_ERR_UNSUPPORTED, "the max-plus operator is compiled for fp32");
    if (e && e->kind != GK_EPILOGUE_DEFAULT && cd != GK_F32) return fail(GK_ERR_UNSUPPORTED, "the bias epilogue is fp32 (src/epilogue.jl:44-52)");
  } else {
    const bool cd16_ok = c->global_a_layout.kind != GK_LAYOUT_DIAGONAL;
    auto cd_ok = [&](int dt) { return dt == GK_F32 || (cd16_ok && (dt == GK_F16 || dt == GK_BF16)); };
    if (!cd_ok(c->global_d_layout.eltype))
      return fail(GK_ERR_UNSUPPORTED, "element type %d of D is not available with this operator", c->global_d_layout.eltype);
    if (c->global_c_layout.kind != GK_LAYOUT_ZERO && !cd_ok(c->global_c_layout.eltype))
      return fail(GK_ERR_UNSUPPORTED, "element type %d of C is not available with this operator", c->global_c_layout.eltype);
  }

  // src/matmul.jl:34-36 (decidable from the configuration alone, so it is checked before the
  // instance lookup)
  if (kernel != GK_KERNEL_SINGLESTAGE && b.K < 2 * os.K)
    return fail(GK_ERR_STAGES, "Need at least two stages to use a pipelined kernel, i.e. BLOCK_K >= 2 * OPERATOR_K");

  // the instance that would run; its LDS request is what Kernel.shmem_size returns
  int rc = GK_OK;
  if (custom) {      // a kernel specialised at run time: its resources are known to the caller
    rc = make_key_as_configured(c, t, e, key, allow_ragged_fast);     // (compiled for exactly this configuration)
    *info = *custom;
  } else {
    rc = find_instance(c, t, e, key, info, allow_ragged_fast);
  }
  if (rc != GK_OK) return rc;

  long long lds_max = 0;
  int threads_max = 0;
  device_limits(&lds_max, &threads_max);
  // src/matmul.jl:28-31
  if (info->lds_bytes > lds_max)
    return fail(GK_ERR_LDS, "Requested too much shared memory: The current GPU can use at most %lld bytes, while this configuration required %d bytes",
                lds_max, info->lds_bytes);
  // src/matmul.jl:41
  const long long threads = (long long)c->warps_per_block * gk::kWaveSize;
  if (threads > threads_max)
    return fail(GK_ERR_THREADS, "Requested too many threads for this kernel: This kernel can be launched using at most %d threads, while this configuration required %lld",
                threads_max, threads);
  // (the instance that runs may be the eight-wave arrangement of a four-wave configuration, see make_key)
  const long long configured_waves = (long long)(c->block_shape.M / c->compute_warp.M) * (c->block_shape.N / c->compute_warp.N);
  const bool other_arrangement = key->waves_m * key->waves_n != configured_waves;
  if (other_arrangement && info->threads > threads_max)
    return fail(GK_ERR_THREADS, "Requested too many threads for this kernel: This kernel can be launched using at most %d threads, while this configuration required %d",
                threads_max, info->threads);
  if (!other_arrangement && threads != info->threads)
    return fail(GK_ERR_UNSUPPORTED, "warps_per_block = %d does not match the %d waves of block_shape / compute_warp", c->warps_per_block,
                info->threads / gk::kWaveSize);
  if (other_arrangement && c->warps_per_block != configured_waves)
    return fail(GK_ERR_UNSUPPORTED, "warps_per_block = %d does not match the %lld waves of block_shape / compute_warp", c->warps_per_block, configured_waves);
  return GK_OK;
}

}  // namespace

extern "C" {

int gk_version(void) { return GK_VERSION; }

size_t gk_last_error(char* buf, size_t n) {
  if (buf && n > 0) {
    size_t m = g_last_error.size() < n - 1 ? g_last_error.size() : n - 1;
    memcpy(buf, g_last_error.data(), m);
    buf[m] = 0;
  }
  return g_last_error.size();
}

const char* gk_status_string(int status) {
  switch (status) {
    case GK_OK: return "GK_OK";
    case GK_ERR_INVALID_ARGUMENT: return "GK_ERR_INVALID_ARGUMENT";
    case GK_ERR_LDS: return "GK_ERR_LDS";
    case GK_ERR_STAGES: return "GK_ERR_STAGES";
    case GK_ERR_THREADS: return "GK_ERR_THREADS";
    case GK_ERR_BLOCK_SHAPE: return "GK_ERR_BLOCK_SHAPE";
    case GK_ERR_OP_SHAPE: return "GK_ERR_OP_SHAPE";
    case GK_ERR_MEM_TILE: return "GK_ERR_MEM_TILE";
    case GK_ERR_TILE_MULTIPLE: return "GK_ERR_TILE_MULTIPLE";
    case GK_ERR_ALIGNMENT: return "GK_ERR_ALIGNMENT";
    case GK_ERR_UNSUPPORTED: return "GK_ERR_UNSUPPORTED";
    case GK_ERR_DIMENSION_MISMATCH: return "GK_ERR_DIMENSION_MISMATCH";
    case GK_ERR_HIP: return "GK_ERR_HIP";
    default: return "GK_ERR_UNKNOWN";
  }
}

int gk_set_device_limits(int64_t lds_bytes, int32_t max_threads) {
  g_lds_override.store(lds_bytes > 0 ? lds_bytes : 0);
  g_threads_override.store(max_threads > 0 ? max_threads : 0);
  return GK_OK;
}

int gk_validate(const gk_config* conf, int32_t kernel) {
  gk::InstanceKey key;
  gk::InstanceInfo info;
  return validate_config(conf, kernel, nullptr, nullptr, &key, &info);
}

int gk_number_of_blocks(const gk_config* conf, int32_t* blocks_x, int32_t* blocks_y) {
  if (!conf || !blocks_x || !blocks_y) return fail(GK_ERR_INVALID_ARGUMENT, "NULL argument");
  if (conf->block_shape.M <= 0 || conf->block_shape.N <= 0) return fail(GK_ERR_BLOCK_SHAPE, "block_shape must be positive");
  int gx = 0, gy = 0;
  gk::number_of_blocks(conf->cta_swizzle.kind, conf->cta_swizzle.param, conf->matmul_shape.M, conf->matmul_shape.N,
                       conf->block_shape.M, conf->block_shape.N, gx, gy);
  *blocks_x = gx;
  *blocks_y = gy;
  return GK_OK;
}

int gk_cta_swizzle(const gk_config* conf, int32_t block_x, int32_t block_y, int32_t* block_i, int32_t* block_j) {
  if (!conf || !block_i || !block_j) return fail(GK_ERR_INVALID_ARGUMENT, "NULL argument");
  const int nbm = (conf->matmul_shape.M + conf->block_shape.M - 1) / conf->block_shape.M;
  const int nbn = (conf->matmul_shape.N + conf->block_shape.N - 1) / conf->block_shape.N;
  int ti = 0, tj = 0;
  gk::cta_swizzle(conf->cta_swizzle.kind, conf->cta_swizzle.param, block_x, block_y, nbm, nbn, ti, tj);
  *block_i = ti * conf->block_shape.M;
  *block_j = tj * conf->block_shape.N;
  return GK_OK;
}

int64_t gk_shmem_size(const gk_config* conf, int32_t kernel) {
  (void)kernel;
  if (!conf) { fail(GK_ERR_INVALID_ARGUMENT, "config is NULL"); return -1; }
  gk::InstanceKey key;
  gk::InstanceInfo info;
  if (find_instance(conf, nullptr, nullptr, &key, &info) != GK_OK) return -1;
  return info.lds_bytes;
}

int32_t gk_threads_per_block(const gk_config* conf) {
  if (!conf) return -1;
  return conf->warps_per_block * gk::kWaveSize;
}

int gk_kernel_name(const gk_config* conf, const gk_transforms* transforms, const gk_epilogue* epilogue, int32_t kernel,
                   char* buf, size_t n) {
  if (!conf || !buf || n == 0) return fail(GK_ERR_INVALID_ARGUMENT, "NULL argument");
  gk::InstanceKey key;
  gk::InstanceInfo info;
  int rc = validate_config(conf, kernel, transforms, epilogue, &key, &info);      // a name only for a launch that would pass
  if (rc != GK_OK) return rc;
  snprintf(buf, n, "%s", info.name);
  return GK_OK;
}

}  // extern "C"

namespace {
// bytes of a rows x cols tile in a shared layout: Layout.physical_size (src/layout.jl:76, 113, 152,
// 194, 246, 342-345, 381-383): padding goes to the leading physical dimension, planar complex
// layouts hold two planes, interleaved ones two reals per element
long long shared_tile_bytes(const gk_layout* l, long long rows, long long cols) {
  const bool row = is_row_major(l->kind) || l->kind == GK_LAYOUT_SPLIT_ROW_MAJOR;
  long long lead = row ? cols : rows, other = row ? rows : cols;
  long long n = (lead + l->pad) * other;
  if (l->kind == GK_LAYOUT_SPLIT_COL_MAJOR || l->kind == GK_LAYOUT_SPLIT_ROW_MAJOR ||
      l->kind == GK_LAYOUT_INTERLEAVED_COL_MAJOR || l->kind == GK_LAYOUT_INTERLEAVED_ROW_MAJOR)
    n *= 2;
  return n * dtype_size(l->eltype);
}
}  // namespace

extern "C" {

int64_t gk_reference_shmem_size(const gk_config* conf) {
  if (!conf) { fail(GK_ERR_INVALID_ARGUMENT, "config is NULL"); return -1; }
  const gk_layout* ls[4] = {&conf->shared_a_layout, &conf->shared_b_layout, &conf->shared_c_layout, &conf->shared_d_layout};
  for (const gk_layout* l : ls)
    if (!valid_layout_kind(l->kind) || dtype_size(l->eltype) == 0) { fail(GK_ERR_INVALID_ARGUMENT, "unknown layout kind or element type"); return -1; }
  const gk_shape& b = conf->block_shape;
  const long long size_a = shared_tile_bytes(ls[0], b.M, b.K), size_b = shared_tile_bytes(ls[1], b.K, b.N);
  const long long size_c = shared_tile_bytes(ls[2], b.M, b.N), size_d = shared_tile_bytes(ls[3], b.M, b.N);
  return std::max(size_c, std::max(size_a + size_b, size_d));
}

int gk_heuristic_block_shape(const gk_layout* sa, const gk_layout* sb, const gk_layout* sc, const gk_layout* sd, gk_shape* out) {
  if (!sa || !sb || !sc || !sd || !out) return fail(GK_ERR_INVALID_ARGUMENT, "NULL argument");
  const gk_layout* ls[4] = {sa, sb, sc, sd};
  for (const gk_layout* l : ls)
    if (!valid_layout_kind(l->kind) || dtype_size(l->eltype) == 0) return fail(GK_ERR_INVALID_ARGUMENT, "unknown layout kind or element type");
  auto nbytes = shared_tile_bytes;
  const long long limit = 64 * 1024;
  long long M = 1, N = 1, K = 1;
  for (;;) {     // src/config.jl:104-110
    const long long m2 = (M == N) ? 2 * M : M, n2 = (M == N) ? N : 2 * N;
    const long long cd = std::max(nbytes(sc, m2, n2), nbytes(sd, m2, n2));
    if (cd > limit) break;
    M = m2; N = n2;
  }
  while (nbytes(sa, M, 2 * K) + nbytes(sb, 2 * K, N) <= limit) K *= 2;   // src/config.jl:112-117
  out->M = (int32_t)M; out->N = (int32_t)N; out->K = (int32_t)K;
  return GK_OK;
}

}  // extern "C"

namespace gk_internal {

// Everything gk_matmul does before the launch: configuration checks, operand checks, kernel
// arguments and grid.  `custom` replaces the lookup of a compiled instance (run-time compiled kernels).
int prepare_launch(const gk_config* conf, const void* a, const void* b, const void* c, void* d, const gk_transforms* transforms,
                   const gk_epilogue* epilogue, int32_t kernel, const gk::InstanceInfo* custom, Launch* out) {
  gk::InstanceKey& key = out->key;
  gk::InstanceInfo& info = out->info;
  int rc = validate_config(conf, kernel, transforms, epilogue, &key, &info, custom);
  if (rc != GK_OK) return rc;
  out->ragged = false;
  if (key.family == gk::FAMILY_MFMA && ragged_fast_path(conf)) {
    if ((((uintptr_t)a | (uintptr_t)b) & 1u) != 0) return fail(GK_ERR_ALIGNMENT, "A and B must be aligned to their 2-byte elements");
    out->ragged = needs_tail_tile(conf);
  }

  const bool a_zero = conf->global_a_layout.kind == GK_LAYOUT_ZERO, b_zero = conf->global_b_layout.kind == GK_LAYOUT_ZERO;
  if ((!a_zero && !a) || (!b_zero && !b) || !d) return fail(GK_ERR_INVALID_ARGUMENT, "a, b and d must not be NULL");
  if (conf->global_c_layout.kind != GK_LAYOUT_ZERO && !c) return fail(GK_ERR_INVALID_ARGUMENT, "c must not be NULL unless its layout is Zero");
  if (epilogue && epilogue->kind != GK_EPILOGUE_DEFAULT && !epilogue->bias) return fail(GK_ERR_INVALID_ARGUMENT, "bias epilogue without a bias pointer");

  gk::GemmArgs& args = out->args;
  make_args(conf, a, b, c, d, transforms, epilogue, &args);
  const bool solo_edges = key.family == gk::FAMILY_MFMA && key.fused == 0 && (args.M % 256 != 0 || args.N % 256 != 0 || args.K % 64 != 0);
  // (16-byte accesses to an FP32 C / D: at 16-byte boundaries for a contraction, at those of an element for a product with tiles over its edges)
  const bool cd_fit = solo_edges ? ((((uintptr_t)args.d) | (args.c_mode != 0 ? (uintptr_t)args.c : 0)) & 3u) == 0 : gk::solo_cd_path(args) != 0;
  if (!custom && (key.family == gk::FAMILY_GETT || solo_edges) && key.BM == 256 && key.BN == 256 && key.BK == 64 && key.waves_m == 2 && key.waves_n == 2 &&
      !cd_fit) {
    // a contraction on the four-wave arrangement, and a product with tiles over its edges, move C and D 16 bytes at a
    // time: pointers that do not allow it run the eight-wave arrangement (see make_key)
    key.waves_n = 4;
    gk::FamilyFn fn8 = family_fn(key);
    hipError_t e8 = hipSuccess;
    if (!fn8 || !fn8(key, args, dim3(1), nullptr, 0, &info, &e8)) return fail(GK_ERR_UNSUPPORTED, "no compiled kernel instance for this %s", solo_edges ? "product" : "contraction");
  }

  if (!custom && key.family == gk::FAMILY_MFMA && wide_tile(key) && key.waves_m == 2 && key.waves_n == 2 && gk::solo_cd_path(args) == 0) {
    // the four waves of a tile with a side of 192 move an FP32 C / D 16 bytes at a time as well
    wide_tile_on_eight_waves(&key);
    gk::FamilyFn fn8 = family_fn(key);
    hipError_t e8 = hipSuccess;
    if (!fn8 || !fn8(key, args, dim3(1), nullptr, 0, &info, &e8)) return fail(GK_ERR_UNSUPPORTED, "no compiled kernel instance for this product");
  }

  // aligned layouts move 16-byte vectors (reference src/layout.jl:22-34 traps on the device; here it is a host check)
  auto check_aligned = [&](const gk_layout& l, const void* p, long long ld, const char* what) -> int {
    const bool interleaved = l.kind == GK_LAYOUT_INTERLEAVED_COL_MAJOR || l.kind == GK_LAYOUT_INTERLEAVED_ROW_MAJOR;
    if (l.kind != GK_LAYOUT_ALIGNED_COL_MAJOR && l.kind != GK_LAYOUT_ALIGNED_ROW_MAJOR && !interleaved && !is_split_layout(l.kind)) return GK_OK;
    const int es = dtype_size(l.eltype);   // ld already counts real elements for interleaved data
    if (es == 0) return fail(GK_ERR_INVALID_ARGUMENT, "unknown element type of %s", what);
    if (((uintptr_t)p & 15u) != 0) return fail(GK_ERR_ALIGNMENT, "%s is not aligned to 16 bytes", what);
    if ((ld * es) % 16 != 0) return fail(GK_ERR_ALIGNMENT, "leading dimension of %s (%lld elements) is not a multiple of 16 bytes", what, ld);
    return GK_OK;
  };
  if ((rc = check_aligned(conf->global_a_layout, a, args.lda, "A")) != GK_OK) return rc;
  if ((rc = check_aligned(conf->global_b_layout, b, args.ldb, "B")) != GK_OK) return rc;
  if ((rc = check_aligned(conf->global_c_layout, c, args.ldc, "C")) != GK_OK) return rc;
  if ((rc = check_aligned(conf->global_d_layout, d, args.ldd, "D")) != GK_OK) return rc;

  if (key.family == gk::FAMILY_DIAGONAL && (((uintptr_t)a & 15u) != 0))
    return fail(GK_ERR_ALIGNMENT, "the diagonal of A must be aligned to 16 bytes");
  if (key.family == gk::FAMILY_GETT && ((((uintptr_t)a | (uintptr_t)b) & 15u) != 0))
    return fail(GK_ERR_ALIGNMENT, "tensor operands must be aligned to 16 bytes");

  // leading dimensions must cover the operand
  {
    const bool a_row = is_row_major(conf->global_a_layout.kind), b_row = is_row_major(conf->global_b_layout.kind);
    // extents in the unit the leading dimensions count: real elements (two per complex number of an
    // interleaved matrix, one per complex number of a plane)
    const bool planar = is_split_layout(conf->global_a_layout.kind);
    const bool cplx = conf->op.kind == GK_OP_MFMA_COMPLEX || conf->op.kind == GK_OP_MFMA_DUAL;
    const long long em = planar ? conf->matmul_shape.M : args.M, en = planar ? conf->matmul_shape.N : args.N;
    const long long ek = (cplx && !planar) ? 2ll * conf->matmul_shape.K : conf->matmul_shape.K;
    if (!a_zero && conf->global_a_layout.kind != GK_LAYOUT_DIAGONAL && conf->global_a_layout.kind != GK_LAYOUT_GETT &&
        args.lda < (a_row ? ek : em))
      return fail(GK_ERR_DIMENSION_MISMATCH, "lda = %lld is smaller than the leading extent of A", args.lda);
    if (!b_zero && conf->global_b_layout.kind != GK_LAYOUT_GETT && args.ldb < (b_row ? en : ek))
      return fail(GK_ERR_DIMENSION_MISMATCH, "ldb = %lld is smaller than the leading extent of B", args.ldb);
    if (conf->global_d_layout.kind != GK_LAYOUT_GETT && (args.ldd < em || (args.c_mode && args.ldc < em)))
      return fail(GK_ERR_DIMENSION_MISMATCH, "ldc/ldd is smaller than M");
    // the kernels keep per-lane tile offsets in 32 bits
    const long long span_a = (long long)(a_row ? conf->block_shape.M : conf->block_shape.K) * args.lda * 2;
    const long long span_b = (long long)(b_row ? conf->block_shape.K : conf->block_shape.N) * args.ldb * 2;
    if (span_a + 2 * args.plane_a >= (1ll << 31) || span_b >= (1ll << 31))
      return fail(GK_ERR_UNSUPPORTED, "leading dimension too large for 32-bit tile offsets");
  }

  int gx = 0, gy = 0;
  gk::number_of_blocks(args.swz_kind, args.swz_param, conf->matmul_shape.M, conf->matmul_shape.N, conf->block_shape.M,
                       conf->block_shape.N, gx, gy);
  if (gx <= 0 || gy <= 0) return fail(GK_ERR_INVALID_ARGUMENT, "empty grid");

  out->gx = gx;
  out->gy = gy;
  return GK_OK;
}

}  // namespace gk_internal

extern "C" {

int gk_matmul(const gk_config* conf, const void* a, const void* b, const void* c, void* d, const gk_transforms* transforms,
              const gk_epilogue* epilogue, int32_t kernel, void* stream) {
  gk_internal::Launch L;
  int rc = gk_internal::prepare_launch(conf, a, b, c, d, transforms, epilogue, kernel, nullptr, &L);
  if (rc != GK_OK) return rc;
  gk::FamilyFn fn = family_fn(L.key);
  hipError_t err = hipSuccess;
  if (kernel == GK_KERNEL_SPLIT_K)
    return fail(GK_ERR_INVALID_ARGUMENT, "the K-split kernel needs a workspace for the partial tiles of its slices: call gk_matmul_split_k");
  if (!fn || !fn(L.key, L.args, dim3((unsigned)L.gx, (unsigned)L.gy), (hipStream_t)stream, 1, &L.info, &err))
    return fail(GK_ERR_UNSUPPORTED, "no compiled kernel instance");
  if (err != hipSuccess) return fail(GK_ERR_HIP, "HIP launch of %s failed: %s", L.info.name, hipGetErrorString(err));
  return GK_OK;
}

}  // extern "C"

namespace {

// The arrival counters of a K-split launch take a region of fixed size at the head of the workspace, whatever the
// product: a launch is split only when its tiles leave CUs idle (split_k_slices gives one slice from 2 * kNumCUs tiles
// on), so kSplitCounterBytes / 4 counters are enough for every launch that uses them.  With a region whose size followed
// the tile count, a workspace reused by a product with more tiles would have found the float bits of old partial sums
// where its counters are.
constexpr size_t kSplitCounterBytes = 2048;
static_assert(kSplitCounterBytes / sizeof(unsigned) >= 2 * (size_t)gk::kNumCUs - 1, "one counter for every tile of a launch that is split");

// K slices of a K-split launch, from a sweep of slice counts on 4096 x 64 x 4096, 256 x 256 x 16384 and
// 8192 x 128 x 8192: about two workgroups per CU, and slices at least 1024 deep in K -- a slice pays for its
// prologue, for the trip of its partial tile to memory and for the arrival counter (about 3 us on the last
// workgroup's path), which shorter slices do not earn back (4096 x 64 x 4096: 4 slices 12.4 us, 8 slices 14.1 us,
// 16 slices 19.4 us).
int split_k_slices(int tiles, int k_tiles, int block_k) {
  int slices = (2 * gk::kNumCUs + tiles - 1) / tiles;
  const int min_tiles = (1024 + block_k - 1) / block_k;
  if (slices > k_tiles / min_tiles) slices = k_tiles / min_tiles;
  return slices < 1 ? 1 : slices;
}

}  // namespace

namespace gk_internal {

// Launches a K-split product whose partial tiles meet in [counters | partial tiles] at `workspace`
// (`whose` names the workspace in the message that refuses a launch it cannot hold).
int launch_split_k(const gk_config* conf, const void* a, const void* b, const void* c, void* d, const gk_transforms* transforms,
                   const gk_epilogue* epilogue, void* workspace, size_t workspace_bytes, const char* whose, void* stream) {
  gk_internal::Launch L;
  int rc = gk_internal::prepare_launch(conf, a, b, c, d, transforms, epilogue, GK_KERNEL_SPLIT_K, nullptr, &L);
  if (rc != GK_OK) return rc;
  if (L.key.family != gk::FAMILY_MFMA && L.key.family != gk::FAMILY_MFMA_CHECKED)
    return fail(GK_ERR_UNSUPPORTED, "the K-split kernel runs the real MFMA operator");
  gk::FamilyFn fn = family_fn(L.key);
  hipError_t err = hipSuccess;
  const int tiles = L.gx * L.gy;
  const int kt = (conf->matmul_shape.K + conf->block_shape.K - 1) / conf->block_shape.K;   // bounds-checked layouts: the last tile may be partial
  int slices = split_k_slices(tiles, kt, conf->block_shape.K);
  gk::InstanceInfo sk_info;
  // K-split instances exist for the small tiles that skinny products run; anything else (a large tile,
  // generic A / B hooks, a partial last K tile on the aligned kernel) runs unsplit.  The bounds-checked
  // kernel takes its K range from the launch arguments, the aligned kernels have instances of their own.
  gk::FamilyFn sk_fn = L.key.family == gk::FAMILY_MFMA_CHECKED ? fn : gk::family_mfma_splitk;
  if (slices > 1 && !L.ragged && sk_fn && sk_fn(L.key, L.args, dim3(1), nullptr, 0, &sk_info, &err)) {
    const int per = (kt + slices - 1) / slices;
    slices = (kt + per - 1) / per;           // no empty slice: every slice arrives at its tile's counter
    const size_t counters = kSplitCounterBytes;
    if ((size_t)tiles * sizeof(unsigned) > counters)
      return fail(GK_ERR_INVALID_ARGUMENT, "a K-split launch of %d tiles has no room for its arrival counters (%zu bytes)", tiles, counters);
    const size_t need = counters + (size_t)tiles * slices * conf->block_shape.M * conf->block_shape.N * sizeof(float);
    if (!workspace || workspace_bytes < need)
      return fail(GK_ERR_INVALID_ARGUMENT, "the K-split launch needs a workspace of %zu bytes (%d tiles x %d slices of %d x %d floats); %s holds %zu",
                  need, tiles, slices, conf->block_shape.M, conf->block_shape.N, whose, workspace_bytes);
    if (((uintptr_t)workspace & 15u) != 0) return fail(GK_ERR_ALIGNMENT, "the workspace is not aligned to 16 bytes");
    gk::GemmArgs sk = L.args;
    sk.k_steps = per; sk.k_slices = slices;
    sk.ws_counters = (unsigned*)workspace;
    sk.ws_partials = (char*)workspace + counters;
    sk_fn(L.key, sk, dim3((unsigned)L.gx, (unsigned)L.gy, (unsigned)slices), (hipStream_t)stream, 1, &sk_info, &err);
    if (err != hipSuccess) return fail(GK_ERR_HIP, "HIP launch of %s failed: %s", sk_info.name, hipGetErrorString(err));
    return GK_OK;
  }
  if (!fn || !fn(L.key, L.args, dim3((unsigned)L.gx, (unsigned)L.gy), (hipStream_t)stream, 1, &L.info, &err))
    return fail(GK_ERR_UNSUPPORTED, "no compiled kernel instance");
  if (err != hipSuccess) return fail(GK_ERR_HIP, "HIP launch of %s failed: %s", L.info.name, hipGetErrorString(err));
  return GK_OK;
}

}  // namespace gk_internal

extern "C" {

int gk_split_k_workspace_size(const gk_config* conf, size_t* bytes) {
  if (!conf || !bytes) return fail(GK_ERR_INVALID_ARGUMENT, "NULL argument");
  const gk_shape& g = conf->matmul_shape;
  const gk_shape& b = conf->block_shape;
  if (g.M <= 0 || g.N <= 0 || g.K <= 0 || b.M <= 0 || b.N <= 0 || b.K <= 0) return fail(GK_ERR_INVALID_ARGUMENT, "shapes must be positive");
  const long long tiles = (long long)((g.M + b.M - 1) / b.M) * ((g.N + b.N - 1) / b.N);
  const int kt = (g.K + b.K - 1) / b.K;
  const long long slices = split_k_slices((int)(tiles > (1 << 30) ? (1 << 30) : tiles), kt, b.K);
  if (slices < 2) { *bytes = 0; return GK_OK; }      // runs unsplit
  *bytes = kSplitCounterBytes + (size_t)tiles * (size_t)slices * b.M * b.N * sizeof(float);
  return GK_OK;
}

int gk_matmul_split_k(const gk_config* conf, const void* a, const void* b, const void* c, void* d, const gk_transforms* transforms,
                      const gk_epilogue* epilogue, void* workspace, size_t workspace_bytes, void* stream) {
  return gk_internal::launch_split_k(conf, a, b, c, d, transforms, epilogue, workspace, workspace_bytes, "the caller's workspace", stream);
}

int gk_dev_alloc(size_t bytes, void** ptr) {
  if (!ptr) return fail(GK_ERR_INVALID_ARGUMENT, "ptr is NULL");
  *ptr = nullptr;
  hipError_t e = hipMalloc(ptr, bytes ? bytes : 1);
  if (e != hipSuccess) return fail(GK_ERR_HIP, "hipMalloc of %zu bytes failed: %s", bytes, hipGetErrorString(e));
  return GK_OK;
}

int gk_dev_free(void* ptr) {
  hipError_t e = hipFree(ptr);
  if (e != hipSuccess) return fail(GK_ERR_HIP, "hipFree failed: %s", hipGetErrorString(e));
  return GK_OK;
}

int gk_copy_to_device(void* dst, const void* src, size_t bytes) {
  hipError_t e = hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice);
  if (e != hipSuccess) return fail(GK_ERR_HIP, "host to device copy of %zu bytes failed: %s", bytes, hipGetErrorString(e));
  return GK_OK;
}

int gk_copy_to_host(void* dst, const void* src, size_t bytes) {
  hipError_t e = hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost);
  if (e != hipSuccess) return fail(GK_ERR_HIP, "device to host copy of %zu bytes failed: %s", bytes, hipGetErrorString(e));
  return GK_OK;
}

int gk_synchronize(void) {
  hipError_t e = hipDeviceSynchronize();
  if (e != hipSuccess) return fail(GK_ERR_HIP, "hipDeviceSynchronize failed: %s", hipGetErrorString(e));
  return GK_OK;
}

int32_t gk_sizeof(int32_t which) {
  switch (which) {
    case 0: return (int32_t)sizeof(gk_config);
    case 1: return (int32_t)sizeof(gk_layout);
    case 2: return (int32_t)sizeof(gk_operator);
    case 3: return (int32_t)sizeof(gk_transforms);
    case 4: return (int32_t)sizeof(gk_epilogue);
    case 5: return (int32_t)sizeof(gk_gett);
    default: return -1;
  }
}

}  // extern "C"
