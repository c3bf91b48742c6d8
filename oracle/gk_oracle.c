/*
 * CPU oracle for the tiled GEMM hot path.  TEST INFRASTRUCTURE ONLY: it is linked or loaded by
 * tests, by the smoke check and by the cpu_baseline leg of the benchmark, never by the product
 * library.
 *
 * It restates, value by value, the order of operations of the reference kernels
 * (reference src/kernel.jl:167-187 C load + two transforms, :224-236 / :311-319 A and B
 * load + two transforms each, :322-326 inner product, :337-347 accumulator store + transform,
 * src/epilogue.jl:67-70 bias-then-transform), with the layouts of src/layout.jl
 * (ColMajor :117-148, RowMajor :156-184, Diagonal :225-236, Interleaved* :276-334, Zero :82-89),
 * the inner products of src/operator.jl (FPUOp.mma :139-153 sequential fma in ascending k,
 * TropicalFPUOp :134-137, WMMAComplexOp.mma :307-311, WMMADualOp.mma :366-369) and the
 * alpha/beta convention of src/matmul.jl:185-204.
 *
 * Rounding points (reference: the LDS copy has the shared layout's eltype, fragments have the
 * operator's compute type, accumulators its accumulator type):
 *   a' = round_compute( T_sh2rf_a( round_shared( T_gl2sh_a( A[i,k] ) ) ) )      (same for b')
 *   c0 = round_accum ( T_sh2rf_c( round_shared_c( T_gl2sh_c( C[i,j] ) ) ) )
 *   acc = c0 (+)= a' * b'   for k ascending, in the accumulator type
 *   d  = round_d( T_sh2gl_d( [ + bias ] round_shared_d( T_rf2sh_d( acc ) ) ) )
 * Transform ops are evaluated in fp32 (fp64 when the value type is fp64) and rounded to the
 * destination type with round-to-nearest-even.
 *
 * Parity pinning: the real/complex/tropical/dual GEMM functions are pinned in tests/ against
 * numpy float64 matmul, closed forms (identity, all-ones, single non-zero, diagonal product),
 * brute force on tiny shapes and linearity; layouts against index-distinct prime fixtures; the
 * integer element types (Int16 / Int32 / Int64, configs/configs.jl:495-497) against exact Python
 * integers reduced modulo 2^bits with magnitudes that overflow; Float32 -> Float64 and Float64
 * against numpy float64 matmul on dyadic inputs (bit-exact) and a math.fma chain; every elementwise
 * op (float and integer evaluation) against hand-typed value tables and numpy closed forms through an
 * identity product; the bfloat16 conversions exhaustively against torch.bfloat16; the dual-number
 * product against a0*b0 and a0*b1 + a1*b0 in float64.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- dtypes ---- */
enum { GKO_F16 = 0, GKO_BF16 = 1, GKO_F32 = 2, GKO_F64 = 3, GKO_I16 = 4, GKO_I32 = 5, GKO_I64 = 6 };

/* ---- layout kinds ---- */
enum {
  GKO_L_ZERO = 0,
  GKO_L_COL = 1,        /* element (r,c) at p[r + c*ld]            */
  GKO_L_ROW = 2,        /* element (r,c) at p[c + r*ld]            */
  GKO_L_DIAG = 3,       /* element (r,c) = p[c] if r == c else 0   */
  GKO_L_ICOL = 4,       /* interleaved complex, col-major          */
  GKO_L_IROW = 5,       /* interleaved complex, row-major          */
  GKO_L_GETT = 6        /* offset = sum_row-modes + sum_col-modes  */
};

/* ---- operator kinds ---- */
enum { GKO_OP_FMA = 0, GKO_OP_TROPICAL = 1, GKO_OP_COMPLEX = 2, GKO_OP_DUAL = 3 };

/* ---- transform ops ---- */
enum { GKO_T_IDENTITY = 0, GKO_T_SCALE = 1, GKO_T_ADD = 2, GKO_T_RELU = 3, GKO_T_NEG = 4, GKO_T_ABS = 5, GKO_T_CLAMP = 6, GKO_T_SQUARE = 7 };

typedef struct { int32_t kind; float p0, p1; } gko_op;
typedef struct { int32_t n; gko_op ops[4]; } gko_transform;

typedef struct {
  int32_t kind, dtype;
  int64_t ld;
  int32_t nmodes[2];           /* GETT: modes forming the row index, modes forming the col index */
  int64_t extent[2][4];        /* fastest digit first */
  int64_t stride[2][4];
} gko_layout;

typedef struct {
  int64_t M, N, K;
  gko_layout a, b, c, d;
  int32_t shared_a_dtype, shared_b_dtype, shared_c_dtype, shared_d_dtype;
  int32_t compute_dtype, accum_dtype;
  int32_t op_kind;
  int32_t wide_accum;          /* 1: accumulate in fp64 without intermediate rounding (error-norm reference) */
  gko_transform t[8];          /* gl2sh a,b,c ; sh2gl d ; sh2rf a,b,c ; rf2sh d  (reference src/matmul.jl:8-15) */
  int32_t epilogue;            /* 0 default, 1 bias per column (reference src/epilogue.jl:44-52), 2 bias per row */
  const float* bias;
} gko_problem;

/* ---------------- scalar conversions ---------------- */
static float half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ffu, bits;
  if (exp == 0) {
    if (man == 0) bits = sign;
    else {
      int e = -1;
      do { man <<= 1; ++e; } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) bits = sign | 0x7f800000u | (man << 13);
  else bits = sign | ((exp + 112) << 23) | (man << 13);
  float f; memcpy(&f, &bits, 4); return f;
}

/* double -> half, round to nearest even, done directly from the double so that there is a
 * single rounding. */
static uint16_t double_to_half(double x) {
  uint64_t bits; memcpy(&bits, &x, 8);
  uint16_t sign = (uint16_t)((bits >> 48) & 0x8000u);
  int64_t exp = (int64_t)((bits >> 52) & 0x7ff);
  uint64_t man = bits & 0xfffffffffffffull;
  if (exp == 0x7ff) return (uint16_t)(sign | 0x7c00u | (man ? 0x200u : 0));
  if (exp == 0 && man == 0) return sign;
  int64_t e = exp - 1023;                     /* unbiased */
  if (e > 15) return (uint16_t)(sign | 0x7c00u);
  uint64_t sig = man | (1ull << 52);          /* 53-bit significand, value = sig * 2^(e-52) */
  int shift;                                  /* number of low bits to drop */
  int64_t hexp;
  if (e >= -14) { shift = 42; hexp = e + 15; }          /* normal half: keep 11 bits */
  else { shift = (int)(42 + (-14 - e)); hexp = 0; }     /* subnormal */
  if (exp == 0) return sign;                  /* double subnormal: far below half range */
  if (shift > 63) return sign;
  uint64_t kept = sig >> shift;
  uint64_t rem = sig & ((1ull << shift) - 1);
  uint64_t halfway = 1ull << (shift - 1);
  if (rem > halfway || (rem == halfway && (kept & 1))) ++kept;
  uint32_t out;
  if (hexp == 0) out = (uint32_t)kept;                         /* may carry into exponent 1: fine */
  else out = (uint32_t)(((uint64_t)hexp << 10) + (kept - 0x400u)); /* carry propagates to exponent */
  if (out >= 0x7c00u) out = 0x7c00u;
  return (uint16_t)(sign | out);
}

static float bf16_to_float(uint16_t h) { uint32_t b = (uint32_t)h << 16; float f; memcpy(&f, &b, 4); return f; }
static uint16_t float_to_bf16(float f) {
  uint32_t b; memcpy(&b, &f, 4);
  if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((b >> 16) | 0x40u);
  uint32_t lsb = (b >> 16) & 1u;
  b += 0x7fffu + lsb;
  return (uint16_t)(b >> 16);
}

/* round a double value to the given dtype, returned as double (exactly representable) */
static double round_to(int dtype, double x) {
  switch (dtype) {
    case GKO_F16: return (double)half_to_float(double_to_half(x));
    case GKO_BF16: return (double)bf16_to_float(float_to_bf16((float)x)); /* values reaching here are fp32 already */
    case GKO_F32: return (double)(float)x;
    default: return x;
  }
}

static double load_scalar(int dtype, const void* p, int64_t idx) {
  switch (dtype) {
    case GKO_F16: return (double)half_to_float(((const uint16_t*)p)[idx]);
    case GKO_BF16: return (double)bf16_to_float(((const uint16_t*)p)[idx]);
    case GKO_F32: return (double)((const float*)p)[idx];
    default: return ((const double*)p)[idx];
  }
}

static void store_scalar(int dtype, void* p, int64_t idx, double v) {
  switch (dtype) {
    case GKO_F16: ((uint16_t*)p)[idx] = double_to_half(v); break;
    case GKO_BF16: ((uint16_t*)p)[idx] = float_to_bf16((float)v); break;
    case GKO_F32: ((float*)p)[idx] = (float)v; break;
    default: ((double*)p)[idx] = v; break;
  }
}

/* exported for the tests that pin the conversions */
uint16_t gko_double_to_half(double x) { return double_to_half(x); }
float gko_half_to_float(uint16_t h) { return half_to_float(h); }
uint16_t gko_float_to_bf16(float f) { return float_to_bf16(f); }
float gko_bf16_to_float(uint16_t h) { return bf16_to_float(h); }
/* vector forms of the same two functions (the exhaustive tests convert 2^16 x several patterns) */
void gko_float_to_bf16_n(const float* x, uint16_t* out, int64_t n) { for (int64_t i = 0; i < n; ++i) out[i] = float_to_bf16(x[i]); }
void gko_bf16_to_float_n(const uint16_t* x, float* out, int64_t n) { for (int64_t i = 0; i < n; ++i) out[i] = bf16_to_float(x[i]); }

/* ---------------- transforms ---------------- */
/* fp32 evaluation (fp64 when wide != 0), no contraction: one rounding per op */
static double apply_transform(const gko_transform* t, double x, int wide) {
  for (int i = 0; i < t->n; ++i) {
    const gko_op* o = &t->ops[i];
    if (wide) {
      double p0 = (double)o->p0, p1 = (double)o->p1;
      switch (o->kind) {
        case GKO_T_SCALE: x = x * p0; break;
        case GKO_T_ADD: x = x + p0; break;
        case GKO_T_RELU: x = x > 0.0 ? x : 0.0; break;
        case GKO_T_NEG: x = -x; break;
        case GKO_T_ABS: x = fabs(x); break;
        case GKO_T_CLAMP: x = x < p0 ? p0 : (x > p1 ? p1 : x); break;
        case GKO_T_SQUARE: x = x * x; break;
        default: break;
      }
    } else {
      volatile float f = (float)x;   /* volatile: forbid fused multiply-add / excess precision */
      float p0 = o->p0, p1 = o->p1;
      switch (o->kind) {
        case GKO_T_SCALE: f = f * p0; break;
        case GKO_T_ADD: f = f + p0; break;
        case GKO_T_RELU: f = f > 0.0f ? f : 0.0f; break;
        case GKO_T_NEG: f = -f; break;
        case GKO_T_ABS: f = fabsf(f); break;
        case GKO_T_CLAMP: f = f < p0 ? p0 : (f > p1 ? p1 : f); break;
        case GKO_T_SQUARE: f = f * f; break;
        default: break;
      }
      x = (double)f;
    }
  }
  return x;
}

/* One part (0: real, 1: imaginary) of a hook applied to a complex number.  The reference hands tiles of the
 * layout's element type to the transform (src/kernel.jl:167-187, 337-347, src/transform.jl:20-30), so a hook of a
 * complex product sees Complex values: z * p0 and -z act on both parts, z + p0 (p0 real) on the real part only.
 * The other ops have no complex method of the same type (max / clamp) or change the type (abs): not defined here,
 * complex_transform_ok() says so. */
static double apply_transform_part(const gko_transform* t, double x, int part, int wide) {
  for (int i = 0; i < t->n; ++i) {
    gko_transform one;
    one.n = 1;
    one.ops[0] = t->ops[i];
    if (one.ops[0].kind == GKO_T_ADD && part == 1) continue;
    x = apply_transform(&one, x, wide);
  }
  return x;
}
static int complex_transform_ok(const gko_transform* t) {
  for (int i = 0; i < t->n; ++i) {
    const int k = t->ops[i].kind;
    if (k != GKO_T_SCALE && k != GKO_T_ADD && k != GKO_T_NEG && k != 0) return 0;
  }
  return 1;
}

/* ---------------- layouts ---------------- */
static int64_t gett_offset(const gko_layout* L, int which, int64_t idx) {
  int64_t off = 0;
  for (int m = 0; m < L->nmodes[which]; ++m) {
    int64_t e = L->extent[which][m];
    off += (idx % e) * L->stride[which][m];
    idx /= e;
  }
  return off;
}

/* load logical element (r,c) of a real layout */
static double layout_load(const gko_layout* L, const void* p, int64_t r, int64_t c) {
  switch (L->kind) {
    case GKO_L_ZERO: return 0.0;
    case GKO_L_COL: return load_scalar(L->dtype, p, r + c * L->ld);
    case GKO_L_ROW: return load_scalar(L->dtype, p, c + r * L->ld);
    case GKO_L_DIAG: return r == c ? load_scalar(L->dtype, p, c) : 0.0;
    case GKO_L_GETT: return load_scalar(L->dtype, p, gett_offset(L, 0, r) + gett_offset(L, 1, c));
    default: return 0.0;
  }
}

static void layout_load_complex(const gko_layout* L, const void* p, int64_t r, int64_t c, double* re, double* im) {
  int64_t idx;
  switch (L->kind) {
    case GKO_L_ICOL: idx = r + c * L->ld; break;
    case GKO_L_IROW: idx = c + r * L->ld; break;
    default: *re = 0.0; *im = 0.0; return;
  }
  *re = load_scalar(L->dtype, p, 2 * idx);
  *im = load_scalar(L->dtype, p, 2 * idx + 1);
}

static int64_t layout_store_index(const gko_layout* L, int64_t r, int64_t c) {
  switch (L->kind) {
    case GKO_L_COL: case GKO_L_ICOL: return r + c * L->ld;
    case GKO_L_ROW: case GKO_L_IROW: return c + r * L->ld;
    case GKO_L_GETT: return gett_offset(L, 0, r) + gett_offset(L, 1, c);
    default: return -1;
  }
}

/* ---------------- the GEMM ---------------- */
static int is_complex_layout(const gko_layout* L) { return L->kind == GKO_L_ICOL || L->kind == GKO_L_IROW; }

/* ---------------- integer element types ---------------- */
/* FPUOp with Int16 / Int32 / Int64 (reference configs/configs.jl:495-497): Julia's fma on integers
 * is a*b + c with wrap-around, and so is every elementwise op.  Values are carried in uint64 and
 * wrapped to the element width after each operation, which is the same residue class. */
static int64_t wrap_int(int dtype, uint64_t x) {
  switch (dtype) {
    case GKO_I16: return (int64_t)(int16_t)(uint16_t)x;
    case GKO_I32: return (int64_t)(int32_t)(uint32_t)x;
    default: return (int64_t)x;
  }
}

static int64_t load_int(int dtype, const void* p, int64_t idx) {
  switch (dtype) {
    case GKO_I16: return ((const int16_t*)p)[idx];
    case GKO_I32: return ((const int32_t*)p)[idx];
    default: return ((const int64_t*)p)[idx];
  }
}

static void store_int(int dtype, void* p, int64_t idx, int64_t v) {
  switch (dtype) {
    case GKO_I16: ((int16_t*)p)[idx] = (int16_t)v; break;
    case GKO_I32: ((int32_t*)p)[idx] = (int32_t)v; break;
    default: ((int64_t*)p)[idx] = v; break;
  }
}

static int64_t apply_transform_int(const gko_transform* t, int dtype, int64_t x) {
  for (int i = 0; i < t->n; ++i) {
    const gko_op* o = &t->ops[i];
    const int64_t q0 = wrap_int(dtype, (uint64_t)(int64_t)o->p0), q1 = wrap_int(dtype, (uint64_t)(int64_t)o->p1);
    switch (o->kind) {
      case GKO_T_SCALE: x = wrap_int(dtype, (uint64_t)x * (uint64_t)q0); break;
      case GKO_T_ADD: x = wrap_int(dtype, (uint64_t)x + (uint64_t)q0); break;
      case GKO_T_RELU: x = x > 0 ? x : 0; break;
      case GKO_T_NEG: x = wrap_int(dtype, (uint64_t)0 - (uint64_t)x); break;
      case GKO_T_ABS: x = x < 0 ? wrap_int(dtype, (uint64_t)0 - (uint64_t)x) : x; break;
      case GKO_T_CLAMP: x = x < q0 ? q0 : (x > q1 ? q1 : x); break;
      case GKO_T_SQUARE: x = wrap_int(dtype, (uint64_t)x * (uint64_t)x); break;
      default: break;
    }
  }
  return x;
}

static int64_t layout_load_int(const gko_layout* L, const void* p, int64_t r, int64_t c) {
  switch (L->kind) {
    case GKO_L_COL: return load_int(L->dtype, p, r + c * L->ld);
    case GKO_L_ROW: return load_int(L->dtype, p, c + r * L->ld);
    default: return 0;     /* Layout.Zero */
  }
}

static int gko_matmul_int(const gko_problem* P, const void* a, const void* b, const void* c, void* d) {
  const int64_t M = P->M, N = P->N, K = P->K;
  const int dt = P->accum_dtype;
  if (P->op_kind != GKO_OP_FMA || P->epilogue != 0) return 1;
  const gko_layout* Ls[4] = {&P->a, &P->b, &P->c, &P->d};
  for (int i = 0; i < 4; ++i)
    if (Ls[i]->kind != GKO_L_ZERO && Ls[i]->kind != GKO_L_COL && Ls[i]->kind != GKO_L_ROW) return 1;
  int64_t* out = (int64_t*)malloc(sizeof(int64_t) * (size_t)M * (size_t)N);
  if (!out) return 2;
  for (int64_t j = 0; j < N; ++j)
    for (int64_t i = 0; i < M; ++i) {
      int64_t acc = 0;
      if (P->c.kind != GKO_L_ZERO) {
        acc = apply_transform_int(&P->t[2], dt, layout_load_int(&P->c, c, i, j));
        acc = apply_transform_int(&P->t[6], dt, acc);
      }
      for (int64_t k = 0; k < K; ++k) {      /* ascending k, one wrapped a*b + c per step (src/operator.jl:139-153) */
        int64_t x = apply_transform_int(&P->t[4], P->a.dtype, apply_transform_int(&P->t[0], P->a.dtype, layout_load_int(&P->a, a, i, k)));
        int64_t y = apply_transform_int(&P->t[5], P->b.dtype, apply_transform_int(&P->t[1], P->b.dtype, layout_load_int(&P->b, b, k, j)));
        acc = wrap_int(dt, (uint64_t)x * (uint64_t)y + (uint64_t)acc);
      }
      acc = apply_transform_int(&P->t[7], dt, acc);
      out[(size_t)j * M + i] = apply_transform_int(&P->t[3], dt, acc);
    }
  for (int64_t j = 0; j < N; ++j)
    for (int64_t i = 0; i < M; ++i) {
      int64_t idx = layout_store_index(&P->d, i, j);
      if (idx >= 0) store_int(P->d.dtype, d, idx, out[(size_t)j * M + i]);
    }
  free(out);
  return 0;
}

/*
 * D = epilogue(T_d(sum_k T_a(A) * T_b(B) + T_c(C))).  Returns 0 on success.
 * a, b, c, d are host pointers in the layouts of the problem; d may alias c.
 */
int gko_matmul(const gko_problem* P, const void* a, const void* b, const void* c, void* d) {
  if (P->accum_dtype >= GKO_I16) return gko_matmul_int(P, a, b, c, d);
  const int64_t M = P->M, N = P->N, K = P->K;
  const int two = (P->op_kind == GKO_OP_COMPLEX || P->op_kind == GKO_OP_DUAL) ? 2 : 1;
  const int wide_t = (P->compute_dtype == GKO_F64);   /* transforms of A/B in fp64 only for fp64 data */
  const int wide_cd = (P->accum_dtype == GKO_F64);
  if (two == 2 && !(is_complex_layout(&P->a) && is_complex_layout(&P->b))) return 1;
  if (two == 2)
    for (int h = 0; h < 8; ++h)
      if (!complex_transform_ok(&P->t[h])) return 3;

  /* transformed operands, k-contiguous: At[i*K + k], Bt[j*K + k]; planes for complex/dual */
  double* At = (double*)malloc(sizeof(double) * (size_t)M * (size_t)K * two);
  double* Bt = (double*)malloc(sizeof(double) * (size_t)N * (size_t)K * two);
  if (!At || !Bt) { free(At); free(Bt); return 2; }
  const size_t planeA = (size_t)M * (size_t)K, planeB = (size_t)N * (size_t)K;

#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < M; ++i)
    for (int64_t k = 0; k < K; ++k) {
      double v[2] = {0.0, 0.0};
      if (two == 2) layout_load_complex(&P->a, a, i, k, &v[0], &v[1]);
      else v[0] = layout_load(&P->a, a, i, k);
      for (int q = 0; q < two; ++q) {
        double x = round_to(P->shared_a_dtype, apply_transform_part(&P->t[0], v[q], q, wide_t));
        x = round_to(P->compute_dtype, apply_transform_part(&P->t[4], x, q, wide_t));
        At[q * planeA + (size_t)i * K + k] = x;
      }
    }
#pragma omp parallel for schedule(static)
  for (int64_t j = 0; j < N; ++j)
    for (int64_t k = 0; k < K; ++k) {
      double v[2] = {0.0, 0.0};
      if (two == 2) layout_load_complex(&P->b, b, k, j, &v[0], &v[1]);
      else v[0] = layout_load(&P->b, b, k, j);
      for (int q = 0; q < two; ++q) {
        double x = round_to(P->shared_b_dtype, apply_transform_part(&P->t[1], v[q], q, wide_t));
        x = round_to(P->compute_dtype, apply_transform_part(&P->t[5], x, q, wide_t));
        Bt[q * planeB + (size_t)j * K + k] = x;
      }
    }

  /* results are staged so that d may alias c */
  double* out = (double*)malloc(sizeof(double) * (size_t)M * (size_t)N * two);
  if (!out) { free(At); free(Bt); return 2; }
  const size_t planeD = (size_t)M * (size_t)N;
  const int acc32 = (P->accum_dtype != GKO_F64) && !P->wide_accum;
  const int acc16 = (P->accum_dtype == GKO_F16 || P->accum_dtype == GKO_BF16) && !P->wide_accum;

#pragma omp parallel for schedule(static)
  for (int64_t j = 0; j < N; ++j)
    for (int64_t i = 0; i < M; ++i) {
      double c0[2] = {0.0, 0.0};
      if (P->c.kind != GKO_L_ZERO) {
        if (two == 2) layout_load_complex(&P->c, c, i, j, &c0[0], &c0[1]);
        else c0[0] = layout_load(&P->c, c, i, j);
        for (int q = 0; q < two; ++q) {
          double x = round_to(P->shared_c_dtype, apply_transform_part(&P->t[2], c0[q], q, wide_cd));
          c0[q] = round_to(P->accum_dtype, apply_transform_part(&P->t[6], x, q, wide_cd));
        }
      }
      const double* ar = At + (size_t)i * K;
      const double* br = Bt + (size_t)j * K;
      double res[2] = {c0[0], c0[1]};
      if (P->op_kind == GKO_OP_FMA) {
        if (acc16) {
          double acc = c0[0];
          for (int64_t k = 0; k < K; ++k) acc = round_to(P->accum_dtype, fma(ar[k], br[k], acc));
          res[0] = acc;
        } else if (acc32) {
          float acc = (float)c0[0];
          for (int64_t k = 0; k < K; ++k) acc = fmaf((float)ar[k], (float)br[k], acc);
          res[0] = (double)acc;
        } else {
          double acc = c0[0];
          for (int64_t k = 0; k < K; ++k) acc = fma(ar[k], br[k], acc);
          res[0] = acc;
        }
      } else if (P->op_kind == GKO_OP_TROPICAL) {
        if (acc32) {
          float acc = (float)c0[0];
          for (int64_t k = 0; k < K; ++k) { float s = (float)ar[k] + (float)br[k]; acc = s > acc ? s : acc; }
          res[0] = (double)acc;
        } else {
          double acc = c0[0];
          for (int64_t k = 0; k < K; ++k) { double s = ar[k] + br[k]; acc = s > acc ? s : acc; }
          res[0] = acc;
        }
      } else {
        const double* ai = ar + planeA; const double* bi = br + planeB;
        if (acc32) {
          float re = (float)c0[0], im = (float)c0[1];
          for (int64_t k = 0; k < K; ++k) {
            re = fmaf((float)ar[k], (float)br[k], re);
            if (P->op_kind == GKO_OP_COMPLEX) re = fmaf(-(float)ai[k], (float)bi[k], re);
            im = fmaf((float)ar[k], (float)bi[k], im);
            im = fmaf((float)ai[k], (float)br[k], im);
          }
          res[0] = (double)re; res[1] = (double)im;
        } else {
          double re = c0[0], im = c0[1];
          for (int64_t k = 0; k < K; ++k) {
            re = fma(ar[k], br[k], re);
            if (P->op_kind == GKO_OP_COMPLEX) re = fma(-ai[k], bi[k], re);
            im = fma(ar[k], bi[k], im);
            im = fma(ai[k], br[k], im);
          }
          res[0] = re; res[1] = im;
        }
      }
      for (int q = 0; q < two; ++q) {
        double x = round_to(P->shared_d_dtype, apply_transform_part(&P->t[7], res[q], q, wide_cd));
        /* a bias value is real: on a complex D it goes to the real part (the reference's apply_bias,
         * src/epilogue.jl:45-53, takes Float32 tiles only and has no complex method) */
        if (P->epilogue == 1 && P->bias && q == 0) { volatile float s = (float)x + P->bias[j]; x = (double)s; }
        else if (P->epilogue == 2 && P->bias && q == 0) { volatile float s = (float)x + P->bias[i]; x = (double)s; }
        x = apply_transform_part(&P->t[3], x, q, wide_cd);
        out[q * planeD + (size_t)j * M + i] = x;
      }
    }

  for (int64_t j = 0; j < N; ++j)
    for (int64_t i = 0; i < M; ++i) {
      int64_t idx = layout_store_index(&P->d, i, j);
      if (idx < 0) continue;
      if (two == 2) {
        store_scalar(P->d.dtype, d, 2 * idx, out[(size_t)j * M + i]);
        store_scalar(P->d.dtype, d, 2 * idx + 1, out[planeD + (size_t)j * M + i]);
      } else store_scalar(P->d.dtype, d, idx, out[(size_t)j * M + i]);
    }
  free(At); free(Bt); free(out);
  return 0;
}

int gko_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

int gko_struct_sizes(int which) {
  switch (which) {
    case 0: return (int)sizeof(gko_problem);
    case 1: return (int)sizeof(gko_layout);
    case 2: return (int)sizeof(gko_transform);
    default: return 0;
  }
}
