// D = diag(a) * B (+ C): the GEMM whose A operand is Layout.Diagonal (reference
// src/layout.jl:225-236, run by matmul_singlestage with threadblock_condition, src/kernel.jl:60).
//
// The reference builds the dense tile of A in shared memory and skips the K blocks that hold no
// diagonal element.  Taken to its end that skip leaves exactly one product per output element,
// D[i,j] = fma(a[i], B[i,j], C[i,j]), which is what this kernel computes: every other term of the
// sum is an exact zero, so the result is bit-identical to the full product.  The work is pure
// streaming (read B, read C, write D), bound by HBM bandwidth: each lane moves 16-byte vectors and
// a workgroup covers its block_shape.M x block_shape.N tile of D in one pass.
#pragma once
#include "common.hpp"
#include <type_traits>

#ifndef GK_DIAG_U
#define GK_DIAG_U 8      // 4-row chunks in flight per lane without C
#endif
#ifndef GK_DIAG_U_C
#define GK_DIAG_U_C 4    // ... and with C
#endif

namespace gk {

// B_ROWMAJOR: B is the 'T' operand, stored N x K with K = M contiguous along j ... i.e. element
// (i, j) lives at b[j + i*ldb]; otherwise at b[i + j*ldb].
template <bool B_ROWMAJOR, typename T>
__global__ void __launch_bounds__(1024) diagonal_gemm_kernel(const GemmArgs args, int BM, int BN) {
  typedef T vec8 __attribute__((ext_vector_type(8)));
  extern __shared__ __attribute__((aligned(16))) char smem[];
  int ti, tj;
  cta_swizzle(args.swz_kind, args.swz_param, (int)blockIdx.x, (int)blockIdx.y, args.nbm, args.nbn, ti, tj);
  if (ti >= args.nbm || tj >= args.nbn) return;
  const int m0 = ti * BM, n0 = tj * BN;
  const T* A = (const T*)args.a;
  const T* B = (const T*)args.b;
  const float* C = (const float*)args.c;
  float* D = (float*)args.d;
  const bool xf_a = args.t[H_GL2SH_A].n > 0 || args.t[H_SH2RF_A].n > 0;
  const bool xf_b = args.t[H_GL2SH_B].n > 0 || args.t[H_SH2RF_B].n > 0;
  const bool xf_c = args.t[H_GL2SH_C].n > 0 || args.t[H_SH2RF_C].n > 0;
  const bool xf_d = args.t[H_RF2SH_D].n > 0 || args.t[H_SH2GL_D].n > 0 || args.epi_kind != 0;

  // c_in: the 8 values of C for this chunk (ignored when C is Layout.Zero)
  auto finish = [&](int i, int j, const float (&av)[8], const float (&bv)[8], const float4v c0, const float4v c1) {
    float c[8];
    if (args.c_mode != 0) {
#pragma unroll
      for (int e = 0; e < 4; ++e) { c[e] = c0[e]; c[4 + e] = c1[e]; }
      if (xf_c) { apply_list_regs<8>(args.t[H_GL2SH_C], c); apply_list_regs<8>(args.t[H_SH2RF_C], c); }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) c[e] = 0.0f;
    }
    float x[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = __builtin_fmaf(av[e], bv[e], c[e]);
    if (xf_d) {
      apply_list_regs<8>(args.t[H_RF2SH_D], x);
      if (args.epi_kind == 1) {
        const float bj = args.bias[j];
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = x[e] + bj;
      } else if (args.epi_kind == 2) {
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = x[e] + args.bias[i + e];
      }
      apply_list_regs<8>(args.t[H_SH2GL_D], x);
    }
    *(float4v*)&D[i + (long long)j * args.ldd] = (float4v){x[0], x[1], x[2], x[3]};
    *(float4v*)&D[i + 4 + (long long)j * args.ldd] = (float4v){x[4], x[5], x[6], x[7]};
  };
  auto load_c = [&](int i, int j, float4v& c0, float4v& c1) {
    if (args.c_mode != 0) {
      c0 = *(const float4v*)&C[i + (long long)j * args.ldc];
      c1 = *(const float4v*)&C[i + 4 + (long long)j * args.ldc];
    }
  };
  auto prep = [&](vec8 v, bool xf, const OpList& t0, const OpList& t1, float (&out)[8]) {
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = (float)v[e];
    if (xf) {
      if (t0.n > 0) {
        apply_list_regs<8>(t0, out);
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = (float)(T)out[e];
      }
      if (t1.n > 0) {
        apply_list_regs<8>(t1, out);
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = (float)(T)out[e];
      }
    }
  };

  if (!B_ROWMAJOR) {
    // chunk = 8 consecutive rows i of one column j.  A lane keeps U chunks in flight: all their
    // loads are issued before the first result is needed, which is what fills the memory pipeline
    // when a workgroup is the only one on its CU.
    const int chunks_m = BM / 8, total = chunks_m * BN;
    auto sweep = [&](auto u_c, auto plain_c) {
      constexpr int U = decltype(u_c)::value;
      constexpr bool PLAIN = decltype(plain_c)::value;     // no transform, no bias: nothing but the fma
      const int stride = (int)blockDim.x;
      for (int q0 = (int)threadIdx.x; q0 < total; q0 += U * stride) {
        vec8 bq[U], aq[U];
        float4v c0[U], c1[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int q = q0 + u * stride;
          if (q < total) {
            const int i = m0 + (q % chunks_m) * 8, j = n0 + q / chunks_m;
            bq[u] = *(const vec8*)&B[i + (long long)j * args.ldb];
            aq[u] = *(const vec8*)&A[i];
            load_c(i, j, c0[u], c1[u]);
          }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int q = q0 + u * stride;
          if (q < total) {
            const int i = m0 + (q % chunks_m) * 8, j = n0 + q / chunks_m;
            if constexpr (PLAIN) {
              float x[8];
#pragma unroll
              for (int e = 0; e < 8; ++e) {
                const float c = args.c_mode != 0 ? (e < 4 ? c0[u][e] : c1[u][e - 4]) : 0.0f;
                x[e] = __builtin_fmaf((float)aq[u][e], (float)bq[u][e], c);
              }
              // plain stores: streaming (non-temporal) loads and stores measured 20-40 % slower here
              *(float4v*)&D[i + (long long)j * args.ldd] = (float4v){x[0], x[1], x[2], x[3]};
              *(float4v*)&D[i + 4 + (long long)j * args.ldd] = (float4v){x[4], x[5], x[6], x[7]};
            } else {
              float av[8], bv[8];
              prep(aq[u], xf_a, args.t[H_GL2SH_A], args.t[H_SH2RF_A], av);
              prep(bq[u], xf_b, args.t[H_GL2SH_B], args.t[H_SH2RF_B], bv);
              finish(i, j, av, bv, c0[u], c1[u]);
            }
          }
        }
      }
    };
    // No transform and no bias: chunks of 4 rows, so that one store instruction of a wave writes 1 KiB
    // of consecutive addresses (with 8-row chunks the two 16-byte stores of a lane each fill every other
    // half of the 32-byte pieces, i.e. partial lines per instruction) and one load reads 512 B.
    auto sweep4 = [&](auto u_c) {
      constexpr int U = decltype(u_c)::value;
      typedef T vec4 __attribute__((ext_vector_type(4)));
      const int chunks4 = BM / 4, total4 = chunks4 * BN;
      const int stride = (int)blockDim.x;
      for (int q0 = (int)threadIdx.x; q0 < total4; q0 += U * stride) {
        vec4 bq[U], aq[U];
        float4v cq[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int q = q0 + u * stride;
          if (q < total4) {
            const int i = m0 + (q % chunks4) * 4, j = n0 + q / chunks4;
            bq[u] = *(const vec4*)&B[i + (long long)j * args.ldb];
            aq[u] = *(const vec4*)&A[i];
            if (args.c_mode != 0) cq[u] = *(const float4v*)&C[i + (long long)j * args.ldc];
          }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int q = q0 + u * stride;
          if (q < total4) {
            const int i = m0 + (q % chunks4) * 4, j = n0 + q / chunks4;
            float4v x;
#pragma unroll
            for (int e = 0; e < 4; ++e) x[e] = __builtin_fmaf((float)aq[u][e], (float)bq[u][e], args.c_mode != 0 ? cq[u][e] : 0.0f);
            *(float4v*)&D[i + (long long)j * args.ldd] = x;
          }
        }
      }
    };
    typedef std::true_type Plain;
    typedef std::false_type Generic;
    (void)Plain{};
    if (xf_a || xf_b || xf_c || xf_d) sweep(std::integral_constant<int, 1>{}, Generic{});
    else if (args.c_mode != 0) sweep4(std::integral_constant<int, GK_DIAG_U_C>{});
    else sweep4(std::integral_constant<int, GK_DIAG_U>{});
  } else {
    // transpose 64 (i) x 64 (j) sub-tiles of B through LDS so that both the loads (along j) and the
    // stores (along i) are 16-byte vectors
    T* tile = (T*)smem;                   // [64 i][64 + 8 j]
    constexpr int PITCH = 72;
    for (int sm = 0; sm < BM; sm += 64)
      for (int sn = 0; sn < BN; sn += 64) {
        __syncthreads();
        for (int q = (int)threadIdx.x; q < 64 * 8; q += (int)blockDim.x) {
          const int il = q / 8, jl = (q % 8) * 8;
          *(vec8*)&tile[il * PITCH + jl] = *(const vec8*)&B[(n0 + sn + jl) + (long long)(m0 + sm + il) * args.ldb];
        }
        __syncthreads();
        for (int q = (int)threadIdx.x; q < 8 * 64; q += (int)blockDim.x) {
          const int il = (q % 8) * 8, jl = q / 8;
          vec8 bvec;
#pragma unroll
          for (int e = 0; e < 8; ++e) bvec[e] = tile[(il + e) * PITCH + jl];
          const int i = m0 + sm + il, j = n0 + sn + jl;
          float av[8], bv[8];
          float4v c0, c1;
          load_c(i, j, c0, c1);
          prep(*(const vec8*)&A[i], xf_a, args.t[H_GL2SH_A], args.t[H_SH2RF_A], av);
          prep(bvec, xf_b, args.t[H_GL2SH_B], args.t[H_SH2RF_B], bv);
          finish(i, j, av, bv, c0, c1);
        }
      }
  }
}

}  // namespace gk
