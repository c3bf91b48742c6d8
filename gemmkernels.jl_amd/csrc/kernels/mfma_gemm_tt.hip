// MFMA GEMM instances for the 'TT' transpose pair (A K-major, B N-major in memory).
#define GK_A_KMAJOR true
#define GK_B_KMAJOR false
#define GK_FAMILY_FN family_mfma_tt
#define GK_STREAM_FN family_mfma_stream_tt
#define GK_TAG "tt"
#include "mfma_instances.inc"
