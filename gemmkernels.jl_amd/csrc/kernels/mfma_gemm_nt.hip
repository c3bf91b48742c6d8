// MFMA GEMM instances for the 'NT' transpose pair (A M-major, B N-major in memory).
#define GK_A_KMAJOR false
#define GK_B_KMAJOR false
#define GK_FAMILY_FN family_mfma_nt
#define GK_STREAM_FN family_mfma_stream_nt
#define GK_TAG "nt"
#include "mfma_instances.inc"
