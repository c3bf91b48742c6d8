// MFMA GEMM instances for the 'TN' transpose pair (A K-major, B K-major in memory).
#define GK_A_KMAJOR true
#define GK_B_KMAJOR true
#define GK_FAMILY_FN family_mfma_tn
#define GK_STREAM_FN family_mfma_stream_tn
#define GK_TAG "tn"
#include "mfma_instances.inc"
