// MFMA GEMM instances for the 'NN' transpose pair (A M-major, B K-major in memory).
#define GK_A_KMAJOR false
#define GK_B_KMAJOR true
#define GK_FAMILY_FN family_mfma_nn
#define GK_STREAM_FN family_mfma_stream_nn
#define GK_TAG "nn"
#include "mfma_instances.inc"
