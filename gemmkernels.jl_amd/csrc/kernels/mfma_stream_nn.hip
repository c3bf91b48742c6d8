// The 256 x 256 x 64 four-wave instances that stream C in, for the 'NN' transpose pair (A M-major, B K-major in memory).
#define GK_A_KMAJOR false
#define GK_B_KMAJOR true
#define GK_FAMILY_FN family_mfma_stream_nn
#define GK_FAMILY_FN_BF16 family_mfma_stream_nn_bf16
#define GK_TAG "nn"
#include "mfma_stream_instances.inc"
