// The BF16 ones of the 256 x 256 x 64 four-wave instances that stream C in, for the 'TN' transpose pair (A K-major, B K-major in memory).
#define GK_STREAM_BF16
#define GK_A_KMAJOR true
#define GK_B_KMAJOR true
#define GK_FAMILY_FN family_mfma_stream_tn
#define GK_FAMILY_FN_BF16 family_mfma_stream_tn_bf16
#define GK_TAG "tn"
#include "mfma_stream_instances.inc"
