// Four-wave instances of the 256 x 192 x 64 tile (192 x 256 x 64: mfma_wide_tn_192x256.hip) for the 'TN' transpose pair (A K-major, B K-major in memory).
#define GK_A_KMAJOR true
#define GK_B_KMAJOR true
#define GK_FAMILY_FN family_mfma_wide_tn
#define GK_TAG "tn"
#include "mfma_wide_instances.inc"
