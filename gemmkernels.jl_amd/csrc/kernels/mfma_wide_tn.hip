// Four-wave instances of the tiles with a side of 192 for the 'TN' transpose pair (A K-major, B K-major in memory).
#define GK_A_KMAJOR true
#define GK_B_KMAJOR true
#define GK_FAMILY_FN family_mfma_wide_tn
#define GK_TAG "tn"
#include "mfma_wide_instances.inc"
