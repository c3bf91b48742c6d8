// Four-wave instances of the tiles with a side of 192 for the 'TT' transpose pair (A K-major, B N-major in memory).
#define GK_A_KMAJOR true
#define GK_B_KMAJOR false
#define GK_FAMILY_FN family_mfma_wide_tt
#define GK_TAG "tt"
#include "mfma_wide_instances.inc"
