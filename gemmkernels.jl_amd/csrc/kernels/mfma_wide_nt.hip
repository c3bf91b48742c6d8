// Four-wave instances of the tiles with a side of 192 for the 'NT' transpose pair (A M-major, B N-major in memory).
#define GK_A_KMAJOR false
#define GK_B_KMAJOR false
#define GK_FAMILY_FN family_mfma_wide_nt
#define GK_TAG "nt"
#include "mfma_wide_instances.inc"
