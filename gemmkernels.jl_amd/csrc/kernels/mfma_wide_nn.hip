// Four-wave instances of the tiles with a side of 192 for the 'NN' transpose pair (A M-major, B K-major in memory).
#define GK_A_KMAJOR false
#define GK_B_KMAJOR true
#define GK_FAMILY_FN family_mfma_wide_nn
#define GK_TAG "nn"
#include "mfma_wide_instances.inc"
