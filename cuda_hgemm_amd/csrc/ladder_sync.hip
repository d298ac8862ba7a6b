// Ladder steps 1-3: LDS-staged 256x128x32 tile with register-staged copies, eight
// wavefronts as 4 (M) x 2 (N) with 64x64 wave tiles -- the block / warp shape of the
// reference's tiled kernels (reference src/mma/mma_base.cu:13-29).
#include "variant_def.h"

using namespace hgemm;

//                                      BM   BN  BK  WM WN ST  loader    layout      ps2r
HGEMM_DEFINE_TILED_VARIANT(hgemm_mfma_base, 256, 128, 32, 4, 2, 1, LOAD_REG, LDS_LINEAR, false)
HGEMM_DEFINE_TILED_VARIANT(hgemm_mfma_padding, 256, 128, 32, 4, 2, 1, LOAD_REG, LDS_PADDED, false)
HGEMM_DEFINE_TILED_VARIANT(hgemm_mfma_swizzle, 256, 128, 32, 4, 2, 1, LOAD_REG, LDS_SWIZZLE, false)
