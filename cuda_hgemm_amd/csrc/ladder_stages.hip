// Ladder steps 7-9: K_STAGE-deep LDS ring with s_waitcnt vmcnt((K_STAGE-2) * loads) in
// the steady state (reference src/mma/mma_async_stage4.cu:234,383 wait_group(2)).
// The 2-deep ring uses the wider 64-half K chunk so it differs from the pg2s+ps2r step.
#include "variant_def.h"

using namespace hgemm;

HGEMM_DEFINE_TILED_VARIANT(hgemm_mfma_async_stage2, 256, 128, 64, 4, 2, 2, LOAD_DMA, LDS_SWIZZLE, true)
HGEMM_DEFINE_TILED_VARIANT(hgemm_mfma_async_stage3, 256, 128, 32, 4, 2, 3, LOAD_DMA, LDS_SWIZZLE, true)
HGEMM_DEFINE_TILED_VARIANT(hgemm_mfma_async_stage4, 256, 128, 32, 4, 2, 4, LOAD_DMA, LDS_SWIZZLE, true)
// The same kernel on a 64x64x64 tile, four waves of one 32x32 MFMA tile each, 5-stage ring with the barrier one
// chunk ahead and whole chunks of operands in registers: what hgemm_auto runs on small grids of whole tiles
// (no counterpart in the reference, whose tiles are 256x128).
HGEMM_DEFINE_TILED_VARIANT(hgemm_mfma_tiled_64x64, 64, 64, 64, 2, 2, 5, LOAD_DMA, LDS_SWIZZLE, true, true)
