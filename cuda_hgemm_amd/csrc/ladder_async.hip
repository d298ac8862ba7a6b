// Ladder steps 4-6: copies go global -> LDS without passing through registers, then two
// LDS buffers, then double-buffered operand registers.
#include "variant_def.h"

using namespace hgemm;

HGEMM_DEFINE_TILED_VARIANT(hgemm_mfma_async, 256, 128, 32, 4, 2, 1, LOAD_DMA, LDS_SWIZZLE, false)
HGEMM_DEFINE_TILED_VARIANT(hgemm_mfma_async_pg2s, 256, 128, 32, 4, 2, 2, LOAD_DMA, LDS_SWIZZLE, false)
HGEMM_DEFINE_TILED_VARIANT(hgemm_mfma_async_pg2s_ps2r, 256, 128, 32, 4, 2, 2, LOAD_DMA, LDS_SWIZZLE, true)
