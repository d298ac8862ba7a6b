// Glue that turns one TileConfig into an exported entry point plus its shape predicate.
#pragma once

#include "../../include/hgemm.h"
#include "mfma_tiled.h"

#define HGEMM_DEFINE_TILED_VARIANT(symbol, ...)                                                              \
    extern "C" void symbol(const hgemm_half *A, const hgemm_half *B, hgemm_half *C, size_t M, size_t N,      \
                           size_t K) {                                                                       \
        hgemm::launch_tiled<hgemm::TileConfig<__VA_ARGS__>>(A, B, C, M, N, K, #symbol);                      \
    }                                                                                                        \
    extern "C" int symbol##_supports(size_t M, size_t N, size_t K) {                                         \
        return hgemm::TileConfig<__VA_ARGS__>::supports(M, N, K) ? 1 : 0;                                    \
    }

#define HGEMM_DECLARE_SUPPORTS(symbol) extern "C" int symbol##_supports(size_t M, size_t N, size_t K)
