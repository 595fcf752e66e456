// Internal interface of the matrix-core Q8_0 GEMV (q8_mfma.hip).
#pragma once
#include "tsp_common.hpp"

namespace tsp {

// raw GGUF Q8_0 rows, columns a multiple of 256 up to 2048, at least 32 rows, 16-byte aligned matrix and activations
bool q8_mfma_supported(const void* matrix, const float* x, uint32_t columns, uint32_t rows);
// nine to sixteen token rows in one pass over the matrix: also columns a multiple of 1024, rows a multiple of 4, y 16-byte aligned
bool q8_mfma_supported_16(const void* matrix, const float* x, const float* y, uint32_t columns, uint32_t rows);
// x token-major [width, columns], y token-major [width, rows]; width <= 8, or <= 16 where q8_mfma_supported_16 holds
int q8_mfma(const void* matrix, const float* x, float* y, uint32_t columns, uint32_t rows, uint32_t width, uint32_t* error_word, hipStream_t stream);
// q8_lanes_v1 rows on the same path: columns a multiple of 512 up to 2048, at least 16 rows, 16-byte aligned matrix and activations
bool q8_lanes_mfma_supported(const void* matrix, const float* x, uint32_t columns, uint32_t rows);
// nine to sixteen token rows in one pass over the matrix: also columns a multiple of 1024, at least 32 rows in multiples of 4, y 16-byte aligned
bool q8_lanes_mfma_supported_16(const void* matrix, const float* x, const float* y, uint32_t columns, uint32_t rows);
// width <= 8, or <= 16 where q8_lanes_mfma_supported_16 holds
int q8_lanes_mfma(const void* matrix, const float* x, float* y, uint32_t columns, uint32_t rows, uint32_t width, uint32_t* error_word, hipStream_t stream);

}  // namespace tsp
