// Internal interface of the dense Q4_K GEMM for many activation rows (dense_tall.hip): raw GGUF rows, a 256 x 256 output tile
// per workgroup, weights decoded to halves once per 128 activation rows.
#pragma once
#include "tsp_common.hpp"

namespace tsp {

struct DenseTallArgs {
    const _Float16* a;   // activation rows as halves (bf16 values), a_stride halves apart, columns of every eight in the order
                         // (0, 2, 1, 3, 4, 6, 5, 7): the order in which a word of nibbles unpacks two at a time
    uint32_t a_stride;
    const uint8_t* w;    // [n rows][k / 256 blocks of 144 B]
    uint32_t m, n, k;
    void* out;           // f32 or bf16 rows, out_stride bytes apart
    uint64_t out_stride;
    int out_bf16;
    uint32_t* error_word;
};

// Enough rows to fill the chip with 256-row tiles; activations and weights addressed with 32-bit offsets.
bool dense_tall_takes(uint32_t tokens, uint32_t rows, uint32_t columns, uint64_t matrix_bytes);
int launch_dense_tall(const DenseTallArgs& a, hipStream_t stream);

}  // namespace tsp
