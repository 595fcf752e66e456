// Internal interface of the dense Q4_K GEMM for few activation rows (dense_ksplit.hip): raw GGUF rows, a 64 x 64 output tile
// per workgroup with the columns split over the workgroup's waves, exact integer weight factors.
#pragma once
#include "tsp_common.hpp"

namespace tsp {

struct DenseKsplitArgs {
    const _Float16* a;   // activation rows as halves (bf16 values), k halves apart, columns of every eight in the order
                         // (0, 2, 1, 3, 4, 6, 5, 7): the order in which a word of nibbles unpacks two at a time
    const _Float16* sx;  // per row and 256-column super-block: the eight 32-column sums as high halves, then their residuals
    const uint8_t* w;    // [n rows][k / 256 blocks of 144 B]
    uint32_t m, n, k;
    void* out;           // f32 or bf16 rows, out_stride bytes apart
    uint64_t out_stride;
    int out_bf16;
    uint32_t* error_word;
};

// 512, 1024 or 2048 columns (two, four or eight waves of one super-block each) and at most 384 activation rows
bool dense_ksplit_takes(uint32_t tokens, uint32_t rows, uint32_t columns);
int launch_dense_ksplit(const DenseKsplitArgs& a, hipStream_t stream);

}  // namespace tsp
