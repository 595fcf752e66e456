// Q8_0 GEMV for 1, 2, 4 or 8 token rows (LM head / MTP verify): each weight byte is read once
// and decoded once for all token rows.
//
// Raw GGUF Q8_0 rows are 34-byte blocks (f16 scale + 32 int8), so blocks are only 2-byte aligned,
// but a row of K columns is K*17/16 bytes: a whole number of dwords whenever K % 64 == 0. The
// kernel therefore streams a row as a flat dword array, lane i taking dwords i, i+64, ... (fully
// coalesced), and works out per dword which block it lies in. A dword holds up to four quants of
// ONE block (the two bytes of a scale field that may share the dword are masked to a neutral
// code). The scale of that block is fetched with a 2-byte load that hits the same cache lines.
//
//   sum_k d*q_k*x_k with q_k = u_k - 128 (u = q ^ 0x80) = d * (sum_k u_k*x_k - 128 * sum_k x_k)
//
// so the four bytes convert with v_cvt_f32_ubyte0..3 and a masked byte (u = 0x80) contributes 0.
#include "decode.hpp"
#include "q8_mfma.hpp"

using namespace tsp;

namespace {

struct Q8Args {
    const uint8_t* matrix;
    const float* x;   // token-major [M, columns]
    float* y;         // token-major [M, rows]
    uint32_t columns, rows;
    uint32_t* error_word;
};

__device__ __forceinline__ float ubf(uint32_t w, int i) { return float((w >> (8 * i)) & 0xffu); }

// M token rows; activations live in LDS as [M][columns + 4] with two zero floats either side so the
// neutral positions of a straddling dword read in-bounds, finite values.
template <int M>
__global__ __launch_bounds__(256) void q8_flat(Q8Args a) {
    extern __shared__ float lds[];
    const uint32_t stride = a.columns + 4;
    for (uint32_t i = threadIdx.x; i < M * stride; i += blockDim.x) {
        const uint32_t m = i / stride, c = i % stride;
        lds[i] = (c >= 2 && c < a.columns + 2) ? a.x[m * a.columns + (c - 2)] : 0.0f;
    }
    __syncthreads();

    const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const uint32_t row_dwords = a.columns / 32 * 34 / 4;
    const uint32_t waves = gridDim.x * (blockDim.x / kWave);
    for (uint32_t row = blockIdx.x * (blockDim.x / kWave) + wave; row < a.rows; row += waves) {
        const uint8_t* data = a.matrix + uint64_t(row) * row_dwords * 4;
        float acc[M];
#pragma unroll
        for (int m = 0; m < M; ++m) acc[m] = 0;
        for (uint32_t dw = lane; dw < row_dwords; dw += kWave) {
            const uint32_t w = *reinterpret_cast<const uint32_t*>(data + dw * 4);
            const uint32_t byte0 = dw * 4, block = byte0 / 34, pos = byte0 - block * 34;  // pos even, 0..32
            // bytes of this dword that are quants of `block`: pos == 0 -> bytes 2,3; pos == 32 -> bytes 0,1
            const uint32_t vmask = pos == 0 ? 0xffff0000u : pos == 32 ? 0x0000ffffu : 0xffffffffu;
            const uint32_t u = ((w ^ 0x80808080u) & vmask) | (0x80808080u & ~vmask);
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t*>(data + block * 34));
            // element index of byte 0 within the row, shifted by the two leading pad floats
            const uint32_t e0 = block * 32 + pos;  // = (block*32 + pos - 2) + 2
            const float u0 = ubf(u, 0), u1 = ubf(u, 1), u2 = ubf(u, 2), u3 = ubf(u, 3);
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const float* xs = lds + m * stride + e0;
                const float x0 = xs[0], x1 = xs[1], x2 = xs[2], x3 = xs[3];
                float t = -128.0f * ((x0 + x1) + (x2 + x3));
                t = __builtin_fmaf(u0, x0, t);
                t = __builtin_fmaf(u1, x1, t);
                t = __builtin_fmaf(u2, x2, t);
                t = __builtin_fmaf(u3, x3, t);
                acc[m] = __builtin_fmaf(d, t, acc[m]);
            }
        }
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const float total = wave_sum(acc[m]);
            if (lane == 0) {
                if (nonfinite(total)) atomicOr(a.error_word, TSP_ERRBIT_NONFINITE);
                a.y[uint64_t(m) * a.rows + row] = total;
            }
        }
    }
}

// q8_lanes_v1 rows: [f16 scale x blocks][runs of 16 blocks x 512 B, byte = index*width + block%16].
// One lane takes the `width` bytes of one (run, index): element `index` of up to 16 blocks.
template <int M>
__global__ __launch_bounds__(256) void q8_lanes(Q8Args a) {
    const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const uint32_t blocks = a.columns / 32, row_bytes = blocks * 34, runs = (blocks + 15) / 16;
    const uint32_t waves = gridDim.x * (blockDim.x / kWave);
    for (uint32_t row = blockIdx.x * (blockDim.x / kWave) + wave; row < a.rows; row += waves) {
        const uint8_t* data = a.matrix + uint64_t(row) * row_bytes;
        float acc[M];
#pragma unroll
        for (int m = 0; m < M; ++m) acc[m] = 0;
        for (uint32_t item = lane; item < runs * 32; item += kWave) {
            const uint32_t run = item / 32, index = item % 32;
            const uint32_t width = blocks - run * 16 < 16 ? blocks - run * 16 : 16;
            const uint8_t* q = data + blocks * 2 + run * 512 + index * width;
            for (uint32_t b = 0; b < width; ++b) {
                const uint32_t block = run * 16 + b;
                const float wv = half_bits_to_float(ld16(data + block * 2)) * float(int(int8_t(q[b])));
#pragma unroll
                for (int m = 0; m < M; ++m) acc[m] = __builtin_fmaf(wv, a.x[uint64_t(m) * a.columns + block * 32 + index], acc[m]);
            }
        }
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const float total = wave_sum(acc[m]);
            if (lane == 0) {
                if (nonfinite(total)) atomicOr(a.error_word, TSP_ERRBIT_NONFINITE);
                a.y[uint64_t(m) * a.rows + row] = total;
            }
        }
    }
}

// Any K (multiple of 32) and any alignment: wave per row, lane per block.
template <int M>
__global__ __launch_bounds__(256) void q8_blocks(Q8Args a) {
    const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const uint32_t blocks = a.columns / 32;
    const uint32_t waves = gridDim.x * (blockDim.x / kWave);
    for (uint32_t row = blockIdx.x * (blockDim.x / kWave) + wave; row < a.rows; row += waves) {
        const uint8_t* data = a.matrix + uint64_t(row) * blocks * 34;
        float acc[M];
#pragma unroll
        for (int m = 0; m < M; ++m) acc[m] = 0;
        for (uint32_t b = lane; b < blocks; b += kWave) {
            const uint8_t* block = data + b * 34;
            const float d = half_bits_to_float(ld16(block));
            for (uint32_t i = 0; i < 32; ++i) {
                const float wv = d * float(int(int8_t(block[2 + i])));
#pragma unroll
                for (int m = 0; m < M; ++m) acc[m] = __builtin_fmaf(wv, a.x[uint64_t(m) * a.columns + b * 32 + i], acc[m]);
            }
        }
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const float total = wave_sum(acc[m]);
            if (lane == 0) {
                if (nonfinite(total)) atomicOr(a.error_word, TSP_ERRBIT_NONFINITE);
                a.y[uint64_t(m) * a.rows + row] = total;
            }
        }
    }
}

template <int M>
int launch(uint32_t layout, const Q8Args& a, hipStream_t stream) {
    const uint32_t grid = (a.rows + 3) / 4 > 4096 ? 4096 : (a.rows + 3) / 4;
    if (layout == TSP_LAYOUT_Q8_LANES_V1) {
        TSP_LAUNCH("q8_lanes", stream, q8_lanes<M><<<grid, 256, 0, stream>>>(a));
        return launch_status("q8_lanes");
    }
    const uint64_t lds_bytes = uint64_t(M) * (a.columns + 4) * 4;
    if (a.columns % 64 == 0 && reinterpret_cast<uintptr_t>(a.matrix) % 4 == 0 && lds_bytes <= 96 * 1024) {
        static std::atomic<uint64_t> raised{0};  // one per instantiation (M)
        int device = 0;
        if (lds_bytes > 48 * 1024 && setup_pending(raised, &device)) {
            TSP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&q8_flat<M>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
            setup_done(raised, device);
        }
        TSP_LAUNCH("q8_flat", stream, q8_flat<M><<<grid, 256, lds_bytes, stream>>>(a));
        return launch_status("q8_flat");
    }
    TSP_LAUNCH("q8_blocks", stream, q8_blocks<M><<<grid, 256, 0, stream>>>(a));
    return launch_status("q8_blocks");
}

}  // namespace

extern "C" int tsp_q8_matvec_many(uint32_t layout, const void* matrix, uint64_t matrix_bytes, const float* x, float* y,
                                  uint32_t columns, uint32_t rows, uint32_t width, uint32_t* error_word, void* stream) {
    TSP_REQUIRE(columns && columns <= 65536 && columns % 32 == 0 && rows && rows <= 1000000 &&
                    (width == 1 || width == 2 || width == 4 || width == 8),
                "unsupported Q8-many projection shape");
    TSP_REQUIRE(layout == TSP_LAYOUT_GGUF || layout == TSP_LAYOUT_Q8_LANES_V1, "Q8-many layout");
    TSP_REQUIRE(uint64_t(columns / 32) * rows * 34 == matrix_bytes, "Q8-many matrix byte span mismatch");
    TSP_REQUIRE(matrix && x && y && error_word, "null device pointer");
    const uint64_t x_span = uint64_t(columns) * width * 4, y_span = uint64_t(rows) * width * 4;
    TSP_REQUIRE(!ranges_overlap(y, y_span, matrix, matrix_bytes) && !ranges_overlap(y, y_span, x, x_span), "Q8-many output overlaps an input");
    const Q8Args a{static_cast<const uint8_t*>(matrix), x, y, columns, rows, error_word};
    const auto s = static_cast<hipStream_t>(stream);
    if (layout == TSP_LAYOUT_GGUF && q8_mfma_supported(matrix, x, columns, rows)) return q8_mfma(matrix, x, y, columns, rows, width, error_word, s);
    if (layout == TSP_LAYOUT_Q8_LANES_V1 && q8_lanes_mfma_supported(matrix, x, columns, rows))
        return q8_lanes_mfma(matrix, x, y, columns, rows, width, error_word, s);
    switch (width) {
    case 1: return launch<1>(layout, a, s);
    case 2: return launch<2>(layout, a, s);
    case 4: return launch<4>(layout, a, s);
    default: return launch<8>(layout, a, s);
    }
}

extern "C" int tsp_dense_mm_q8(uint32_t layout, const void* matrix, uint64_t matrix_bytes, const float* input, uint64_t input_stride_bytes,
                               float* output, uint64_t output_stride_bytes, uint32_t tokens, uint32_t columns, uint32_t rows,
                               uint32_t* error_word, void* stream) {
    TSP_REQUIRE(tokens && tokens <= 65536 && input_stride_bytes % 4 == 0 && output_stride_bytes % 4 == 0 &&
                    input_stride_bytes >= uint64_t(columns) * 4 && output_stride_bytes >= uint64_t(rows) * 4,
                "dense Q8_0 GEMM row geometry mismatch");
    TSP_REQUIRE(input && output, "null device pointer");
    const uint64_t in_span = uint64_t(tokens - 1) * input_stride_bytes + uint64_t(columns) * 4;
    const uint64_t out_span = uint64_t(tokens - 1) * output_stride_bytes + uint64_t(rows) * 4;
    TSP_REQUIRE(!ranges_overlap(output, out_span, matrix, matrix_bytes) && !ranges_overlap(output, out_span, input, in_span),
                "dense Q8_0 GEMM output overlaps an input");
    // Token rows that lie back to back go eight, four, two, one at a time (each weight decoded once for the group, the
    // width sequence of src/q8_many.cpp:20-29); rows with padding between them go one by one.
    const bool packed = input_stride_bytes == uint64_t(columns) * 4 && output_stride_bytes == uint64_t(rows) * 4;
    // Nine or more packed rows left: up to sixteen go through the matrix-core kernel in one pass over the weights.
    const bool whole = packed && matrix && error_word && columns % 32 == 0 && rows <= 1000000 && uint64_t(columns / 32) * rows * 34 == matrix_bytes;
    const bool lanes = layout == TSP_LAYOUT_Q8_LANES_V1;
    const bool sixteen = whole && (layout == TSP_LAYOUT_GGUF ? q8_mfma_supported_16(matrix, input, output, columns, rows)
                                                            : lanes && q8_lanes_mfma_supported_16(matrix, input, output, columns, rows));
    for (uint32_t done = 0; done < tokens;) {
        if (sixteen && tokens - done > 8) {
            const uint32_t width = tokens - done < 16 ? tokens - done : 16;
            const int rc = (lanes ? q8_lanes_mfma : q8_mfma)(matrix, input + uint64_t(done) * columns, output + uint64_t(done) * rows, columns, rows, width,
                                                             error_word, static_cast<hipStream_t>(stream));
            if (rc != TSP_OK) return rc;
            done += width;
            continue;
        }
        uint32_t width = 1;
        if (packed) tsp_q8_many_width(tokens - done, &width);
        const int rc = tsp_q8_matvec_many(layout, matrix, matrix_bytes,
                                          reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(input) + uint64_t(done) * input_stride_bytes),
                                          reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(output) + uint64_t(done) * output_stride_bytes),
                                          columns, rows, width, error_word, stream);
        if (rc != TSP_OK) return rc;
        done += width;
    }
    return TSP_OK;
}
