// Decode / verify GEMV over block-quantised rows: y[r] = sum_c dec(W[r,c]) * x[c], f32 decode and
// f32 accumulate. HBM-bound work: every kernel streams each weight byte exactly once with 16-byte
// coalesced loads, keeps the activation slice a lane needs in registers across rows, unpacks
// nibbles and scales in registers and finishes with DPP reductions inside the wave.
//
//  gemv_generic   wave per row, any decodable encoding and any K: the scalar control arm.
//  gemv_q4k       Q4_K, raw GGUF rows or one planar v3 expert; a lane owns one 32-byte nibble pair
//                 (two 32-weight sub-blocks), 4 lanes per super-block. The lane's 64 activations are
//                 kept as three planes of signed bytes under a per-sub-block scale (24 bits of each
//                 value), and the nibbles multiply them four at a time with v_dot4_i32_i8: the sums
//                 of q * x are exact integers, scaled by d * sc in f32 once per sub-block.
//  gemv_q8        Q8_0 raw rows as a flat dword stream (row bytes are a multiple of 4).
//  gemv_q6k       Q6_K planar expert planes.
#include "decode.hpp"

using namespace tsp;

namespace {

struct GemvArgs {
    const uint8_t* matrix;       // first row of expert 0
    const float* x;
    float* y;
    const uint32_t* ids;         // per blockIdx.y expert id, or nullptr
    uint64_t expert_stride;      // bytes between experts
    uint64_t x_stride, y_stride; // bytes between blockIdx.y slices of x / y
    uint32_t columns, rows, experts, count;
    uint32_t* error_word;
    tsp_planar_spec spec;        // planar layouts only
};

// Resolves the blockIdx.y slice: returns false (after zero-filling and flagging) for a bad expert id.
__device__ __forceinline__ bool resolve(const GemvArgs& a, const uint8_t*& w, const float*& x, float*& y) {
    const uint32_t slice = blockIdx.y;
    w = a.matrix;
    x = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(a.x) + slice * a.x_stride);
    y = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.y) + slice * a.y_stride);
    if (a.ids) {
        const uint32_t e = a.ids[slice];
        if (e >= a.experts) {
            if (threadIdx.x == 0 && blockIdx.x == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
            for (uint32_t r = blockIdx.x * blockDim.x + threadIdx.x; r < a.rows; r += gridDim.x * blockDim.x) y[r] = 0;
            return false;
        }
        w += e * a.expert_stride;
    }
    return true;
}

// ------------------------------------------------------------------------------------ generic
template <uint32_t T>
__global__ __launch_bounds__(256) void gemv_generic(GemvArgs a) {
    constexpr uint32_t E = BlockGeometry<T>::elements, B = BlockGeometry<T>::bytes;
    const uint8_t* w; const float* x; float* y;
    if (!resolve(a, w, x, y)) return;
    const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const uint64_t row_bytes = uint64_t(a.columns / E) * B;
    for (uint32_t row = blockIdx.x * 4 + wave; row < a.rows; row += gridDim.x * 4) {
        const uint8_t* data = w + row * row_bytes;
        float acc = 0;
        for (uint32_t c = lane; c < a.columns; c += kWave) acc = __builtin_fmaf(decode_element<T>(data + (c / E) * B, c % E), x[c], acc);
        const float total = wave_sum(acc);
        if (lane == 0) {
            if (nonfinite(total)) atomicOr(a.error_word, TSP_ERRBIT_NONFINITE);
            y[row] = total;
        }
    }
}

// ------------------------------------------------------------------------------------ Q4_K

// Sum over aligned groups of N lanes (N = 8, 16, 32, 64); every lane of a group gets the sum.
template <int N>
__device__ __forceinline__ float group_sum(float v) {
    v = dpp_add<0xB1>(v);
    v = dpp_add<0x4E>(v);
    v = dpp_add<0x141>(v);
    if constexpr (N >= 16) v = dpp_add<0x140>(v);
    if constexpr (N >= 32) v += __shfl_xor(v, 16, kWave);
    if constexpr (N >= 64) v += __shfl_xor(v, 32, kWave);
    return v;
}

// BPR = super-blocks per row (K / 256), one of 2, 4, 8, 16. A wave covers 16 super-blocks per step
// (16 / BPR rows); lane = (block-in-step, pair) owns 64 weights and keeps their 64 activations in
// registers for every row it visits.
template <int BPR, bool PLANAR>
__global__ __launch_bounds__(256) void gemv_q4k(GemvArgs a) {
    constexpr int LPR = 4 * BPR;        // lanes per row
    constexpr int RPS = kWave / LPR;    // rows per wave step
    // per sub-block of 32 activations: three planes of eight dwords (four signed bytes each), then 1 / scale, the sum, a flag
    constexpr uint32_t kSubWords = 3 * 8 + 4;
    __shared__ __attribute__((aligned(16))) uint32_t planes[BPR * 8 * kSubWords];
    const uint8_t* w; const float* x; float* y;
    if (!resolve(a, w, x, y)) return;
    const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const uint32_t pair = lane % 4, blk_in_row = (lane / 4) % BPR, row_in_step = lane / LPR;
    const uint32_t steps = (a.rows + RPS - 1) / RPS;
    const uint32_t waves = gridDim.x * (blockDim.x / kWave);

    // The bytes of one step as they come from memory: nothing is computed on them until they are needed, so that a step's
    // requests can be in flight while something else happens (the activations being staged, the step before being summed).
    struct Raw { uint4 q0, q1, hdr; uint32_t sc, mn, dm; };
    auto fetch = [&](uint32_t step) {
        const uint32_t row = step * RPS + row_in_step;
        const uint64_t blk = uint64_t(row < a.rows ? row : a.rows - 1) * BPR + blk_in_row;
        Raw r{};
        if constexpr (PLANAR) {
            const uint8_t* qs = w + a.spec.qs_offset + blk * 128 + pair * 32;
            r.q0 = *reinterpret_cast<const uint4*>(qs);
            r.q1 = *reinterpret_cast<const uint4*>(qs + 16);
            const uint8_t* sm = w + a.spec.sm_offset + blk * 16 + pair * 2;
            r.sc = *reinterpret_cast<const uint16_t*>(sm);
            r.mn = *reinterpret_cast<const uint16_t*>(sm + 8);
            r.dm = *reinterpret_cast<const uint32_t*>(w + a.spec.dm_offset + blk * 4);
        } else {
            const uint8_t* block = w + blk * 144;
            r.hdr = *reinterpret_cast<const uint4*>(block);
            r.q0 = *reinterpret_cast<const uint4*>(block + 16 + pair * 32);
            r.q1 = *reinterpret_cast<const uint4*>(block + 32 + pair * 32);
        }
        return r;
    };

    // The activations are asked for first (a few cached kilobytes: they come back first), the wave's first weight bytes right
    // behind them; the activations are staged and summed while the weights travel.
    constexpr uint32_t kQuads = BPR * 64;                // float4 in a row of activations
    constexpr uint32_t kMine = (kQuads + 255) / 256;     // per thread: 1 (K = 512, half the threads) .. 16 (K = 4096)
    float4 xv[kMine];
    const bool x_quads = reinterpret_cast<uintptr_t>(x) % 16 == 0;  // else a row that only floats align
#pragma unroll
    for (uint32_t j = 0; j < kMine; ++j) {
        const uint32_t quad = threadIdx.x + j * 256;
        if (kQuads % 256 == 0 || quad < kQuads) {
            if (x_quads) xv[j] = reinterpret_cast<const float4*>(x)[quad];
            else xv[j] = make_float4(x[4 * quad], x[4 * quad + 1], x[4 * quad + 2], x[4 * quad + 3]);
        }
    }
    uint32_t step = blockIdx.x * (blockDim.x / kWave) + wave;
    Raw cur = fetch(step < steps ? step : 0);
    // The activations become integers, once per workgroup: per sub-block of 32 one scale that brings the largest magnitude to
    // 8 290 000 (just under 127 * 2^16 + 2^15, the most that three signed bytes hold), every value rounded to the nearest
    // integer of that grid (2^-24 of the sub-block's largest value: the precision of the f32 operand itself for the values
    // that matter) and written as three signed base-256 digits, x = (a 2^16 + b 2^8 + c) / scale with a, b, c in [-128, 127].
    // Four activations' digits share a dword, in the order of the four bytes of a word of nibbles, so that v_dot4_i32_i8
    // multiplies four weights per instruction and plane: three integer instructions per four weights where the f32 form
    // spends a conversion and a multiply-add per weight. The integer sums are exact; the three of a sub-block recombine in f32.
    // A thread turns the quads it loaded into digits; the eight threads of a sub-block are neighbours and agree on its scale
    // with three cross-lane steps.
#pragma unroll
    for (uint32_t j = 0; j < kMine; ++j) {
        const uint32_t quad = threadIdx.x + j * 256;
        const bool mine = kQuads % 256 == 0 || quad < kQuads;  // uniform over every group of eight lanes
        const float v4[4] = {mine ? xv[j].x : 0.0f, mine ? xv[j].y : 0.0f, mine ? xv[j].z : 0.0f, mine ? xv[j].w : 0.0f};
        float biggest = fmaxf(fmaxf(fabsf(v4[0]), fabsf(v4[1])), fmaxf(fabsf(v4[2]), fabsf(v4[3])));
        float sum = (v4[0] + v4[1]) + (v4[2] + v4[3]);
        uint32_t flag = (nonfinite(v4[0]) || nonfinite(v4[1]) || nonfinite(v4[2]) || nonfinite(v4[3])) ? 1u : 0u;
        biggest = dpp_max<0xB1>(biggest); biggest = dpp_max<0x4E>(biggest); biggest = dpp_max<0x141>(biggest);
        sum = octet_sum(sum);
        flag |= uint32_t(__builtin_amdgcn_update_dpp(0, int(flag), 0xB1, 0xf, 0xf, true));
        flag |= uint32_t(__builtin_amdgcn_update_dpp(0, int(flag), 0x4E, 0xf, 0xf, true));
        flag |= uint32_t(__builtin_amdgcn_update_dpp(0, int(flag), 0x141, 0xf, 0xf, true));
        // a sub-block of zeros, of subnormals only, or with something not finite in it keeps scale 1 (its integers are zeros)
        const bool usable = biggest >= 1.1754944e-38f && !nonfinite(biggest) && flag == 0;
        const float scale = usable ? 8290000.0f / biggest : 1.0f;
        uint32_t w2 = 0, w1 = 0, w0 = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int xi = usable ? __float2int_rn(v4[e] * scale) : 0;
            const int c = ((xi + 128) & 255) - 128, upper = (xi - c) >> 8;
            const int b = ((upper + 128) & 255) - 128, a8 = (upper - b) >> 8;
            w2 |= uint32_t(a8 & 0xff) << (8 * e);
            w1 |= uint32_t(b & 0xff) << (8 * e);
            w0 |= uint32_t(c & 0xff) << (8 * e);
        }
        if (mine) {
            uint32_t* sub = planes + (quad / 8) * kSubWords;
            sub[16 + quad % 8] = w2; sub[8 + quad % 8] = w1; sub[quad % 8] = w0;
            if (quad % 8 == 0) {
                sub[24] = __float_as_uint(usable ? biggest / 8290000.0f : 1.0f);
                sub[25] = __float_as_uint(sum);
                sub[26] = flag;
            }
        }
    }
    __syncthreads();

    uint32_t pa[3][8], pb[3][8];
    float sxa, sxb, inv_a, inv_b;
    bool x_bad;
    {
        const uint32_t* sa = planes + (blk_in_row * 8 + pair * 2) * kSubWords;
        const uint32_t* sb = sa + kSubWords;
#pragma unroll
        for (int p = 0; p < 3; ++p)
#pragma unroll
            for (int k = 0; k < 8; ++k) { pa[p][k] = sa[p * 8 + k]; pb[p][k] = sb[p * 8 + k]; }
        inv_a = __uint_as_float(sa[24]); sxa = __uint_as_float(sa[25]);
        inv_b = __uint_as_float(sb[24]); sxb = __uint_as_float(sb[25]);
        x_bad = (sa[26] | sb[26]) != 0;
    }

    for (; step < steps; step += waves) {
        const uint32_t row = step * RPS + row_in_step;
        const bool live = row < a.rows;
        const Raw now = cur;
        cur = fetch(step + waves < steps ? step + waves : step);  // the next step's bytes travel while this one is summed
        float d, dmin;
        uint32_t sc_a, sc_b, mn_a, mn_b;
        if constexpr (PLANAR) {
            sc_a = now.sc & 0xffu; sc_b = now.sc >> 8; mn_a = now.mn & 0xffu; mn_b = now.mn >> 8;
            d = half_bits_to_float(now.dm & 0xffffu); dmin = half_bits_to_float(now.dm >> 16);
        } else {
            const uint4 hdr = now.hdr;
            d = half_bits_to_float(hdr.x & 0xffffu); dmin = half_bits_to_float(hdr.x >> 16);
            // sub-blocks 2*pair and 2*pair+1: byte j = (2*pair) & 3 (and j+1) of the three header words
            const uint32_t sh = (pair & 1u) * 16u;
            const uint32_t s2 = (hdr.y >> sh) & 0xffffu, m2 = (hdr.z >> sh) & 0xffffu, e2 = (hdr.w >> sh) & 0xffffu;
            if (pair < 2) {
                sc_a = s2 & 63u; sc_b = (s2 >> 8) & 63u; mn_a = m2 & 63u; mn_b = (m2 >> 8) & 63u;
            } else {
                sc_a = (e2 & 15u) | (((s2 >> 6) & 3u) << 4);
                sc_b = ((e2 >> 8) & 15u) | (((s2 >> 14) & 3u) << 4);
                mn_a = ((e2 >> 4) & 15u) | (((m2 >> 6) & 3u) << 4);
                mn_b = ((e2 >> 12) & 15u) | (((m2 >> 14) & 3u) << 4);
            }
        }
        const uint32_t words[8] = {now.q0.x, now.q0.y, now.q0.z, now.q0.w, now.q1.x, now.q1.y, now.q1.z, now.q1.w};
        int a2 = 0, a1 = 0, a0 = 0, b2 = 0, b1 = 0, b0 = 0;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int lo = int(words[k] & 0x0f0f0f0fu), hi = int((words[k] >> 4) & 0x0f0f0f0fu);
            a2 = __builtin_amdgcn_sdot4(lo, int(pa[2][k]), a2, false);
            a1 = __builtin_amdgcn_sdot4(lo, int(pa[1][k]), a1, false);
            a0 = __builtin_amdgcn_sdot4(lo, int(pa[0][k]), a0, false);
            b2 = __builtin_amdgcn_sdot4(hi, int(pb[2][k]), b2, false);
            b1 = __builtin_amdgcn_sdot4(hi, int(pb[1][k]), b1, false);
            b0 = __builtin_amdgcn_sdot4(hi, int(pb[0][k]), b0, false);
        }
        // each plane's sum is below 2^16 and exact as a float; the three recombine with two roundings to f32
        const float dot_a = __builtin_fmaf(float(a2), 65536.0f, __builtin_fmaf(float(a1), 256.0f, float(a0))) * inv_a;
        const float dot_b = __builtin_fmaf(float(b2), 65536.0f, __builtin_fmaf(float(b1), 256.0f, float(b0))) * inv_b;
        // sum_c ((d*sc)*q - dmin*mn) * x = (d*sc) * sum q x - (dmin*mn) * sum x, per sub-block
        float part = (d * float(sc_a)) * dot_a - (dmin * float(mn_a)) * sxa;
        part += (d * float(sc_b)) * dot_b - (dmin * float(mn_b)) * sxb;
        if (x_bad) part = __uint_as_float(0x7fc00000u);  // a non-finite activation: the row's sum is not a number, and the batch is refused
        const float total = group_sum<LPR>(part);
        if (live && lane % LPR == 0) {
            if (nonfinite(total)) atomicOr(a.error_word, TSP_ERRBIT_NONFINITE);
            y[row] = total;
        }
    }
}

// ------------------------------------------------------------------------------------ launch
uint32_t grid_rows(uint32_t work_items, uint32_t per_block) {
    const uint32_t blocks = (work_items + per_block - 1) / per_block;
    return blocks < 1 ? 1 : blocks > 2048 ? 2048 : blocks;
}

int launch_gemv(uint32_t encoding, uint32_t layout, GemvArgs a, hipStream_t stream) {
    const bool aligned = reinterpret_cast<uintptr_t>(a.matrix) % 16 == 0 && a.expert_stride % 16 == 0;
    if (encoding == 12 && aligned && (layout == TSP_LAYOUT_GGUF || layout == TSP_LAYOUT_PLANAR_V3)) {
        const uint32_t bpr = a.columns / 256;
        const bool planar = layout == TSP_LAYOUT_PLANAR_V3;
#define TSP_Q4K_CASE(N)                                                                                                   \
    if (bpr == N) {                                                                                                       \
        /* at most 1024 workgroups, four per compute unit of a 256-unit GPU: sixteen waves per unit with a step in flight each */ \
        /* keep memory as busy as thirty-two do, and a workgroup's set-up (the activations' digit planes) serves more steps */    \
        /* (measured at 65 536 and 262 144 rows of 2048 columns: 15.2 and 59.4 us against 16.3 and 60.0; two steps in flight */   \
        /* per wave: no faster) */                                                                                              \
        uint32_t blocks = grid_rows((a.rows + 64 / (4 * N) - 1) / (64 / (4 * N)), 4);                                     \
        if (a.count == 1 && blocks > 1024) blocks = 1024;                                                                 \
        const dim3 grid(blocks, a.count);                                                                                 \
        if (planar) TSP_LAUNCH("gemv_q4k", stream, gemv_q4k<N, true><<<grid, 256, 0, stream>>>(a));                                                       \
        else TSP_LAUNCH("gemv_q4k", stream, gemv_q4k<N, false><<<grid, 256, 0, stream>>>(a));                                                             \
        return launch_status("gemv_q4k");                                                                                 \
    }
        TSP_Q4K_CASE(2) TSP_Q4K_CASE(4) TSP_Q4K_CASE(8) TSP_Q4K_CASE(16)
#undef TSP_Q4K_CASE
    }
    TSP_REQUIRE(layout == TSP_LAYOUT_GGUF, "no GEMV kernel for this layout/encoding/shape");
    const dim3 grid(grid_rows(a.rows, 4), a.count);
    const bool ok = dispatch_encoding(encoding, [&]<uint32_t T>() { TSP_LAUNCH("gemv_generic", stream, gemv_generic<T><<<grid, 256, 0, stream>>>(a)); });
    TSP_REQUIRE(ok, "no owned numerical decoder for this encoding");
    return launch_status("gemv_generic");
}

int check_shape(uint32_t encoding, uint32_t layout, uint64_t matrix_bytes, uint32_t columns, uint32_t rows, uint32_t experts,
                tsp_planar_spec* spec, uint64_t* expert_stride) {
    TSP_REQUIRE(tsp_can_decode(encoding) && columns && columns <= 65536 && rows && rows <= 1000000, "unsupported graph GEMV shape/type");
    const auto* enc = find_encoding(encoding);
    TSP_REQUIRE(columns % enc->elements == 0, "GEMV row is not block-aligned");
    std::memset(spec, 0, sizeof *spec);
    if (layout == TSP_LAYOUT_PLANAR_V3) {
        const int rc = tsp_make_expert_spec(encoding, columns, rows, spec);
        if (rc != TSP_OK) return rc;
        *expert_stride = spec->planar_expert_bytes;
    } else {
        TSP_REQUIRE(layout == TSP_LAYOUT_GGUF || (layout == TSP_LAYOUT_Q8_LANES_V1 && encoding == 8), "layout/encoding mismatch");
        *expert_stride = uint64_t(columns / enc->elements) * enc->bytes * rows;
    }
    TSP_REQUIRE(!mul_overflows(*expert_stride, experts) && *expert_stride * experts == matrix_bytes, "graph GEMV buffer shape mismatch");
    return TSP_OK;
}

}  // namespace

extern "C" int tsp_gemv_rows(uint32_t encoding, uint32_t layout, const void* matrix, uint64_t matrix_bytes, const float* x,
                             uint64_t x_stride_bytes, float* y, uint64_t y_stride_bytes, uint32_t count, uint32_t columns,
                             uint32_t rows, uint32_t* error_word, void* stream) {
    GemvArgs a{};
    if (encoding == 8 && count == 1 && layout != TSP_LAYOUT_PLANAR_V3)
        return tsp_q8_matvec_many(layout, matrix, matrix_bytes, x, y, columns, rows, 1, error_word, stream);
    const int rc = check_shape(encoding, layout, matrix_bytes, columns, rows, 1, &a.spec, &a.expert_stride);
    if (rc != TSP_OK) return rc;
    TSP_REQUIRE(matrix && x && y && error_word, "null device pointer");
    TSP_REQUIRE(count && count <= 65535 && x_stride_bytes % 4 == 0 && y_stride_bytes % 4 == 0 &&
                    (count == 1 || (x_stride_bytes >= uint64_t(columns) * 4 && y_stride_bytes >= uint64_t(rows) * 4)),
                "graph GEMV row extent mismatch");
    const uint64_t x_span = uint64_t(count - 1) * x_stride_bytes + uint64_t(columns) * 4;
    const uint64_t y_span = uint64_t(count - 1) * y_stride_bytes + uint64_t(rows) * 4;
    TSP_REQUIRE(!ranges_overlap(y, y_span, matrix, matrix_bytes) && !ranges_overlap(y, y_span, x, x_span),
                "GEMV output overlaps an input");
    a.matrix = static_cast<const uint8_t*>(matrix); a.x = x; a.y = y; a.ids = nullptr;
    a.x_stride = x_stride_bytes; a.y_stride = y_stride_bytes;
    a.columns = columns; a.rows = rows; a.experts = 1; a.count = count; a.error_word = error_word;
    return launch_gemv(encoding, layout, a, static_cast<hipStream_t>(stream));
}

extern "C" int tsp_gemv(uint32_t encoding, uint32_t layout, const void* matrix, uint64_t matrix_bytes, const float* x, float* y,
                        uint32_t columns, uint32_t rows, uint32_t* error_word, void* stream) {
    return tsp_gemv_rows(encoding, layout, matrix, matrix_bytes, x, 0, y, 0, 1, columns, rows, error_word, stream);
}

extern "C" int tsp_routed_gemv(uint32_t encoding, const void* matrices, uint64_t matrices_bytes, const uint32_t* ids, const float* x,
                               float* y, uint32_t columns, uint32_t rows, uint32_t experts, uint32_t selected, int broadcast_input,
                               uint32_t* error_word, void* stream) {
    GemvArgs a{};
    TSP_REQUIRE(experts && experts <= 4096 && selected && selected <= 64, "invalid routed GEMV routing shape");
    const int rc = check_shape(encoding, TSP_LAYOUT_GGUF, matrices_bytes, columns, rows, experts, &a.spec, &a.expert_stride);
    if (rc != TSP_OK) return rc;
    TSP_REQUIRE(matrices && ids && x && y && error_word, "null device pointer");
    const uint64_t x_span = uint64_t(broadcast_input ? 1 : selected) * columns * 4, y_span = uint64_t(selected) * rows * 4;
    TSP_REQUIRE(!ranges_overlap(y, y_span, matrices, matrices_bytes) && !ranges_overlap(y, y_span, x, x_span) &&
                    !ranges_overlap(y, y_span, ids, uint64_t(selected) * 4),
                "routed GEMV output overlaps an input");
    a.matrix = static_cast<const uint8_t*>(matrices); a.x = x; a.y = y; a.ids = ids;
    a.x_stride = broadcast_input ? 0 : uint64_t(columns) * 4; a.y_stride = uint64_t(rows) * 4;
    a.columns = columns; a.rows = rows; a.experts = experts; a.count = selected; a.error_word = error_word;
    return launch_gemv(encoding, TSP_LAYOUT_GGUF, a, static_cast<hipStream_t>(stream));
}
