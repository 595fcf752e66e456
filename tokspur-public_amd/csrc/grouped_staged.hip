// Grouped dequant-GEMM over expert stacks in the encodings and row layouts that the integer-factor Q4_K kernel does not
// take: Q5_1, Q8_0 and Q5_K in GGUF rows, Q8_0 in q8_lanes_v1 rows, Q5_1 in q51_lanes_v1 rows.
//
// The arithmetic is the engine's declared one for this operator (kernels/grouped_mm.metal:24-243): every weight is decoded in
// f32 and rounded once to half, every activation is rounded once to half, products accumulate in f32.
//
// One workgroup of four waves works off one 32-route task (the engine's task list: tasks[2 + 2 t] = expert, start) for 128
// weight rows; a wave owns 32 of them. Per 32-column block a lane decodes sixteen weights of its row straight into the B
// fragments of two v_mfma_f32_32x32x16_f16 and converts sixteen activations of its route into the A fragments: lane
// (r = lane % 32, h = lane / 32) takes columns 16 h .. 16 h + 15 of the block on both sides, so the order in which columns
// meet inside an instruction is the same for A and B. Nothing goes through LDS and there is no barrier; the four waves
// re-read the task's activation rows through the caches.
#include "grouped_staged.hpp"

using namespace tsp;

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float half_at(const uint8_t* p) { return half_bits_to_float(uint32_t(p[0]) | (uint32_t(p[1]) << 8)); }

// sixteen weights of one row: block `kb` of 32 columns, half `h` of it, as halves
template <int ENC, int LAYOUT>
__device__ __forceinline__ void decode16(const uint8_t* __restrict__ row, uint32_t kb, uint32_t h, uint32_t blocks, _Float16 (&out)[16]) {
    if constexpr (ENC == 8 && LAYOUT == TSP_LAYOUT_GGUF) {
        const uint8_t* p = row + uint64_t(kb) * 34;
        const float d = half_at(p);
        const uint16_t* q = reinterpret_cast<const uint16_t*>(p + 2 + 16 * h);  // rows and blocks are even-sized: 2-byte aligned
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t two = q[i];
            out[2 * i] = _Float16(d * float(int8_t(two & 0xff)));
            out[2 * i + 1] = _Float16(d * float(int8_t(two >> 8)));
        }
    } else if constexpr (ENC == 8) {  // q8_lanes_v1: [f16 scales x blocks][runs of 16 blocks: quant i of the run's blocks side by side]
        const float d = half_at(row + 2 * kb);
        const uint32_t run = kb / 16, left = blocks - run * 16, width = left < 16 ? left : 16;
        const uint8_t* q = row + 2 * uint64_t(blocks) + uint64_t(run) * 512 + kb % 16;
#pragma unroll
        for (int i = 0; i < 16; ++i) out[i] = _Float16(d * float(int8_t(q[(16 * h + i) * width])));
    } else if constexpr (ENC == 7) {
        const uint8_t* head = LAYOUT == TSP_LAYOUT_GGUF ? row + uint64_t(kb) * 24 : row + uint64_t(kb) * 8;
        const float d = half_at(head), m = half_at(head + 2);
        const uint32_t qh = *reinterpret_cast<const uint32_t*>(head + 4) >> (16 * h);
        uint32_t width = 1;
        const uint8_t* q = head + 8;
        if constexpr (LAYOUT != TSP_LAYOUT_GGUF) {  // q51_lanes_v1: [8-byte heads x blocks][runs of 16 blocks: quant byte i side by side]
            const uint32_t run = kb / 16, left = blocks - run * 16;
            width = left < 16 ? left : 16;
            q = row + 8 * uint64_t(blocks) + uint64_t(run) * 256 + kb % 16;
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t v = ((uint32_t(q[i * width]) >> (4 * h)) & 15u) | (((qh >> i) & 1u) << 4);
            out[i] = _Float16(d * float(v) + m);
        }
    } else {  // Q5_K: 176 bytes per 256 columns: d, dmin, 12 bytes of 6-bit scales and minima, 32 bytes of fifth bits, 128 of nibbles
        const uint8_t* p = row + uint64_t(kb / 8) * 176;
        const uint32_t g = kb % 8;
        const uint8_t* s = p + 4;
        uint32_t sc, mn;
        if (g < 4) { sc = s[g] & 63u; mn = s[4 + g] & 63u; }
        else { sc = (s[4 + g] & 15u) | ((s[g - 4] >> 6) << 4); mn = (s[4 + g] >> 4) | ((s[g] >> 6) << 4); }
        const float dl = half_at(p) * float(sc), ml = half_at(p + 2) * float(mn);
        const uint8_t* fifth = p + 16 + 16 * h;
        const uint8_t* nib = p + 48 + (g / 2) * 32 + 16 * h;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t v = ((uint32_t(nib[i]) >> (4 * (g & 1))) & 15u) | (((uint32_t(fifth[i]) >> g) & 1u) << 4);
            out[i] = _Float16(dl * float(v) - ml);
        }
    }
}

template <int ENC, int LAYOUT>
__global__ __launch_bounds__(256) void grouped_staged_kernel(GroupedStagedArgs a) {
    const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, r = lane % 32, h = lane / 32;
    const uint32_t task = blockIdx.y;
    const uint32_t listed = a.tasks[0];
    if (listed > a.maximum_tasks || a.tasks[1] != a.tokens * a.selected) {  // a task list that is not this call's
        if (threadIdx.x == 0 && blockIdx.x == 0 && task == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
        return;
    }
    if (task >= listed) return;
    const uint32_t expert = a.tasks[2 + 2 * task], start = a.tasks[3 + 2 * task];
    const uint32_t count = expert < a.experts ? a.counts[expert] : 0;
    if (expert >= a.experts || start >= a.tokens || count > a.tokens || start >= count) {
        if (threadIdx.x == 0 && blockIdx.x == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
        return;
    }
    const uint32_t n = count - start < 32 ? count - start : 32;
    // the route of this lane's activation row; rows past the task's end re-read its first route and are never stored
    uint32_t rid = a.token_map[uint64_t(expert) * a.tokens + start + (r < n ? r : 0)];
    uint32_t bad = 0;
    if (rid >= a.tokens * a.selected || a.ids[rid] != expert) { bad = TSP_ERRBIT_INDEX; rid = 0xffffffffu; }
    const uint32_t in_row = rid == 0xffffffffu ? 0 : a.broadcast ? rid / a.selected : rid;
    const float* x = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(a.input) + uint64_t(in_row) * a.input_stride) + 16 * h;

    const uint32_t first = blockIdx.x * 128 + wave * 32;
    if (first >= a.rows) { publish_error(bad, a.error_word); return; }
    const uint32_t wrow = first + r < a.rows ? first + r : a.rows - 1;  // a ragged last tile re-reads the last row
    const uint8_t* w = a.matrices + uint64_t(expert) * a.expert_stride + uint64_t(wrow) * a.row_bytes;
    const uint32_t blocks = a.columns / 32;

    f32x16 acc = {};
    for (uint32_t kb = 0; kb < blocks; ++kb) {
        _Float16 wv[16];
        decode16<ENC, LAYOUT>(w, kb, h, blocks, wv);
        const float4* xp = reinterpret_cast<const float4*>(x + kb * 32);
        const float4 x0 = xp[0], x1 = xp[1], x2 = xp[2], x3 = xp[3];
        const f16x8 a0 = {_Float16(x0.x), _Float16(x0.y), _Float16(x0.z), _Float16(x0.w), _Float16(x1.x), _Float16(x1.y), _Float16(x1.z), _Float16(x1.w)};
        const f16x8 a1 = {_Float16(x2.x), _Float16(x2.y), _Float16(x2.z), _Float16(x2.w), _Float16(x3.x), _Float16(x3.y), _Float16(x3.z), _Float16(x3.w)};
        const f16x8 b0 = {wv[0], wv[1], wv[2], wv[3], wv[4], wv[5], wv[6], wv[7]};
        const f16x8 b1 = {wv[8], wv[9], wv[10], wv[11], wv[12], wv[13], wv[14], wv[15]};
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, b0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b1, acc, 0, 0, 0);
    }
    // D[i][j]: j = lane % 32 is the weight row, i = 8 (v / 4) + 4 (lane / 32) + v % 4 the route of the task
    const bool row_live = first + r < a.rows;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const uint32_t i = 8 * (v / 4) + 4 * h + v % 4;
        const uint32_t dest = __shfl(rid, i, kWave);  // lane i (< 32) holds route i
        if (i < n && dest != 0xffffffffu && row_live) {
            const float value = acc[v];
            bad |= nonfinite(value) ? TSP_ERRBIT_NONFINITE : 0u;
            reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.output) + uint64_t(dest) * a.output_stride)[first + r] = value;
        }
    }
    publish_error(bad, a.error_word);
}

template <int ENC, int LAYOUT>
int launch_as(const GroupedStagedArgs& a, hipStream_t s) {
    const dim3 grid((a.rows + 127) / 128, a.maximum_tasks);
    TSP_LAUNCH("gemm_grouped_staged", s, grouped_staged_kernel<ENC, LAYOUT><<<grid, 256, 0, s>>>(a));
    return launch_status("gemm_grouped_staged");
}

}  // namespace

namespace tsp {

bool grouped_staged_takes(uint32_t encoding, uint32_t layout) {
    return (layout == TSP_LAYOUT_GGUF && (encoding == 7 || encoding == 8 || encoding == 13)) || (layout == TSP_LAYOUT_Q8_LANES_V1 && encoding == 8) ||
           (layout == TSP_LAYOUT_Q51_LANES_V1 && encoding == 7);
}

int launch_grouped_staged(uint32_t encoding, uint32_t layout, const GroupedStagedArgs& a, hipStream_t s) {
    if (layout == TSP_LAYOUT_Q8_LANES_V1) return launch_as<8, TSP_LAYOUT_Q8_LANES_V1>(a, s);
    if (layout == TSP_LAYOUT_Q51_LANES_V1) return launch_as<7, TSP_LAYOUT_Q51_LANES_V1>(a, s);
    if (encoding == 7) return launch_as<7, TSP_LAYOUT_GGUF>(a, s);
    if (encoding == 8) return launch_as<8, TSP_LAYOUT_GGUF>(a, s);
    return launch_as<13, TSP_LAYOUT_GGUF>(a, s);
}

}  // namespace tsp
