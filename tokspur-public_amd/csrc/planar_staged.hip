// The grouped MoE products for the planar kinds the integer-factor kernels have no unpacking for: Q5_K and Q8_0 co-located gate / up
// (include/tokspur/planar_pack_v3.hpp kinds 4-7) with fused SwiGLU, Q5_1 and Q8_0 planes down (kinds 8, 9). They plug into the same
// pipeline as the Q4_K / Q6_K kernels: the same 64-row task list, the same f16 activation rows, the same h rows (the half nearest
// h / 256, grouped by task slot), so any gate/up kind combines with any down kind.
//
// Arithmetic: every weight is decoded in f32 from its planes and rounded once to half (the engine stages halves the same way,
// kernels/planar_moe_v3.metal:2406-2483); activations are the f16 rows the pipeline already holds; f32 accumulation.
// One workgroup of four waves works off one task for 128 output columns; a wave owns 32 of them and both 32-row tiles of the
// task. A lane (c = lane % 32, s = lane / 32) decodes columns 16 s .. 16 s + 15 of every 32-column block of its weight row
// straight into the B fragments of two v_mfma_f32_32x32x16_f16 and reads the same columns of its activation rows as the A
// fragments. No LDS, no barrier.
#include "planar_staged.hpp"

using namespace tsp;

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float half_at(const uint8_t* p) { return half_bits_to_float(*reinterpret_cast<const uint16_t*>(p)); }
__device__ __forceinline__ uint32_t byte_of(const uint4& v, int i) { return ((i < 4 ? v.x : i < 8 ? v.y : i < 12 ? v.z : v.w) >> (8 * (i % 4))) & 0xffu; }

// sixteen weights of row `row` of one planar expert: columns 32 kb + 16 s .. + 15, as halves
template <int T>
__device__ __forceinline__ void planar16(const uint8_t* __restrict__ e, const tsp_planar_spec& p, uint32_t row, uint32_t kb, uint32_t s, f16x8& lo, f16x8& hi) {
    _Float16 out[16];
    if constexpr (T == 12 || T == 13) {
        const uint64_t blk = uint64_t(row) * p.blocks_per_row + kb / 8;
        const uint32_t g = kb % 8;
        const uint4 nib = *reinterpret_cast<const uint4*>(e + p.qs_offset + blk * 128 + (g >> 1) * 32 + 16 * s);
        uint4 fifth = {0, 0, 0, 0};
        if constexpr (T == 13) fifth = *reinterpret_cast<const uint4*>(e + p.qh_offset + blk * 32 + 16 * s);
        const uint8_t* sm = e + p.sm_offset + blk * 16;
        const uint8_t* dm = e + p.dm_offset + blk * 4;
        const float dl = half_at(dm) * float(sm[g]), ml = half_at(dm + 2) * float(sm[8 + g]);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            uint32_t q = (byte_of(nib, i) >> ((g & 1u) * 4u)) & 15u;
            if constexpr (T == 13) q |= ((byte_of(fifth, i) >> g) & 1u) << 4;
            out[i] = _Float16(dl * float(q) - ml);
        }
    } else if constexpr (T == 7) {
        const uint64_t blk = uint64_t(row) * p.blocks_per_row + kb;
        const uint4 nib = *reinterpret_cast<const uint4*>(e + p.qs_offset + blk * 16);
        const uint32_t qh = *reinterpret_cast<const uint32_t*>(e + p.qh_offset + blk * 4) >> (16 * s);
        const uint8_t* dm = e + p.dm_offset + blk * 4;
        const float d = half_at(dm), m = half_at(dm + 2);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t q = ((byte_of(nib, i) >> (4 * s)) & 15u) | (((qh >> i) & 1u) << 4);
            out[i] = _Float16(d * float(q) + m);
        }
    } else {
        static_assert(T == 8);
        const uint64_t blk = uint64_t(row) * p.blocks_per_row + kb;
        const uint4 q = *reinterpret_cast<const uint4*>(e + p.qs_offset + blk * 32 + 16 * s);
        const float d = half_at(e + p.dm_offset + blk * 2);
#pragma unroll
        for (int i = 0; i < 16; ++i) out[i] = _Float16(d * float(int(int8_t(byte_of(q, i)))));
    }
    lo = f16x8{out[0], out[1], out[2], out[3], out[4], out[5], out[6], out[7]};
    hi = f16x8{out[8], out[9], out[10], out[11], out[12], out[13], out[14], out[15]};
}

// The task of this workgroup and the routes of its rows: lane c of every wave holds the routes of rows c and c + 32.
struct Task {
    uint32_t expert, nrows, rid[2];
    uint32_t bad;
    bool live;
};
__device__ __forceinline__ Task resolve(const PlanarStagedArgs& a, uint32_t task, uint32_t c, bool reporter) {
    Task t{0, 0, {0xffffffffu, 0xffffffffu}, 0, false};
    const uint32_t listed = a.task_list[0];
    if (listed > a.task_slots || a.task_list[1] != a.tokens * a.selected) {
        if (reporter && task == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
        return t;
    }
    if (task >= listed) return t;
    t.expert = a.task_list[2 + 2 * task];
    const uint32_t start = a.task_list[3 + 2 * task];
    const uint32_t count = t.expert < a.experts ? a.counts[t.expert] : 0;
    if (t.expert >= a.experts || count > a.tokens || start >= count) {
        if (reporter) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
        return t;
    }
    t.nrows = count - start < 64 ? count - start : 64;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t r = c + 32 * i;
        uint32_t rid = a.token_map[uint64_t(t.expert) * a.tokens + start + (r < t.nrows ? r : 0)];  // rows past the end re-read the first
        if (rid >= a.tokens * a.selected || a.ids[rid] != t.expert) { t.bad = TSP_ERRBIT_INDEX; rid = 0xffffffffu; }
        t.rid[i] = rid;
    }
    t.live = true;
    return t;
}

__device__ __forceinline__ f16x8 halves8(const _Float16* p) { return *reinterpret_cast<const f16x8*>(p); }

// h[task slot, unit] = silu(gate_e . x) * (up_e . x), stored as the half nearest h / 256
template <int T>
__global__ __launch_bounds__(256) void planar_staged_gate_up(PlanarStagedArgs a) {
    const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, c = lane % 32, s = lane / 32;
    const uint32_t task = blockIdx.y;
    Task t = resolve(a, task, c, threadIdx.x == 0 && blockIdx.x == 0);
    if (!t.live) return;
    const uint32_t first = blockIdx.x * 128 + wave * 32;
    if (first >= a.hidden) { publish_error(t.bad, a.error_word); return; }
    const uint32_t unit = first + c < a.hidden ? first + c : a.hidden - 1;
    const uint32_t half_experts = a.experts / 2;
    const uint8_t* gate = (t.expert < half_experts ? a.pair_lo : a.pair_hi) + uint64_t(t.expert < half_experts ? t.expert : t.expert - half_experts) * 2 * a.spec.planar_expert_bytes;
    const uint8_t* up = gate + a.spec.planar_expert_bytes;
    const _Float16* x[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) x[i] = a.xh + uint64_t(t.rid[i] == 0xffffffffu ? 0 : t.rid[i] / a.selected) * a.channels + 16 * s;
    const bool two = t.nrows > 32;

    f32x16 g[2] = {}, u[2] = {};
    const uint32_t blocks = a.channels / 32;
    for (uint32_t kb = 0; kb < blocks; ++kb) {
        f16x8 g0, g1, u0, u1;
        planar16<T>(gate, a.spec, unit, kb, s, g0, g1);
        planar16<T>(up, a.spec, unit, kb, s, u0, u1);
        const f16x8 a0 = halves8(x[0] + kb * 32), a1 = halves8(x[0] + kb * 32 + 8);
        g[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, g0, g[0], 0, 0, 0);
        u[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, u0, u[0], 0, 0, 0);
        g[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, g1, g[0], 0, 0, 0);
        u[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, u1, u[0], 0, 0, 0);
        if (two) {
            const f16x8 b0 = halves8(x[1] + kb * 32), b1 = halves8(x[1] + kb * 32 + 8);
            g[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b0, g0, g[1], 0, 0, 0);
            u[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b0, u0, u[1], 0, 0, 0);
            g[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b1, g1, g[1], 0, 0, 0);
            u[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b1, u1, u[1], 0, 0, 0);
        }
    }
    uint32_t bad = t.bad;
    const bool unit_live = first + c < a.hidden;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t row = 32 * i + 8 * (v / 4) + 4 * s + v % 4;  // D[row][unit]: unit = lane % 32
            if (row < t.nrows && unit_live) {
                const float gv = g[i][v];
                const float h = gv * sigmoid_stable(gv) * u[i][v];
                const _Float16 carried = _Float16(h * (1.0f / 256.0f));
                bad |= (nonfinite(h) || (__builtin_bit_cast(uint16_t, carried) & 0x7c00u) == 0x7c00u) ? TSP_ERRBIT_NONFINITE : 0u;
                a.hbuf[(uint64_t(task) * 64 + row) * a.hidden + first + c] = carried;
            }
        }
    }
    publish_error(bad, a.error_word);
}

// y[rid, channel] = 256 * (down_e[channel, :] . hbuf[task slot, :])
template <int T>
__global__ __launch_bounds__(256) void planar_staged_down(PlanarStagedArgs a) {
    const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, c = lane % 32, s = lane / 32;
    const uint32_t task = blockIdx.y;
    Task t = resolve(a, task, c, threadIdx.x == 0 && blockIdx.x == 0);
    if (!t.live) return;
    const uint32_t first = blockIdx.x * 128 + wave * 32;
    if (first >= a.channels) return;  // the route check is reported by the first column tile's waves
    const uint32_t channel = first + c < a.channels ? first + c : a.channels - 1;
    const uint8_t* down = a.down + uint64_t(t.expert) * a.down_spec.planar_expert_bytes;
    const _Float16* h[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) h[i] = a.hbuf + (uint64_t(task) * 64 + (c + 32 * i < t.nrows ? c + 32 * i : 0)) * a.hidden + 16 * s;
    const bool two = t.nrows > 32;

    f32x16 acc[2] = {};
    const uint32_t blocks = a.hidden / 32;
    for (uint32_t kb = 0; kb < blocks; ++kb) {
        f16x8 w0, w1;
        planar16<T>(down, a.down_spec, channel, kb, s, w0, w1);
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(halves8(h[0] + kb * 32), w0, acc[0], 0, 0, 0);
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(halves8(h[0] + kb * 32 + 8), w1, acc[0], 0, 0, 0);
        if (two) {
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(halves8(h[1] + kb * 32), w0, acc[1], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(halves8(h[1] + kb * 32 + 8), w1, acc[1], 0, 0, 0);
        }
    }
    uint32_t bad = t.bad;
    const bool channel_live = first + c < a.channels;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t in_tile = 8 * (v / 4) + 4 * s + v % 4, row = 32 * i + in_tile;
            const uint32_t dest = __shfl(t.rid[i], in_tile, kWave);  // lane r (< 32) holds the routes of rows r and r + 32
            if (row < t.nrows && dest != 0xffffffffu && channel_live) {
                const float value = acc[i][v] * 256.0f;
                bad |= nonfinite(value) ? TSP_ERRBIT_NONFINITE : 0u;
                reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.y) + uint64_t(dest) * a.y_stride)[first + c] = value;
            }
        }
    }
    publish_error(bad, a.error_word);
}

}  // namespace

namespace tsp {

bool planar_staged_gate_up_takes(uint32_t gate_kind, uint32_t up_kind) {
    return (gate_kind == TSP_KIND_Q5K_COLOC_GATE && up_kind == TSP_KIND_Q5K_COLOC_UP) || (gate_kind == TSP_KIND_Q8_COLOC_GATE && up_kind == TSP_KIND_Q8_COLOC_UP);
}
bool planar_staged_down_takes(uint32_t down_kind) { return down_kind == TSP_KIND_Q51_PLANAR || down_kind == TSP_KIND_Q8_PLANAR; }

int launch_planar_staged_gate_up(const PlanarStagedArgs& a, hipStream_t s) {
    const dim3 grid((a.hidden + 127) / 128, a.task_slots);
    if (a.spec.source_type == 13) TSP_LAUNCH("gemm_gate_up_swiglu_staged", s, planar_staged_gate_up<13><<<grid, 256, 0, s>>>(a));
    else TSP_LAUNCH("gemm_gate_up_swiglu_staged", s, planar_staged_gate_up<8><<<grid, 256, 0, s>>>(a));
    return launch_status("gemm_gate_up_swiglu_staged");
}
int launch_planar_staged_down(const PlanarStagedArgs& a, hipStream_t s) {
    const dim3 grid((a.channels + 127) / 128, a.task_slots);
    if (a.down_spec.source_type == 7) TSP_LAUNCH("gemm_down_staged", s, planar_staged_down<7><<<grid, 256, 0, s>>>(a));
    else TSP_LAUNCH("gemm_down_staged", s, planar_staged_down<8><<<grid, 256, 0, s>>>(a));
    return launch_status("gemm_down_staged");
}

}  // namespace tsp
