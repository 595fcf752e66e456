// The grouped MoE products for the planar kinds the integer-factor kernels have no unpacking for: Q5_K and Q8_0 co-located gate / up
// (include/tokspur/planar_pack_v3.hpp kinds 4-7) with fused SwiGLU, Q5_1 and Q8_0 planes down (kinds 8, 9). They plug into the same
// pipeline as the Q4_K / Q6_K kernels: the same 64-row task list, the same f16 activation rows, the same h rows (the half nearest
// h / 256, grouped by task slot), so any gate/up kind combines with any down kind.
//
// Arithmetic: every weight is decoded in f32 from its planes and rounded once to half (the engine stages halves the same way,
// kernels/planar_moe_v3.metal:2406-2483); activations are the f16 rows the pipeline already holds; f32 accumulation.
// One workgroup of four waves works off one task for 128 hidden units (gate/up: a wave owns 32 units, i.e. 32 gate rows and 32
// up rows) or 256 output channels (down: 64 per wave) and both 32-row tiles of the task. A lane (c = lane % 32, s = lane / 32) decodes columns 16 s .. 16 s + 15 of every 32-column block of its weight row
// straight into the B fragments of two v_mfma_f32_32x32x16_f16 and reads the same columns of its activation rows as the A
// fragments; the next block's bytes are requested before the current block is decoded. No LDS, no barrier.
#include "planar_staged.hpp"

#include "mfma_quant.hpp"

using namespace tsp;

namespace {

__device__ __forceinline__ float half_at(const uint8_t* p) { return half_bits_to_float(*reinterpret_cast<const uint16_t*>(p)); }
__device__ __forceinline__ uint32_t byte_of(const uint4& v, int i) { return ((i < 4 ? v.x : i < 8 ? v.y : i < 12 ? v.z : v.w) >> (8 * (i % 4))) & 0xffu; }

// The bytes of sixteen weights of row `row` of one planar expert (columns 32 kb + 16 s .. + 15) as they come from memory, and
// their decoding to halves: two steps, so that the next block's bytes can be on their way while this block is multiplied.
struct Raw16 {
    uint4 q;       // nibbles (K kinds, Q5_1) or int8 quants (Q8_0)
    uint4 fifth;   // Q5_K: the bytes holding the fifth bits; Q5_1: .x = the block's 32 fifth bits
    float a, b;    // K kinds: d * sc and dmin * mn; Q5_1: d and m; Q8_0: d
    uint32_t g;    // K kinds: the sub-block within its super-block
};
template <int T>
__device__ __forceinline__ Raw16 fetch16(const uint8_t* __restrict__ e, const tsp_planar_spec& p, uint32_t row, uint32_t kb, uint32_t s) {
    Raw16 r{};
    if constexpr (T == 12 || T == 13) {
        const uint64_t blk = uint64_t(row) * p.blocks_per_row + kb / 8;
        r.g = kb % 8;
        r.q = *reinterpret_cast<const uint4*>(e + p.qs_offset + blk * 128 + (r.g >> 1) * 32 + 16 * s);
        if constexpr (T == 13) r.fifth = *reinterpret_cast<const uint4*>(e + p.qh_offset + blk * 32 + 16 * s);
        const uint8_t* sm = e + p.sm_offset + blk * 16;
        const uint8_t* dm = e + p.dm_offset + blk * 4;
        r.a = half_at(dm) * float(sm[r.g]);
        r.b = half_at(dm + 2) * float(sm[8 + r.g]);
    } else if constexpr (T == 7) {
        const uint64_t blk = uint64_t(row) * p.blocks_per_row + kb;
        r.q = *reinterpret_cast<const uint4*>(e + p.qs_offset + blk * 16);
        r.fifth.x = *reinterpret_cast<const uint32_t*>(e + p.qh_offset + blk * 4) >> (16 * s);
        const uint8_t* dm = e + p.dm_offset + blk * 4;
        r.a = half_at(dm);
        r.b = half_at(dm + 2);
    } else {
        static_assert(T == 8);
        const uint64_t blk = uint64_t(row) * p.blocks_per_row + kb;
        r.q = *reinterpret_cast<const uint4*>(e + p.qs_offset + blk * 32 + 16 * s);
        r.a = half_at(e + p.dm_offset + blk * 2);
    }
    return r;
}
template <int T>
__device__ __forceinline__ void decode16(const Raw16& r, uint32_t s, f16x8& lo, f16x8& hi) {
    _Float16 out[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        if constexpr (T == 12 || T == 13) {
            uint32_t q = (byte_of(r.q, i) >> ((r.g & 1u) * 4u)) & 15u;
            if constexpr (T == 13) q |= ((byte_of(r.fifth, i) >> r.g) & 1u) << 4;
            out[i] = _Float16(r.a * float(q) - r.b);
        } else if constexpr (T == 7) {
            const uint32_t q = ((byte_of(r.q, i) >> (4 * s)) & 15u) | (((r.fifth.x >> i) & 1u) << 4);
            out[i] = _Float16(r.a * float(q) + r.b);
        } else {
            out[i] = _Float16(r.a * float(int(int8_t(byte_of(r.q, i)))));
        }
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
    Raw16 rg = fetch16<T>(gate, a.spec, unit, 0, s), ru = fetch16<T>(up, a.spec, unit, 0, s);
    f16x8 a0 = halves8(x[0]), a1 = halves8(x[0] + 8), b0 = halves8(x[1]), b1 = halves8(x[1] + 8);
    for (uint32_t kb = 0; kb < blocks; ++kb) {
        // the next block's bytes are requested before this block is decoded (the last step re-reads its own)
        const uint32_t nb = kb + 1 < blocks ? kb + 1 : kb;
        const Raw16 ng = fetch16<T>(gate, a.spec, unit, nb, s), nu = fetch16<T>(up, a.spec, unit, nb, s);
        const f16x8 na0 = halves8(x[0] + nb * 32), na1 = halves8(x[0] + nb * 32 + 8);
        const f16x8 nb0 = halves8(x[1] + nb * 32), nb1 = halves8(x[1] + nb * 32 + 8);
        f16x8 g0, g1, u0, u1;
        decode16<T>(rg, s, g0, g1);
        decode16<T>(ru, s, u0, u1);
        g[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, g0, g[0], 0, 0, 0);
        u[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, u0, u[0], 0, 0, 0);
        g[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, g1, g[0], 0, 0, 0);
        u[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, u1, u[0], 0, 0, 0);
        if (two) {
            g[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b0, g0, g[1], 0, 0, 0);
            u[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b0, u0, u[1], 0, 0, 0);
            g[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b1, g1, g[1], 0, 0, 0);
            u[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b1, u1, u[1], 0, 0, 0);
        }
        rg = ng; ru = nu; a0 = na0; a1 = na1; b0 = nb0; b1 = nb1;
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

// y[rid, channel] = 256 * (down_e[channel, :] . hbuf[task slot, :]). A wave owns 64 channels (two column tiles), so that one set
// of A fragments serves twice the weights: what these launches ask of the L1 path is mostly the tasks' h rows.
//
// STAGED: the task's h rows (64 consecutive rows of hbuf, at most 64 KB) are brought into LDS once per workgroup by direct global ->
// LDS loads, a kilobyte of consecutive bytes per instruction, and every A fragment is an LDS read. Read straight from memory, a
// fragment load touches 32 different cache lines (one per row), four times per block and wave, and the address path of the L1
// bounds the launch. 16-byte chunk j of row r sits at slot j ^ (r % 16) of its row, so that the 16 rows a quarter-wave reads at
// once fall into different banks. For 128 <= hidden <= 512 in multiples of 128; other widths read from memory.
//
// A workgroup's life starts with a chain of dependent look-ups (task list -> counts -> token_map -> ids); with two workgroups per
// CU nothing hides them, so everything that does not need their results is requested first: the h rows need only the task's
// slot, the first weight bytes only the expert id, and the routes are not needed before the epilogue.
template <int T, bool STAGED>
__global__ __launch_bounds__(256) void planar_staged_down(PlanarStagedArgs a) {
    extern __shared__ __align__(16) uint8_t staged_rows[];
    const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, c = lane % 32, s = lane / 32;
    const uint32_t task = blockIdx.y;
    const bool reporter = threadIdx.x == 0 && blockIdx.x == 0;
    const uint32_t row_bytes = a.hidden * 2;
    if constexpr (STAGED) {
        const uint32_t per_row = row_bytes / 16, chunks = 64 * per_row;  // slots of 16 bytes; all 64 rows are loaded: hbuf has them
        const uint8_t* rows = reinterpret_cast<const uint8_t*>(a.hbuf + uint64_t(task) * 64 * a.hidden);
        for (uint32_t at = wave * kWave; at < chunks; at += 4 * kWave) {
            const uint32_t slot = at + lane, r = slot / per_row, j = slot % per_row;
            load_to_lds_16(rows, r * row_bytes + ((j ^ (r % 16)) * 16), uint32_t(__builtin_amdgcn_readfirstlane(int(lds_address(staged_rows) + at * 16))));
        }
    }
    // a workgroup that has nothing to do still waits for the bytes it asked to be written into its LDS
    const auto leave = [&](bool flag) {
        if (flag && reporter) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
        if constexpr (STAGED) wait_all_loads();
    };
    const uint32_t listed = a.task_list[0];
    if (listed > a.task_slots || a.task_list[1] != a.tokens * a.selected) { leave(task == 0); return; }
    if (task >= listed) { leave(false); return; }
    const uint32_t expert = a.task_list[2 + 2 * task], start = a.task_list[3 + 2 * task];
    if (expert >= a.experts) { leave(true); return; }
    const uint32_t first = blockIdx.x * 256 + wave * 64;
    const bool wave_live = first < a.channels;
    uint32_t channel[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) channel[j] = first + 32 * j + c < a.channels ? first + 32 * j + c : a.channels - 1;
    const uint8_t* down = a.down + uint64_t(expert) * a.down_spec.planar_expert_bytes;
    const uint32_t blocks = a.hidden / 32;
    constexpr uint32_t kQuad = 4;
    Raw16 cur[2][kQuad], nxt[2][kQuad];
    const auto fetch_quad = [&](Raw16 (&into)[2][kQuad], uint32_t kb0) {
#pragma unroll
        for (uint32_t q = 0; q < kQuad; ++q) {
            const uint32_t kb = kb0 + q < blocks ? kb0 + q : blocks - 1;  // past the end: the last block again, never multiplied
#pragma unroll
            for (int j = 0; j < 2; ++j) into[j][q] = fetch16<T>(down, a.down_spec, channel[j], kb, s);
        }
    };
    fetch_quad(cur, 0);
    const uint32_t count = a.counts[expert];
    if (count > a.tokens || start >= count) { leave(true); return; }
    Task t{expert, count - start < 64 ? count - start : 64, {0xffffffffu, 0xffffffffu}, 0, true};
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t r = c + 32 * i;
        uint32_t rid = a.token_map[uint64_t(expert) * a.tokens + start + (r < t.nrows ? r : 0)];  // rows past the end re-read the first
        if (rid >= a.tokens * a.selected || a.ids[rid] != expert) { t.bad = TSP_ERRBIT_INDEX; rid = 0xffffffffu; }
        t.rid[i] = rid;
    }
    if constexpr (STAGED) {
        wait_all_loads();
        __syncthreads();
    }
    if (!wave_live) return;  // the route check is reported by the first column tile's waves
    const _Float16* h[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) h[i] = a.hbuf + (uint64_t(task) * 64 + (c + 32 * i < t.nrows ? c + 32 * i : 0)) * a.hidden + 16 * s;
    const bool two = t.nrows > 32;

    f32x16 acc[2][2] = {};  // [row tile][column tile]
    // fragment f (0, 1) of row tile i for block kb: halves 32 kb + 16 s + 8 f .. + 7 of row 32 i + c
    const auto fragment = [&](uint32_t i, uint32_t kb, uint32_t f) {
        if constexpr (STAGED) {
            const uint32_t r = 32 * i + c, j = kb * 4 + 2 * s + f;
            return *reinterpret_cast<const f16x8*>(staged_rows + r * row_bytes + ((j ^ (r % 16)) * 16));
        } else {
            return halves8(h[i] + kb * 32 + 8 * f);
        }
    };
    // Four blocks (128 columns: one cache line of a Q8_0 row's quants) per step; the next step's weight bytes are requested
    // before this step is decoded, so a round trip to memory is paid once per four blocks and hidden behind them.
    for (uint32_t kb0 = 0; kb0 < blocks; kb0 += kQuad) {
        fetch_quad(nxt, kb0 + kQuad);
#pragma unroll
        for (uint32_t q = 0; q < kQuad; ++q) {
            const uint32_t kb = kb0 + q;
            if (kb < blocks) {  // uniform
                f16x8 w0, w1, v0, v1;
                decode16<T>(cur[0][q], s, w0, w1);
                decode16<T>(cur[1][q], s, v0, v1);
                const f16x8 a0 = fragment(0, kb, 0), a1 = fragment(0, kb, 1);
                acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, w0, acc[0][0], 0, 0, 0);
                acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, v0, acc[0][1], 0, 0, 0);
                acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, w1, acc[0][0], 0, 0, 0);
                acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, v1, acc[0][1], 0, 0, 0);
                if (two) {
                    const f16x8 b0 = fragment(1, kb, 0), b1 = fragment(1, kb, 1);
                    acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b0, w0, acc[1][0], 0, 0, 0);
                    acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b0, v0, acc[1][1], 0, 0, 0);
                    acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b1, w1, acc[1][0], 0, 0, 0);
                    acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b1, v1, acc[1][1], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (uint32_t q = 0; q < kQuad; ++q) {
#pragma unroll
            for (int j = 0; j < 2; ++j) cur[j][q] = nxt[j][q];
        }
    }
    uint32_t bad = t.bad;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t in_tile = 8 * (v / 4) + 4 * s + v % 4, row = 32 * i + in_tile;
            const uint32_t dest = __shfl(t.rid[i], in_tile, kWave);  // lane r (< 32) holds the routes of rows r and r + 32
            if (row < t.nrows && dest != 0xffffffffu) {
                float* out = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.y) + uint64_t(dest) * a.y_stride);
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    if (first + 32 * j + c >= a.channels) continue;
                    const float value = acc[i][j][v] * 256.0f;
                    bad |= nonfinite(value) ? TSP_ERRBIT_NONFINITE : 0u;
                    out[first + 32 * j + c] = value;
                }
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
    const dim3 grid((a.channels + 255) / 256, a.task_slots);
    const bool staged = a.hidden >= 128 && a.hidden <= 512 && a.hidden % 128 == 0;
    const uint32_t lds = staged ? 64 * a.hidden * 2 : 0;  // at most 64 KB: the default limit, no attribute to raise
    if (a.down_spec.source_type == 7) {
        if (staged) TSP_LAUNCH("gemm_down_staged", s, planar_staged_down<7, true><<<grid, 256, lds, s>>>(a));
        else TSP_LAUNCH("gemm_down_staged", s, planar_staged_down<7, false><<<grid, 256, 0, s>>>(a));
    } else {
        if (staged) TSP_LAUNCH("gemm_down_staged", s, planar_staged_down<8, true><<<grid, 256, lds, s>>>(a));
        else TSP_LAUNCH("gemm_down_staged", s, planar_staged_down<8, false><<<grid, 256, 0, s>>>(a));
    }
    return launch_status("gemm_down_staged");
}

}  // namespace tsp
