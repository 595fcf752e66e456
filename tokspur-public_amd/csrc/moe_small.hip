// Routed MoE for 1..8 token rows (decode and speculative verify) on Pack v3 planar experts:
//   h[rid, r] = silu(Wg[e] x_t . r) * (Wu[e] x_t . r)      gate + up + SwiGLU, one kernel
//   y[rid, c] = Wd[e] h[rid] . c                            down projection
// with rid = t*selected + slot and e = ids[rid]. HBM-bound: the union records (one per distinct
// expert, up to 8 tokens each) let every expert's weights be streamed from HBM once for all the
// tokens that route to it. f32 decode, f32 accumulate, no narrowing.
//
// Fast arms: Q4_K gate/up with K a multiple of 512 (a lane owns one 32-byte nibble pair and keeps
// the activations of its 64 columns in registers; the two half-waves of a step take the gate row
// and the up row of the same hidden unit, so SwiGLU needs one cross-lane move), and Q6_K planes
// for the down projection. Every other planar encoding goes through the generic arm.
#include "decode.hpp"
#include "record_resident.hpp"
#include "skinny.hpp"

using namespace tsp;

namespace {

struct SmallMoeArgs {
    const uint8_t* pair_lo;   // experts 0..E/2-1 as [gate_e, up_e]
    const uint8_t* pair_hi;   // experts E/2..E-1
    const uint8_t* down;      // [experts] planar
    const uint32_t* ids;      // [tokens*selected]
    uint32_t* meta;           // union block, or nullptr for tokens == 1
    const float* x;           // [tokens] rows, x_stride bytes apart
    float* h;                 // [tokens*selected] rows, h_stride bytes apart
    float* y;                 // [tokens*selected] rows, y_stride bytes apart
    uint64_t x_stride, h_stride, y_stride;
    uint32_t channels, hidden, experts, selected, tokens;
    tsp_planar_spec gu, dn;
    uint32_t* error_word;
};

struct Record { uint32_t expert, count; uint32_t token[8], route[8]; };

// Record `index` of the launch: a union record, or a single route when there is no union block.
__device__ __forceinline__ bool load_record(const SmallMoeArgs& a, uint32_t index, Record& r) {
    if (a.meta) {
        if (index >= a.meta[6]) return false;
        r.expert = a.meta[8 + index];
        r.count = a.meta[136 + index];
#pragma unroll
        for (int k = 0; k < 8; ++k) { r.token[k] = a.meta[264 + index * 8 + k]; r.route[k] = a.meta[1288 + index * 8 + k]; }
    } else {
        if (index >= a.tokens * a.selected) return false;
        r.expert = a.ids[index];
        r.count = 1;
#pragma unroll
        for (int k = 0; k < 8; ++k) { r.token[k] = index / a.selected; r.route[k] = index; }
    }
    return true;
}

__device__ __forceinline__ float silu_mul(float g, float u) {
    const float s = sigmoid_stable(g);
    return (g * s) * u;
}

__device__ __forceinline__ float ubyte(uint32_t w, int i) { return float((w >> (8 * i)) & 0xffu); }

template <int N>
__device__ __forceinline__ float lanes_sum(float v) {
    v = dpp_add<0xB1>(v);
    v = dpp_add<0x4E>(v);
    v = dpp_add<0x141>(v);
    if constexpr (N >= 16) v = dpp_add<0x140>(v);
    if constexpr (N >= 32) v += __shfl_xor(v, 16, kWave);
    if constexpr (N >= 64) v += __shfl_xor(v, 32, kWave);
    return v;
}

// ------------------------------------------------------------------------------------ planar element decode (generic arm)
template <uint32_t T>
__device__ __forceinline__ float planar_element(const uint8_t* base, const tsp_planar_spec& s, uint64_t blk, uint32_t e) {
    if constexpr (T == 12 || T == 13) {
        const uint32_t grp = e / 32, l = e % 32;
        uint32_t q = (uint32_t(base[s.qs_offset + blk * 128 + (grp >> 1) * 32 + l]) >> ((grp & 1u) * 4u)) & 15u;
        if constexpr (T == 13) q |= ((uint32_t(base[s.qh_offset + blk * 32 + l]) >> grp) & 1u) << 4;
        const uint8_t* sm = base + s.sm_offset + blk * 16;
        const uint8_t* dm = base + s.dm_offset + blk * 4;
        return (half_bits_to_float(ld16(dm)) * float(sm[grp])) * float(q) - half_bits_to_float(ld16(dm + 2)) * float(sm[8 + grp]);
    } else if constexpr (T == 14) {
        const uint32_t sec = e / 128, t = e % 128;
        const uint32_t low = (uint32_t(base[s.qs_offset + blk * 128 + sec * 64 + t % 64]) >> (4 * (t / 64))) & 15u;
        const uint32_t high = (uint32_t(base[s.qh_offset + blk * 64 + sec * 32 + t % 32]) >> (2 * (t / 32))) & 3u;
        return (half_bits_to_float(ld16(base + s.dm_offset + blk * 2)) * float(int(int8_t(base[s.sm_offset + blk * 16 + e / 16])))) *
               float(int(low | (high << 4)) - 32);
    } else if constexpr (T == 7) {
        const uint32_t low = (uint32_t(base[s.qs_offset + blk * 16 + e % 16]) >> (4 * (e / 16))) & 15u;
        const uint32_t q = low | (((ld32(base + s.qh_offset + blk * 4) >> e) & 1u) << 4);
        const uint8_t* dm = base + s.dm_offset + blk * 4;
        return half_bits_to_float(ld16(dm)) * float(q) + half_bits_to_float(ld16(dm + 2));
    } else {
        static_assert(T == 8);
        return half_bits_to_float(ld16(base + s.dm_offset + blk * 2)) * float(int(int8_t(base[s.qs_offset + blk * 32 + e])));
    }
}

template <uint32_t T> constexpr uint32_t planar_block_elements() { return (T == 7 || T == 8) ? 32u : 256u; }

__device__ __forceinline__ const uint8_t* pair_base(const SmallMoeArgs& a, uint32_t expert) {
    const uint32_t half = a.experts / 2;
    const uint8_t* base = expert < half ? a.pair_lo : a.pair_hi;
    return base + uint64_t(expert < half ? expert : expert - half) * 2 * a.gu.planar_expert_bytes;
}

// grid (ceil(hidden/4), records): one wave per hidden unit, all tokens of the record.
template <uint32_t T>
__global__ __launch_bounds__(256) void gate_up_generic(SmallMoeArgs a) {
    Record rec;
    if (!load_record(a, blockIdx.y, rec)) return;
    uint32_t bad = 0;
    if (rec.expert >= a.experts) {
        if (threadIdx.x == 0 && blockIdx.x == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
        return;
    }
    constexpr uint32_t E = planar_block_elements<T>();
    const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const uint32_t r = blockIdx.x * 4 + wave;
    if (r >= a.hidden) return;
    const uint8_t* gate = pair_base(a, rec.expert);
    const uint8_t* up = gate + a.gu.planar_expert_bytes;
    const uint32_t bpr = a.channels / E;
    for (uint32_t k = 0; k < rec.count; ++k) {
        const float* x = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(a.x) + rec.token[k] * a.x_stride);
        float g = 0, u = 0;
        for (uint32_t c = lane; c < a.channels; c += kWave) {
            const uint64_t blk = uint64_t(r) * bpr + c / E;
            const float xv = x[c];
            g = __builtin_fmaf(planar_element<T>(gate, a.gu, blk, c % E), xv, g);
            u = __builtin_fmaf(planar_element<T>(up, a.gu, blk, c % E), xv, u);
        }
        g = wave_sum(g);
        u = wave_sum(u);
        if (lane == 0) {
            const float act = silu_mul(g, u);
            if (nonfinite(g) || nonfinite(u) || nonfinite(act)) bad = TSP_ERRBIT_NONFINITE;
            reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.h) + rec.route[k] * a.h_stride)[r] = act;
        }
    }
    publish_error(bad, a.error_word);
}

// grid (ceil(channels/4), records)
template <uint32_t T>
__global__ __launch_bounds__(256) void down_generic(SmallMoeArgs a) {
    Record rec;
    if (!load_record(a, blockIdx.y, rec)) return;
    if (rec.expert >= a.experts) return;  // flagged by the gate/up kernel of the same batch
    constexpr uint32_t E = planar_block_elements<T>();
    const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const uint32_t r = blockIdx.x * 4 + wave;
    if (r >= a.channels) return;
    const uint8_t* w = a.down + uint64_t(rec.expert) * a.dn.planar_expert_bytes;
    const uint32_t bpr = a.hidden / E;
    uint32_t bad = 0;
    for (uint32_t k = 0; k < rec.count; ++k) {
        const float* hrow = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(a.h) + rec.route[k] * a.h_stride);
        float acc = 0;
        for (uint32_t c = lane; c < a.hidden; c += kWave)
            acc = __builtin_fmaf(planar_element<T>(w, a.dn, uint64_t(r) * bpr + c / E, c % E), hrow[c], acc);
        acc = wave_sum(acc);
        if (lane == 0) {
            if (nonfinite(acc)) bad = TSP_ERRBIT_NONFINITE;
            reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.y) + rec.route[k] * a.y_stride)[r] = acc;
        }
    }
    publish_error(bad, a.error_word);
}

// ------------------------------------------------------------------------------------ Q4_K gate/up fast arm
// BPR super-blocks per row (2, 4 or 8). A wave step covers 16 super-blocks = RPS rows; the first
// RPS/2 are gate rows of hidden units u0.., the others the up rows of the same units. TOK tokens of
// the record are processed per pass with their activations in registers.
template <int BPR, int TOK>
__global__ __launch_bounds__(256) void gate_up_q4k(SmallMoeArgs a) {
    constexpr int LPR = 4 * BPR, RPS = kWave / LPR, UPS = RPS / 2;  // units per step
    static_assert(RPS >= 2);
    Record rec;
    if (!load_record(a, blockIdx.y, rec)) return;
    if (rec.expert >= a.experts) {
        if (threadIdx.x == 0 && blockIdx.x == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
        return;
    }
    const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, nwaves = blockDim.x / kWave;
    const uint32_t pair = lane % 4, blk_in_row = (lane / 4) % BPR, row_in_step = lane / LPR;
    const bool is_up = row_in_step >= UPS;
    const uint32_t unit_in_step = row_in_step % UPS;
    const uint8_t* w = pair_base(a, rec.expert) + (is_up ? a.gu.planar_expert_bytes : 0);
    const uint32_t steps = (a.hidden + UPS - 1) / UPS;
    const uint32_t passes = (rec.count + TOK - 1) / TOK;
    uint32_t bad = 0;
    // work item = (step, pass); consecutive waves take the passes of one step so they share its weights in L1
    const uint32_t items = steps * passes;
    uint32_t held_pass = 0xffffffffu;
    float xa[TOK][32], xb[TOK][32], sxa[TOK], sxb[TOK];
    for (uint32_t item = blockIdx.x * nwaves + wave; item < items; item += gridDim.x * nwaves) {
        const uint32_t step = item / passes, pass = item % passes;
        if (pass != held_pass) {
            held_pass = pass;
#pragma unroll
            for (int t = 0; t < TOK; ++t) {
                const uint32_t k = pass * TOK + t < rec.count ? pass * TOK + t : rec.count - 1;
                const float* src = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(a.x) + rec.token[k] * a.x_stride) +
                                   blk_in_row * 256 + pair * 64;
                sxa[t] = 0; sxb[t] = 0;
#pragma unroll
                for (int i = 0; i < 32; i += 4) {
                    const float4 va = *reinterpret_cast<const float4*>(src + i), vb = *reinterpret_cast<const float4*>(src + 32 + i);
                    xa[t][i] = va.x; xa[t][i + 1] = va.y; xa[t][i + 2] = va.z; xa[t][i + 3] = va.w;
                    xb[t][i] = vb.x; xb[t][i + 1] = vb.y; xb[t][i + 2] = vb.z; xb[t][i + 3] = vb.w;
                    sxa[t] += (va.x + va.y) + (va.z + va.w);
                    sxb[t] += (vb.x + vb.y) + (vb.z + vb.w);
                }
            }
        }
        const uint32_t unit = step * UPS + unit_in_step;
        const bool live = unit < a.hidden;
        const uint64_t blk = uint64_t(live ? unit : a.hidden - 1) * BPR + blk_in_row;
        const uint8_t* qs = w + a.gu.qs_offset + blk * 128 + pair * 32;
        const uint4 q0 = *reinterpret_cast<const uint4*>(qs), q1 = *reinterpret_cast<const uint4*>(qs + 16);
        const uint8_t* sm = w + a.gu.sm_offset + blk * 16 + pair * 2;
        const uint32_t sc = *reinterpret_cast<const uint16_t*>(sm), mn = *reinterpret_cast<const uint16_t*>(sm + 8);
        const uint32_t dm = *reinterpret_cast<const uint32_t*>(w + a.gu.dm_offset + blk * 4);
        const float d = half_bits_to_float(dm & 0xffffu), dmin = half_bits_to_float(dm >> 16);
        const float dl_a = d * float(sc & 0xffu), dl_b = d * float(sc >> 8);
        const float ml_a = dmin * float(mn & 0xffu), ml_b = dmin * float(mn >> 8);
        const uint32_t words[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        float dot_a[TOK], dot_b[TOK];
#pragma unroll
        for (int t = 0; t < TOK; ++t) { dot_a[t] = 0; dot_b[t] = 0; }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint32_t lo = words[k] & 0x0f0f0f0fu, hi = (words[k] >> 4) & 0x0f0f0f0fu;
            const float l0 = ubyte(lo, 0), l1 = ubyte(lo, 1), l2 = ubyte(lo, 2), l3 = ubyte(lo, 3);
            const float h0 = ubyte(hi, 0), h1 = ubyte(hi, 1), h2 = ubyte(hi, 2), h3 = ubyte(hi, 3);
#pragma unroll
            for (int t = 0; t < TOK; ++t) {
                dot_a[t] = __builtin_fmaf(l0, xa[t][4 * k], dot_a[t]);
                dot_a[t] = __builtin_fmaf(l1, xa[t][4 * k + 1], dot_a[t]);
                dot_a[t] = __builtin_fmaf(l2, xa[t][4 * k + 2], dot_a[t]);
                dot_a[t] = __builtin_fmaf(l3, xa[t][4 * k + 3], dot_a[t]);
                dot_b[t] = __builtin_fmaf(h0, xb[t][4 * k], dot_b[t]);
                dot_b[t] = __builtin_fmaf(h1, xb[t][4 * k + 1], dot_b[t]);
                dot_b[t] = __builtin_fmaf(h2, xb[t][4 * k + 2], dot_b[t]);
                dot_b[t] = __builtin_fmaf(h3, xb[t][4 * k + 3], dot_b[t]);
            }
        }
#pragma unroll
        for (int t = 0; t < TOK; ++t) {
            float part = dl_a * dot_a[t] - ml_a * sxa[t];
            part += dl_b * dot_b[t] - ml_b * sxb[t];
            const float total = lanes_sum<LPR>(part);
            // lane of the gate row fetches the up row's total: same unit, UPS rows further on
            const float other = __shfl(total, (lane + UPS * LPR) % kWave, kWave);
            const uint32_t k = pass * TOK + t;
            if (live && !is_up && lane % LPR == 0 && k < rec.count) {
                const float act = silu_mul(total, other);
                if (nonfinite(total) || nonfinite(other) || nonfinite(act)) bad = TSP_ERRBIT_NONFINITE;
                reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.h) + rec.route[k] * a.h_stride)[unit] = act;
            }
        }
    }
    publish_error(bad, a.error_word);
}

// ------------------------------------------------------------------------------------ Q6_K down fast arm
// Planes [ql 128][qh 64][sc 16][d 2] per block. A lane owns four byte positions j..j+3 of one
// 128-weight section: 16 weights (elements j, 32+j, 64+j, 96+j and their three neighbours).
// 16 lanes per block; BPR = blocks per row (hidden / 256) in {1, 2, 4}.
template <int BPR, int TOK>
__global__ __launch_bounds__(256) void down_q6k(SmallMoeArgs a) {
    constexpr int LPR = 16 * BPR, RPS = kWave / LPR;
    Record rec;
    if (!load_record(a, blockIdx.y, rec)) return;
    if (rec.expert >= a.experts) return;
    const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, nwaves = blockDim.x / kWave;
    const uint32_t jq = lane % 8, sec = (lane / 8) % 2, blk_in_row = (lane / 16) % BPR, row_in_step = lane / LPR;
    const uint8_t* w = a.down + uint64_t(rec.expert) * a.dn.planar_expert_bytes;
    const uint32_t steps = (a.channels + RPS - 1) / RPS;
    const uint32_t passes = (rec.count + TOK - 1) / TOK;
    const uint32_t items = steps * passes;
    uint32_t bad = 0, held_pass = 0xffffffffu;
    float xv[TOK][16], sx[TOK][4];  // [quarter q][i]: element sec*128 + q*32 + jq*4 + i
    for (uint32_t item = blockIdx.x * nwaves + wave; item < items; item += gridDim.x * nwaves) {
        const uint32_t step = item / passes, pass = item % passes;
        if (pass != held_pass) {
            held_pass = pass;
#pragma unroll
            for (int t = 0; t < TOK; ++t) {
                const uint32_t k = pass * TOK + t < rec.count ? pass * TOK + t : rec.count - 1;
                const float* src = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(a.h) + rec.route[k] * a.h_stride) +
                                   blk_in_row * 256 + sec * 128 + jq * 4;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 v = *reinterpret_cast<const float4*>(src + q * 32);
                    xv[t][4 * q] = v.x; xv[t][4 * q + 1] = v.y; xv[t][4 * q + 2] = v.z; xv[t][4 * q + 3] = v.w;
                    sx[t][q] = (v.x + v.y) + (v.z + v.w);
                }
            }
        }
        const uint32_t row = step * RPS + row_in_step;
        const bool live = row < a.channels;
        const uint64_t blk = uint64_t(live ? row : a.channels - 1) * BPR + blk_in_row;
        const uint8_t* ql = w + a.dn.qs_offset + blk * 128 + sec * 64 + jq * 4;
        const uint32_t la = *reinterpret_cast<const uint32_t*>(ql), lb = *reinterpret_cast<const uint32_t*>(ql + 32);
        const uint32_t qh = *reinterpret_cast<const uint32_t*>(w + a.dn.qh_offset + blk * 64 + sec * 32 + jq * 4);
        const float d = half_bits_to_float(*reinterpret_cast<const uint16_t*>(w + a.dn.dm_offset + blk * 2));
        // sub-scales of the four 16-weight groups this lane touches: sec*8 + 2*q + (jq*4)/16
        const uint8_t* scp = w + a.dn.sm_offset + blk * 16 + sec * 8 + jq / 4;
        // 6-bit codes, four per dword, one dword per quarter q (elements q*32 + jq*4 + 0..3)
        const uint32_t code[4] = {
            (la & 0x0f0f0f0fu) | ((qh << 4) & 0x30303030u),
            (lb & 0x0f0f0f0fu) | ((qh << 2) & 0x30303030u),
            ((la >> 4) & 0x0f0f0f0fu) | (qh & 0x30303030u),
            ((lb >> 4) & 0x0f0f0f0fu) | ((qh >> 2) & 0x30303030u),
        };
        float part[TOK];
#pragma unroll
        for (int t = 0; t < TOK; ++t) part[t] = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float ds = d * float(int(int8_t(scp[2 * q])));
            const float c0 = ubyte(code[q], 0), c1 = ubyte(code[q], 1), c2 = ubyte(code[q], 2), c3 = ubyte(code[q], 3);
#pragma unroll
            for (int t = 0; t < TOK; ++t) {
                float dot = -32.0f * sx[t][q];  // sum (c - 32) x = sum c x - 32 sum x
                dot = __builtin_fmaf(c0, xv[t][4 * q], dot);
                dot = __builtin_fmaf(c1, xv[t][4 * q + 1], dot);
                dot = __builtin_fmaf(c2, xv[t][4 * q + 2], dot);
                dot = __builtin_fmaf(c3, xv[t][4 * q + 3], dot);
                part[t] = __builtin_fmaf(ds, dot, part[t]);
            }
        }
#pragma unroll
        for (int t = 0; t < TOK; ++t) {
            const float total = lanes_sum<LPR>(part[t]);
            const uint32_t k = pass * TOK + t;
            if (live && lane % LPR == 0 && k < rec.count) {
                if (nonfinite(total)) bad = TSP_ERRBIT_NONFINITE;
                reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.y) + rec.route[k] * a.y_stride)[row] = total;
            }
        }
    }
    publish_error(bad, a.error_word);
}

// ------------------------------------------------------------------------------------ host side
bool coloc_pair_kinds(uint32_t gate_kind, uint32_t up_kind, uint32_t* type) {
    if (gate_kind == TSP_KIND_Q4K_COLOC_GATE && up_kind == TSP_KIND_Q4K_COLOC_UP) { *type = 12; return true; }
    if (gate_kind == TSP_KIND_Q5K_COLOC_GATE && up_kind == TSP_KIND_Q5K_COLOC_UP) { *type = 13; return true; }
    if (gate_kind == TSP_KIND_Q8_COLOC_GATE && up_kind == TSP_KIND_Q8_COLOC_UP) { *type = 8; return true; }
    return false;
}

int fill_common(const tsp_small_moe* m, SmallMoeArgs* a, bool need_down) {
    TSP_REQUIRE(m, "null small MoE description");
    uint32_t gu_type = 0;
    TSP_REQUIRE(coloc_pair_kinds(m->gate_kind, m->up_kind, &gu_type), "planar v3 co-located gate/up registration mismatch");
    TSP_REQUIRE(m->experts >= 2 && m->experts <= 512 && m->experts % 2 == 0, "co-located planar v3 requires even experts >= 2");
    TSP_REQUIRE(m->tokens >= 1 && m->tokens <= 8 && m->selected >= 1 && m->selected <= 16 && m->selected <= m->experts,
                "planar v3 gate/up row or stride geometry mismatch");
    TSP_REQUIRE(m->x_stride_bytes >= uint64_t(m->channels) * 4 && m->x_stride_bytes % 4 == 0 &&
                    m->h_stride_bytes >= uint64_t(m->hidden) * 4 && m->h_stride_bytes % 4 == 0,
                "planar v3 gate/up row or stride geometry mismatch");
    int rc = tsp_make_expert_spec(gu_type, m->channels, m->hidden, &a->gu);
    if (rc != TSP_OK) return rc;
    TSP_REQUIRE(m->pair_lo && m->pair_hi && m->ids && m->x && m->h && m->error_word, "null device pointer");
    TSP_REQUIRE(m->tokens == 1 || m->union_meta, "planar v3 small MoE requires the union block for more than one token");
    TSP_REQUIRE(reinterpret_cast<uintptr_t>(m->pair_lo) % 16 == 0 && reinterpret_cast<uintptr_t>(m->pair_hi) % 16 == 0,
                "planar v3 matrices require 16-byte alignment");
    const uint32_t routes = m->tokens * m->selected;
    const uint64_t pair_bytes = uint64_t(m->experts / 2) * 2 * a->gu.planar_expert_bytes;
    const uint64_t x_span = uint64_t(m->tokens - 1) * m->x_stride_bytes + uint64_t(m->channels) * 4;
    const uint64_t h_span = uint64_t(routes - 1) * m->h_stride_bytes + uint64_t(m->hidden) * 4;
    TSP_REQUIRE(!ranges_overlap(m->h, h_span, m->pair_lo, pair_bytes) && !ranges_overlap(m->h, h_span, m->pair_hi, pair_bytes) &&
                    !ranges_overlap(m->h, h_span, m->x, x_span) && !ranges_overlap(m->h, h_span, m->ids, uint64_t(routes) * 4) &&
                    !ranges_overlap(m->h, h_span, m->union_meta, m->union_meta ? 9280 : 0),
                "planar v3 small MoE outputs overlap inputs");
    a->pair_lo = static_cast<const uint8_t*>(m->pair_lo); a->pair_hi = static_cast<const uint8_t*>(m->pair_hi);
    a->ids = m->ids; a->meta = m->tokens > 1 ? m->union_meta : nullptr; a->x = m->x; a->h = m->h;
    a->x_stride = m->x_stride_bytes; a->h_stride = m->h_stride_bytes;
    a->channels = m->channels; a->hidden = m->hidden; a->experts = m->experts; a->selected = m->selected; a->tokens = m->tokens;
    a->error_word = m->error_word;
    if (need_down) {
        const uint32_t dn_type = m->down_kind == TSP_KIND_Q51_PLANAR ? 7u : m->down_kind == TSP_KIND_Q8_PLANAR ? 8u :
                                 m->down_kind == TSP_KIND_Q6K_PLANAR_X ? 14u : 0u;
        TSP_REQUIRE(dn_type, "planar v3 down registration mismatch");
        rc = tsp_make_expert_spec(dn_type, m->hidden, m->channels, &a->dn);
        if (rc != TSP_OK) return rc;
        TSP_REQUIRE(m->down && m->y && reinterpret_cast<uintptr_t>(m->down) % 16 == 0, "planar v3 down pointer/alignment");
        TSP_REQUIRE(m->y_stride_bytes >= uint64_t(m->channels) * 4 && m->y_stride_bytes % 4 == 0, "planar v3 down output geometry mismatch");
        const uint64_t y_span = uint64_t(routes - 1) * m->y_stride_bytes + uint64_t(m->channels) * 4;
        const uint64_t dn_bytes = uint64_t(m->experts) * a->dn.planar_expert_bytes;
        TSP_REQUIRE(!ranges_overlap(m->y, y_span, m->down, dn_bytes) && !ranges_overlap(m->y, y_span, m->h, h_span) &&
                        !ranges_overlap(m->y, y_span, m->x, x_span) && !ranges_overlap(m->y, y_span, m->ids, uint64_t(routes) * 4) &&
                        !ranges_overlap(m->y, y_span, m->pair_lo, pair_bytes) && !ranges_overlap(m->y, y_span, m->pair_hi, pair_bytes) &&
                        !ranges_overlap(m->y, y_span, m->union_meta, m->union_meta ? 9280 : 0) &&
                        !ranges_overlap(m->h, h_span, m->down, dn_bytes),
                    "planar v3 small MoE outputs overlap inputs");
        a->down = static_cast<const uint8_t*>(m->down); a->y = m->y; a->y_stride = m->y_stride_bytes;
    }
    return TSP_OK;
}

uint32_t record_slots(const SmallMoeArgs& a) {
    const uint32_t routes = a.tokens * a.selected;
    return routes < 128 ? routes : 128;
}

SkinnyMoe skinny_view(const SmallMoeArgs& a, const tsp_shared_rows* shared = nullptr) {
    SkinnyMoe v{a.pair_lo, a.pair_hi, a.down, a.ids, a.meta, a.x, a.h, a.y, a.x_stride, a.h_stride, a.y_stride,
                a.channels, a.hidden, a.experts, a.selected, a.tokens, record_slots(a), a.gu, a.dn, a.error_word};
    if (shared) {
        v.shared_gate = static_cast<const uint8_t*>(shared->gate); v.shared_up = static_cast<const uint8_t*>(shared->up);
        v.shared_down = static_cast<const uint8_t*>(shared->down);
        v.shared_h = shared->h; v.shared_h_stride = shared->h_stride_bytes; v.shared_y = shared->y; v.shared_y_stride = shared->y_stride_bytes;
    }
    return v;
}

// The record-resident gate/up launch builds the union records itself (and leaves them in `meta` for the down launch): no
// launch of the union kernel goes before it.
bool gate_up_builds_union(const SmallMoeArgs& a, const tsp_shared_rows* shared = nullptr) {
    return skinny_moe_supported(a.gu.source_type, a.dn.source_type, a.channels, a.hidden, a.x, a.x_stride, a.h, a.h_stride, false) &&
           record_gate_up_takes(skinny_view(a, shared));
}

int launch_gate_up(const SmallMoeArgs& a, hipStream_t s, const tsp_shared_rows* shared = nullptr) {
    const uint32_t records = record_slots(a);
    if (skinny_moe_supported(a.gu.source_type, a.dn.source_type, a.channels, a.hidden, a.x, a.x_stride, a.h, a.h_stride, false)) {
        const SkinnyMoe view = skinny_view(a, shared);
        return record_gate_up_takes(view) ? launch_record_gate_up(view, s) : skinny_moe_gate_up(view, s);
    }
    TSP_REQUIRE(!shared, "the always-on expert rides only on the matrix-core small-row kernels");
    const bool x_aligned = reinterpret_cast<uintptr_t>(a.x) % 16 == 0 && a.x_stride % 16 == 0;
    if (a.gu.source_type == 12 && x_aligned && (a.channels == 512 || a.channels == 1024 || a.channels == 2048)) {
        const uint32_t bpr = a.channels / 256;
        const uint32_t units_per_step = 64 / (4 * bpr) / 2;
        const uint32_t steps = (a.hidden + units_per_step - 1) / units_per_step;
        // tokens == 1: one pass per step; otherwise up to 4 passes of 2 tokens, one per wave of the block
        const dim3 grid(a.tokens == 1 ? (steps + 3) / 4 : steps, records);
#define TSP_GU(N)                                                             \
    if (bpr == N) {                                                           \
        if (a.tokens == 1) TSP_LAUNCH("gate_up_q4k", s, gate_up_q4k<N, 1><<<grid, 256, 0, s>>>(a));         \
        else TSP_LAUNCH("gate_up_q4k", s, gate_up_q4k<N, 2><<<grid, 256, 0, s>>>(a));                       \
        return launch_status("gate_up_q4k");                                  \
    }
        TSP_GU(2) TSP_GU(4) TSP_GU(8)
#undef TSP_GU
    }
    const dim3 grid((a.hidden + 3) / 4, records);
    switch (a.gu.source_type) {
    case 12: TSP_LAUNCH("gate_up_generic", s, gate_up_generic<12><<<grid, 256, 0, s>>>(a)); break;
    case 13: TSP_LAUNCH("gate_up_generic", s, gate_up_generic<13><<<grid, 256, 0, s>>>(a)); break;
    default: TSP_LAUNCH("gate_up_generic", s, gate_up_generic<8><<<grid, 256, 0, s>>>(a)); break;
    }
    return launch_status("gate_up_generic");
}

int launch_down(const SmallMoeArgs& a, hipStream_t s, const tsp_shared_rows* shared = nullptr) {
    const uint32_t records = record_slots(a);
    if (a.dn.source_type == 14 && a.hidden % 256 == 0 && a.hidden <= 2048 && reinterpret_cast<uintptr_t>(a.h) % 16 == 0 && a.h_stride % 16 == 0) {
        const SkinnyMoe view = skinny_view(a, shared);
        return skinny_moe_down(view, s);
    }
    TSP_REQUIRE(!shared, "the always-on expert rides only on the matrix-core small-row kernels");
    const bool h_aligned = reinterpret_cast<uintptr_t>(a.h) % 16 == 0 && a.h_stride % 16 == 0;
    if (a.dn.source_type == 14 && h_aligned && (a.hidden == 256 || a.hidden == 512 || a.hidden == 1024)) {
        const uint32_t bpr = a.hidden / 256;
        const uint32_t rps = 64 / (16 * bpr);
        const uint32_t steps = (a.channels + rps - 1) / rps;
        const dim3 grid(a.tokens == 1 ? (steps + 3) / 4 : steps, records);
#define TSP_DN(N)                                                          \
    if (bpr == N) {                                                        \
        if (a.tokens == 1) TSP_LAUNCH("down_q6k", s, down_q6k<N, 1><<<grid, 256, 0, s>>>(a));         \
        else TSP_LAUNCH("down_q6k", s, down_q6k<N, 2><<<grid, 256, 0, s>>>(a));                       \
        return launch_status("down_q6k");                                  \
    }
        TSP_DN(1) TSP_DN(2) TSP_DN(4)
#undef TSP_DN
    }
    const dim3 grid((a.channels + 3) / 4, records);
    switch (a.dn.source_type) {
    case 7: TSP_LAUNCH("down_generic", s, down_generic<7><<<grid, 256, 0, s>>>(a)); break;
    case 8: TSP_LAUNCH("down_generic", s, down_generic<8><<<grid, 256, 0, s>>>(a)); break;
    default: TSP_LAUNCH("down_generic", s, down_generic<14><<<grid, 256, 0, s>>>(a)); break;
    }
    return launch_status("down_generic");
}

}  // namespace

extern "C" int tsp_planar_moe_gate_up_swiglu_m8(const tsp_small_moe* m, void* stream) {
    SmallMoeArgs a{};
    int rc = fill_common(m, &a, false);
    if (rc != TSP_OK) return rc;
    const auto s = static_cast<hipStream_t>(stream);
    if (m->tokens > 1 && !gate_up_builds_union(a)) {
        rc = tsp_planar_union_build(m->ids, m->union_meta, m->experts, m->selected, m->tokens, m->hidden, m->channels, m->error_word, stream);
        if (rc != TSP_OK) return rc;
    }
    return launch_gate_up(a, s);
}

extern "C" int tsp_planar_moe_routed_m8(const tsp_small_moe* m, void* stream) {
    SmallMoeArgs a{};
    int rc = fill_common(m, &a, true);
    if (rc != TSP_OK) return rc;
    const auto s = static_cast<hipStream_t>(stream);
    if (m->tokens > 1 && !gate_up_builds_union(a)) {
        rc = tsp_planar_union_build(m->ids, m->union_meta, m->experts, m->selected, m->tokens, m->hidden, m->channels, m->error_word, stream);
        if (rc != TSP_OK) return rc;
    }
    rc = launch_gate_up(a, s);
    if (rc != TSP_OK) return rc;
    return launch_down(a, s);
}

extern "C" int tsp_planar_moe_routed_m8_shared(const tsp_small_moe* m, const tsp_shared_rows* shared, void* stream) {
    TSP_REQUIRE(shared, "null shared expert description");
    SmallMoeArgs a{};
    int rc = fill_common(m, &a, true);
    if (rc != TSP_OK) return rc;
    TSP_REQUIRE(shared->gate && shared->up && shared->down && shared->h && shared->y, "null device pointer");
    TSP_REQUIRE(skinny_moe_supported(a.gu.source_type, a.dn.source_type, a.channels, a.hidden, a.x, a.x_stride, a.h, a.h_stride, true) &&
                    a.gu.source_type == 12 && a.dn.source_type == 14,
                "the always-on expert rides only with Q4_K co-located gate/up and Q6_K planes down, 16-byte aligned rows");
    TSP_REQUIRE(reinterpret_cast<uintptr_t>(shared->gate) % 16 == 0 && reinterpret_cast<uintptr_t>(shared->up) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(shared->down) % 16 == 0 && reinterpret_cast<uintptr_t>(shared->h) % 16 == 0 &&
                    shared->h_stride_bytes % 16 == 0 && shared->h_stride_bytes >= uint64_t(m->hidden) * 4 && shared->y_stride_bytes % 4 == 0 &&
                    shared->y_stride_bytes >= uint64_t(m->channels) * 4,
                "planar v3 small MoE shape or stride mismatch");
    const uint64_t h_span = uint64_t(m->tokens - 1) * shared->h_stride_bytes + uint64_t(m->hidden) * 4;
    const uint64_t y_span = uint64_t(m->tokens - 1) * shared->y_stride_bytes + uint64_t(m->channels) * 4;
    const uint32_t routes = m->tokens * m->selected;
    const void* others[] = {m->x, m->ids, m->h, m->y, shared->gate, shared->up, shared->down, m->union_meta};
    const uint64_t spans[] = {uint64_t(m->tokens - 1) * m->x_stride_bytes + uint64_t(m->channels) * 4, uint64_t(routes) * 4,
                              uint64_t(routes - 1) * m->h_stride_bytes + uint64_t(m->hidden) * 4, uint64_t(routes - 1) * m->y_stride_bytes + uint64_t(m->channels) * 4,
                              a.gu.planar_expert_bytes, a.gu.planar_expert_bytes, a.dn.planar_expert_bytes, m->union_meta ? 9280u : 0u};
    for (int i = 0; i < 8; ++i)
        TSP_REQUIRE(!ranges_overlap(shared->h, h_span, others[i], spans[i]) && !ranges_overlap(shared->y, y_span, others[i], spans[i]),
                    "planar v3 small MoE outputs overlap inputs");
    TSP_REQUIRE(!ranges_overlap(shared->h, h_span, shared->y, y_span), "planar v3 small MoE outputs overlap inputs");
    const auto s = static_cast<hipStream_t>(stream);
    if (m->tokens > 1 && !gate_up_builds_union(a, shared)) {
        rc = tsp_planar_union_build(m->ids, m->union_meta, m->experts, m->selected, m->tokens, m->hidden, m->channels, m->error_word, stream);
        if (rc != TSP_OK) return rc;
    }
    rc = launch_gate_up(a, s, shared);
    if (rc != TSP_OK) return rc;
    return launch_down(a, s, shared);
}
