// The T <= 8 routed MoE (decode, verify) as two activation-resident streaming kernels: gate/up + SwiGLU for 2048-column
// Q4_K experts and the down product for 512-column Q6_K experts, over the union records (one per distinct expert, at most
// eight rows each) and, riding along as one more record, the layer's always-on expert.
//
// These launches move about a megabyte of weights per distinct expert and compute next to nothing: they are streams from
// HBM, and are built like the grouped prefill kernels (gate_up_resident.hip, down_resident.hip) around that stream.
//
//   * One persistent workgroup of eight waves per CU takes an equal contiguous share of the launch's (record, unit) items,
//     in record order; a unit is 32 hidden units (gate/up) or 128 output channels (down).
//   * K is split over the waves (gate/up: wave w owns super-block w of 2048 columns; down: waves w and w + 4 own the two
//     super-blocks of the same 32 channels). A wave's operands, its 256 columns of the record's rows, are read once per
//     record as f32, scaled by a power of two chosen from the largest magnitude among them, split into a high and a low
//     half (22 significant bits together) and kept in registers as MFMA A fragments: rows 0..7 of the 32-row operand hold
//     the high halves, rows 8..15 the low halves, and the two sums meet when the accumulators are read. Nothing but exact
//     integers (sc * q, sc * (q - 32)) meets them on the matrix cores, the block scales are applied in f32, and the
//     power of two is taken off again before partial sums of different waves meet.
//   * Weight tiles go global -> LDS directly into a wave-private ring, requested ahead by a cursor that runs across record
//     boundaries; inside the tile loop nothing but these requests and the tile's stores uses the vector memory counter, so
//     every wait is an exact count. A row a record does not have repeats its first row, operand and destination alike
//     (the union block pads its records that way), so every lane always stores.
//   * The K slices add up through LDS in wave order: results do not depend on timing, nor on which other records ride in
//     the launch.
#include "record_resident.hpp"

#include <type_traits>

#include "mfma_quant.hpp"

using namespace tsp;

namespace {

constexpr int kWaves = 8, kThreads = kWaves * kWave;
constexpr uint32_t kRecordRows = 8, kMaxRecords = 128;
constexpr uint32_t kInfoSlots = 32;  // records of a workgroup's share kept in LDS: a share spans at most records / groups + 2

struct RecordArgs {
    const float* x;            // operand rows: token rows (gate/up) or the routes' h rows (down), x_stride bytes apart
    uint64_t x_stride;
    const float* shared_x;     // the always-on expert's operand rows, by token
    uint64_t shared_x_stride;
    const uint8_t* w0;         // gate/up: experts 0..E/2-1 as [gate_e, up_e]; down: the experts' planes
    const uint8_t* w1;         // gate/up: experts E/2..E-1
    const uint8_t* shared_w0;  // the always-on expert: gate, or down
    const uint8_t* shared_w1;  // up
    tsp_planar_spec spec;
    const uint32_t* meta;      // the union block
    float* out;                // result rows by route, out_stride bytes apart
    uint64_t out_stride;
    float* shared_out;         // by token
    uint64_t shared_out_stride;
    uint32_t experts, tokens, selected, records, n;  // n: hidden units (gate/up) or channels (down)
    uint32_t* error_word;
};

// ---------------------------------------------------------------- records
struct Record { uint32_t index, expert, count; bool shared, ok; };

__device__ __forceinline__ uint4 pack_record(const Record& r) {
    return uint4{r.index, r.expert, r.count | (r.shared ? 256u : 0u) | (r.ok ? 512u : 0u), 0u};
}
// every lane read the same slot: the words go to scalar registers
__device__ __forceinline__ Record unpack_record(const uint4& v) {
    Record r;
    r.index = __builtin_amdgcn_readfirstlane(v.x);
    r.expert = __builtin_amdgcn_readfirstlane(v.y);
    const uint32_t w = __builtin_amdgcn_readfirstlane(v.z);
    r.count = w & 255u; r.shared = (w & 256u) != 0; r.ok = (w & 512u) != 0;
    return r;
}
// List position k: union record k, or, after the `live` union records, the always-on expert with the tokens as its rows. A
// record that does not check out keeps every address inside the tensors (expert 0, row 0); whoever resolves it flags the batch.
__device__ __forceinline__ Record resolve_record(const RecordArgs& a, uint32_t k, uint32_t live) {
    Record r;
    r.shared = a.shared_w0 != nullptr && k == live;
    r.index = k < kMaxRecords ? k : 0;
    r.expert = r.shared ? 0 : a.meta[8 + r.index];
    r.count = r.shared ? a.tokens : a.meta[136 + r.index];
    r.ok = r.count >= 1 && r.count <= kRecordRows && (r.shared || (k < live && r.expert < a.experts));
    if (!r.ok) { r.expert = 0; r.count = 0; r.shared = false; }
    return r;
}

// A pointer that is the same in every lane, moved to scalar registers (the address operand of the stores below has to be one).
__device__ __forceinline__ uint8_t* uniform_pointer(uint8_t* p) {
    const uint64_t bits = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(bits))), hi = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(bits >> 32)));
    return reinterpret_cast<uint8_t*>(uint64_t(hi) << 32 | lo);
}

// ---------------------------------------------------------------- operand rows
template <int Ctrl>
__device__ __forceinline__ uint32_t dpp_max_u32(uint32_t v) {
    const uint32_t moved = uint32_t(__builtin_amdgcn_update_dpp(0, int(v), Ctrl, 0xf, 0xf, true));
    return v > moved ? v : moved;
}
__device__ __forceinline__ uint32_t wave_largest_u32(uint32_t v) {
    v = dpp_max_u32<0xB1>(v);
    v = dpp_max_u32<0x4E>(v);
    v = dpp_max_u32<0x141>(v);
    v = dpp_max_u32<0x140>(v);
    const uint32_t a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
    const uint32_t c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
    const uint32_t ab = a > b ? a : b, cd = c > d ? c : d;
    return ab > cd ? ab : cd;
}

// A wave's 256 columns of the record's rows as MFMA A fragments. `row` is the lane's operand row at the wave's first column
// plus the lane's k-half (16 columns); lane (n, k-half) of fragment t holds eight columns of row n % 8, their high halves
// where n % 16 < 8 and their low halves above. Q4_K fragments take the columns of every eight in the order (0, 2, 1, 3, 4,
// 6, 5, 7), the order in which a dword of nibbles unpacks, and come with the sums of the eight 32-column sub-blocks (over
// 32, as high and low halves: the operand of the minima term, zero in the low-half rows). Returns the power of two that
// takes the scaling off again.
template <bool Q4>
__device__ __forceinline__ float stage_record_rows(const float* row, uint32_t lane, f16x8 (&A)[16], f16x8& sxA, uint32_t& bad) {
    const bool low_half = (lane & 8u) != 0;
    float4 raw[16][2];
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        const int c0 = Q4 ? (t / 4) * 64 + ((t / 2) % 2) * 32 + (t % 2) * 8 : (t / 8) * 128 + ((t / 2) % 4) * 32 + (t % 2) * 8;
        raw[t][0] = *reinterpret_cast<const float4*>(row + c0);
        raw[t][1] = *reinterpret_cast<const float4*>(row + c0 + 4);
    }
    // the largest magnitude as bits: an infinity or a NaN is larger than any finite value's
    uint32_t top = 0;
#pragma unroll
    for (int t = 0; t < 16; ++t)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const float4 v = raw[t][h];
            const uint32_t b0 = __float_as_uint(v.x) & 0x7fffffffu, b1 = __float_as_uint(v.y) & 0x7fffffffu;
            const uint32_t b2 = __float_as_uint(v.z) & 0x7fffffffu, b3 = __float_as_uint(v.w) & 0x7fffffffu;
            const uint32_t m01 = b0 > b1 ? b0 : b1, m23 = b2 > b3 ? b2 : b3, m = m01 > m23 ? m01 : m23;
            top = top > m ? top : m;
        }
    top = wave_largest_u32(top);
    // scale = 2^(13 - exponent(largest)): the largest |x * scale| is below 2^14, and so are the sub-block sums / 32
    float scale = 1.0f, inv_scale = 1.0f;
    if (top >= 0x7f800000u) {
        bad |= TSP_ERRBIT_NONFINITE;
    } else if (top != 0) {
        const int e = int(top >> 23) - 127;
        int shift = 13 - e;
        shift = shift > 100 ? 100 : shift < -100 ? -100 : shift;
        scale = __uint_as_float(uint32_t(127 + shift) << 23);
        inv_scale = __uint_as_float(uint32_t(127 - shift) << 23);
    }
    float part[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        const float s[8] = {raw[t][0].x * scale, raw[t][0].y * scale, raw[t][0].z * scale, raw[t][0].w * scale,
                            raw[t][1].x * scale, raw[t][1].y * scale, raw[t][1].z * scale, raw[t][1].w * scale};
        _Float16 p[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const _Float16 hi = _Float16(s[e]);
            const _Float16 lo = _Float16(s[e] - float(hi));
            p[e] = low_half ? lo : hi;
        }
        if constexpr (Q4) {
            A[t] = f16x8{p[0], p[2], p[1], p[3], p[4], p[6], p[5], p[7]};
            part[t / 2] += ((s[0] + s[1]) + (s[2] + s[3])) + ((s[4] + s[5]) + (s[6] + s[7]));
        } else {
            A[t] = f16x8{p[0], p[1], p[2], p[3], p[4], p[5], p[6], p[7]};
        }
    }
    if constexpr (Q4) {
        // a sub-block's 32 columns are fragments 2s and 2s + 1 of the two k-halves: lanes l and l ^ 32
        const bool second = (lane & 32u) != 0;
        _Float16 h8[8];
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            const float other = __shfl_xor(part[sb], 32, kWave);
            const float sum = second ? other + part[sb] : part[sb] + other;  // the same order in both lanes
            const float s32 = sum * 0.03125f;
            const _Float16 hi = _Float16(s32);
            const _Float16 lo = _Float16(s32 - float(hi));
            h8[sb] = low_half ? _Float16(0.0f) : second ? lo : hi;
        }
        sxA = f16x8{h8[0], h8[1], h8[2], h8[3], h8[4], h8[5], h8[6], h8[7]};
    }
    return inv_scale;
}

// ---------------------------------------------------------------- gate/up + SwiGLU, Q4_K planes of 2048 columns
constexpr int kGuStageBytes = 5120;  // 32 rows x 128 B of nibbles, 32 x 16 B of scales / minima, 32 x 16 B holding d / dmin
constexpr int kGuStages = 3;
constexpr int kGuTileLoads = 5;
constexpr int kSumBytes = 4 * kWave * 4;             // a wave's partial sums of one tile: [4 rows per lane][64 lanes] f32
constexpr int kGuPhaseBytes = 2 * kWaves * kSumBytes;  // gate and up

__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void record_gate_up_kernel(RecordArgs a) {
    // LDS: [2 phases][gate, up][8 waves][1 KB of partial sums] | [32 records of the share] | [8 waves][3 stages][5 KB weight tile]
    constexpr int kInfoAt = 2 * kGuPhaseBytes, kStagesAt = kInfoAt + kInfoSlots * 16;
    __shared__ __attribute__((aligned(16))) uint8_t lds_raw[kStagesAt + kWaves * kGuStages * kGuStageBytes];
    static_assert(sizeof(lds_raw) <= 160 * 1024, "one workgroup per compute unit");
    uint4* const info = reinterpret_cast<uint4*>(lds_raw + kInfoAt);

    const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const uint32_t n = lane % 32, khalf = lane / 32;
    constexpr uint32_t bpr = 8;  // 2048 columns
    const uint32_t units = a.n / 32;

    const uint32_t listed = a.meta[6];
    const uint32_t live = listed < a.records ? listed : a.records;
    if (listed > a.records && tid == 0 && blockIdx.x == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
    const uint32_t total = live + (a.shared_w0 ? 1 : 0);
    const uint32_t groups = gridDim.x, share = blockIdx.x;
    const uint32_t items = total * units;
    const uint32_t it0 = uint32_t(uint64_t(items) * share / groups), it1 = uint32_t(uint64_t(items) * (share + 1) / groups);
    if (it0 >= it1) return;
    const uint32_t k0 = it0 / units, k1 = (it1 - 1) / units;  // first and last record of the share
    auto first_unit = [&](uint32_t k) { return k == k0 ? it0 % units : 0; };
    auto end_unit = [&](uint32_t k) { return k == k1 ? (it1 - 1) % units + 1 : units; };

    // ---- the share's records, looked up once into LDS. Every wave writes the whole table for itself (the same words) and
    // reads only what it wrote: a vector load inside the tile loop would have the compiler drain the requests in flight.
    if (lane < kInfoSlots && k0 + lane <= k1) {
        const Record r = resolve_record(a, k0 + lane, live);
        if (!r.ok) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
        info[lane] = pack_record(r);
    }
    auto info_at = [&](uint32_t k) { return unpack_record(k - k0 < kInfoSlots ? info[k - k0] : pack_record(resolve_record(a, k, live))); };

    uint8_t* const my_stage = lds_raw + kStagesAt + wave * (kGuStages * kGuStageBytes);
    const uint32_t my_stage_lds = __builtin_amdgcn_readfirstlane(lds_address(my_stage));

    // ---- per-lane parts of the request addresses (the per-tile parts are uniform and stay in scalar registers)
    // nibbles: request q covers rows 8q .. 8q+7 of the tile, eight lanes per row (one 128-byte line: the row's super-block);
    // lane l sits at 16-byte slot l % 8 of its row in LDS and fetches chunk (l % 8) ^ (row % 8)
    const uint32_t qs_lane = uint32_t(a.spec.qs_offset) + (lane / 8) * (bpr * 128) + wave * 128 + (((lane % 8) ^ ((lane / 8) & 7)) * 16);
    // lanes 0..31: scales and minima of row l (16 B); lanes 32..63: the 16 bytes holding d / dmin of row l - 32
    const uint32_t hdr_lane = lane < 32 ? uint32_t(a.spec.sm_offset) + lane * (bpr * 16) + wave * 16
                                        : uint32_t(a.spec.dm_offset) + (lane - 32) * (bpr * 4) + (wave / 4) * 16;
    const uint32_t hdr_unit_step = lane < 32 ? 32 * bpr * 16 : 32 * bpr * 4;
    auto weight_bases = [&](const Record& r, const uint8_t*& gate, const uint8_t*& up) {
        if (r.shared) { gate = a.shared_w0; up = a.shared_w1; return; }
        const uint32_t half_e = a.experts / 2;
        const uint8_t* pair = (r.expert < half_e ? a.w0 : a.w1) + uint64_t(r.expert < half_e ? r.expert : r.expert - half_e) * 2 * a.spec.planar_expert_bytes;
        gate = pair;
        up = pair + a.spec.planar_expert_bytes;
    };
    auto request_tile = [&](const uint8_t* base, uint32_t unit, uint32_t stage_offset) {  // base: one expert (under 4 GiB), uniform
        const uint8_t* qs = base + uint64_t(unit) * (32 * bpr * 128);
        const uint32_t dst = my_stage_lds + stage_offset;
#pragma unroll
        for (int q = 0; q < 4; ++q) load_to_lds_16(qs + q * (8 * bpr * 128), qs_lane, dst + q * 1024);
        load_to_lds_16(base, hdr_lane + unit * hdr_unit_step, dst + 4096);
    };

    uint32_t bad = 0, phase = 0;
    const Q4Consts q4c = q4_consts();
    const Q4ScaleConsts q4s = q4_scale_consts();

    // ---- the request cursor runs three tiles ahead of the arithmetic: (record, unit, gate or up)
    uint32_t rk = k0, runit = first_unit(k0), rj = 0, rstage = 0;
    bool rdone = false;
    const uint8_t *rgate, *rup;
    weight_bases(info_at(k0), rgate, rup);
    auto request_next = [&]() {  // past the end of the share the last tile is requested again (unused)
        request_tile(rj == 0 ? rgate : rup, runit, rstage);
        rstage = rstage + kGuStageBytes == kGuStages * kGuStageBytes ? 0 : rstage + kGuStageBytes;
        if (rdone) return;
        if (rj == 0) { rj = 1; return; }
        if (runit + 1 < end_unit(rk)) { rj = 0; ++runit; return; }
        if (rk == k1) { rdone = true; return; }
        ++rk;
        rj = 0;
        runit = 0;
        weight_bases(info_at(rk), rgate, rup);
    };
#pragma unroll
    for (int s = 0; s < kGuStages; ++s) request_next();
    uint32_t stage = 0;  // byte offset of the stage the next tile sits in

    f16x8 A[16];   // operand fragments: [k16 step of the super-block]
    f16x8 sxA;     // sub-block sums (k-half 0: the high halves, k-half 1: the residuals)
    float inv_scale = 1.0f;
    uint32_t store_at = 0;       // where this lane's result of a unit goes, from the first byte of the unit's columns in the output
    uint8_t* out_base = nullptr;
    auto load_rows = [&](uint32_t k) {
        const Record cur = info_at(k);
        // operand row n % 8: its token; the reducing waves' result row 4 * k-half + wave: its route (the always-on expert: the token)
        const uint32_t op = n % 8, res = 4 * khalf + wave % 4;
        uint32_t token, dst;
        if (cur.shared) {
            token = op < a.tokens ? op : 0;
            dst = res < a.tokens ? res : 0;
        } else {
            token = a.meta[264 + cur.index * 8 + op];
            dst = a.meta[1288 + cur.index * 8 + res];
            if (token >= a.tokens || dst >= a.tokens * a.selected) { if (cur.ok) bad |= TSP_ERRBIT_INDEX; token = 0; dst = 0; }
        }
        if (!cur.ok) { token = 0; dst = 0; }  // flagged already: the batch is refused whatever lands in row 0
        out_base = uniform_pointer(reinterpret_cast<uint8_t*>(cur.shared ? a.shared_out : a.out));  // scalar registers: the unit's columns are added there
        store_at = dst * uint32_t(cur.shared ? a.shared_out_stride : a.out_stride) + n * 4;
        const float* row = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(cur.shared ? a.shared_x : a.x) +
                                                          uint64_t(token) * (cur.shared ? a.shared_x_stride : a.x_stride)) + wave * 256 + khalf * 16;
        const float back = stage_record_rows<true>(row, lane, A, sxA, bad);
        inv_scale = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(back)));  // the same in every lane
        // The rows are needed at once. Naming every fragment as an operand here makes the compiler wait for their loads now:
        // left to itself it may wait at the fragments' first uses inside the tile loop, with counts that know nothing of the
        // requests in flight and so drain them tile after tile.
#pragma unroll
        for (int t = 0; t < 16; ++t) asm volatile("" : "+v"(A[t]));
        asm volatile("" : "+v"(sxA), "+v"(store_at));
    };

    // ---- one tile: unpack, multiply, park the wave's partial sums; after the up tile the eight waves' sums meet
    auto tile = [&](uint32_t unit, auto j_tag) {
        constexpr int J = decltype(j_tag)::value;
        // Wait for the tile's five requests. Younger than those are the ten of the other two stages and, in the waves that
        // store, the store of the unit before (everything completes in issue order; at a record's first tiles nothing
        // older than the record's rows is outstanding at all).
        if (wave < 4) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kGuStages - 1) * kGuTileLoads + 1) : "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kGuStages - 1) * kGuTileLoads) : "memory");
        const uint8_t* st = my_stage + stage;
        u32x4 raw[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) raw[p] = *reinterpret_cast<const u32x4*>(st + n * 128 + (((2 * p + khalf) ^ (n & 7)) * 16));
        const uint4 sm = *reinterpret_cast<const uint4*>(st + 4096 + n * 16);
        const uint32_t dm = *reinterpret_cast<const uint32_t*>(st + 4096 + 512 + n * 16 + (wave % 4) * 4);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        request_next();  // the stage is free again: the tile three ahead goes there
        stage = stage + kGuStageBytes == kGuStages * kGuStageBytes ? 0 : stage + kGuStageBytes;
        const float d = half_bits_to_float(dm & 0xffffu), dmin = half_bits_to_float(dm >> 16);

        f32x16 blk;
        auto steps = [&](auto p_tag) {
            constexpr int P = decltype(p_tag)::value;
            const Q4PairScale sc = q4_pair_scale<P>(sm.x, sm.y, q4s);
#pragma unroll
            for (int hi = 0; hi < 2; ++hi) {
                f16x8 f[2];
                frags_q4k_pair(raw[P], sc, hi, q4c, f);
#pragma unroll
                for (int ff = 0; ff < 2; ++ff) {
                    if (P == 0 && hi == 0 && ff == 0) {
                        const f32x16 zero{};
                        blk = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[0], f[0], zero, 0, 0, 0);
                    } else {
                        blk = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[P * 4 + hi * 2 + ff], f[ff], blk, 0, 0, 0);
                    }
                }
            }
        };
        steps(std::integral_constant<int, 0>{});
        steps(std::integral_constant<int, 1>{});
        steps(std::integral_constant<int, 2>{});
        steps(std::integral_constant<int, 3>{});
        HdrQ4 hdr;
        hdr.mn[0] = sm.z; hdr.mn[1] = sm.w;
        const f16x8 mn = minima_frag(hdr);
        const f32x16 zero{};
        const f32x16 mblk = __builtin_amdgcn_mfma_f32_32x32x16_f16(sxA, mn, zero, 0, 0, 0);
        // Accumulator v of the 32 x 32 tile is operand row 8 (v / 4) + 4 khalf + v % 4: v < 4 the high halves of record rows
        // 4 khalf + v, v + 4 their low halves. partial = (d * sum(x * sc*q) - 32 dmin * sum(Sx / 32 * mn)) / scale
        float* const park = reinterpret_cast<float*>(lds_raw + (phase & 1) * kGuPhaseBytes + (J * kWaves + wave) * kSumBytes) + lane;
#pragma unroll
        for (int e = 0; e < 4; ++e) park[e * kWave] = __builtin_fmaf(-32.0f * dmin, mblk[e], d * (blk[e] + blk[e + 4])) * inv_scale;
        if constexpr (J == 1) {
            lds_barrier();
            if (wave < 4) {
                // wave e adds up row 4 khalf + e of the eight waves' gate and up tiles, in wave order, and stores the unit's h
                const float* in = reinterpret_cast<const float*>(lds_raw + (phase & 1) * kGuPhaseBytes) + wave * kWave + lane;
                float g = 0.0f, u = 0.0f;
#pragma unroll
                for (int w = 0; w < kWaves; ++w) {
                    g += in[w * (kSumBytes / 4)];
                    u += in[(kWaves + w) * (kSumBytes / 4)];
                }
                const float h = (g * sigmoid_stable(g)) * u;
                if (nonfinite(g) || nonfinite(u) || nonfinite(h)) bad |= TSP_ERRBIT_NONFINITE;
                // uniform base (the output, the unit's columns) + 32-bit lane offset, spelled out: the compiler would form a
                // 64-bit address per store
                uint8_t* const base = out_base + unit * 128;
                const uint32_t at = store_at;
                asm volatile("global_store_dword %0, %1, %2" ::"v"(at), "v"(h), "s"(base) : "memory");
            }
            ++phase;
        }
    };

    for (uint32_t k = k0; k <= k1; ++k) {
        load_rows(k);
        const uint32_t u1 = end_unit(k);
        for (uint32_t unit = first_unit(k); unit < u1; ++unit) {
            tile(unit, std::integral_constant<int, 0>{});
            tile(unit, std::integral_constant<int, 1>{});
        }
    }
    wait_all_loads();  // the last requests fetched tiles nobody reads: they must have landed before the stages are given away
    publish_error(bad, a.error_word);
}

// ---------------------------------------------------------------- down, Q6_K planes of 512 columns
// A stage holds one tile, 32 weight rows x one super-block:
//   [32 rows x 128 B low nibbles][32 x 64 B high bits][32 x 16 B sub-scales][128 B of d: 32 rows x 2 super-blocks][pad]
constexpr int kDnStageBytes = 7168, kDnStages = 2, kDnTileLoads = 7, kDnTileStores = 2;
constexpr int kQlAt = 0, kQhAt = 4096, kScAt = 6144, kDAt = 6656;
constexpr int kHandBytes = kWave * 8;              // what a wave hands its partner per tile: two sums per lane
constexpr int kDnPhaseBytes = kWaves * kHandBytes;

__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void record_down_kernel(RecordArgs a) {
    // LDS: [2 phases][8 waves][512 B handed over] | [32 records of the share] | [8 waves][2 stages][7 KB weight tile]
    constexpr int kInfoAt = 2 * kDnPhaseBytes, kStagesAt = kInfoAt + kInfoSlots * 16;
    __shared__ __attribute__((aligned(16))) uint8_t lds_raw[kStagesAt + kWaves * kDnStages * kDnStageBytes];
    static_assert(sizeof(lds_raw) <= 160 * 1024, "one workgroup per compute unit");
    uint4* const info = reinterpret_cast<uint4*>(lds_raw + kInfoAt);

    const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const uint32_t n = lane % 32, khalf = (lane / 32) & 1;
    const uint32_t kh = wave / 4, nq = wave % 4;  // super-block, channel tile of the item
    constexpr uint32_t bpr = 2;                   // 512 columns
    const uint32_t units = a.n / 128;

    const uint32_t listed = a.meta[6];
    const uint32_t live = listed < a.records ? listed : a.records;
    if (listed > a.records && tid == 0 && blockIdx.x == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
    const uint32_t total = live + (a.shared_w0 ? 1 : 0);
    const uint32_t groups = gridDim.x, share = blockIdx.x;
    const uint32_t items = total * units;
    const uint32_t it0 = uint32_t(uint64_t(items) * share / groups), it1 = uint32_t(uint64_t(items) * (share + 1) / groups);
    if (it0 >= it1) return;
    const uint32_t k0 = it0 / units, k1 = (it1 - 1) / units;
    auto first_unit = [&](uint32_t k) { return k == k0 ? it0 % units : 0; };
    auto end_unit = [&](uint32_t k) { return k == k1 ? (it1 - 1) % units + 1 : units; };

    if (lane < kInfoSlots && k0 + lane <= k1) {
        const Record r = resolve_record(a, k0 + lane, live);
        if (!r.ok) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
        info[lane] = pack_record(r);
    }
    auto info_at = [&](uint32_t k) { return unpack_record(k - k0 < kInfoSlots ? info[k - k0] : pack_record(resolve_record(a, k, live))); };

    uint8_t* const my_stage = lds_raw + kStagesAt + wave * (kDnStages * kDnStageBytes);
    const uint32_t my_stage_lds = __builtin_amdgcn_readfirstlane(lds_address(my_stage));

    // ---- per-lane parts of the request addresses, from the first byte of the expert (the per-tile parts are uniform)
    // low nibbles: request q covers rows 8q .. 8q+7 of the tile, eight lanes per row (one 128-byte line: the row's
    // super-block kh); lane l sits at 16-byte slot l % 8 of its row in LDS and fetches chunk (l % 8) ^ (row % 8)
    const uint32_t ql_lane = uint32_t(a.spec.qs_offset) + (lane / 8) * (bpr * 128) + kh * 128 + (((lane % 8) ^ ((lane / 8) & 7)) * 16);
    // high bits: request q covers rows 16q .. 16q+15, four lanes per row (64 bytes); slot l % 4 holds chunk (l % 4) ^ ((row / 4) % 4)
    const uint32_t qh_lane = uint32_t(a.spec.qh_offset) + (lane / 4) * (bpr * 64) + kh * 64 + (((lane % 4) ^ ((lane / 16) & 3)) * 16);
    // lanes 0..31: the sixteen sub-scales of row l; lanes 32..39: the 128 bytes of d of the tile's rows; the rest repeat lane 39
    const uint32_t tail = lane < 40 ? lane - 32 : 7;
    const uint32_t hdr_lane = lane < 32 ? uint32_t(a.spec.sm_offset) + lane * (bpr * 16) + kh * 16 : uint32_t(a.spec.dm_offset) + tail * 16;
    const uint32_t hdr_tile_step = lane < 32 ? 32 * bpr * 16 : 32 * bpr * 2;
    auto request_tile = [&](const uint8_t* base, uint32_t unit, uint32_t stage_offset) {  // base: one expert (under 4 GiB), uniform
        const uint32_t tile = unit * 4 + nq;
        const uint32_t dst = my_stage_lds + stage_offset;
        const uint8_t* ql = base + uint64_t(tile) * (32 * bpr * 128);
        const uint8_t* qh = base + uint64_t(tile) * (32 * bpr * 64);
#pragma unroll
        for (int q = 0; q < 4; ++q) load_to_lds_16(ql + q * (8 * bpr * 128), ql_lane, dst + kQlAt + q * 1024);
#pragma unroll
        for (int q = 0; q < 2; ++q) load_to_lds_16(qh + q * (16 * bpr * 64), qh_lane, dst + kQhAt + q * 1024);
        load_to_lds_16(base, hdr_lane + tile * hdr_tile_step, dst + kScAt);
    };
    auto weight_base_of = [&](const Record& r) { return r.shared ? a.shared_w0 : a.w0 + uint64_t(r.expert) * a.spec.planar_expert_bytes; };

    uint32_t bad = 0, phase = 0;
    uint32_t biggest = 0;  // the largest result's bits without the sign: anything not finite shows at the end

    // ---- the request cursor runs two tiles ahead of the arithmetic: (record, unit)
    uint32_t rk = k0, runit = first_unit(k0), rstage = 0;
    bool rdone = false;
    const uint8_t* rbase = weight_base_of(info_at(k0));
    auto request_next = [&]() {  // past the end of the share the last tile is requested again (unused)
        request_tile(rbase, runit, rstage);
        rstage = rstage + kDnStageBytes == kDnStages * kDnStageBytes ? 0 : rstage + kDnStageBytes;
        if (rdone) return;
        if (runit + 1 < end_unit(rk)) { ++runit; return; }
        if (rk == k1) { rdone = true; return; }
        ++rk;
        runit = 0;
        rbase = weight_base_of(info_at(rk));
    };
#pragma unroll
    for (int s = 0; s < kDnStages; ++s) request_next();
    uint32_t stage = 0;

    f16x8 A[16];  // operand fragments: [section * 8 + quarter * 2 + fragment]
    float inv_scale = 1.0f;
    uint32_t store_at[2] = {0, 0};  // where this lane's two results of a tile go, from the first byte of the tile's columns in the output
    uint8_t* out_base = nullptr;
    auto load_rows = [&](uint32_t k) {
        const Record cur = info_at(k);
        // operand row n % 8: its route's h row; this wave finishes record rows 4 * k-half + 2 kh + {0, 1}
        const uint32_t op = n % 8;
        uint32_t src, dst[2];
        if (cur.shared) {
            src = op < a.tokens ? op : 0;
#pragma unroll
            for (int j = 0; j < 2; ++j) { const uint32_t res = 4 * khalf + 2 * kh + j; dst[j] = res < a.tokens ? res : 0; }
        } else {
            src = a.meta[1288 + cur.index * 8 + op];
#pragma unroll
            for (int j = 0; j < 2; ++j) dst[j] = a.meta[1288 + cur.index * 8 + 4 * khalf + 2 * kh + j];
            if (src >= a.tokens * a.selected || dst[0] >= a.tokens * a.selected || dst[1] >= a.tokens * a.selected) {
                if (cur.ok) bad |= TSP_ERRBIT_INDEX;
                src = 0; dst[0] = 0; dst[1] = 0;
            }
        }
        if (!cur.ok) { src = 0; dst[0] = 0; dst[1] = 0; }  // flagged already: the batch is refused whatever lands in row 0
        out_base = uniform_pointer(reinterpret_cast<uint8_t*>(cur.shared ? a.shared_out : a.out));
        const uint32_t out_stride = uint32_t(cur.shared ? a.shared_out_stride : a.out_stride);
        store_at[0] = dst[0] * out_stride + n * 4;
        store_at[1] = dst[1] * out_stride + n * 4;
        const float* row = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(cur.shared ? a.shared_x : a.x) +
                                                          uint64_t(src) * (cur.shared ? a.shared_x_stride : a.x_stride)) + kh * 256 + khalf * 16;
        f16x8 unused;
        const float back = stage_record_rows<false>(row, lane, A, unused, bad);
        inv_scale = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(back)));  // the same in every lane
#pragma unroll
        for (int t = 0; t < 16; ++t) asm volatile("" : "+v"(A[t]));
        asm volatile("" : "+v"(store_at[0]), "+v"(store_at[1]));
    };

    auto tile = [&](uint32_t unit) {
        // Wait for the tile's seven requests, which went out two tiles ago, ahead of that tile's two stores: younger than
        // they are those stores, the seven requests of the other stage and the two stores of the tile before (everything
        // completes in issue order; at a record's first tiles nothing older than the record's rows is outstanding at all)
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kDnStages - 1) * kDnTileLoads + 2 * kDnTileStores) : "memory");
        const uint8_t* st = my_stage + stage;
        RawQ6 raw[2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            raw[s].la = *reinterpret_cast<const u32x4*>(st + kQlAt + n * 128 + (((4 * s + khalf) ^ (n & 7)) * 16));
            raw[s].lb = *reinterpret_cast<const u32x4*>(st + kQlAt + n * 128 + (((4 * s + 2 + khalf) ^ (n & 7)) * 16));
            raw[s].qh = *reinterpret_cast<const u32x4*>(st + kQhAt + n * 64 + (((2 * s + khalf) ^ ((n >> 2) & 3)) * 16));
        }
        const uint4 sc = *reinterpret_cast<const uint4*>(st + kScAt + n * 16);
        const uint32_t dd = *reinterpret_cast<const uint32_t*>(st + kDAt + n * 4);  // d of super-blocks 0 and 1 of row n
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        request_next();  // the stage is free again: the tile two ahead goes there
        stage = stage + kDnStageBytes == kDnStages * kDnStageBytes ? 0 : stage + kDnStageBytes;
        raw[0].sc[0] = sc.x; raw[0].sc[1] = sc.y; raw[1].sc[0] = sc.z; raw[1].sc[1] = sc.w;
        const float d = half_bits_to_float(kh ? dd >> 16 : dd & 0xffffu);
        f32x16 blk;
        auto quarter = [&](auto s_tag, auto q_tag) {
            constexpr int S = decltype(s_tag)::value, Q = decltype(q_tag)::value;
            f16x8 f[2];
            frags_q6k<Q>(raw[S], khalf, f);
#pragma unroll
            for (int ff = 0; ff < 2; ++ff) {
                if (S == 0 && Q == 0 && ff == 0) {
                    const f32x16 zero{};
                    blk = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[0], f[0], zero, 0, 0, 0);
                } else {
                    blk = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[S * 8 + Q * 2 + ff], f[ff], blk, 0, 0, 0);
                }
            }
        };
        quarter(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
        quarter(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{});
        quarter(std::integral_constant<int, 0>{}, std::integral_constant<int, 2>{});
        quarter(std::integral_constant<int, 0>{}, std::integral_constant<int, 3>{});
        quarter(std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{});
        quarter(std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{});
        quarter(std::integral_constant<int, 1>{}, std::integral_constant<int, 2>{});
        quarter(std::integral_constant<int, 1>{}, std::integral_constant<int, 3>{});
        // Accumulator v < 4 is the high-half sum of record row 4 khalf + v, v + 4 its low-half sum. The wave's part of that
        // row's result is (d * sum) / scale; the partner wave holds the other super-block's part. Each hands the other two of
        // its four parts and finishes the other two: part of super-block 0 + part of super-block 1, whichever wave adds them.
        float part[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) part[e] = (d * (blk[e] + blk[e + 4])) * inv_scale;
        uint8_t* const tile_base = out_base + (unit * 4 + nq) * 128;  // uniform
        auto finish = [&](auto kh_tag) {
            constexpr int KH = decltype(kh_tag)::value;
            float2* const hand = reinterpret_cast<float2*>(lds_raw + (phase & 1) * kDnPhaseBytes + wave * kHandBytes) + lane;
            *hand = float2{part[2 * (1 - KH)], part[2 * (1 - KH) + 1]};
            lds_barrier();
            const float2 theirs = *(reinterpret_cast<const float2*>(lds_raw + (phase & 1) * kDnPhaseBytes + (wave ^ 4) * kHandBytes) + lane);
            ++phase;
            const float t2[2] = {theirs.x, theirs.y};
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const float mine = part[2 * KH + j];
                const float val = KH == 0 ? mine + t2[j] : t2[j] + mine;
                const uint32_t magnitude = __float_as_uint(val) & 0x7fffffffu;
                biggest = biggest > magnitude ? biggest : magnitude;
                // uniform base + 32-bit lane offset, spelled out: the compiler would form 64-bit addresses
                const uint32_t at = store_at[j];
                uint8_t* const base = tile_base;
                asm volatile("global_store_dword %0, %1, %2" ::"v"(at), "v"(val), "s"(base) : "memory");
            }
        };
        if (kh == 0) finish(std::integral_constant<int, 0>{});
        else finish(std::integral_constant<int, 1>{});
    };

    for (uint32_t k = k0; k <= k1; ++k) {
        load_rows(k);
        const uint32_t u1 = end_unit(k);
        for (uint32_t unit = first_unit(k); unit < u1; ++unit) tile(unit);
    }
    wait_all_loads();  // the last requests fetched tiles nobody reads: they must have landed before the stages are given away
    if (biggest >= 0x7f800000u) bad |= TSP_ERRBIT_NONFINITE;
    publish_error(bad, a.error_word);
}

int compute_units(int* out) {
    static std::atomic<uint64_t> seen{0};
    static int cus[64];
    int device = 0;
    if (first_use_on_device(seen, &device) || cus[device] == 0) {
        int n = 0;
        TSP_HIP(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device));
        cus[device] = n >= 1 ? n : 1;
    }
    *out = cus[device];
    return TSP_OK;
}

bool aligned16(const void* p, uint64_t stride) { return reinterpret_cast<uintptr_t>(p) % 16 == 0 && stride % 16 == 0; }

// results are addressed as a 32-bit offset from the output's first byte
bool spans_under_4g(uint32_t rows, uint64_t stride) { return rows == 0 || uint64_t(rows) * stride < (1ull << 32); }

}  // namespace

namespace tsp {

bool record_gate_up_takes(const SkinnyMoe& m) {
    if (!m.meta || m.tokens < 2 || m.tokens > kRecordRows || m.records > kMaxRecords) return false;
    if (m.gu.source_type != 12 || m.channels != 2048 || m.hidden % 32 || m.hidden < 32 || m.experts % 2) return false;
    if (!aligned16(m.x, m.x_stride) || !spans_under_4g(m.tokens * m.selected, m.h_stride)) return false;
    if (m.shared_gate && !spans_under_4g(m.tokens, m.shared_h_stride)) return false;
    return true;
}

int launch_record_gate_up(const SkinnyMoe& m, hipStream_t s) {
    RecordArgs a{};
    a.x = m.x; a.x_stride = m.x_stride; a.shared_x = m.x; a.shared_x_stride = m.x_stride;
    a.w0 = m.pair_lo; a.w1 = m.pair_hi; a.shared_w0 = m.shared_gate; a.shared_w1 = m.shared_up; a.spec = m.gu; a.meta = m.meta;
    a.out = m.h; a.out_stride = m.h_stride; a.shared_out = m.shared_h; a.shared_out_stride = m.shared_h_stride;
    a.experts = m.experts; a.tokens = m.tokens; a.selected = m.selected; a.records = m.records; a.n = m.hidden;
    a.error_word = m.error_word;
    int cus = 0;
    const int rc = compute_units(&cus);
    if (rc != TSP_OK) return rc;
    TSP_LAUNCH("record_gate_up_swiglu", s, record_gate_up_kernel<<<cus, kThreads, 0, s>>>(a));
    return launch_status("record_gate_up");
}

bool record_down_takes(const SkinnyMoe& m) {
    if (!m.meta || m.tokens < 2 || m.tokens > kRecordRows || m.records > kMaxRecords) return false;
    if (m.dn.source_type != 14 || m.hidden != 512 || m.channels % 128 || m.channels < 128) return false;
    if (!aligned16(m.h, m.h_stride) || !spans_under_4g(m.tokens * m.selected, m.y_stride)) return false;
    if (m.shared_down && (!aligned16(m.shared_h, m.shared_h_stride) || !spans_under_4g(m.tokens, m.shared_y_stride))) return false;
    return true;
}

int launch_record_down(const SkinnyMoe& m, hipStream_t s) {
    RecordArgs a{};
    a.x = m.h; a.x_stride = m.h_stride; a.shared_x = m.shared_h; a.shared_x_stride = m.shared_h_stride;
    a.w0 = m.down; a.shared_w0 = m.shared_down; a.spec = m.dn; a.meta = m.meta;
    a.out = m.y; a.out_stride = m.y_stride; a.shared_out = m.shared_y; a.shared_out_stride = m.shared_y_stride;
    a.experts = m.experts; a.tokens = m.tokens; a.selected = m.selected; a.records = m.records; a.n = m.channels;
    a.error_word = m.error_word;
    int cus = 0;
    const int rc = compute_units(&cus);
    if (rc != TSP_OK) return rc;
    TSP_LAUNCH("record_down", s, record_down_kernel<<<cus, kThreads, 0, s>>>(a));
    return launch_status("record_down");
}

}  // namespace tsp
