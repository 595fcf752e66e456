// Gate/up + SwiGLU of the T <= 8 routed MoE (decode, verify) for 2048-column Q4_K experts, over the union records (one per
// distinct expert, at most eight rows each) and, riding along as one more record, the layer's always-on expert.
//
// The launch moves about a megabyte of weights per distinct expert and is built, like the grouped prefill kernel
// (gate_up_resident.hip), around that stream:
//
//   * One persistent workgroup of eight waves per CU takes an equal contiguous share of the launch's (record, 32 hidden
//     units) items, in record order. The union block is copied to LDS once, by all threads, and the share's records are
//     kept in a small table there: inside the tile loop nothing is read from memory but weights.
//   * K is split over the waves: wave w owns super-block w of the 2048 columns. Every record multiplies rows of the same
//     few tokens, so a wave keeps the TOKENS' rows, its 256 columns of them, for the whole launch: read once as f32, scaled
//     by a power of two chosen from the largest magnitude among them, split into a high and a low half (22 significant
//     bits together) and held in registers as MFMA A fragments. Rows 0..7 of the 32-row operand are the tokens' high
//     halves, rows 8..15 their low halves; the two sums meet when the accumulators are read. Nothing but exact integers
//     (sc * q) meets them on the matrix cores, the block scales are applied in f32, and the power of two is taken off
//     again before partial sums of different waves meet.
//   * Weight tiles go global -> LDS directly into a wave-private ring of three stages, requested ahead by a cursor that
//     runs across record boundaries; nothing but these requests and the stores uses the vector memory counter inside
//     the loop, so every wait is an exact count.
//   * The K slices add up through LDS in wave order, and that is where a record's rows are found again: the lane that
//     finishes record row r reads the partial sums of operand row token[r]. A row a record does not have repeats its first
//     row, operand and destination alike (the union block pads its records that way), so every lane of the finishing
//     waves always stores; the two halves of the workgroup take turns finishing. Results do not depend on timing, nor on
//     which other records ride in the launch.
//
// The down product of these batches stays with the one-super-block-per-wave kernel (skinny.hip): its operand rows are a
// record's own h rows, so they change with the record, and built this way (rows turned into halves by the workgroup
// through LDS at every record) it measured 23.5 us a launch against 21.4.
#include "record_resident.hpp"

#include <type_traits>

#include "grouping_device.hpp"
#include "mfma_quant.hpp"

using namespace tsp;

namespace {

constexpr int kWaves = 8, kThreads = kWaves * kWave;
constexpr uint32_t kRecordRows = 8, kMaxRecords = 128;
constexpr uint32_t kInfoSlots = 32;  // records of a workgroup's share kept in LDS: a share spans at most records / groups + 2

struct RecordArgs {
    const float* x;            // token rows, x_stride bytes apart
    uint64_t x_stride;
    const uint8_t* w0;         // experts 0..E/2-1 as [gate_e, up_e]
    const uint8_t* w1;         // experts E/2..E-1
    const uint8_t* shared_w0;  // the always-on expert: gate
    const uint8_t* shared_w1;  // up
    tsp_planar_spec spec;
    const uint32_t* ids;       // the routes' expert ids, [tokens][selected]
    uint32_t* meta;            // the union block: written by workgroup 0 for the launches that follow
    float* out;                // h rows by route, out_stride bytes apart
    uint64_t out_stride;
    float* shared_out;         // the always-on expert's h rows, by token
    uint64_t shared_out_stride;
    uint32_t experts, tokens, selected, records, n;  // n: hidden units
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

// A wave's 256 columns of eight rows as MFMA A fragments: lane (n, k-half) of fragment t holds eight columns of row n % 8,
// their high halves where n % 16 < 8 and their low halves above. The fragments take the columns of every eight in the order
// (0, 2, 1, 3, 4, 6, 5, 7), the order in which a dword of nibbles unpacks, and come with the sums of the eight 32-column
// sub-blocks (over 32, as high and low halves: the operand of the minima term, zero in the low-half rows). Returns the
// power of two that takes the scaling off again.
// The rows are loaded the cheap way: lane l holds columns 4l .. 4l+3 of each of the eight rows (a row of the wave's 256
// columns is one contiguous kilobyte, one request), scales and splits its 32 values, and the wave turns the rows into
// fragments through 8.25 KB of LDS of its own: [high plane][low plane], a plane 8 rows x 512 B, 16-byte chunk c of row r
// at position c ^ r, then [8 rows][8 sums / 32 high halves, 8 residuals]. (Requesting every lane's own sixteen
// columns of its own row instead costs the memory pipeline ~50 cycles per request, 32 requests per wave: 6 us a launch.)
constexpr int kRowScratchBytes = 2 * 8 * 512 + 8 * 32;
__device__ __forceinline__ float rows_to_fragments(const float4 (&v)[8], uint32_t lane, uint8_t* scratch, f16x8 (&A)[16], f16x8& sxA, uint32_t& bad) {
    uint32_t top = 0;  // the largest magnitude as bits: an infinity or a NaN is larger than any finite value's
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t b0 = __float_as_uint(v[j].x) & 0x7fffffffu, b1 = __float_as_uint(v[j].y) & 0x7fffffffu;
        const uint32_t b2 = __float_as_uint(v[j].z) & 0x7fffffffu, b3 = __float_as_uint(v[j].w) & 0x7fffffffu;
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
    _Float16* const sums = reinterpret_cast<_Float16*>(scratch + 2 * 8 * 512);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float s4[4] = {v[j].x * scale, v[j].y * scale, v[j].z * scale, v[j].w * scale};
        _Float16 hi[4], lo[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            hi[e] = _Float16(s4[e]);
            lo[e] = _Float16(s4[e] - float(hi[e]));
        }
        // this lane's half of chunk l / 2, in the fragments' column order
        uint8_t* const at = scratch + j * 512 + (((lane / 2) ^ j) * 16) + (lane % 2) * 8;
        *reinterpret_cast<f16x4*>(at) = f16x4{hi[0], hi[2], hi[1], hi[3]};
        *reinterpret_cast<f16x4*>(at + 8 * 512) = f16x4{lo[0], lo[2], lo[1], lo[3]};
        float sum = (s4[0] + s4[1]) + (s4[2] + s4[3]);  // eight neighbouring lanes hold one 32-column sub-block
        sum = octet_sum(sum);
        if (lane % 8 == 0) {
            const float s32 = sum * 0.03125f;
            const _Float16 h = _Float16(s32);
            sums[j * 16 + lane / 8] = h;
            sums[j * 16 + 8 + lane / 8] = _Float16(s32 - float(h));
        }
    }
    // the planes are read back by other lanes of this same wave only: LDS serves a wave's requests in order
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const uint32_t r = lane % 8, khalf = (lane / 32) & 1;
    const uint8_t* const plane = scratch + ((lane & 8u) ? 8 * 512 : 0) + r * 512;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        const int c0 = (t / 4) * 64 + ((t / 2) % 2) * 32 + (t % 2) * 8;  // fragment t: pair of sub-blocks t / 4, low or high nibbles, first or second eight
        A[t] = *reinterpret_cast<const f16x8*>(plane + (((c0 / 8 + 2 * khalf) ^ r) * 16));
    }
    const f16x8 mine = *reinterpret_cast<const f16x8*>(sums + r * 16 + khalf * 8);
    const f16x8 none{};
    sxA = (lane & 8u) ? none : mine;
    return inv_scale;
}

// ---------------------------------------------------------------- a workgroup's share of the launch
constexpr int kMetaBytes = 9280;  // the union block
constexpr int kSlotBytes = 80;    // a record of the share: (index, expert, rows | flags), its 8 tokens, its 8 routes

// The union block, built by every workgroup for itself in LDS from the routes' expert ids (one load per thread instead of a
// launch of its own before this one); workgroup 0 also writes it to memory, where the down product's launch reads it. False
// when an id is out of range: the block's header is then zero in memory, the error bit set, and every workgroup leaves.
__device__ __forceinline__ bool build_union_block(const RecordArgs& a, uint32_t mine, uint32_t* block, uint32_t* scratch, uint32_t tid) {
    const bool writer = blockIdx.x == 0;
    return union_block(mine, tid, uint32_t(kThreads), a.experts, a.selected, a.tokens, a.n, 2048u, scratch,
                       [&](uint32_t word, uint32_t value) { block[word] = value; if (writer) a.meta[word] = value; },
                       [&]() { if (writer) atomicOr(a.error_word, TSP_ERRBIT_INDEX); });
}

// The launch's (record, unit) items, in record order, cut into equal contiguous shares, one per workgroup.
struct Share { uint32_t live, units, it0, it1, k0, k1; };
__device__ __forceinline__ Share share_of(const RecordArgs& a, const uint32_t* meta, uint32_t units, uint32_t tid) {
    Share s;
    const uint32_t listed = __builtin_amdgcn_readfirstlane(meta[6]);
    s.live = listed < a.records ? listed : a.records;
    if (listed > a.records && tid == 0 && blockIdx.x == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
    s.units = units;
    const uint32_t items = (s.live + (a.shared_w0 ? 1 : 0)) * units;  // at most 129 records x 512 units: the products below fit 32 bits
    s.it0 = items * blockIdx.x / gridDim.x;
    s.it1 = items * (blockIdx.x + 1) / gridDim.x;
    s.k0 = s.it0 / units;
    s.k1 = s.it1 > s.it0 ? (s.it1 - 1) / units : s.k0;
    return s;
}
__device__ __forceinline__ uint32_t first_unit(const Share& s, uint32_t k) { return k == s.k0 ? s.it0 % s.units : 0; }
__device__ __forceinline__ uint32_t end_unit(const Share& s, uint32_t k) { return k == s.k1 ? (s.it1 - 1) % s.units + 1 : s.units; }

// The share's records into their table: lane l looks after record k0 + l. Every wave writes the whole table for itself (the
// same words) and reads only what it wrote. A record that does not check out keeps every address inside the tensors
// (expert 0, token 0, route 0) and is flagged: the batch is refused whatever lands in row 0. A share spans at most
// records / groups + 2 records, far fewer than the table holds.
__device__ __forceinline__ void build_record_table(const RecordArgs& a, const uint32_t* meta, const Share& s, uint32_t lane, uint8_t* slots) {
    if (lane < kInfoSlots && s.k0 + lane <= s.k1) {
        const uint32_t k = s.k0 + lane;
        Record r;
        r.shared = a.shared_w0 != nullptr && k == s.live;
        r.index = k < kMaxRecords ? k : 0;
        r.expert = r.shared ? 0 : meta[8 + r.index];
        r.count = r.shared ? a.tokens : meta[136 + r.index];
        r.ok = r.count >= 1 && r.count <= kRecordRows && (r.shared || (k < s.live && r.expert < a.experts));
        uint32_t token[8], route[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            token[j] = r.shared ? (uint32_t(j) < a.tokens ? j : 0) : meta[264 + r.index * 8 + j];
            route[j] = r.shared ? token[j] : meta[1288 + r.index * 8 + j];
            if (token[j] >= a.tokens || route[j] >= a.tokens * a.selected) r.ok = false;
        }
        if (!r.ok) {
            atomicOr(a.error_word, TSP_ERRBIT_INDEX);
            r.expert = 0; r.count = 0; r.shared = false;
#pragma unroll
            for (int j = 0; j < 8; ++j) token[j] = route[j] = 0;
        }
        uint4* slot = reinterpret_cast<uint4*>(slots + lane * kSlotBytes);
        slot[0] = pack_record(r);
        slot[1] = uint4{token[0], token[1], token[2], token[3]};
        slot[2] = uint4{token[4], token[5], token[6], token[7]};
        slot[3] = uint4{route[0], route[1], route[2], route[3]};
        slot[4] = uint4{route[4], route[5], route[6], route[7]};
    }
}
__device__ __forceinline__ const uint8_t* slot_of(const uint8_t* slots, const Share& s, uint32_t k) {
    return slots + (k - s.k0 < kInfoSlots ? k - s.k0 : 0) * kSlotBytes;
}

// ---------------------------------------------------------------- gate/up + SwiGLU, Q4_K planes of 2048 columns
constexpr int kGuStageBytes = 5120;  // 32 rows x 128 B of nibbles, 32 x 16 B of scales / minima, 32 x 16 B holding d / dmin
constexpr int kGuStages = 3;
constexpr int kGuTileLoads = 5;
constexpr int kSumBytes = 4 * kWave * 4;               // a wave's partial sums of one tile: [4 rows per lane][64 lanes] f32
constexpr int kGuPhaseBytes = 2 * kWaves * kSumBytes;  // gate and up

// Every record multiplies rows of the same few tokens, so the tokens, not the records' rows, are what a wave keeps: operand
// row t is token t (high half; t + 8 the low half), for all of the launch, and a record's row r is found again when the
// partial sums are added up, by reading the sums of operand row token[r]. Between two records nothing is read from memory.
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void record_gate_up_kernel(RecordArgs a) {
    // LDS: [2 phases][gate, up][8 waves][1 KB of partial sums] (first: the union block) | [32 records of the share] | [8 waves][3 stages][5 KB weight tile]
    constexpr int kInfoAt = 2 * kGuPhaseBytes, kStagesAt = kInfoAt + kInfoSlots * kSlotBytes;
    static_assert(kMetaBytes <= kInfoAt);
    __shared__ __attribute__((aligned(16))) uint8_t lds_raw[kStagesAt + kWaves * kGuStages * kGuStageBytes];
    static_assert(sizeof(lds_raw) <= 160 * 1024, "one workgroup per compute unit");
    uint8_t* const slots = lds_raw + kInfoAt;

    const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const uint32_t n = lane % 32, khalf = lane / 32;
    constexpr uint32_t bpr = 8;  // 2048 columns
    const uint32_t units = a.n / 32;
    uint32_t bad = 0, phase = 0;

    // ---- the tokens' rows, this wave's 256 columns of them (a kilobyte per row and request)
    // the thread's route id first: the union records are built from the ids while the rows travel
    const uint32_t my_id = tid < a.tokens * a.selected ? a.ids[tid] : 0xffffffffu;
    float4 rows[8];
    {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t token = uint32_t(j) < a.tokens ? j : 0;  // a token the batch does not have repeats the first; nobody reads its sums
            rows[j] = *reinterpret_cast<const float4*>(reinterpret_cast<const uint8_t*>(a.x) + uint64_t(token) * a.x_stride + (wave * 256 + lane * 4) * 4);
        }
    }
    static_assert(kUnionScratchWords * 4 <= kGuStages * kGuStageBytes);
    if (!build_union_block(a, my_id, reinterpret_cast<uint32_t*>(lds_raw), reinterpret_cast<uint32_t*>(lds_raw + kStagesAt), tid)) return;
    __syncthreads();  // the block is complete; the scratch (the first wave's ring of stages) is free again
    const uint32_t* meta = reinterpret_cast<const uint32_t*>(lds_raw);
    const Share sh = share_of(a, meta, units, tid);
    if (sh.it0 >= sh.it1) return;
    const uint32_t k0 = sh.k0, k1 = sh.k1;  // first and last record of the share
    build_record_table(a, meta, sh, lane, slots);
    lds_barrier();  // every wave has taken what it needs from the union block: the partial sums live there from now on
    auto info_at = [&](uint32_t k) { return unpack_record(*reinterpret_cast<const uint4*>(slot_of(slots, sh, k))); };  // uniform

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

    // ---- the request cursor runs three tiles ahead of the arithmetic: (record, unit, gate or up)
    uint32_t rk = k0, runit = first_unit(sh, k0), rj = 0, rstage = 0;
    bool rdone = false;
    const uint8_t *rgate, *rup;
    weight_bases(info_at(k0), rgate, rup);
    auto request_next = [&]() {  // past the end of the share the last tile is requested again (unused)
        request_tile(rj == 0 ? rgate : rup, runit, rstage);
        rstage = rstage + kGuStageBytes == kGuStages * kGuStageBytes ? 0 : rstage + kGuStageBytes;
        if (rdone) return;
        if (rj == 0) { rj = 1; return; }
        if (runit + 1 < end_unit(sh, rk)) { rj = 0; ++runit; return; }
        if (rk == k1) { rdone = true; return; }
        ++rk;
        rj = 0;
        runit = 0;
        weight_bases(info_at(rk), rgate, rup);
    };
    // ---- the rows become operands through the wave's own ring of stages, which is idle until the first request: the
    // requests go out once the fragments have been read back
    f16x8 A[16];   // operand fragments: [k16 step of the super-block]
    f16x8 sxA;     // sub-block sums (k-half 0: the high halves, k-half 1: the residuals)
    static_assert(kRowScratchBytes <= kGuStages * kGuStageBytes);
    const float back = rows_to_fragments(rows, lane, my_stage, A, sxA, bad);
    const float inv_scale = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(back)));  // the same in every lane
    // Naming the fragments as operands makes the compiler wait for their LDS reads here, before the requests overwrite the planes
    // (and not at their first uses inside the tile loop).
#pragma unroll
    for (int t = 0; t < 16; ++t) asm volatile("" : "+v"(A[t]));
    asm volatile("" : "+v"(sxA));
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int s = 0; s < kGuStages; ++s) request_next();
    uint32_t stage = 0;  // byte offset of the stage the next tile sits in
    const Q4Consts q4c = q4_consts();
    const Q4ScaleConsts q4s = q4_scale_consts();

    // ---- what changes from record to record: where a reducing lane finds its row's sums, and where its result goes
    uint32_t sums_at = 0;   // float index, within a wave's partial sums, of the operand row that is this lane's record row
    uint32_t store_at = 0;  // byte offset of this lane's result from the first byte of the unit's columns in the output
    uint8_t* out_base = nullptr;
    auto enter_record = [&](uint32_t k) {
        const Record cur = info_at(k);
        const uint32_t* ids = reinterpret_cast<const uint32_t*>(slot_of(slots, sh, k) + 16);
        const uint32_t r = 4 * khalf + wave % 4;  // the record row this lane finishes when it is its half's turn
        const uint32_t token = ids[r], route = ids[8 + r];
        // operand row `token` is accumulator token % 4 of the lanes of k-half token / 4
        sums_at = (token % 4) * kWave + (token / 4) * 32 + n;
        out_base = uniform_pointer(reinterpret_cast<uint8_t*>(cur.shared ? a.shared_out : a.out));  // scalar registers: the unit's columns are added there
        store_at = route * uint32_t(cur.shared ? a.shared_out_stride : a.out_stride) + n * 4;
    };

    // ---- one tile: unpack, multiply, park the wave's partial sums; after the up tile the eight waves' sums meet
    auto tile = [&](uint32_t unit, auto j_tag) {
        constexpr int J = decltype(j_tag)::value;
        // Wait for the tile's five requests, which went out three tiles ago. Younger than those are the ten of the other two
        // stages and this wave's stores since: it stores in every other unit (`phase` counts the units), so for a gate tile
        // one of the two units before, for an up tile the unit before or none (everything completes in issue order).
        const uint32_t half = wave / 4;  // waves 0..3 finish the even units, waves 4..7 the odd ones
        const bool one_store = J == 0 ? phase >= 2 || (phase == 1 && half == 0) : phase >= 1 && ((phase - 1) & 1) == half;
        if (one_store) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kGuStages - 1) * kGuTileLoads + 1) : "memory");
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
        // Accumulator v of the 32 x 32 tile is operand row 8 (v / 4) + 4 khalf + v % 4: v < 4 the high halves of tokens
        // 4 khalf + v, v + 4 their low halves. partial = (d * sum(x * sc*q) - 32 dmin * sum(Sx / 32 * mn)) / scale
        float* const park = reinterpret_cast<float*>(lds_raw + (phase & 1) * kGuPhaseBytes + (J * kWaves + wave) * kSumBytes) + lane;
#pragma unroll
        for (int e = 0; e < 4; ++e) park[e * kWave] = __builtin_fmaf(-32.0f * dmin, mblk[e], d * (blk[e] + blk[e + 4])) * inv_scale;
        if constexpr (J == 1) {
            lds_barrier();
            if ((phase & 1) == wave / 4) {
                // a lane of wave e (or e + 4) adds up, in wave order, the eight waves' gate and up sums of the token that is row
                // 4 khalf + e of the record, and stores that row's h; the two halves of the workgroup take turns
                const float* in = reinterpret_cast<const float*>(lds_raw + (phase & 1) * kGuPhaseBytes) + sums_at;
                float g = 0.0f, u = 0.0f;
#pragma unroll
                for (int w = 0; w < kWaves; ++w) {
                    g += in[w * (kSumBytes / 4)];
                    u += in[(kWaves + w) * (kSumBytes / 4)];
                }
                const float h = (g * sigmoid_fast(g)) * u;
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
        enter_record(k);
        const uint32_t u1 = end_unit(sh, k);
        for (uint32_t unit = first_unit(sh, k); unit < u1; ++unit) {
            tile(unit, std::integral_constant<int, 0>{});
            tile(unit, std::integral_constant<int, 1>{});
        }
    }
    wait_all_loads();  // the last requests fetched tiles nobody reads: they must have landed before the stages are given away
    publish_error(bad, a.error_word);
}

int compute_units(int* out) {
    static std::atomic<uint64_t> seen{0};
    static int cus[64];
    int device = 0;
    if (setup_pending(seen, &device)) {
        int n = 0;
        TSP_HIP(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device));
        cus[device] = n >= 1 ? n : 1;
        setup_done(seen, device);
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
    if (!aligned16(m.x, m.x_stride) || !aligned16(m.meta, 0) || !spans_under_4g(m.tokens * m.selected, m.h_stride)) return false;
    if (m.shared_gate && !spans_under_4g(m.tokens, m.shared_h_stride)) return false;
    return true;
}

int launch_record_gate_up(const SkinnyMoe& m, hipStream_t s) {
    RecordArgs a{};
    a.x = m.x; a.x_stride = m.x_stride;
    a.w0 = m.pair_lo; a.w1 = m.pair_hi; a.shared_w0 = m.shared_gate; a.shared_w1 = m.shared_up; a.spec = m.gu; a.ids = m.ids; a.meta = m.meta;
    a.out = m.h; a.out_stride = m.h_stride; a.shared_out = m.shared_h; a.shared_out_stride = m.shared_h_stride;
    a.experts = m.experts; a.tokens = m.tokens; a.selected = m.selected; a.records = m.records; a.n = m.hidden;
    a.error_word = m.error_word;
    int cus = 0;
    const int rc = compute_units(&cus);
    if (rc != TSP_OK) return rc;
    TSP_LAUNCH("record_gate_up_swiglu", s, record_gate_up_kernel<<<cus, kThreads, 0, s>>>(a));
    return launch_status("record_gate_up");
}

}  // namespace tsp
