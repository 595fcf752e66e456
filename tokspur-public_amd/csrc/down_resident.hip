// Grouped down GEMM for 512-column experts in Q6_K planes (ql / qh / sc / d), Q8_0 planes (quants / d) or Q5_1 planes
// (nibbles / fifth bits / d, m), the task's h rows resident in registers.
//
// The companion of the activation-resident gate/up kernel, built the same way around the stream of expert weights:
//
//   * One persistent workgroup of eight waves per CU takes an equal contiguous share of the launch's (task, 128 output
//     channels) items, in task order; consecutive shares go to workgroups of one XCD.
//   * K = 512 is two super-blocks. Wave w multiplies super-block w / 4 of the 32 output channels w % 4 of the item: its A
//     operands, the task's <= 64 rows of h (halves of h / 256, by task slot) in those 256 columns, are loaded once per task
//     into registers (64 or 128 VGPRs) and stay there while the expert's 2048 weight rows stream past.
//   * A weight tile (32 rows x one super-block: 4 KB of low nibbles, 2 KB of high bit pairs, 512 B of sub-scales, the
//     rows' d) comes global -> LDS directly into a wave-private ring of two stages, requested two tiles ahead by a cursor
//     that runs across task boundaries. Nothing but these requests and the tile's stores uses the vector memory counter
//     inside the loop, so every wait is an exact count.
//   * The two waves that hold the two super-blocks of the same channels exchange the halves of their 32 x 32 f32 sums
//     through LDS (one LDS-only barrier per 32 rows) and each finishes 16 rows: out = fma(d1, sum1, d0 * sum0) * scale,
//     the order and the roundings of a sequential pass over the two super-blocks, whichever wave computes it.
//   * Every lane stores, always: a row past the task's end repeats the task's first row, operands and destination alike
//     (the same values to the same address), so the number of stores in flight is a constant too. Where a lane's sixteen
//     results go is worked out once per task (32-bit offsets from the output's first byte, a table in LDS), the share's
//     tasks are looked up once per pass (a table in LDS), and the routes are those the gate/up product of the same call
//     has already checked against the expert: inside the tile loop nothing is read from memory but weights.
#include "down_resident.hpp"
#include "mfma_quant.hpp"
#include "resident_tasks.hpp"

#include <type_traits>

using namespace tsp;

namespace {

constexpr int kWaves = 8, kThreads = kWaves * kWave;
constexpr int kTaskRows = 64;
// A stage holds one tile, 32 weight rows x one super-block (256 columns):
//   Q6_K planes: [32 rows x 128 B low nibbles][32 x 64 B high bits][32 x 16 B sub-scales][128 B of d: 32 rows x 2 super-blocks][pad]
//   Q8_0 planes: [32 rows x 256 B quants][32 x 16 B of d: eight blocks]
//   Q5_1 planes: [32 rows x 128 B nibbles][32 x 32 B fifth bits: eight blocks][32 x 32 B of d, m: eight blocks]
constexpr int kQ6 = 14, kQ8 = 8, kQ51 = 7;  // the planes' source types
constexpr int kQlAt = 0, kQhAt = 4096, kScAt = 6144, kDAt = 6656;
constexpr int kQ8dAt = 8192;
constexpr int kQ51hAt = 4096, kQ51dAt = 5120;
template <int KIND> constexpr int kStageBytes = KIND == kQ6 ? 7168 : KIND == kQ8 ? 8704 : 6144;
template <int KIND> constexpr int kTileLoads = KIND == kQ6 ? 7 : KIND == kQ8 ? 9 : 6;  // direct-to-LDS requests per tile and wave
// Q6_K exchanges through two buffers in turn (one barrier per exchange); the larger Q8_0 stages leave room for one buffer,
// which a second barrier hands back
template <int KIND> constexpr int kPhases = KIND == kQ8 ? 1 : 2;
constexpr int kStages = 2;
constexpr int kExchangeBytes = 2048;        // what a wave hands its partner per 32 rows: eight accumulators per lane
constexpr int kPhaseBytes = kWaves * kExchangeBytes;
constexpr uint32_t kInfoSlots = kResidentInfoSlots;

template <int KIND>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void down_resident_kernel(ResidentDownArgs a) {
    // LDS: [1 or 2 phases][8 waves][2 KB exchange] | [2 passes][32 tasks of the share] | [2 tasks][64 row offsets] | [8 waves][2 stages][weight tile]
    constexpr int kStageBytes = ::kStageBytes<KIND>, kTileLoads = ::kTileLoads<KIND>, kPhases = ::kPhases<KIND>;
    constexpr int kInfoAt = kPhases * kPhaseBytes, kRowsAt = kInfoAt + 2 * kInfoSlots * 16, kStagesAt = kRowsAt + 2 * kTaskRows * 4;
    __shared__ __attribute__((aligned(16))) uint8_t lds_raw[kStagesAt + kWaves * kStages * kStageBytes];
    static_assert(sizeof(lds_raw) <= 160 * 1024, "one workgroup per compute unit");
    uint4* const info_tables = reinterpret_cast<uint4*>(lds_raw + kInfoAt);
    uint32_t* const row_at = reinterpret_cast<uint32_t*>(lds_raw + kRowsAt);

    const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const uint32_t kh = wave / 4, nq = wave % 4;  // super-block, channel tile of the item
    constexpr uint32_t bpr = 2;                   // 512 columns
    const uint32_t units = a.channels / 128;

    const uint32_t bound = a.task_slots;
    const uint32_t listed = a.tasks[0];
    if (listed > bound || a.tasks[1] != a.tokens * a.selected || a.classes[0] + a.classes[1] != listed) {
        if (tid == 0 && blockIdx.x == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
        return;
    }
    const uint32_t groups = gridDim.x, share = (blockIdx.x % 8) * (groups / 8) + blockIdx.x / 8;

    uint8_t* const my_stage = lds_raw + kStagesAt + wave * (kStages * kStageBytes);
    const uint32_t my_stage_lds = __builtin_amdgcn_readfirstlane(lds_address(my_stage));

    // ---- per-lane parts of the request addresses, from the first byte of the expert (the per-tile parts are uniform)
    // Q6_K low nibbles: request q covers rows 8q .. 8q+7 of the tile, eight lanes per row (one 128-byte line: the row's
    // super-block kh); lane l sits at 16-byte slot l % 8 of its row in LDS and fetches chunk (l % 8) ^ (row % 8)
    const uint32_t ql_lane = uint32_t(a.spec.qs_offset) + (lane / 8) * (bpr * 128) + kh * 128 + (((lane % 8) ^ ((lane / 8) & 7)) * 16);
    // high bits: request q covers rows 16q .. 16q+15, four lanes per row (64 bytes); slot l % 4 holds chunk (l % 4) ^ ((row / 4) % 4)
    const uint32_t qh_lane = uint32_t(a.spec.qh_offset) + (lane / 4) * (bpr * 64) + kh * 64 + (((lane % 4) ^ ((lane / 16) & 3)) * 16);
    // lanes 0..31: the sixteen sub-scales of row l; lanes 32..39: the 128 bytes of d of the tile's rows; the rest repeat lane 39
    const uint32_t tail = lane < 40 ? lane - 32 : 7;
    const uint32_t hdr_lane = lane < 32 ? uint32_t(a.spec.sm_offset) + lane * (bpr * 16) + kh * 16 : uint32_t(a.spec.dm_offset) + tail * 16;
    const uint32_t hdr_tile_step = lane < 32 ? 32 * bpr * 16 : 32 * bpr * 2;
    // Q8_0 quants: a row is 16 blocks x 32 bytes; request q covers rows 4q .. 4q+3, sixteen lanes per row (the 256 bytes of the
    // row's super-block kh); slot l % 16 of row r holds chunk (l % 16) ^ (r % 16), and r % 16 = (l / 16) | (4q % 16), so request q
    // flips bits 2..3 of the chunk index of request 0: an exclusive or with (4q % 16) << 4 on the byte offset, whose bits 4..7
    // are the chunk's alone (row stride 512, super-block 256)
    const uint32_t q8_lane = (lane / 16) * 512 + kh * 256 + (((lane % 16) ^ (lane / 16)) * 16);
    // d: lanes 0..31 fetch the 16 bytes holding the eight d of row l's super-block kh; lanes 32..63 sit out
    const uint32_t q8d_lane = uint32_t(a.spec.dm_offset) + (lane % 32) * 32 + kh * 16;
    // Q5_1: the nibbles of a row's super-block are one 128-byte line, requested like the Q6_K low nibbles (ql_lane: row stride 256
    // either way); fifth bits and (d, m) are 4 bytes per block, 32 bytes per row and super-block: two lanes per row
    const uint32_t q51_lane = (lane / 2) * 64 + kh * 32 + (lane % 2) * 16;

    auto request_tile = [&](const uint8_t* base, uint32_t unit, uint32_t stage_offset) {  // base: one expert (under 4 GiB), uniform
        const uint32_t tile = unit * 4 + nq;
        const uint32_t dst = my_stage_lds + stage_offset;
        if constexpr (KIND == kQ6) {
            const uint8_t* ql = base + uint64_t(tile) * (32 * bpr * 128);
            const uint8_t* qh = base + uint64_t(tile) * (32 * bpr * 64);
#pragma unroll
            for (int q = 0; q < 4; ++q) load_to_lds_16(ql + q * (8 * bpr * 128), ql_lane, dst + kQlAt + q * 1024);
#pragma unroll
            for (int q = 0; q < 2; ++q) load_to_lds_16(qh + q * (16 * bpr * 64), qh_lane, dst + kQhAt + q * 1024);
            load_to_lds_16(base, hdr_lane + tile * hdr_tile_step, dst + kScAt);
        } else if constexpr (KIND == kQ8) {
            const uint8_t* qs = base + a.spec.qs_offset + uint64_t(tile) * (32 * 512);
#pragma unroll
            for (int q = 0; q < 8; ++q) load_to_lds_16(qs + q * (4 * 512), q8_lane ^ (((4 * q) & 15) << 4), dst + q * 1024);
            if (lane < 32) load_to_lds_16(base, q8d_lane + tile * (32 * 32), dst + kQ8dAt);  // one request of the wave, half its lanes
        } else {
            const uint8_t* qs = base + uint64_t(tile) * (32 * 256);
#pragma unroll
            for (int q = 0; q < 4; ++q) load_to_lds_16(qs + q * (8 * 256), ql_lane, dst + q * 1024);
            load_to_lds_16(base + a.spec.qh_offset + uint64_t(tile) * (32 * 64), q51_lane, dst + kQ51hAt);
            load_to_lds_16(base + a.spec.dm_offset + uint64_t(tile) * (32 * 64), q51_lane, dst + kQ51dAt);
        }
    };

    uint32_t bad = 0, phase = 0, parity = 0;
    uint32_t biggest = 0;  // the largest result's bits without the sign: anything not finite shows at the end
    const float s256 = a.out_scale;

    auto pass = [&](auto mt_tag) {
        constexpr int MT = decltype(mt_tag)::value;
        const uint32_t of_kind = a.classes[MT - 1];
        const uint32_t* list = a.classes + 2 + (MT - 1) * bound;
        const uint32_t items = of_kind * units;
        const uint32_t it0 = uint32_t(uint64_t(items) * share / groups), it1 = uint32_t(uint64_t(items) * (share + 1) / groups);
        if (it0 >= it1) return;
        const uint32_t k0 = it0 / units, k1 = (it1 - 1) / units;  // first and last position in the kind's list
        auto first_unit = [&](uint32_t k) { return k == k0 ? it0 % units : 0; };
        auto end_unit = [&](uint32_t k) { return k == k1 ? (it1 - 1) % units + 1 : units; };

        // ---- the share's tasks, looked up once: (task, expert, first row, rows | shared << 8 | ok << 9) per list position, in
        // LDS. Every wave writes the whole table for itself (the same words), so nothing inside the tile loop reads task lists
        // from memory: a vector load there would have the compiler drain the requests in flight before it goes on.
        uint4* const info = info_tables + (MT - 1) * kInfoSlots;  // a table per pass: a wave may start the second pass while others finish the first
        auto resolve = [&](uint32_t k) { return resolve_resident_task(a.tasks, a.counts, list[k], listed, a.experts, a.tokens, a.shared_down != nullptr); };
        if (lane < kInfoSlots && k0 + lane <= k1) {
            const ResidentTask t = resolve(k0 + lane);
            if (!t.ok) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
            info[lane] = pack_resident_task(t);
        }
        using Info = ResidentTask;
        auto info_at = [&](uint32_t k) {  // uniform; a share of more tasks than the table holds resolves the rest the slow way
            return unpack_resident_task(k - k0 < kInfoSlots ? info[k - k0] : pack_resident_task(resolve(k)));
        };
        auto weight_base_of = [&](const Info& t) { return t.shared ? a.shared_down : a.down + uint64_t(t.expert) * a.spec.planar_expert_bytes; };

        f16x8 A[MT][16];        // h fragments: [row tile][section * 8 + quarter * 2 + fragment]
        // ---- the request cursor runs two tiles ahead of the arithmetic: (list position, unit)
        uint32_t rk = k0, runit = first_unit(k0), rstage = 0;
        bool rdone = false;
        const uint8_t* rbase = weight_base_of(info_at(k0));
        auto request_next = [&]() {  // past the end of the share the last tile is requested again (unused)
            request_tile(rbase, runit, rstage);
            rstage = rstage + kStageBytes == kStages * kStageBytes ? 0 : rstage + kStageBytes;
            if (rdone) return;
            if (runit + 1 < end_unit(rk)) { ++runit; return; }
            if (rk == k1) { rdone = true; return; }
            ++rk;
            runit = 0;
            rbase = weight_base_of(info_at(rk));
        };
        request_next();
        request_next();
        uint32_t stage = 0;  // byte offset of the stage the next tile sits in

        uint8_t* out_base = nullptr;  // the rows the task's results go to
        auto load_rows = [&](uint32_t k) {  // the task at list position k: this wave's 256 columns of its h rows, and where its results go
            const Info cur = info_at(k);
            out_base = reinterpret_cast<uint8_t*>(cur.shared ? a.shared_y : a.y);
            const uint32_t out_stride = uint32_t(cur.shared ? a.shared_y_stride : a.y_stride);
            const uint32_t n = lane % 32, khalf = lane / 32;
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const uint32_t r = i * 32 + n, rr = r < cur.nrows ? r : 0;  // a row past the end repeats the first
                const _Float16* row = a.hbuf + (uint64_t(cur.task) * kTaskRows + rr) * (bpr * 256) + kh * 256 + khalf * 16;
#pragma unroll
                for (int t = 0; t < 16; ++t) {
                    // Q6_K: section t / 8, quarter (t / 2) % 4, fragment t % 2; Q8_0, Q5_1: block t / 2, fragment t % 2. Either way a
                    // lane's k-half takes sixteen consecutive columns of every 32.
                    if constexpr (KIND == kQ6) A[i][t] = *reinterpret_cast<const f16x8*>(row + (t / 8) * 128 + ((t / 2) % 4) * 32 + (t % 2) * 8);
                    else A[i][t] = *reinterpret_cast<const f16x8*>(row + (t / 2) * 32 + (t % 2) * 8);
                }
            }
            // Lane l looks up where task row l goes: its route (for the always-on expert its token). The gate/up product of
            // the same call has checked every route against the expert; here the index only has to stay inside the output.
            const uint32_t rr = lane < cur.nrows ? lane : 0;
            uint32_t dst;
            if (cur.shared) {
                dst = cur.start + rr;
            } else {
                dst = a.token_map[uint64_t(cur.expert) * a.tokens + cur.start + rr];
                if (dst >= a.tokens * a.selected) { if (cur.ok) bad |= TSP_ERRBIT_INDEX; dst = 0; }
            }
            if (!cur.ok) dst = 0;  // a task that does not check out is flagged; the batch is refused whatever lands in row 0
            // where the 64 task rows go, as byte offsets from the output's first byte: a table per wave (all eight write the same
            // words, each reads its own), two of them in turn because a wave may be a task ahead of its partner's last reads
            parity ^= 1;
            row_at[parity * kTaskRows + lane] = dst * out_stride;  // a row past the end has looked up the first row's
            // The rows are needed at once. Naming every fragment as an operand here makes the compiler wait for their loads now:
            // left to itself it waits at the fragments' first uses inside the tile loop, in every pass of the loop, with counts
            // that know nothing of the requests in flight and so drain them tile after tile.
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int t = 0; t < 16; ++t) asm volatile("" : "+v"(A[i][t]));
        };

        auto tile = [&](uint32_t unit) {
            // wait for the tile's seven requests, which went out in the tile before last, ahead of that tile's stores: younger than
            // they are those stores, the seven requests of the other stage and the stores of the tile before (everything
            // completes in issue order; at a task's first tiles nothing older than the task's rows is outstanding at all)
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kStages - 1) * kTileLoads + 16 * MT) : "memory");
            uint32_t lane_now = lane;
            if constexpr (MT == 2) asm volatile("" : "+v"(lane_now));  // lane-derived addresses are derived again per tile, not kept
            const uint32_t n = lane_now % 32, khalf = (lane_now / 32) & 1;  // & 1: the compiler must see that khalf picks no sub-scale word
            const uint8_t* st = my_stage + stage;
            f32x16 blk[MT];
            float d0 = 0, d1 = 0;
            if constexpr (KIND == kQ6) {
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
                raw[0].sc[0] = sc.x; raw[0].sc[1] = sc.y; raw[1].sc[0] = sc.z; raw[1].sc[1] = sc.w;
                // the output scale is a power of two: folded into d it changes no rounding
                d0 = half_bits_to_float(dd & 0xffffu) * s256;
                d1 = half_bits_to_float(dd >> 16) * s256;
                auto quarter = [&](auto s_tag, auto q_tag) {
                    constexpr int S = decltype(s_tag)::value, Q = decltype(q_tag)::value;
                    f16x8 f[2];
                    frags_q6k<Q>(raw[S], khalf, f);
#pragma unroll
                    for (int ff = 0; ff < 2; ++ff)
#pragma unroll
                        for (int i = 0; i < MT; ++i) {
                            if (S == 0 && Q == 0 && ff == 0) {
                                const f32x16 zero{};
                                blk[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[i][0], f[0], zero, 0, 0, 0);
                            } else {
                                blk[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[i][S * 8 + Q * 2 + ff], f[ff], blk[i], 0, 0, 0);
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
            } else if constexpr (KIND == kQ51) {
                // Q5_1: element e of a block is nibble e % 16 (low for e < 16, high above) of byte e % 16 with bit e of the
                // block's fifth-bit word on top; the lane's k-half takes elements 16 khalf .. 16 khalf + 15. A weight is the
                // half nearest to d * q + m: q exact as a half, one packed fused multiply-add, one rounding (the f32
                // evaluation rounds the sum to f32 first, which can move the half only when that sum sits on a tie).
                u32x4 q[8];
#pragma unroll
                for (int b = 0; b < 8; ++b) q[b] = *reinterpret_cast<const u32x4*>(st + n * 128 + ((b ^ (n & 7)) * 16));
                u32x4 fifth[2], dm[2];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    fifth[h] = *reinterpret_cast<const u32x4*>(st + kQ51hAt + n * 32 + h * 16);
                    dm[h] = *reinterpret_cast<const u32x4*>(st + kQ51dAt + n * 32 + h * 16);
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                request_next();  // the stage is free again: the tile two ahead goes there
#pragma unroll
                for (int b = 0; b < 8; ++b) {
                    const uint32_t pair = dm[b / 4][b % 4];  // d in the low half, m in the high half
                    const f16x2 d2 = as_h2(__builtin_amdgcn_perm(pair, pair, 0x05040504u)), m2 = as_h2(__builtin_amdgcn_perm(pair, pair, 0x07060706u));
                    const uint32_t bits = fifth[b / 4][b % 4] >> (16 * khalf);
                    const f16x2 off = splat(-1024.0f);
                    f16x8 f[2];
#pragma unroll
                    for (int ff = 0; ff < 2; ++ff) {
                        f16x2 p[4];
#pragma unroll
                        for (int j = 0; j < 2; ++j) {
                            const int w = 2 * ff + j;  // bytes 4 w .. 4 w + 3 of the block: elements 16 khalf + 4 w .. + 3
                            const uint32_t nibbles = (q[b][w] >> (4 * khalf)) & 0x0f0f0f0fu;
                            // bits 4 w .. 4 w + 3 of the fifth-bit half-word to bit 0 of four bytes: no two partial products share a bit
                            const uint32_t four = ((bits >> (4 * w)) & 15u) * 0x00204081u & 0x01010101u;
                            const uint32_t codes = nibbles | (four << 4);
                            p[2 * j] = fma2(as_h2(spread01(codes, 0x64646464u)) + off, d2, m2);
                            p[2 * j + 1] = fma2(as_h2(spread23(codes, 0x64646464u)) + off, d2, m2);
                        }
                        f[ff] = f16x8{p[0][0], p[0][1], p[1][0], p[1][1], p[2][0], p[2][1], p[3][0], p[3][1]};
                    }
#pragma unroll
                    for (int ff = 0; ff < 2; ++ff)
#pragma unroll
                        for (int i = 0; i < MT; ++i) {
                            if (b == 0 && ff == 0) {
                                const f32x16 zero{};
                                blk[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[i][0], f[0], zero, 0, 0, 0);
                            } else {
                                blk[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[i][b * 2 + ff], f[ff], blk[i], 0, 0, 0);
                            }
                        }
                }
            } else {
                // Q8_0: sixteen quants of row n per block (the lane's k-half of the block's 32) and the row's eight d. A weight
                // is the half nearest to d * q, the engine's arithmetic for this kind: q is exact as a half and so is d, so one
                // packed half multiply rounds once, as the f32 product rounded to half does.
                u32x4 q[8];
#pragma unroll
                for (int b = 0; b < 8; ++b) q[b] = *reinterpret_cast<const u32x4*>(st + n * 256 + (((2 * b + khalf) ^ (n & 15)) * 16));
                const u32x4 dd = *reinterpret_cast<const u32x4*>(st + kQ8dAt + n * 16);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                request_next();  // the stage is free again: the tile two ahead goes there
#pragma unroll
                for (int b = 0; b < 8; ++b) {
                    const uint32_t pair = dd[b / 2];
                    const f16x2 d2 = as_h2(b % 2 ? __builtin_amdgcn_perm(pair, pair, 0x07060706u) : __builtin_amdgcn_perm(pair, pair, 0x05040504u));
                    f16x8 f[2];
#pragma unroll
                    for (int ff = 0; ff < 2; ++ff) {
                        const f16x8 whole = quants8(q[b][2 * ff], q[b][2 * ff + 1]);
                        const f16x2 p0 = f16x2{whole[0], whole[1]} * d2, p1 = f16x2{whole[2], whole[3]} * d2;
                        const f16x2 p2 = f16x2{whole[4], whole[5]} * d2, p3 = f16x2{whole[6], whole[7]} * d2;
                        f[ff] = f16x8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
                    }
#pragma unroll
                    for (int ff = 0; ff < 2; ++ff)
#pragma unroll
                        for (int i = 0; i < MT; ++i) {
                            if (b == 0 && ff == 0) {
                                const f32x16 zero{};
                                blk[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[i][0], f[0], zero, 0, 0, 0);
                            } else {
                                blk[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[i][b * 2 + ff], f[ff], blk[i], 0, 0, 0);
                            }
                        }
                }
            }
            stage = stage + kStageBytes == kStages * kStageBytes ? 0 : stage + kStageBytes;

            // Accumulator v of a 32 x 32 tile is row 8 (v / 4) + 4 khalf + v % 4, column n. The wave of super-block 0 finishes
            // rows 0..15 (v < 8), its partner rows 16..31: each hands over the eight sums of the other's rows. Which of the two a
            // wave is, is a scalar: one branch per tile instead of a select per value.
            uint8_t* const tile_base = out_base + (unit * 4 + nq) * 128;  // uniform
            auto finish = [&](auto kh_tag) {
                constexpr int KH = decltype(kh_tag)::value;
#pragma unroll
                for (int i = 0; i < MT; ++i) {
                    uint8_t* out = lds_raw + (phase % kPhases) * kPhaseBytes + wave * kExchangeBytes + lane_now * 16;
#pragma unroll
                    for (int c = 0; c < 2; ++c) {
                        f32x4 v;
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = blk[i][8 * (1 - KH) + 4 * c + e];
                        *reinterpret_cast<f32x4*>(out + c * 1024) = v;
                    }
                    lds_barrier();
                    const uint8_t* in = lds_raw + (phase % kPhases) * kPhaseBytes + (wave ^ 4) * kExchangeBytes + lane_now * 16;
                    ++phase;
                    f32x4 theirs[2];
#pragma unroll
                    for (int c = 0; c < 2; ++c) theirs[c] = *reinterpret_cast<const f32x4*>(in + c * 1024);
                    if constexpr (kPhases == 1) lds_barrier();  // both have read: the one buffer may be written again
#pragma unroll
                    for (int c = 0; c < 2; ++c) {
                        // accumulator 4 c + e of the wave's half of the row tile is task row 32 i + 16 KH + 8 c + 4 khalf + e
                        const u32x4 to = *reinterpret_cast<const u32x4*>(&row_at[parity * kTaskRows + i * 32 + 16 * KH + 8 * c + 4 * khalf]);
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float mine = blk[i][8 * KH + 4 * c + e];
                            const float sum0 = KH == 0 ? mine : theirs[c][e], sum1 = KH == 0 ? theirs[c][e] : mine;
                            // Q6_K: the integer sums of the two super-blocks times their d, in the order of a sequential pass;
                            // Q8_0, Q5_1: the weights carried their scales, the two halves of K just add
                            const float val = KIND == kQ6 ? __builtin_fmaf(d1, sum1, d0 * sum0) : (sum0 + sum1) * s256;
                            const uint32_t magnitude = __float_as_uint(val) & 0x7fffffffu;
                            biggest = biggest > magnitude ? biggest : magnitude;
                            // uniform base + 32-bit lane offset, spelled out: the compiler would form 64-bit addresses
                            const uint32_t at = to[e] + n * 4;
                            uint8_t* const base = tile_base;
                            asm volatile("global_store_dword %0, %1, %2" ::"v"(at), "v"(val), "s"(base) : "memory");
                        }
                    }
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
        wait_all_loads();  // the last requests fetched tiles nobody reads: they must have landed before the stages are reused or given away
    };
    pass(std::integral_constant<int, 2>{});
    pass(std::integral_constant<int, 1>{});
    if (biggest >= 0x7f800000u) bad |= TSP_ERRBIT_NONFINITE;
    publish_error(bad, a.error_word);
}

}  // namespace

namespace tsp {

bool resident_down_takes(uint32_t source_type, uint32_t channels, uint32_t hidden) {
    return (source_type == kQ6 || source_type == kQ8 || source_type == kQ51) && hidden == 512 && channels % 128 == 0 && channels >= 128;
}

int launch_resident_down(const ResidentDownArgs& a, hipStream_t s) {
    static std::atomic<uint64_t> seen{0};
    static int cus[64];
    int device = 0;
    if (setup_pending(seen, &device)) {
        int n = 0;
        TSP_HIP(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device));
        cus[device] = n >= 8 ? n / 8 * 8 : 8;
        setup_done(seen, device);
    }
    if (a.spec.source_type == kQ6) TSP_LAUNCH("gemm_down", s, down_resident_kernel<kQ6><<<cus[device], kThreads, 0, s>>>(a));
    else if (a.spec.source_type == kQ8) TSP_LAUNCH("gemm_down", s, down_resident_kernel<kQ8><<<cus[device], kThreads, 0, s>>>(a));
    else TSP_LAUNCH("gemm_down", s, down_resident_kernel<kQ51><<<cus[device], kThreads, 0, s>>>(a));
    return launch_status("down_resident");
}

}  // namespace tsp
