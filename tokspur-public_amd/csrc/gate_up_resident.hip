// Grouped gate/up GEMM with fused SwiGLU for 2048-column Q4_K experts, activations resident in registers.
//
// The ragged grouped product is bound by the expert weights streaming in from HBM, so the kernel is built around that
// stream and keeps everything else off the memory pipeline:
//
//   * One persistent workgroup of eight waves per CU. The launch's work, the (task, 32 hidden units) items in task order,
//     is cut into equal contiguous shares, one per workgroup; consecutive shares go to workgroups of the same XCD so that
//     the tasks of one expert meet in one L2.
//   * The K dimension is split over the waves: wave w owns super-block w (columns 256 w .. 256 w + 255) of every weight
//     row. Its A operands, the task's <= 64 activation rows of those 256 columns, are loaded ONCE per task into registers
//     (64 or 128 VGPRs as MFMA fragments) and stay there while all of the expert's rows stream past. No activation byte is
//     read twice per task and none passes through LDS.
//   * Weights go global -> LDS directly (no registers in between), a tile of 32 rows x one 128-byte line of nibbles +
//     the rows' scale bytes and d/dmin per request, into a wave-private ring of two stages. Eight neighbouring lanes fetch
//     one whole cache line. Nothing but these requests and the epilogue's stores uses the vector memory counter inside
//     the loop, so each wave waits with an exact count, and since the ring is private no barrier guards it.
//   * A wave's product over its super-block, d * sum(x * sc*q) - dmin * sum(Sx * mn), is a partial result of a 32 x 32
//     tile; the eight partials add up through LDS in wave order (a fixed order: results are reproducible bit for bit) with
//     one barrier per tile, and the threads that hold gate and up of the same hidden units apply SwiGLU and store h / 256
//     as halves, the format the down GEMM reads.
//   * A wave issues at most one instruction every four cycles and two waves share a SIMD, so what a wave executes per
//     tile is kept short: unpacking is one mask-or and one packed multiply-add per pair of weights, scales are set up two
//     sub-blocks at a time, the sigmoid uses the hardware exponential and reciprocal, every lane stores (rows a task
//     does not have repeat its first row, value and slot alike), and the tasks of at most 32 rows run in a loop of their own that keeps
//     every address in registers. Measured with the arithmetic, the requests or the barrier taken out in turn, no single
//     one of them bounds the kernel: what is left is the chain of latencies of one tile (arrival, LDS, matrix results,
//     barrier, sum) at two waves per SIMD.
#include "gate_up_resident.hpp"
#include "mfma_quant.hpp"
#include "resident_tasks.hpp"

#include <type_traits>

using namespace tsp;

namespace {

constexpr int kWaves = 8, kThreads = kWaves * kWave;
constexpr int kTaskRows = 64;              // rows of a task (the grouped GEMMs' own task list)
constexpr int kStageBytes = 5120;          // 32 rows x 128 B of nibbles, 32 x 16 B of scales / minima, 32 x 16 B holding d / dmin
constexpr int kStages = 2;
constexpr int kPartialBytes = 4096;        // one wave's 32 x 32 f32 partial tile
constexpr int kPhaseBytes = kWaves * kPartialBytes;
constexpr int kTileLoads = 5;              // direct-to-LDS requests per tile and wave
constexpr uint32_t kInfoSlots = kResidentInfoSlots;

__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void gate_up_resident_kernel(ResidentGateUpArgs a) {
    // LDS: [2 phases][8 waves][4 KB partial tile] | [2 passes][32 tasks of the share] | [8 waves][2 stages][5 KB weight tile]
    constexpr int kInfoAt = 2 * kPhaseBytes, kStagesAt = kInfoAt + 2 * kInfoSlots * 16;
    __shared__ __attribute__((aligned(16))) uint8_t lds_raw[kStagesAt + kWaves * kStages * kStageBytes];
    uint4* const info_tables = reinterpret_cast<uint4*>(lds_raw + kInfoAt);

    const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const uint32_t n = lane % 32, khalf = lane / 32;
    constexpr uint32_t bpr = 8;  // 2048 columns
    const uint32_t units = a.hidden / 32;

    // ---- the launch's task list must be whole before anything is addressed through it
    const uint32_t bound = a.task_slots;
    const uint32_t listed = a.tasks[0];
    if (listed > bound || a.tasks[1] != a.tokens * a.selected || a.classes[0] + a.classes[1] != listed) {
        if (tid == 0 && blockIdx.x == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
        return;
    }
    const uint32_t groups = gridDim.x, share = (blockIdx.x % 8) * (groups / 8) + blockIdx.x / 8;

    uint8_t* const my_stage = lds_raw + kStagesAt + wave * (kStages * kStageBytes);

    const uint32_t my_stage_lds = __builtin_amdgcn_readfirstlane(lds_address(my_stage));

    // ---- per-lane parts of the request addresses (the per-tile parts are uniform and stay in scalar registers)
    // nibbles: request q covers rows 8q .. 8q+7 of the tile, eight lanes per row; lane l sits at 16-byte slot l % 8 of
    // its row in LDS and fetches chunk (l % 8) ^ (row % 8), so that the fragment reads below spread over all banks
    const uint32_t qs_lane = uint32_t(a.spec.qs_offset) + (lane / 8) * (bpr * 128) + wave * 128 + (((lane % 8) ^ ((lane / 8) & 7)) * 16);
    // lanes 0..31: scales and minima of row l (16 B); lanes 32..63: the 16 bytes holding d / dmin of row l - 32
    const uint32_t hdr_lane = lane < 32 ? uint32_t(a.spec.sm_offset) + lane * (bpr * 16) + wave * 16
                                        : uint32_t(a.spec.dm_offset) + (lane - 32) * (bpr * 4) + (wave / 4) * 16;
    const uint32_t hdr_unit_step = lane < 32 ? 32 * bpr * 16 : 32 * bpr * 4;

    using Info = ResidentTask;
    auto weight_bases = [&](const Info& t, const uint8_t*& gate, const uint8_t*& up) {
        if (t.shared) { gate = a.shared_gate; up = a.shared_up; return; }
        const uint32_t half_e = a.experts / 2;
        const uint8_t* pair = (t.expert < half_e ? a.pair_lo : a.pair_hi) + uint64_t(t.expert < half_e ? t.expert : t.expert - half_e) * 2 * a.spec.planar_expert_bytes;
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
    uint32_t biggest = 0;  // the largest carried half's bits without the sign: anything not finite shows at the end
    const Q4Consts q4c = q4_consts();
    const Q4ScaleConsts q4s = q4_scale_consts();

    // The tasks come in two kinds, those of at most 32 rows (one row tile: 64 registers of activations) and those of 33..64
    // (two row tiles, 128 registers), each with its own loop so that neither carries the other's registers. A workgroup takes
    // the same share of either kind's (task, unit) items: equal work for every workgroup whatever the mix of kinds.
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
        // from memory: a vector load there would have the compiler drain the requests in flight before it goes on. A table per
        // pass: a wave may start the second pass while others finish the first.
        uint4* const info = info_tables + (MT - 1) * kInfoSlots;
        auto resolve = [&](uint32_t k) { return resolve_resident_task(a.tasks, a.counts, list[k], listed, a.experts, a.tokens, a.shared_gate != nullptr); };
        if (lane < kInfoSlots && k0 + lane <= k1) {
            const ResidentTask t = resolve(k0 + lane);
            if (!t.ok) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
            info[lane] = pack_resident_task(t);
        }
        auto info_at = [&](uint32_t k) {  // uniform; a share of more tasks than the table holds resolves the rest the slow way
            return unpack_resident_task(k - k0 < kInfoSlots ? info[k - k0] : pack_resident_task(resolve(k)));
        };

        f16x8 A[MT][16];   // activation fragments: [row tile][k16 step of the super-block]
        f16x8 sxA[MT];     // activation sums (k-half 0: the eight sub-block sums' high halves, k-half 1: the residuals)
        // ---- the request cursor runs two tiles ahead of the arithmetic: (list position, unit, gate or up)
        uint32_t rk = k0, runit = first_unit(k0), rj = 0, rstage = 0;
        bool rdone = false;
        const uint8_t *rgate, *rup;
        weight_bases(info_at(k0), rgate, rup);
        auto request_next = [&]() {  // past the end of the share the last tile is requested again (unused)
            request_tile(rj == 0 ? rgate : rup, runit, rstage);
            rstage = rstage + kStageBytes == kStages * kStageBytes ? 0 : rstage + kStageBytes;
            if (rdone) return;
            if (rj == 0) { rj = 1; return; }
            if (runit + 1 < end_unit(rk)) { rj = 0; ++runit; return; }
            if (rk == k1) { rdone = true; return; }
            ++rk;
            rj = 0;
            runit = 0;
            weight_bases(info_at(rk), rgate, rup);
        };
        request_next();
        request_next();
        uint32_t stage = 0;  // byte offset of the stage the next tile sits in

        uint32_t task = 0, task_rows = 0;
        auto load_rows = [&](uint32_t k) {  // the task at list position k: its activation rows, this wave's 256 columns of them, into registers
            const Info cur = info_at(k);
            task = cur.task;
            task_rows = cur.nrows;
            // every row's route first, then, side by side, the route's expert (checked against the task's) and the row of the
            // route's token: two round trips, not three
            uint32_t rid[MT], token[MT];
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const uint32_t r = i * 32 + n, rr = r < cur.nrows ? r : 0;
                rid[i] = cur.shared ? 0 : a.token_map[uint64_t(cur.expert) * a.tokens + cur.start + rr];
                token[i] = cur.shared ? cur.start + rr : rid[i] / a.selected;
                // A row past the task's end repeats its first row (and stores what it computes, the first row's h, to the first
                // row's slot), and a route outside the batch stands in for token 0 (the batch is refused). So every lane stores,
                // every wave issues the same number of stores per unit, and the waits below can count them.
                if (!cur.shared && rid[i] >= a.tokens * a.selected) { rid[i] = 0; token[i] = 0; if (cur.ok) bad |= TSP_ERRBIT_INDEX; }
                if (!cur.ok) token[i] = 0;
            }
            uint32_t owner[MT];
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                owner[i] = cur.shared ? cur.expert : a.ids[rid[i]];
                const _Float16* row = a.xh + uint64_t(token[i]) * (bpr * 256) + wave * 256 + khalf * 16;
#pragma unroll
                for (int t = 0; t < 16; ++t) A[i][t] = *reinterpret_cast<const f16x8*>(row + (t / 4) * 64 + ((t / 2) % 2) * 32 + (t % 2) * 8);
                sxA[i] = *reinterpret_cast<const f16x8*>(a.sx + (uint64_t(token[i]) * bpr + wave) * 16 + khalf * 8);
            }
#pragma unroll
            for (int i = 0; i < MT; ++i)
                if (owner[i] != cur.expert && cur.ok) bad |= TSP_ERRBIT_INDEX;  // a route that is not the expert's: the batch is refused
            // The rows are needed at once. Naming every fragment as an operand here makes the compiler wait for their loads now:
            // left to itself it waits at the fragments' first uses inside the tile loop, in every pass of the loop, with counts
            // that know nothing of the requests in flight and so drain them tile after tile.
#pragma unroll
            for (int i = 0; i < MT; ++i) {
#pragma unroll
                for (int t = 0; t < 16; ++t) asm volatile("" : "+v"(A[i][t]));
                asm volatile("" : "+v"(sxA[i]));
            }
        };

        // ---- one tile: unpack, multiply, add the eight waves' partial results up, and for an up tile apply SwiGLU and store
        float gate_sum[MT][2];
        auto tile = [&](uint32_t k, uint32_t unit, auto j_tag) {
            constexpr int J = decltype(j_tag)::value;
            // wait for the tile's five requests: younger than those are the five of the other stage and, for a gate tile, the
            // stores of the unit before (loads complete in order; a store that completes early only ends the wait sooner)
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kStages - 1) * kTileLoads + (J == 0 ? 2 * MT : 0)) : "memory");
            // With two row tiles everything a lane derives from its id is derived again per tile from this one register:
            // hoisted out of the loops these addresses would occupy a dozen registers next to the 128 of the activations.
            uint32_t lane_now = lane;
            if constexpr (MT == 2) asm volatile("" : "+v"(lane_now));
            const uint32_t n = lane_now % 32, khalf = lane_now / 32;
            const uint8_t* st = my_stage + stage;
            u32x4 raw[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) raw[p] = *reinterpret_cast<const u32x4*>(st + n * 128 + (((2 * p + khalf) ^ (n & 7)) * 16));
            const uint4 sm = *reinterpret_cast<const uint4*>(st + 4096 + n * 16);
            const uint32_t dm = *reinterpret_cast<const uint32_t*>(st + 4096 + 512 + n * 16 + (wave % 4) * 4);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            // the stage is free again: the tile two ahead goes there
            request_next();
            stage = stage + kStageBytes == kStages * kStageBytes ? 0 : stage + kStageBytes;
            float d = half_bits_to_float(dm & 0xffffu), dmin = half_bits_to_float(dm >> 16);
            asm volatile("" : "+v"(d), "+v"(dmin));  // as floats in registers: folded into the arithmetic as halves they make every multiply-add a mixed-precision one

            f32x16 blk[MT];
            auto steps = [&](auto p_tag) {
                constexpr int P = decltype(p_tag)::value;
                // the scales of sub-blocks 2P (low nibbles) and 2P + 1 (high nibbles, in place as 16 q: scale / 16) as one pair
                const Q4PairScale sc = q4_pair_scale<P>(sm.x, sm.y, q4s);
#pragma unroll
                for (int hi = 0; hi < 2; ++hi) {
                    f16x8 f[2];
                    frags_q4k_pair(raw[P], sc, hi, q4c, f);
#pragma unroll
                    for (int ff = 0; ff < 2; ++ff)
#pragma unroll
                        for (int i = 0; i < MT; ++i) {
                            if (P == 0 && hi == 0 && ff == 0) {
                                const f32x16 zero{};
                                blk[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[i][0], f[0], zero, 0, 0, 0);
                            } else {
                                blk[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[i][P * 4 + hi * 2 + ff], f[ff], blk[i], 0, 0, 0);
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
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                // partial = d * blk - dmin * sum_s Sx(hi + lo)[m, s] * mn[n, s]
                const f32x16 zero{};
                const f32x16 mblk = __builtin_amdgcn_mfma_f32_32x32x16_f16(sxA[i], mn, zero, 0, 0, 0);
                uint8_t* out = lds_raw + (phase & 1) * kPhaseBytes + wave * kPartialBytes + lane_now * 16;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    f32x4 v;
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaf(-dmin, mblk[4 * c + e], d * blk[i][4 * c + e]);
                    *reinterpret_cast<f32x4*>(out + c * 1024) = v;
                }
                lds_barrier();
                // thread tid adds up elements 2 tid, 2 tid + 1 of the eight partial tiles, in wave order
                const uint8_t* in = lds_raw + (phase & 1) * kPhaseBytes + (wave * kWave + lane_now) * 8;
                float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
                for (int w = 0; w < kWaves; ++w) {
                    const float2 p2 = *reinterpret_cast<const float2*>(in + w * kPartialBytes);
                    s0 += p2.x; s1 += p2.y;
                }
                ++phase;
                if constexpr (J == 0) {
                    gate_sum[i][0] = s0; gate_sum[i][1] = s1;
                } else {
                    // element 2 tid + e of the tile is accumulator 4 (wave / 2) + 2 (lane % 2) + e of fragment lane
                    // 32 (wave % 2) + lane / 2: task row 32 i + 4 wave + 2 (lane % 2) + e, hidden unit lane / 2 of the tile
                    const float up_sum[2] = {s0, s1};
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        const uint32_t r = i * 32 + 4 * wave + 2 * (lane_now % 2) + e;
                        const float g = gate_sum[i][e], u = up_sum[e];
                        const float h = (g * sigmoid_fast(g)) * u;
                        // h travels to the down GEMM as the half nearest to h * 2^-8. A gate or up sum that is not finite, or a
                        // product too large for a half, leaves an infinity or a NaN here, and only here is it looked for.
                        const _Float16 carried = _Float16(h * 0.00390625f);
                        const uint32_t bits = __builtin_bit_cast(uint16_t, carried), magnitude = bits & 0x7fffu;
                        biggest = biggest > magnitude ? biggest : magnitude;
                        // uniform base (the task's slots, the unit's columns) + 32-bit lane offset, spelled out: the compiler would
                        // form a 64-bit address per store
                        // a row past the task's end has multiplied the first row's activations: the same bits, stored to the first
                        // row's slot, so that the slots nobody reads cost no traffic (and every lane still stores)
                        const uint32_t at = ((r < task_rows ? r : 0) * a.hidden + lane_now / 2) * 2;
                        const _Float16* const base = a.hbuf + (uint64_t(task) * kTaskRows) * a.hidden + unit * 32;
                        asm volatile("global_store_short %0, %1, %2" ::"v"(at), "v"(bits), "s"(base) : "memory");
                    }
                }
            }
        };

        for (uint32_t k = k0; k <= k1; ++k) {
            load_rows(k);
            const uint32_t u1 = end_unit(k);
            for (uint32_t unit = first_unit(k); unit < u1; ++unit) {
                tile(k, unit, std::integral_constant<int, 0>{});
                tile(k, unit, std::integral_constant<int, 1>{});
            }
        }
        wait_all_loads();  // the last requests fetched tiles nobody reads: they must have landed before the stages are reused or given away
    };
    pass(std::integral_constant<int, 2>{});
    pass(std::integral_constant<int, 1>{});
    if (biggest >= 0x7c00u) bad |= TSP_ERRBIT_NONFINITE;
    publish_error(bad, a.error_word);
}

}  // namespace

namespace tsp {

bool resident_gate_up_takes(uint32_t channels, uint32_t hidden) { return channels == 2048 && hidden % 32 == 0 && hidden >= 32; }

int launch_resident_gate_up(const ResidentGateUpArgs& a, hipStream_t s) {
    static std::atomic<uint64_t> seen{0};
    static int cus[64];
    int device = 0;
    if (setup_pending(seen, &device)) {
        int n = 0;
        TSP_HIP(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device));
        cus[device] = n >= 8 ? n / 8 * 8 : 8;
        setup_done(seen, device);
    }
    TSP_LAUNCH("gemm_gate_up_swiglu", s, gate_up_resident_kernel<<<cus[device], kThreads, 0, s>>>(a));
    return launch_status("gate_up_resident");
}

}  // namespace tsp
