// Prefill dequant-GEMM on the matrix cores: out[m, n] = sum_k x[m, k] * dec(W[n, k]).
//
// K-quant weights factor as  w = d * (sc * q) - dmin * mn  (Q4_K) and  w = d * (sc * (q - 32))  (Q6_K)
// with a per-super-block f16 factor d (dmin) and small INTEGER products sc*q (< 2^10) resp. sc*(q-32)
// (< 2^12). The kernel feeds those integers, which are exact in f16, to v_mfma_f32_32x32x16_f16 against
// the activations (bf16 values carried as f16, exact), accumulates one super-block of 256 columns in a
// scratch accumulator, and applies d once per super-block on the f32 accumulators:
//
//     out += d[n, b] * sum_{k in b} x[m, k] * (sc*q)[n, k]   -   sum_s (dmin*mn)[n, b, s] * Sx[m, b, s]
//
// The second term (Q4_K minima) is one more MFMA per super-block against the per-sub-block activation
// sums Sx, carried as a hi+lo pair of f16. Nothing is rounded to f16 that is not an exact integer (Q6_K
// products above 2048 round to even, a 2^-12 relative step), so results track the f32-dequantised
// reference to f32-accumulation accuracy, and unpacking costs ~1.4 VALU operations per weight (mask,
// byte permute into 1024+q, one packed f16 fma) instead of ~3 for convert + f32 fma + f16 round.
//
// One workgroup = 4 waves = one task (<= 64 activation rows of one expert, or one 64-row slab of a dense
// matrix) x 256 weight rows. Each wave owns 64 weight rows (two 32-wide MFMA column tiles) and all 64
// activation rows (two row tiles).
//   * Quant bytes are loaded row-wise (one instruction = sixteen rows x 64 contiguous bytes), half a super-block ahead,
//     parked in wave-private swizzled LDS and read back in MFMA B-fragment order (lane = (row % 32, k-half)); every
//     weight is unpacked once per task.
//   * Activations are shared by the four waves: 64 rows x 128 bytes per K step go global -> LDS directly (no registers),
//     two and three steps ahead, into a ring of four slabs; one LDS-only barrier per K step.
//   * For gate/up the two column tiles of a wave are the gate rows and the up rows of the same 32 hidden
//     units, so SwiGLU is an element-wise epilogue on accumulator registers.
#include "dense_ksplit.hpp"
#include "dense_tall.hpp"
#include "down_resident.hpp"
#include "gate_up_resident.hpp"
#include "grouped_staged.hpp"
#include "grouping_device.hpp"
#include "planar_staged.hpp"
#include "mfma_quant.hpp"

#include <type_traits>

using namespace tsp;

namespace {

enum Epilogue : int { EPI_F32 = 0, EPI_BF16 = 1, EPI_SWIGLU = 2 };
enum Rows : int { ROWS_DENSE = 0, ROWS_GATHER_TOKENS = 1, ROWS_TASK_SLOTS = 2, ROWS_ROUTES = 3 };

constexpr int kTaskRows = 64;
constexpr int kRowTiles = kTaskRows / 32;

struct GemmArgs {
    const _Float16* a;        // activation rows, a_stride halfs apart
    uint64_t a_stride;
    const _Float16* sx;       // per row, per super-block: 8 sub-block sums (hi) + 8 residuals (lo); Q4_K only
    const uint8_t* w0;        // dense matrix / pair_lo / down experts
    const uint8_t* w1;        // pair_hi
    tsp_planar_spec spec;     // planar layouts (per expert)
    uint32_t experts;
    const uint32_t* tasks;    // grouped: [2 + 2*bound] with kTaskRows-row tiles
    const uint32_t* counts;
    const uint32_t* token_map;
    const uint32_t* ids;
    uint32_t tokens, selected;
    uint32_t m, n, k;         // dense rows; weight rows (or hidden units for SwiGLU); columns
    void* out;
    uint64_t out_stride;      // bytes
    float out_scale;
    uint32_t* error_word;
    uint64_t raw_expert_bytes;       // raw GGUF expert stacks: bytes between experts (0 for one dense matrix)
    uint32_t broadcast;              // ROWS_ROUTES: one input row per token instead of one per route
    uint32_t col_tiles, task_slots;  // logical grid: column tiles x tasks, launched as one linear grid
    // an always-on expert riding in the same launch: tasks whose expert id is `experts` take every token as their rows,
    // these weights (gate / up halves, or the down matrix) and, for the down product, these output rows
    const uint8_t* shared_w0;
    const uint8_t* shared_w1;
    void* shared_out;
    uint64_t shared_out_stride;
};

// ---------------------------------------------------------------- the kernel
template <int BKIND, int EPI, int ROWS>
__global__ __launch_bounds__(256, 2) void gemm_kernel(GemmArgs a) {  // two workgroups per CU: <= 256 registers per lane
    constexpr bool Q6 = BKIND == B_Q6K_PLANAR;
    constexpr int KSTEP = 64;
    // LDS, carved by hand so that two workgroups fit one CU's 160 KB:
    //   [ring of 4 activation slabs, 8 KB each][quant bytes, private to each wave, double buffered][Q4_K: activation sums x 2]
    // One slab = 64 rows x 128 bytes, written by direct global -> LDS loads: 16-byte chunk c of row r sits at position
    // r * 8 + (c ^ (r & 7)), so the loads fill LDS linearly by lane and the fragment reads spread over all banks.
    // Quant bytes, half a super-block at a time: Q4_K [wave][buffer][64 rows][4 chunks of 16 B], Q6_K the same for the low
    // nibbles plus [64 rows][2 chunks] of high bits; chunks are swizzled so that the row-wise stores and the column-wise
    // reads both spread over all banks.
    // The row tables live where no slab is yet (source rows, before the loop: the tail of slab 3) or any more (destination
    // rows, after the loop: the head of slab 0).
    constexpr int RING = 4, SLAB = kTaskRows * KSTEP * 2;
    constexpr int LDS_SX = 24;       // halfs per staged row of activation sums (16 used)
    constexpr int W_AT = RING * SLAB, W_BYTES = Q6 ? 4 * 2 * 64 * 96 : 4 * 2 * 64 * 64;
    constexpr int SX_AT = W_AT + W_BYTES, SX_BYTES = Q6 ? 0 : 2 * kTaskRows * LDS_SX * 2;
    __shared__ __attribute__((aligned(16))) uint8_t lds_raw[SX_AT + SX_BYTES];
    static_assert(sizeof(lds_raw) <= 80 * 1024, "two workgroups per CU");
    uint8_t* const lds_w = lds_raw + W_AT;
    _Float16* const lds_sx = reinterpret_cast<_Float16*>(lds_raw + SX_AT);  // [2][kTaskRows * LDS_SX]
    uint32_t* const row_src = reinterpret_cast<uint32_t*>(lds_raw + 3 * SLAB + SLAB - 512);
    uint32_t* const task_bad_at = row_src + kTaskRows;
    uint32_t* const row_dst = reinterpret_cast<uint32_t*>(lds_raw);
#define task_bad (*task_bad_at)

    const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const uint32_t col = lane % 32, khalf = lane / 32;
    // Logical (column tile, task) from the linear workgroup id. Workgroups go to the eight XCDs round-robin by id and
    // each XCD has its own L2, so ids are dealt out in runs: XCD x gets the x-th eighth of the live (task, tile) pairs in
    // order. All column tiles of a task, and the row slabs of one expert, then meet in one L2: the task's activation
    // rows and the expert's weight bytes are fetched from memory once and hit in L2 for the other workgroups.
    uint32_t live_tasks = a.task_slots;
    if constexpr (ROWS != ROWS_DENSE) {
        const uint32_t listed = a.tasks[0];
        live_tasks = listed < a.task_slots ? listed : a.task_slots;
        if (live_tasks == 0) live_tasks = 1;  // keeps workgroup (0, 0) alive to report a bad task list
    }
    const uint32_t live_groups = live_tasks * a.col_tiles, per_xcd = (live_groups + 7) / 8;
    const uint32_t logical = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (blockIdx.x / 8 >= per_xcd || logical >= live_groups) return;
    const uint32_t task = logical / a.col_tiles, bx = logical % a.col_tiles;

    // ---- task resolution
    uint32_t expert = 0, nrows = 0;
    bool shared = false;
    uint32_t my_dst = 0xffffffffu;  // output row of activation row `tid` (threads 0..63), parked in a register during the loop
    if (tid == 0) task_bad = 0;
    __syncthreads();
    if constexpr (ROWS == ROWS_DENSE) {
        const uint32_t row0 = task * kTaskRows;
        if (row0 >= a.m) return;
        nrows = a.m - row0 < kTaskRows ? a.m - row0 : kTaskRows;
        if (tid < kTaskRows) { row_src[tid] = row0 + (tid < nrows ? tid : 0); my_dst = row0 + tid; }
    } else {
        const uint32_t bound = a.tokens * a.selected / kTaskRows + a.experts + (a.shared_w0 ? (a.tokens + kTaskRows - 1) / kTaskRows : 0);
        const uint32_t live = a.tasks[0];
        if (live > bound || a.tasks[1] != a.tokens * a.selected) {
            if (tid == 0 && bx == 0 && task == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
            return;
        }
        if (task >= live) return;
        expert = a.tasks[2 + 2 * task];
        const uint32_t start = a.tasks[3 + 2 * task];
        shared = a.shared_w0 != nullptr && expert == a.experts;
        const uint32_t count = shared ? a.tokens : expert < a.experts ? a.counts[expert] : 0;
        if ((expert >= a.experts && !shared) || count > a.tokens || start >= count) {
            if (tid == 0 && bx == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
            return;
        }
        nrows = count - start < kTaskRows ? count - start : kTaskRows;
        if (tid < kTaskRows) {
            // rows past the task's end re-read its first row: their accumulators are never stored
            uint32_t rid;
            if (shared) {
                rid = (start + (tid < nrows ? tid : 0)) * a.selected;  // "route 0" of the token: row_src below divides it back
            } else {
                rid = a.token_map[uint64_t(expert) * a.tokens + start + (tid < nrows ? tid : 0)];
                if (rid >= a.tokens * a.selected || a.ids[rid] != expert) { rid = 0xffffffffu; task_bad = 1; }
            }
            // activation row: the route's token (gate/up, broadcast grouped GEMM), the route itself (grouped GEMM with one input
            // row per route) or the task's slot in the intermediate buffer (down); output row: task slot or route
            const uint32_t safe = rid == 0xffffffffu ? 0 : rid;
            row_src[tid] = ROWS == ROWS_GATHER_TOKENS ? safe / a.selected
                         : ROWS == ROWS_ROUTES       ? (a.broadcast ? safe / a.selected : safe)
                                                     : task * kTaskRows + (tid < nrows ? tid : 0);
            my_dst = ROWS == ROWS_GATHER_TOKENS ? task * kTaskRows + tid : shared ? rid / a.selected : rid;
        }
    }
    __syncthreads();
    if (task_bad && tid == 0 && bx == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
    const int mt_live = (nrows + 31) / 32;

    // ---- weight rows of this wave
    const uint8_t* wbase[2];
    uint64_t wrow[2];
    uint32_t out_col[2];
    bool col_live[2];
    if constexpr (EPI == EPI_SWIGLU) {
        const uint32_t unit = bx * 128 + wave * 32 + col;
        const uint32_t half_e = a.experts / 2;
        const uint8_t* pair = (expert < half_e ? a.w0 : a.w1) + uint64_t(expert < half_e ? expert : expert - half_e) * 2 * a.spec.planar_expert_bytes;
        wbase[0] = shared ? a.shared_w0 : pair;
        wbase[1] = shared ? a.shared_w1 : pair + a.spec.planar_expert_bytes;
        col_live[0] = col_live[1] = unit < a.n;
        wrow[0] = wrow[1] = col_live[0] ? unit : a.n - 1;
        out_col[0] = out_col[1] = unit;
    } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t n = bx * 256 + wave * 64 + j * 32 + col;
            col_live[j] = n < a.n;
            wrow[j] = col_live[j] ? n : a.n - 1;
            out_col[j] = n;
            wbase[j] = shared ? a.shared_w0 : a.w0 + uint64_t(expert) * (BKIND == B_Q4K_RAW ? a.raw_expert_bytes : a.spec.planar_expert_bytes);
        }
    }
    const uint32_t bpr = a.k / 256;
    const uint32_t ksteps = a.k / KSTEP;

    f32x16 acc[kRowTiles][2], blk[kRowTiles][2];
#pragma unroll
    for (int i = 0; i < kRowTiles; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // ---- activation staging, global -> LDS directly, two K steps ahead: per step 64 rows x 128 bytes; instruction i of
    // thread t fills LDS position t + 256 i (16-byte units) = slot t % 8 of row t / 8 + 32 i with chunk (t % 8) ^ (row % 8)
    // of that row, so eight neighbouring lanes still read one row's whole 128 bytes
    const uint32_t st_row = tid / 8, st_chunk = (tid % 8) ^ ((tid / 8) & 7);
    const _Float16* st_src0 = a.a + uint64_t(row_src[st_row]) * a.a_stride + st_chunk * 8;
    const _Float16* st_src1 = a.a + uint64_t(row_src[st_row + 32]) * a.a_stride + st_chunk * 8;
    // fragment reads: lane (col, khalf) takes chunk {2 khalf, 2 khalf + 1, 4 + 2 khalf, 5 + 2 khalf}[q] of row col (+ 32 i)
    uint32_t a_off[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) a_off[q] = col * 128 + (((q / 2) * 4 + 2 * khalf + (q % 2)) ^ (col & 7)) * 16;
    // LDS address of this wave's 1 KB share of slab 0, rows 0..31 (uniform over the wave)
    const uint32_t slab_lds = __builtin_amdgcn_readfirstlane(lds_address(lds_raw) + wave * 1024);
    // activation sums of one super-block: 64 rows x 32 bytes, threads 0..127 copy 16 bytes each
    const uint32_t sx_row = (tid / 2) % kTaskRows, sx_seg = tid % 2;
    const uint32_t sx_src = row_src[sx_row];  // read now: the table's LDS becomes a slab once the loop runs
    uint4 sx_stage{};
    auto fetch_sx = [&](uint32_t b) {
        if constexpr (!Q6) {
            // 64 rows x 32 bytes; threads 128..255 repeat the work of 0..127 so that no load sits under a branch
            sx_stage = *reinterpret_cast<const uint4*>(a.sx + (uint64_t(sx_src) * bpr + b) * 16 + sx_seg * 8);
        }
    };
    auto store_sx = [&](int buf) {
        if constexpr (!Q6) {
            *reinterpret_cast<uint4*>(&lds_sx[buf * kTaskRows * LDS_SX + sx_row * LDS_SX + sx_seg * 8]) = sx_stage;
        }
    };
    // The whole K loop is instantiated once per number of live 32-row tiles, so that its body is straight-line code:
    // a branch per tile would cut every step into a dozen basic blocks, each waiting for its own LDS read before its
    // two MFMAs, and nothing could be scheduled across them.
    auto run = [&](auto mt_tag) {
        constexpr int MT = decltype(mt_tag)::value;
        auto dma_a = [&](uint32_t step, int ring) {  // rows 32..63 only when the task has them; steps past the end re-read the last
            step = step < ksteps ? step : ksteps - 1;
            const uint32_t dst = slab_lds + ring * SLAB;
            load_to_lds_16(st_src0 + uint64_t(step) * KSTEP, dst);
            if constexpr (MT == 2) load_to_lds_16(st_src1 + uint64_t(step) * KSTEP, dst + 4096);
        };
        // one k16 MFMA per (row tile, column tile); `first` starts the super-block accumulator from zero
        auto mfma = [&](int ring, int q, const f16x8& b0, const f16x8& b1, bool first) {
    #pragma unroll
            for (int i = 0; i < MT; ++i) {
                const f16x8 af = *reinterpret_cast<const f16x8*>(lds_raw + ring * SLAB + i * 4096 + a_off[q]);
                if (first) {
                    const f32x16 zero{};
                    blk[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, b0, zero, 0, 0, 0);
                    blk[i][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, b1, zero, 0, 0, 0);
                } else {
                    blk[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, b0, blk[i][0], 0, 0, 0);
                    blk[i][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, b1, blk[i][1], 0, 0, 0);
                }
            }
        };
        auto fold = [&](float d0, float d1) {  // acc += d * blk at the end of a super-block
    #pragma unroll
            for (int i = 0; i < MT; ++i) {
    #pragma unroll
                for (int v = 0; v < 16; ++v) {
                    acc[i][0][v] = __builtin_fmaf(d0, blk[i][0][v], acc[i][0][v]);
                    acc[i][1][v] = __builtin_fmaf(d1, blk[i][1][v], acc[i][1][v]);
                }
            }
        };

        dma_a(0, 0);
        dma_a(1, 1);
        if constexpr (Q6) {
            // Q6_K planes. Low nibbles (64 B) and high bit pairs (32 B) of one 128-column section per row travel
            // global -> registers -> LDS -> fragment registers one section (two K steps) ahead, loaded row-wise like
            // the Q4_K bytes below; sub-scales (16 B) and d (2 B) per super-block go straight to registers. All loads
            // are unconditional (clamped past the end) so that outstanding loads are counted exactly.
            uint8_t* const my_w = lds_w + wave * (2 * 64 * 96);  // [2 buffers]{[64 rows][4 chunks] low nibbles, [64 rows][2 chunks] high bits}
            const uint32_t row_ql = bpr * 128, row_qh = bpr * 64;
            const uint32_t sections = 2 * bpr;
            const uint32_t wave_row0 = bx * 256 + wave * 64;
            const uint32_t ql_row = lane / 4, ql_chunk = (lane % 4) ^ ((lane / 8) & 3);  // chunk c of row r sits at position c ^ ((r >> 1) & 3)
            const uint32_t qh_row = lane / 2, qh_chunk = lane % 2;
            u32x4 wstage[6];
            auto clamp_row = [&](uint32_t r) { return r < a.n ? r : a.n - 1; };
            auto fetch_w = [&](uint32_t section) {
                section = section < sections ? section : sections - 1;
                const uint8_t* ql = wbase[0] + a.spec.qs_offset + uint64_t(section / 2) * 128 + (section % 2) * 64;
                const uint8_t* qh = wbase[0] + a.spec.qh_offset + uint64_t(section / 2) * 64 + (section % 2) * 32;
    #pragma unroll
                for (int q = 0; q < 4; ++q) wstage[q] = *reinterpret_cast<const u32x4*>(ql + (clamp_row(wave_row0 + q * 16 + ql_row) * row_ql + ql_chunk * 16));
    #pragma unroll
                for (int q = 0; q < 2; ++q) wstage[4 + q] = *reinterpret_cast<const u32x4*>(qh + (clamp_row(wave_row0 + q * 32 + qh_row) * row_qh + qh_chunk * 16));
            };
            auto store_w = [&](int wbuf) {
    #pragma unroll
                for (int q = 0; q < 6; ++q) *reinterpret_cast<u32x4*>(my_w + wbuf * 6144 + (q * 64 + lane) * 16) = wstage[q];
            };
            struct Scales { uint32_t sc[4]; float d; };
            auto load_scales = [&](uint32_t b, int j) {
                b = b < bpr ? b : bpr - 1;
                const uint64_t blk_at = wrow[j] * bpr + b;
                const uint4 sc16 = *reinterpret_cast<const uint4*>(wbase[j] + a.spec.sm_offset + blk_at * 16);
                Scales r;
                r.sc[0] = sc16.x; r.sc[1] = sc16.y; r.sc[2] = sc16.z; r.sc[3] = sc16.w;
                r.d = half_bits_to_float(*reinterpret_cast<const uint16_t*>(wbase[j] + a.spec.dm_offset + blk_at * 2));
                return r;
            };
            Scales scl[2] = {load_scales(0, 0), load_scales(0, 1)}, scl_next[2] = {scl[0], scl[1]};
            fetch_w(0);
            store_w(0);
            RawQ6 raw[2];
            // K step H of a super-block: section H/2 (128 columns), quarters 2*(H%2) and 2*(H%2)+1 of that section
            auto half_step = [&](uint32_t step, auto h_tag) {
                constexpr int H = decltype(h_tag)::value;
                constexpr int wbuf = H / 2, ring = H;  // step % RING
                const uint32_t b = step / 4;
                // Even steps request the slabs of the steps two and three ahead, as the first loads after their barrier; the
                // only loads younger than those are the section (6) and, at H == 2, scale (4) loads of the same step, and
                // for an odd step the two slabs and the loads of the even step before it. Loads complete in order.
                constexpr int W[4] = {6, 0, 10, 0};
                lds_barrier_after_loads<H % 2 == 0 ? W[(H + 2) % 4] : W[(H + 1) % 4] + 2 * MT + W[(H + 3) % 4]>();  // slab and this wave's section bytes are complete; every wave has left the other buffers
                if (H % 2 == 0) { dma_a(step + 2, (ring + 2) % RING); dma_a(step + 3, (ring + 3) % RING); }
                if (H % 2 == 0) fetch_w(step / 2 + 1);
                if (H == 2) { scl_next[0] = load_scales(b + 1, 0); scl_next[1] = load_scales(b + 1, 1); }
                if (H % 2 == 0) {
    #pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const uint8_t* lo = my_w + wbuf * 6144 + (j * 32 + col) * 64;
                        const uint32_t swz = (col >> 1) & 3;
                        raw[j].la = *reinterpret_cast<const u32x4*>(lo + ((khalf ^ swz) * 16));
                        raw[j].lb = *reinterpret_cast<const u32x4*>(lo + (((2 + khalf) ^ swz) * 16));
                        raw[j].qh = *reinterpret_cast<const u32x4*>(my_w + wbuf * 6144 + 4096 + ((j * 32 + col) * 2 + khalf) * 16);
                        raw[j].sc[0] = scl[j].sc[(H / 2) * 2]; raw[j].sc[1] = scl[j].sc[(H / 2) * 2 + 1];
                    }
                }
                auto quarter = [&](auto q_tag) {
                    constexpr int Q = decltype(q_tag)::value;
                    f16x8 f0[2], f1[2];
                    frags_q6k<Q>(raw[0], khalf, f0);
                    frags_q6k<Q>(raw[1], khalf, f1);
                    mfma(ring, (Q % 2) * 2, f0[0], f1[0], H == 0 && Q == 0);
                    mfma(ring, (Q % 2) * 2 + 1, f0[1], f1[1], false);
                };
                quarter(std::integral_constant<int, 2 * (H % 2)>{});
                quarter(std::integral_constant<int, 2 * (H % 2) + 1>{});
                if (H == 3) fold(scl[0].d, scl[1].d);
                if (H % 2 == 1) store_w(wbuf ^ 1);
                if (H == 3) { scl[0] = scl_next[0]; scl[1] = scl_next[1]; }
            };
            wait_all_loads();  // slabs 0 and 1 (the stores above already waited for younger loads)
            for (uint32_t b = 0; b < bpr; ++b) {
                half_step(b * 4 + 0, std::integral_constant<int, 0>{});
                half_step(b * 4 + 1, std::integral_constant<int, 1>{});
                half_step(b * 4 + 2, std::integral_constant<int, 2>{});
                half_step(b * 4 + 3, std::integral_constant<int, 3>{});
            }
        } else {
            // Q4_K. Quant bytes travel global -> registers -> LDS -> fragment registers, half a super-block (two K steps)
            // ahead. The global loads are issued row-wise (one instruction = sixteen rows x 64 contiguous bytes, lane = 16-byte
            // chunk), so cache lines are requested in whole halves by neighbouring lanes. In LDS lane (row, k-half) then picks
            // its 16 bytes of the step. Headers (scales, minima, d, dmin: 16 + 4 bytes per lane) go straight to registers.
            //
            // Every load in the loop is unconditional (indices past the end are clamped, the data unused): with no branch
            // around a load the compiler can count outstanding loads exactly and waits only for the oldest ones; a
            // conditional load anywhere makes it drain all of them (s_waitcnt vmcnt(0)) at every step, which exposes a full
            // memory round trip per step. Loads return in issue order, so each step requests its activation slab (awaited
            // at the end of the same step) BEFORE the weight bytes (awaited a step later).
            constexpr uint32_t BLK = BKIND == B_Q4K_PLANAR ? 128 : 144, QS_AT = BKIND == B_Q4K_PLANAR ? 0 : 16;
            uint8_t* const my_w = lds_w + wave * (2 * 64 * 64);  // [2 buffers][64 rows][4 chunks of 16 B]
            const uint32_t ld_row = lane / 4, ld_chunk = (lane % 4) ^ ((lane / 8) & 3);  // chunk c of row r sits at position c ^ ((r >> 1) & 3)
            const uint32_t wave_row0 = EPI == EPI_SWIGLU ? bx * 128 + wave * 32 : bx * 256 + wave * 64;
            const uint32_t row_bytes = bpr * BLK;
            const uint32_t halves = 2 * bpr;
            u32x4 wstage[4];
            // instruction Q of a half-block: rows 16Q .. 16Q+15 of the wave's 64 (tile Q / 2)
            auto fetch_w = [&](uint32_t half, auto q_tag) {
                constexpr int Q = decltype(q_tag)::value, J = Q / 2;
                uint32_t row = wave_row0 + (EPI == EPI_SWIGLU ? (Q % 2) * 16 : Q * 16) + ld_row;
                row = row < a.n ? row : a.n - 1;
                // uniform base + 32-bit lane offset (the host refuses matrices whose rows span 4 GiB or more)
                const uint8_t* base = wbase[J] + (BKIND == B_Q4K_PLANAR ? a.spec.qs_offset : 0) + uint64_t(half / 2) * BLK + QS_AT + (half % 2) * 64;
                wstage[Q] = *reinterpret_cast<const u32x4*>(base + (row * row_bytes + ld_chunk * 16));
            };
            auto fetch_w_all = [&](uint32_t half) {
                half = half < halves ? half : halves - 1;
                fetch_w(half, std::integral_constant<int, 0>{});
                fetch_w(half, std::integral_constant<int, 1>{});
                fetch_w(half, std::integral_constant<int, 2>{});
                fetch_w(half, std::integral_constant<int, 3>{});
            };
            auto store_w = [&](int wbuf) {
    #pragma unroll
                for (int q = 0; q < 4; ++q) *reinterpret_cast<u32x4*>(my_w + wbuf * 4096 + (q * 64 + lane) * 16) = wstage[q];
            };
            auto read_w = [&](int wbuf, int j, int p2) {  // row j*32 + col, chunk 2*p2 + khalf
                return *reinterpret_cast<const u32x4*>(my_w + wbuf * 4096 + ((j * 32 + col) * 4 + ((2 * p2 + khalf) ^ ((col >> 1) & 3))) * 16);
            };
            const Q4Consts q4c = q4_consts();
            HdrQ4 hdr[2];
            RawHdrQ4 hdr_next[2];  // requested at P == 2, decoded at the end of P == 3: nothing touches the bytes while they travel
    #pragma unroll
            for (int j = 0; j < 2; ++j) {
                hdr_next[j] = fetch_hdr_q4k<BKIND>(wbase[j], a.spec, wrow[j], bpr, 0);
                hdr[j] = decode_hdr_q4k<BKIND>(hdr_next[j]);
            }
            fetch_w_all(0);
            store_w(0);
            fetch_sx(0);
            store_sx(0);
            auto pair_step = [&](uint32_t step, auto p_tag) {
                constexpr int P = decltype(p_tag)::value;
                constexpr int wbuf = P / 2, ring = P;  // step % RING
                const uint32_t b = step / 4;
                // Even steps request the slabs of the steps two and three ahead, as the first loads after their barrier; the
                // only loads younger than those are the other loads of the same step (W), and for an odd step the two slabs
                // and the loads of the even step before it. Loads complete in order.
                // sums + half-block, -, half-block + headers (planes: scales and d/dmin apart, two loads per tile; GGUF rows: one), -
                constexpr int W[4] = {5, 0, BKIND == B_Q4K_PLANAR ? 8 : 6, 0};
                lds_barrier_after_loads<P % 2 == 0 ? W[(P + 2) % 4] : W[(P + 1) % 4] + 2 * MT + W[(P + 3) % 4]>();  // slab, this wave's weight bytes (and at P == 3 lds_sx[b & 1]) are complete; every wave has left the other buffers
                if (P % 2 == 0) { dma_a(step + 2, (ring + 2) % RING); dma_a(step + 3, (ring + 3) % RING); }
                if (P == 0) fetch_sx(b + 1 < bpr ? b + 1 : b);
                if (P == 0 || P == 2) fetch_w_all(step / 2 + 1);
                if (P == 2) {
    #pragma unroll
                    for (int j = 0; j < 2; ++j) hdr_next[j] = fetch_hdr_q4k<BKIND>(wbase[j], a.spec, wrow[j], bpr, b + 1 < bpr ? b + 1 : b);
                }
                const u32x4 raw0 = read_w(wbuf, 0, P & 1), raw1 = read_w(wbuf, 1, P & 1);
                f16x8 f0[2], f1[2];
                frags_q4k_swapped<P, 0>(raw0, hdr[0], q4c, f0);
                frags_q4k_swapped<P, 0>(raw1, hdr[1], q4c, f1);
                mfma(ring, 0, f0[0], f1[0], P == 0);
                mfma(ring, 1, f0[1], f1[1], false);
                frags_q4k_swapped<P, 1>(raw0, hdr[0], q4c, f0);
                frags_q4k_swapped<P, 1>(raw1, hdr[1], q4c, f1);
                mfma(ring, 2, f0[0], f1[0], false);
                mfma(ring, 3, f0[1], f1[1], false);
                if (P == 3) {
                    fold(hdr[0].d, hdr[1].d);
                    // minima: acc -= dmin * sum_s Sx(hi + lo)[m, s] * mn[n, s]
                    const f16x8 m0 = minima_frag(hdr[0]), m1 = minima_frag(hdr[1]);
    #pragma unroll
                    for (int i = 0; i < MT; ++i) {
                        const f16x8 sf = *reinterpret_cast<const f16x8*>(&lds_sx[(b & 1) * kTaskRows * LDS_SX + (i * 32 + col) * LDS_SX + khalf * 8]);
                        const f32x16 zero{};
                        blk[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sf, m0, zero, 0, 0, 0);
                        blk[i][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sf, m1, zero, 0, 0, 0);
                    }
                    fold(-hdr[0].dmin, -hdr[1].dmin);
                }
                if (P == 1) store_sx((b + 1) & 1);  // read at P == 3 of the next super-block; the buffer was last read at P == 3 of the one before
                if (P == 1 || P == 3) store_w(wbuf ^ 1);  // read again two barriers from now; this buffer was last read a step ago
                if (P == 3) { hdr[0] = decode_hdr_q4k<BKIND>(hdr_next[0]); hdr[1] = decode_hdr_q4k<BKIND>(hdr_next[1]); }
            };
            wait_all_loads();  // slabs 0 and 1 (the stores above already waited for younger loads)
            for (uint32_t b = 0; b < bpr; ++b) {
                pair_step(b * 4 + 0, std::integral_constant<int, 0>{});
                pair_step(b * 4 + 1, std::integral_constant<int, 1>{});
                pair_step(b * 4 + 2, std::integral_constant<int, 2>{});
                pair_step(b * 4 + 3, std::integral_constant<int, 3>{});
            }
        }
    };
    if (mt_live == 1) run(std::integral_constant<int, 1>{});
    else run(std::integral_constant<int, 2>{});
    wait_all_loads();  // the last steps requested slabs that nobody reads: they must have landed before this LDS is reused or given away
    __syncthreads();
    if (tid < kTaskRows) row_dst[tid] = my_dst;
    __syncthreads();

    // ---- epilogue. Accumulator v of tile (i, j): row = i*32 + 8*(v/4) + 4*khalf + v%4, column = col.
    uint32_t bad = 0;
#pragma unroll
    for (int i = 0; i < kRowTiles; ++i) {
        if (i >= mt_live) continue;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t r = i * 32 + 8 * (v / 4) + 4 * khalf + (v % 4);
            if (r >= nrows) continue;
            const uint32_t dst = row_dst[r];
            if (dst == 0xffffffffu) continue;
            if constexpr (EPI == EPI_SWIGLU) {
                if (!col_live[0]) continue;
                const float g = acc[i][0][v], u = acc[i][1][v];
                const float sg = sigmoid_stable(g);
                const float h = (g * sg) * u;
                // h is carried between the two GEMMs as the half nearest to h * 2^-8: 11 significant bits for
                // 0.016 <= |h| < 1.6e7, an absolute step of 2^-16 below that
                const _Float16 carried = _Float16(h * 0.00390625f);
                if (nonfinite(g) || nonfinite(u) || nonfinite(h) || (__builtin_bit_cast(uint16_t, carried) & 0x7c00u) == 0x7c00u) bad = TSP_ERRBIT_NONFINITE;
                reinterpret_cast<_Float16*>(a.out)[uint64_t(dst) * a.n + out_col[0]] = carried;
            } else {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    if (!col_live[j]) continue;
                    const float val = acc[i][j][v] * a.out_scale;
                    if (nonfinite(val)) bad = TSP_ERRBIT_NONFINITE;
                    uint8_t* orow = shared && ROWS == ROWS_TASK_SLOTS ? static_cast<uint8_t*>(a.shared_out) + uint64_t(dst) * a.shared_out_stride
                                                                      : static_cast<uint8_t*>(a.out) + uint64_t(dst) * a.out_stride;
                    if constexpr (EPI == EPI_F32) {
                        reinterpret_cast<float*>(orow)[out_col[j]] = val;
                    } else {
                        const uint32_t vb = __float_as_uint(val);
                        reinterpret_cast<uint16_t*>(orow)[out_col[j]] = uint16_t((vb + 0x7fffu + ((vb >> 16) & 1u)) >> 16);
                    }
                }
            }
        }
    }
    publish_error(bad, a.error_word);
}

// f32 rows -> bf16 (RNE) -> f16, or bf16 rows -> f16, plus the per-sub-block (32 column) sums of the converted
// values as hi + lo f16 pairs: sx[row][block][0..7] = hi, [8..15] = lo. A thread converts 8 columns; four
// neighbouring lanes share one sub-block. Values outside the f16 range are flagged.
// `block` of `blocks` workgroups share the rows (any workgroup size that is a multiple of the wave).
template <bool FROM_BF16>
__device__ __forceinline__ void to_f16_rows_block(const void* __restrict__ src, uint64_t src_stride_bytes, _Float16* __restrict__ dst,
                                                  _Float16* __restrict__ sx, uint32_t rows, uint32_t columns, uint32_t* error_word,
                                                  uint32_t block, uint32_t blocks) {
    uint32_t bad = 0;
    const uint64_t chunks = uint64_t(rows) * (columns / 8);
    const uint64_t span = (chunks + 3) / 4 * 4;  // whole groups of four lanes stay in the loop together
    for (uint64_t i = block * uint64_t(blockDim.x) + threadIdx.x; i < span; i += uint64_t(blocks) * blockDim.x) {
        const bool live = i < chunks;
        const uint64_t r = live ? i / (columns / 8) : 0, c8 = live ? i % (columns / 8) : 0;
        const uint8_t* row = static_cast<const uint8_t*>(src) + r * src_stride_bytes;
        float sum = 0;
        f16x8 out;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            uint32_t bits;
            if constexpr (FROM_BF16) {
                bits = uint32_t(reinterpret_cast<const uint16_t*>(row)[c8 * 8 + e]) << 16;
            } else {
                const uint32_t fb = __float_as_uint(reinterpret_cast<const float*>(row)[c8 * 8 + e]);
                bits = (fb + 0x7fffu + ((fb >> 16) & 1u)) & 0xffff0000u;
                if ((fb & 0x7f800000u) == 0x7f800000u) bits = fb;
            }
            const _Float16 h = _Float16(__uint_as_float(bits));
            if ((bits & 0x7f800000u) == 0x7f800000u || (__builtin_bit_cast(uint16_t, h) & 0x7c00u) == 0x7c00u) bad = TSP_ERRBIT_NONFINITE;
            out[e] = h;
            sum += float(h);
        }
        sum += __shfl_xor(sum, 1, kWave);
        sum += __shfl_xor(sum, 2, kWave);
        if (live) {
            // Q4_K consumers (the ones that ask for sums) unpack a dword of nibbles into the column pairs (0, 2), (1, 3):
            // their activations are stored in that order, columns 1 <-> 2 and 5 <-> 6 of every eight swapped
            if (sx) out = f16x8{out[0], out[2], out[1], out[3], out[4], out[6], out[5], out[7]};
            *reinterpret_cast<f16x8*>(dst + r * columns + c8 * 8) = out;
            if (sx && (c8 & 3) == 0) {
                const uint32_t sub = uint32_t(c8 / 4), b = sub / 8, s = sub % 8;
                const _Float16 hi = _Float16(sum), lo = _Float16(sum - float(hi));
                if ((__builtin_bit_cast(uint16_t, hi) & 0x7c00u) == 0x7c00u) bad = TSP_ERRBIT_NONFINITE;
                _Float16* o = sx + (r * (columns / 256) + b) * 16;
                o[s] = hi;
                o[8 + s] = lo;
            }
        }
    }
    publish_error(bad, error_word);
}

template <bool FROM_BF16>
__global__ __launch_bounds__(256) void to_f16_rows(const void* __restrict__ src, uint64_t src_stride_bytes, _Float16* __restrict__ dst,
                                                   _Float16* __restrict__ sx, uint32_t rows, uint32_t columns, uint32_t* error_word) {
    to_f16_rows_block<FROM_BF16>(src, src_stride_bytes, dst, sx, rows, columns, error_word, blockIdx.x, gridDim.x);
}

// The two task lists of a grouped product (workgroups 0 and 1) and the row conversion (all other workgroups) in one launch:
// neither needs the other, both need only what the route permutation before them wrote or nothing at all, and a launch of
// its own costs each of these small kernels more than its work.
struct TaskLists {
    const uint32_t* counts; uint32_t* tasks0; uint32_t tile0; uint32_t* tasks1; uint32_t tile1; uint32_t experts, selected, tokens;
    bool every_token1;  // list 1 also holds the always-on expert's tasks
    uint32_t* classes1;  // list 1 is a 64-row list: its tasks by number of rows (task_class_lists_block), or null
};
__global__ __launch_bounds__(512) void tasks_and_rows(TaskLists t, const void* __restrict__ src, uint64_t src_stride_bytes, _Float16* __restrict__ dst,
                                                      _Float16* __restrict__ sx, uint32_t rows, uint32_t columns, uint32_t* error_word) {
    __shared__ uint32_t tiles_scan[512];
    __shared__ uint32_t routes_scan[512];
    __shared__ uint32_t third_scan[512];
    if (blockIdx.x < 2) {
        grouped_tasks_block(t.counts, blockIdx.x == 0 ? t.tasks0 : t.tasks1, blockIdx.x == 0 ? t.tile0 : t.tile1, t.experts, t.selected, t.tokens,
                            error_word, tiles_scan, routes_scan, blockIdx.x == 1 && t.every_token1);
        if (blockIdx.x == 1 && t.classes1) task_class_lists_block(t.counts, t.classes1, t.experts, t.selected, t.tokens, t.every_token1, tiles_scan, routes_scan, third_scan);
    } else {
        to_f16_rows_block<false>(src, src_stride_bytes, dst, sx, rows, columns, error_word, blockIdx.x - 2, gridDim.x - 2);
    }
}

template <int BKIND, int EPI, int ROWS>
int launch(const GemmArgs& a, uint32_t col_tiles, uint32_t tasks, hipStream_t s) {
    constexpr const char* name = EPI == EPI_SWIGLU ? "gemm_gate_up_swiglu" : ROWS == ROWS_TASK_SLOTS ? "gemm_down" : ROWS == ROWS_ROUTES ? "gemm_grouped" : "gemm_dense";
    GemmArgs g = a;
    g.col_tiles = col_tiles;
    g.task_slots = tasks;
    const uint32_t groups = (col_tiles * tasks + 7) / 8 * 8;
    TSP_LAUNCH(name, s, gemm_kernel<BKIND, EPI, ROWS><<<groups, 256, 0, s>>>(g));
    return launch_status("dequant_gemm");
}

int convert_rows(const void* src, uint64_t stride, int from_bf16, _Float16* dst, _Float16* sx, uint32_t rows, uint32_t columns,
                 uint32_t* err, hipStream_t s) {
    const uint64_t chunks = uint64_t(rows) * (columns / 8);
    const uint32_t grid = uint32_t((chunks + 255) / 256 > 8192 ? 8192 : (chunks + 255) / 256);
    if (from_bf16) TSP_LAUNCH("to_f16_rows", s, to_f16_rows<true><<<grid, 256, 0, s>>>(src, stride, dst, sx, rows, columns, err));
    else TSP_LAUNCH("to_f16_rows", s, to_f16_rows<false><<<grid, 256, 0, s>>>(src, stride, dst, sx, rows, columns, err));
    return launch_status("to_f16_rows");
}

// f32 rows only; the caller has checked the task geometry (experts <= 512, tiles <= 256)
int lists_and_rows(const TaskLists& t, const void* src, uint64_t stride, _Float16* dst, _Float16* sx, uint32_t rows, uint32_t columns,
                   uint32_t* err, hipStream_t s) {
    const uint64_t chunks = uint64_t(rows) * (columns / 8);
    const uint32_t grid = 2 + uint32_t((chunks + 511) / 512 > 8192 ? 8192 : (chunks + 511) / 512);
    TSP_LAUNCH("tasks_and_rows", s, tasks_and_rows<<<grid, 512, 0, s>>>(t, src, stride, dst, sx, rows, columns, err));
    return launch_status("tasks_and_rows");
}

uint64_t align256(uint64_t v) { return (v + 255) / 256 * 256; }

}  // namespace

// workspace: [f16 rows][activation sums]
extern "C" uint64_t tsp_dense_mm_workspace_bytes(uint32_t tokens, uint32_t columns) {
    return align256(uint64_t(tokens) * columns * 2) + align256(uint64_t(tokens) * (columns / 256) * 32);
}

extern "C" int tsp_dense_mm(uint32_t encoding, uint32_t layout, const void* matrix, uint64_t matrix_bytes, const void* input,
                            uint64_t input_stride_bytes, int input_is_bf16, void* output, uint64_t output_stride_bytes,
                            int output_is_bf16, uint32_t tokens, uint32_t columns, uint32_t rows, void* workspace,
                            uint64_t workspace_bytes, uint32_t* error_word, void* stream) {
    TSP_REQUIRE((encoding == 12 && (layout == TSP_LAYOUT_GGUF || layout == TSP_LAYOUT_PLANAR_V3)) ||
                    (encoding == 14 && layout == TSP_LAYOUT_PLANAR_V3),
                "dense dequant-GEMM supports Q4_K rows/planes and Q6_K planes");
    TSP_REQUIRE(columns && columns <= 65536 && columns % 256 == 0 && rows && rows <= 1000000 && tokens && tokens <= 65536,
                "dense dequant-GEMM geometry");
    GemmArgs a{};
    if (layout == TSP_LAYOUT_PLANAR_V3) {
        const int rc = tsp_make_expert_spec(encoding, columns, rows, &a.spec);
        if (rc != TSP_OK) return rc;
        TSP_REQUIRE(matrix_bytes == a.spec.planar_expert_bytes, "dense dequant-GEMM matrix byte span mismatch");
    } else {
        TSP_REQUIRE(matrix_bytes == uint64_t(columns / 256) * 144 * rows, "dense dequant-GEMM matrix byte span mismatch");
    }
    const uint32_t in_elem = input_is_bf16 ? 2 : 4, out_elem = output_is_bf16 ? 2 : 4;
    TSP_REQUIRE(input_stride_bytes >= uint64_t(columns) * in_elem && input_stride_bytes % in_elem == 0 &&
                    output_stride_bytes >= uint64_t(rows) * out_elem && output_stride_bytes % out_elem == 0,
                "dense dequant-GEMM row stride");
    TSP_REQUIRE(matrix && input && output && workspace && error_word, "null device pointer");
    TSP_REQUIRE(reinterpret_cast<uintptr_t>(matrix) % 16 == 0 && reinterpret_cast<uintptr_t>(workspace) % 16 == 0,
                "dense dequant-GEMM needs 16-byte aligned weights and workspace");
    TSP_REQUIRE(workspace_bytes >= tsp_dense_mm_workspace_bytes(tokens, columns), "dense dequant-GEMM workspace too small");
    TSP_REQUIRE(matrix_bytes < (1ull << 32), "dense dequant-GEMM addresses weight rows with 32-bit offsets: matrix must be under 4 GiB");
    const uint64_t in_span = uint64_t(tokens - 1) * input_stride_bytes + uint64_t(columns) * in_elem;
    const uint64_t out_span = uint64_t(tokens - 1) * output_stride_bytes + uint64_t(rows) * out_elem;
    TSP_REQUIRE(!ranges_overlap(output, out_span, matrix, matrix_bytes) && !ranges_overlap(output, out_span, input, in_span) &&
                    !ranges_overlap(output, out_span, workspace, workspace_bytes) &&
                    !ranges_overlap(workspace, workspace_bytes, matrix, matrix_bytes) && !ranges_overlap(workspace, workspace_bytes, input, in_span),
                "dense dequant-GEMM buffers overlap");
    const auto s = static_cast<hipStream_t>(stream);
    auto* xh = static_cast<_Float16*>(workspace);
    auto* sx = reinterpret_cast<_Float16*>(static_cast<uint8_t*>(workspace) + align256(uint64_t(tokens) * columns * 2));
    if (encoding == 12 && layout == TSP_LAYOUT_GGUF && dense_tall_takes(tokens, rows, columns, matrix_bytes)) {
        // a thousand rows and more: tiles 128 or 256 rows high, weights rounded once to half (the engine's arithmetic for this product)
        int rc = convert_rows(input, input_stride_bytes, input_is_bf16, xh, sx, tokens, columns, error_word, s);  // with the sums come the swapped columns
        if (rc != TSP_OK) return rc;
        DenseTallArgs t{};
        t.a = xh; t.a_stride = columns; t.w = static_cast<const uint8_t*>(matrix); t.m = tokens; t.n = rows; t.k = columns;
        t.out = output; t.out_stride = output_stride_bytes; t.out_bf16 = output_is_bf16; t.error_word = error_word;
        return launch_dense_tall(t, s);
    }
    int rc = convert_rows(input, input_stride_bytes, input_is_bf16, xh, encoding == 12 ? sx : nullptr, tokens, columns, error_word, s);
    if (rc != TSP_OK) return rc;
    if (encoding == 12 && layout == TSP_LAYOUT_GGUF && dense_ksplit_takes(tokens, rows, columns)) {
        // few rows: 64 x 64 tiles with the columns split over a workgroup's waves, so that the chip has tiles enough
        DenseKsplitArgs t{};
        t.a = xh; t.sx = sx; t.w = static_cast<const uint8_t*>(matrix); t.m = tokens; t.n = rows; t.k = columns;
        t.out = output; t.out_stride = output_stride_bytes; t.out_bf16 = output_is_bf16; t.error_word = error_word;
        return launch_dense_ksplit(t, s);
    }
    a.a = xh; a.a_stride = columns; a.sx = sx; a.w0 = static_cast<const uint8_t*>(matrix); a.experts = 1;
    a.m = tokens; a.n = rows; a.k = columns; a.out = output; a.out_stride = output_stride_bytes; a.out_scale = 1.0f;
    a.error_word = error_word;
    const uint32_t col_tiles = (rows + 255) / 256, tasks = (tokens + kTaskRows - 1) / kTaskRows;
    if (encoding == 14) return output_is_bf16 ? launch<B_Q6K_PLANAR, EPI_BF16, ROWS_DENSE>(a, col_tiles, tasks, s)
                                               : launch<B_Q6K_PLANAR, EPI_F32, ROWS_DENSE>(a, col_tiles, tasks, s);
    if (layout == TSP_LAYOUT_PLANAR_V3) return output_is_bf16 ? launch<B_Q4K_PLANAR, EPI_BF16, ROWS_DENSE>(a, col_tiles, tasks, s)
                                                               : launch<B_Q4K_PLANAR, EPI_F32, ROWS_DENSE>(a, col_tiles, tasks, s);
    return output_is_bf16 ? launch<B_Q4K_RAW, EPI_BF16, ROWS_DENSE>(a, col_tiles, tasks, s)
                          : launch<B_Q4K_RAW, EPI_F32, ROWS_DENSE>(a, col_tiles, tasks, s);
}

// ---------------------------------------------------------------- grouped GEMM over raw GGUF expert stacks
namespace {
struct GroupedLayout { uint64_t xh, sx, tasks, total; uint32_t bound, in_rows; };
GroupedLayout grouped_layout(uint32_t tokens, uint32_t selected, uint32_t experts, uint32_t columns, int broadcast) {
    GroupedLayout l{};
    l.in_rows = broadcast ? tokens : tokens * selected;
    l.bound = tokens * selected / kTaskRows + experts;
    l.sx = align256(uint64_t(l.in_rows) * columns * 2);
    l.tasks = l.sx + align256(uint64_t(l.in_rows) * (columns / 256) * 32);
    l.total = l.tasks + align256((2 + 2 * uint64_t(l.bound)) * 4);
    return l;
}
}  // namespace

extern "C" uint64_t tsp_grouped_mm_workspace_bytes(uint32_t tokens, uint32_t selected, uint32_t experts, uint32_t columns, int broadcast) {
    return grouped_layout(tokens, selected, experts, columns, broadcast).total;
}

extern "C" int tsp_grouped_mm(uint32_t encoding, uint32_t layout, const void* matrices, uint64_t matrices_bytes, const uint32_t* ids,
                              const float* input, uint64_t input_stride_bytes, float* output, uint64_t output_stride_bytes,
                              uint32_t* token_map, uint32_t* counts, uint32_t* tasks, uint32_t columns, uint32_t rows, uint32_t experts,
                              uint32_t selected, uint32_t tokens, int broadcast, void* workspace, uint64_t workspace_bytes,
                              uint32_t* error_word, void* stream) {
    if (grouped_staged_takes(encoding, layout)) {
        // src/grouped_mm.cpp:24-47: the planner's geometry and byte spans decide; the routes, counts and 32-route tasks are written for
        // the caller as in the Q4_K arm, and the staged kernel reads that task list itself (the workspace is not used)
        tsp_grouped_mm_plan_t plan;
        const int planned = tsp_grouped_mm_plan(encoding, layout, columns, rows, experts, selected, tokens, input_stride_bytes, output_stride_bytes,
                                                broadcast, 1, &plan);
        if (planned != TSP_OK) return planned;
        TSP_REQUIRE(matrices && ids && input && output && token_map && counts && tasks && error_word, "null device pointer");
        TSP_REQUIRE(matrices_bytes == plan.matrix_bytes && plan.args.expert_stride_bytes < (1ull << 32), "grouped prefill matrix byte span mismatch");
        TSP_REQUIRE(reinterpret_cast<uintptr_t>(matrices) % 16 == 0 && reinterpret_cast<uintptr_t>(input) % 16 == 0 && reinterpret_cast<uintptr_t>(output) % 4 == 0,
                    "grouped prefill buffer span or alignment is invalid");
        const void* ins[] = {matrices, ids, input};
        const uint64_t in_bytes[] = {matrices_bytes, plan.indices_bytes, plan.input_bytes};
        const void* outs[] = {output, token_map, counts, tasks};
        const uint64_t out_bytes[] = {plan.output_bytes, plan.token_map_bytes, plan.counts_bytes, plan.tasks_bytes};
        for (int o = 0; o < 4; ++o) {
            for (int i = 0; i < 3; ++i) TSP_REQUIRE(!ranges_overlap(outs[o], out_bytes[o], ins[i], in_bytes[i]), "grouped prefill outputs overlap inputs");
            for (int q = 0; q < o; ++q) TSP_REQUIRE(!ranges_overlap(outs[o], out_bytes[o], outs[q], out_bytes[q]), "grouped prefill outputs overlap each other");
        }
        int rc = tsp_grouped_routes(ids, token_map, counts, experts, selected, tokens, error_word, stream);
        if (rc == TSP_OK) rc = tsp_grouped_tasks(counts, tasks, experts, selected, tokens, 32, error_word, stream);
        if (rc != TSP_OK) return rc;
        GroupedStagedArgs g{};
        g.matrices = static_cast<const uint8_t*>(matrices); g.input = input; g.output = output;
        g.expert_stride = plan.args.expert_stride_bytes; g.input_stride = input_stride_bytes; g.output_stride = output_stride_bytes;
        g.columns = columns; g.rows = rows; g.row_bytes = plan.args.row_bytes; g.experts = experts; g.selected = selected; g.tokens = tokens;
        g.broadcast = broadcast ? 1 : 0; g.maximum_tasks = plan.args.maximum_tasks;
        g.ids = ids; g.token_map = token_map; g.counts = counts; g.tasks = tasks; g.error_word = error_word;
        return launch_grouped_staged(encoding, layout, g, static_cast<hipStream_t>(stream));
    }
    TSP_REQUIRE(encoding == 12 && layout == TSP_LAYOUT_GGUF, "grouped dequant-GEMM takes Q4_K, Q5_K, Q5_1 and Q8_0 expert stacks in GGUF rows, Q8_0 in q8_lanes_v1 and Q5_1 in q51_lanes_v1 rows");
    TSP_REQUIRE(columns && columns <= 65536 && columns % 256 == 0 && rows && rows <= 32768 && experts >= 1 && experts <= 512 &&
                    selected >= 1 && selected <= 16 && selected <= experts && tokens >= 1 && tokens <= 2048,
                "grouped prefill geometry mismatch");
    const uint64_t expert_bytes = uint64_t(columns / 256) * 144 * rows;
    TSP_REQUIRE(matrices_bytes == expert_bytes * experts && expert_bytes < (1ull << 32), "grouped prefill matrix byte span mismatch");
    TSP_REQUIRE(input_stride_bytes >= uint64_t(columns) * 4 && input_stride_bytes % 4 == 0 && output_stride_bytes >= uint64_t(rows) * 4 &&
                    output_stride_bytes % 4 == 0,
                "grouped prefill row stride");
    TSP_REQUIRE(matrices && ids && input && output && token_map && counts && tasks && workspace && error_word, "null device pointer");
    const GroupedLayout l = grouped_layout(tokens, selected, experts, columns, broadcast);
    TSP_REQUIRE(workspace_bytes >= l.total && reinterpret_cast<uintptr_t>(workspace) % 256 == 0 && reinterpret_cast<uintptr_t>(matrices) % 16 == 0,
                "grouped prefill buffer span or alignment is invalid");
    const uint32_t routes = tokens * selected;
    const uint64_t in_span = uint64_t(l.in_rows - 1) * input_stride_bytes + uint64_t(columns) * 4;
    const uint64_t out_span = uint64_t(routes - 1) * output_stride_bytes + uint64_t(rows) * 4;
    const void* ins[] = {matrices, ids, input};
    const uint64_t in_bytes[] = {matrices_bytes, uint64_t(routes) * 4, in_span};
    const void* outs[] = {output, token_map, counts, tasks, workspace};
    const uint64_t out_bytes[] = {out_span, uint64_t(experts) * tokens * 4, uint64_t(experts) * 4, (2 + 2 * (uint64_t(routes) / 32 + experts)) * 4, l.total};
    for (int o = 0; o < 5; ++o) {
        for (int i = 0; i < 3; ++i) TSP_REQUIRE(!ranges_overlap(outs[o], out_bytes[o], ins[i], in_bytes[i]), "grouped prefill outputs overlap inputs");
        for (int q = 0; q < o; ++q) TSP_REQUIRE(!ranges_overlap(outs[o], out_bytes[o], outs[q], out_bytes[q]), "grouped prefill outputs overlap each other");
    }
    const auto s = static_cast<hipStream_t>(stream);
    auto* ws = static_cast<uint8_t*>(workspace);
    auto* xh = reinterpret_cast<_Float16*>(ws);
    auto* sx = reinterpret_cast<_Float16*>(ws + l.sx);
    auto* task_list = reinterpret_cast<uint32_t*>(ws + l.tasks);
    int rc = tsp_grouped_routes(ids, token_map, counts, experts, selected, tokens, error_word, stream);
    if (rc == TSP_OK) rc = lists_and_rows(TaskLists{counts, tasks, 32, task_list, kTaskRows, experts, selected, tokens, false, nullptr}, input, input_stride_bytes, xh, sx,
                                          l.in_rows, columns, error_word, s);
    if (rc != TSP_OK) return rc;
    GemmArgs a{};
    a.a = xh; a.a_stride = columns; a.sx = sx; a.w0 = static_cast<const uint8_t*>(matrices); a.raw_expert_bytes = expert_bytes;
    a.experts = experts; a.tasks = task_list; a.counts = counts; a.token_map = token_map; a.ids = ids; a.tokens = tokens; a.selected = selected;
    a.broadcast = broadcast ? 1 : 0; a.n = rows; a.k = columns; a.out = output; a.out_stride = output_stride_bytes; a.out_scale = 1.0f;
    a.error_word = error_word;
    return launch<B_Q4K_RAW, EPI_F32, ROWS_ROUTES>(a, (rows + 255) / 256, l.bound, s);
}

// ---------------------------------------------------------------- grouped MoE
namespace {
struct NaxLayout { uint64_t xh, sx, tasks, classes, hbuf, meta, total; uint32_t bound; };
NaxLayout nax_layout(uint32_t tokens, uint32_t selected, uint32_t experts, uint32_t channels, uint32_t hidden, bool shared = false) {
    NaxLayout l{};
    l.bound = tokens * selected / kTaskRows + experts + (shared ? (tokens + kTaskRows - 1) / kTaskRows : 0);
    l.xh = 0;
    l.sx = align256(uint64_t(tokens) * channels * 2);
    l.tasks = l.sx + align256(uint64_t(tokens) * (channels / 256) * 32);
    l.classes = l.tasks + align256((2 + 2 * uint64_t(l.bound)) * 4);  // the 64-row tasks by number of rows: two counts, two index lists
    l.hbuf = l.classes + align256((2 + 2 * uint64_t(l.bound)) * 4);
    l.meta = l.hbuf + align256(uint64_t(l.bound) * kTaskRows * hidden * 2);  // union records of one chunk of eight tokens
    l.total = l.meta + align256(2320 * 4);
    return l;
}

// Every gate/up pair of one encoding (Q4_K, Q5_K or Q8_0 co-located halves) and every down kind runs on the matrix cores
// below. What is left for this arm are gate and up tensors of DIFFERENT encodings (this entry point takes any gate kind
// beside any up kind; the engine's is_planar_moe asks for one encoding, so its compositions never come here): they run through the routed kernels for at most eight tokens, a chunk of eight tokens at a
// time: the same routes, tasks and expert_down rows, computed in f32 on the vector units. h of a chunk (8 * selected rows of
// f32) borrows the buffer the matrix-core path keeps its h rows in, which is never smaller.
int grouped_moe_in_eights(const tsp_grouped_moe* m, const NaxLayout& l, void* stream) {
    auto* ws = static_cast<uint8_t*>(m->workspace);
    TSP_REQUIRE(uint64_t(8) * m->selected * m->hidden * 4 <= l.meta - l.hbuf, "planar v3 NAX scratch too small for requested batch");  // before anything is enqueued
    int rc = tsp_grouped_routes(m->ids, m->token_map, m->counts, m->experts, m->selected, m->tokens, m->error_word, stream);
    if (rc == TSP_OK) rc = tsp_grouped_tasks(m->counts, m->tasks, m->experts, m->selected, m->tokens, 32, m->error_word, stream);
    for (uint32_t t0 = 0; rc == TSP_OK && t0 < m->tokens; t0 += 8) {
        tsp_small_moe c{};
        c.pair_lo = m->pair_lo; c.pair_hi = m->pair_hi; c.down = m->down;
        c.gate_kind = m->gate_kind; c.up_kind = m->up_kind; c.down_kind = m->down_kind;
        c.channels = m->channels; c.hidden = m->hidden; c.experts = m->experts; c.selected = m->selected;
        c.tokens = m->tokens - t0 < 8 ? m->tokens - t0 : 8;
        c.ids = m->ids + uint64_t(t0) * m->selected;
        c.x = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(m->x) + uint64_t(t0) * m->x_stride_bytes);
        c.x_stride_bytes = m->x_stride_bytes;
        c.h = reinterpret_cast<float*>(ws + l.hbuf); c.h_stride_bytes = uint64_t(m->hidden) * 4;
        c.y = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(m->y) + uint64_t(t0) * m->selected * m->y_stride_bytes);
        c.y_stride_bytes = m->y_stride_bytes;
        c.union_meta = reinterpret_cast<uint32_t*>(ws + l.meta);
        c.error_word = m->error_word;
        rc = tsp_planar_moe_routed_m8(&c, stream);  // builds the chunk's union records itself
    }
    return rc;
}
}  // namespace

extern "C" uint64_t tsp_planar_nax_workspace_bytes(uint32_t tokens, uint32_t selected, uint32_t experts, uint32_t channels, uint32_t hidden) {
    return nax_layout(tokens, selected, experts, channels, hidden).total;
}

namespace {
int grouped_moe(const tsp_grouped_moe* m, const tsp_shared_expert* shared, void* stream);
}

extern "C" int tsp_planar_nax_grouped_moe(const tsp_grouped_moe* m, void* stream) { return grouped_moe(m, nullptr, stream); }

extern "C" uint64_t tsp_planar_nax_shared_workspace_bytes(uint32_t tokens, uint32_t selected, uint32_t experts, uint32_t channels, uint32_t hidden) {
    return nax_layout(tokens, selected, experts, channels, hidden, true).total;
}

extern "C" int tsp_planar_nax_grouped_moe_shared(const tsp_grouped_moe* m, const tsp_shared_expert* shared, void* stream) {
    TSP_REQUIRE(shared, "null shared expert description");
    return grouped_moe(m, shared, stream);
}

namespace {
int grouped_moe(const tsp_grouped_moe* m, const tsp_shared_expert* shared, void* stream) {
    TSP_REQUIRE(m, "null grouped MoE description");
    const bool fast_gate_up = m->gate_kind == TSP_KIND_Q4K_COLOC_GATE && m->up_kind == TSP_KIND_Q4K_COLOC_UP;
    const bool fast_down = m->down_kind == TSP_KIND_Q6K_PLANAR_X;
    const bool matrix_cores = (fast_gate_up || planar_staged_gate_up_takes(m->gate_kind, m->up_kind)) && (fast_down || planar_staged_down_takes(m->down_kind));
    // columns of the K kinds come in super-blocks of 256, those of Q5_1 / Q8_0 in blocks of 32; hidden units in multiples of 32
    const uint32_t channel_step = (m->gate_kind == TSP_KIND_Q8_COLOC_GATE) ? 32u : 256u, hidden_step = fast_down ? 256u : 32u;
    TSP_REQUIRE(m->tokens >= 1 && m->tokens <= 2048 && m->selected >= 1 && m->selected <= 16 && m->selected <= m->experts &&
                    m->experts >= 2 && m->experts <= 512 && m->experts % 2 == 0 && m->channels && m->hidden && m->channels % channel_step == 0 &&
                    m->hidden % hidden_step == 0 && m->channels <= 65536 && m->hidden <= 65536,
                "planar v3 NAX grouped MoE shape or stride mismatch");
    TSP_REQUIRE(m->x_stride_bytes >= uint64_t(m->channels) * 4 && m->x_stride_bytes % 4 == 0 &&
                    m->y_stride_bytes >= uint64_t(m->channels) * 4 && m->y_stride_bytes % 4 == 0,
                "planar v3 NAX grouped MoE shape or stride mismatch");
    TSP_REQUIRE(m->pair_lo && m->pair_hi && m->down && m->ids && m->x && m->y && m->token_map && m->counts && m->tasks &&
                    m->workspace && m->error_word,
                "null device pointer");
    TSP_REQUIRE(!shared || (fast_gate_up && fast_down), "the always-on expert rides only with Q4_K co-located gate/up and Q6_K planes down");
    if (!matrix_cores) {
        const NaxLayout lay = nax_layout(m->tokens, m->selected, m->experts, m->channels, m->hidden);
        TSP_REQUIRE(m->workspace_bytes >= lay.total && reinterpret_cast<uintptr_t>(m->workspace) % 256 == 0,
                    "planar v3 NAX scratch too small for requested batch");
        return grouped_moe_in_eights(m, lay, stream);  // kinds, spans and overlaps are checked per chunk
    }
    tsp_planar_spec gu, dn;
    const uint32_t gate_up_type = fast_gate_up ? 12u : m->gate_kind == TSP_KIND_Q5K_COLOC_GATE ? 13u : 8u;
    const uint32_t down_type = fast_down ? 14u : m->down_kind == TSP_KIND_Q51_PLANAR ? 7u : 8u;
    int rc = tsp_make_expert_spec(gate_up_type, m->channels, m->hidden, &gu);
    if (rc == TSP_OK) rc = tsp_make_expert_spec(down_type, m->hidden, m->channels, &dn);
    if (rc != TSP_OK) return rc;
    TSP_REQUIRE(gu.planar_expert_bytes < (1ull << 32) && dn.planar_expert_bytes < (1ull << 32),
                "planar v3 grouped MoE addresses weight rows with 32-bit offsets: one expert must be under 4 GiB");
    const NaxLayout l = nax_layout(m->tokens, m->selected, m->experts, m->channels, m->hidden, shared != nullptr);
    TSP_REQUIRE(m->workspace_bytes >= l.total, "planar v3 NAX scratch too small for requested batch");
    if (shared) {
        TSP_REQUIRE(shared->gate && shared->up && shared->down && shared->y, "null device pointer");
        TSP_REQUIRE(reinterpret_cast<uintptr_t>(shared->gate) % 16 == 0 && reinterpret_cast<uintptr_t>(shared->up) % 16 == 0 &&
                        reinterpret_cast<uintptr_t>(shared->down) % 16 == 0,
                    "planar v3 matrices require 16-byte alignment (workspace 256)");
        TSP_REQUIRE(shared->y_stride_bytes >= uint64_t(m->channels) * 4 && shared->y_stride_bytes % 4 == 0, "planar v3 NAX grouped MoE shape or stride mismatch");
        const uint64_t sy_span = uint64_t(m->tokens - 1) * shared->y_stride_bytes + uint64_t(m->channels) * 4;
        const void* others[] = {m->pair_lo, m->pair_hi, m->down, m->x, m->ids, shared->gate, shared->up, shared->down, m->y, m->token_map, m->counts, m->tasks, m->workspace};
        const uint64_t spans[] = {uint64_t(m->experts) * gu.planar_expert_bytes, uint64_t(m->experts) * gu.planar_expert_bytes, uint64_t(m->experts) * dn.planar_expert_bytes,
                                  uint64_t(m->tokens - 1) * m->x_stride_bytes + uint64_t(m->channels) * 4, uint64_t(m->tokens) * m->selected * 4,
                                  gu.planar_expert_bytes, gu.planar_expert_bytes, dn.planar_expert_bytes,
                                  uint64_t(m->tokens * m->selected - 1) * m->y_stride_bytes + uint64_t(m->channels) * 4, uint64_t(m->experts) * m->tokens * 4,
                                  uint64_t(m->experts) * 4, (2 + 2 * (uint64_t(m->tokens) * m->selected / 32 + m->experts)) * 4, l.total};
        for (int i = 0; i < 13; ++i) TSP_REQUIRE(!ranges_overlap(shared->y, sy_span, others[i], spans[i]), "planar v3 NAX grouped MoE outputs overlap inputs");
        for (int i = 8; i < 13; ++i)
            for (int w = 5; w < 8; ++w) TSP_REQUIRE(!ranges_overlap(others[i], spans[i], others[w], spans[w]), "planar v3 NAX grouped MoE outputs overlap inputs");
    }
    TSP_REQUIRE(reinterpret_cast<uintptr_t>(m->workspace) % 256 == 0 && reinterpret_cast<uintptr_t>(m->pair_lo) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(m->pair_hi) % 16 == 0 && reinterpret_cast<uintptr_t>(m->down) % 16 == 0,
                "planar v3 matrices require 16-byte alignment (workspace 256)");
    const uint32_t routes = m->tokens * m->selected;
    const uint64_t y_span = uint64_t(routes - 1) * m->y_stride_bytes + uint64_t(m->channels) * 4;
    const uint64_t x_span = uint64_t(m->tokens - 1) * m->x_stride_bytes + uint64_t(m->channels) * 4;
    const uint64_t pair_bytes = uint64_t(m->experts / 2) * 2 * gu.planar_expert_bytes, dn_bytes = uint64_t(m->experts) * dn.planar_expert_bytes;
    const uint64_t map_bytes = uint64_t(m->experts) * m->tokens * 4, cnt_bytes = uint64_t(m->experts) * 4;
    const uint64_t tasks_bytes = (2 + 2 * (uint64_t(routes) / 32 + m->experts)) * 4;
    const void* ins[] = {m->pair_lo, m->pair_hi, m->down, m->x, m->ids};
    const uint64_t in_bytes[] = {pair_bytes, pair_bytes, dn_bytes, x_span, uint64_t(routes) * 4};
    const void* outs[] = {m->y, m->token_map, m->counts, m->tasks, m->workspace};
    const uint64_t out_bytes[] = {y_span, map_bytes, cnt_bytes, tasks_bytes, l.total};
    for (int o = 0; o < 5; ++o) {
        for (int i = 0; i < 5; ++i) TSP_REQUIRE(!ranges_overlap(outs[o], out_bytes[o], ins[i], in_bytes[i]), "planar v3 NAX grouped MoE outputs overlap inputs");
        for (int p = 0; p < o; ++p) TSP_REQUIRE(!ranges_overlap(outs[o], out_bytes[o], outs[p], out_bytes[p]), "planar v3 NAX grouped MoE outputs overlap each other");
    }
    const auto s = static_cast<hipStream_t>(stream);
    auto* ws = static_cast<uint8_t*>(m->workspace);
    auto* xh = reinterpret_cast<_Float16*>(ws + l.xh);
    auto* sx = reinterpret_cast<_Float16*>(ws + l.sx);
    auto* task_list = reinterpret_cast<uint32_t*>(ws + l.tasks);
    auto* hbuf = reinterpret_cast<_Float16*>(ws + l.hbuf);

    rc = tsp_grouped_routes(m->ids, m->token_map, m->counts, m->experts, m->selected, m->tokens, m->error_word, stream);
    // only the Q4_K gate/up kernels want the activation sums and the column order that goes with them
    if (rc == TSP_OK) rc = lists_and_rows(TaskLists{m->counts, m->tasks, 32, task_list, kTaskRows, m->experts, m->selected, m->tokens, shared != nullptr, reinterpret_cast<uint32_t*>(ws + l.classes)}, m->x,
                                          m->x_stride_bytes, xh, fast_gate_up ? sx : nullptr, m->tokens, m->channels, m->error_word, s);
    if (rc != TSP_OK) return rc;

    PlanarStagedArgs staged{};
    staged.xh = xh; staged.pair_lo = static_cast<const uint8_t*>(m->pair_lo); staged.pair_hi = static_cast<const uint8_t*>(m->pair_hi);
    staged.down = static_cast<const uint8_t*>(m->down); staged.spec = gu; staged.down_spec = dn;
    staged.channels = m->channels; staged.hidden = m->hidden; staged.experts = m->experts; staged.selected = m->selected; staged.tokens = m->tokens;
    staged.task_list = task_list; staged.task_slots = l.bound; staged.counts = m->counts; staged.token_map = m->token_map; staged.ids = m->ids;
    staged.hbuf = hbuf; staged.y = m->y; staged.y_stride = m->y_stride_bytes; staged.error_word = m->error_word;

    GemmArgs g{};
    g.a = xh; g.a_stride = m->channels; g.sx = sx; g.w0 = static_cast<const uint8_t*>(m->pair_lo); g.w1 = static_cast<const uint8_t*>(m->pair_hi);
    g.spec = gu; g.experts = m->experts; g.tasks = task_list; g.counts = m->counts; g.token_map = m->token_map; g.ids = m->ids;
    g.tokens = m->tokens; g.selected = m->selected; g.n = m->hidden; g.k = m->channels; g.out = hbuf; g.out_scale = 1.0f;
    g.error_word = m->error_word;
    if (shared) { g.shared_w0 = static_cast<const uint8_t*>(shared->gate); g.shared_w1 = static_cast<const uint8_t*>(shared->up); }
    if (!fast_gate_up) {
        rc = launch_planar_staged_gate_up(staged, s);
    } else if (resident_gate_up_takes(m->channels, m->hidden)) {
        ResidentGateUpArgs r{};
        r.xh = xh; r.sx = sx; r.pair_lo = g.w0; r.pair_hi = g.w1; r.shared_gate = g.shared_w0; r.shared_up = g.shared_w1; r.spec = gu;
        r.experts = m->experts; r.tokens = m->tokens; r.selected = m->selected; r.hidden = m->hidden;
        r.tasks = task_list; r.classes = reinterpret_cast<const uint32_t*>(ws + l.classes); r.counts = m->counts; r.token_map = m->token_map; r.ids = m->ids; r.task_slots = l.bound;
        r.hbuf = hbuf; r.error_word = m->error_word;
        rc = launch_resident_gate_up(r, s);
    } else {
        rc = launch<B_Q4K_PLANAR, EPI_SWIGLU, ROWS_GATHER_TOKENS>(g, (m->hidden + 127) / 128, l.bound, s);
    }
    if (rc != TSP_OK) return rc;
    const uint64_t shared_span = shared ? uint64_t(m->tokens) * shared->y_stride_bytes : 0;
    if (resident_down_takes(down_type, m->channels, m->hidden) && uint64_t(routes) * m->y_stride_bytes < (1ull << 32) && shared_span < (1ull << 32)) {
        ResidentDownArgs r{};
        r.hbuf = hbuf; r.down = static_cast<const uint8_t*>(m->down); r.shared_down = shared ? static_cast<const uint8_t*>(shared->down) : nullptr;
        r.spec = dn; r.experts = m->experts; r.tokens = m->tokens; r.selected = m->selected;
        r.channels = m->channels; r.tasks = task_list; r.classes = reinterpret_cast<const uint32_t*>(ws + l.classes); r.counts = m->counts;
        r.token_map = m->token_map; r.ids = m->ids; r.task_slots = l.bound; r.y = static_cast<float*>(m->y); r.y_stride = m->y_stride_bytes;
        r.shared_y = shared ? static_cast<float*>(shared->y) : nullptr; r.shared_y_stride = shared ? shared->y_stride_bytes : 0;
        r.out_scale = 256.0f; r.error_word = m->error_word;
        return launch_resident_down(r, s);
    }
    if (!fast_down) return launch_planar_staged_down(staged, s);

    GemmArgs d{};
    d.a = hbuf; d.a_stride = m->hidden; d.w0 = static_cast<const uint8_t*>(m->down); d.spec = dn; d.experts = m->experts;
    d.tasks = task_list; d.counts = m->counts; d.token_map = m->token_map; d.ids = m->ids; d.tokens = m->tokens; d.selected = m->selected;
    d.n = m->channels; d.k = m->hidden; d.out = m->y; d.out_stride = m->y_stride_bytes; d.out_scale = 256.0f;  // undo the 2^-8 carried by h
    d.error_word = m->error_word;
    if (shared) { d.shared_w0 = static_cast<const uint8_t*>(shared->down); d.shared_out = shared->y; d.shared_out_stride = shared->y_stride_bytes; }
    return launch<B_Q6K_PLANAR, EPI_F32, ROWS_TASK_SLOTS>(d, (m->channels + 255) / 256, l.bound, s);
}
}  // namespace
