// Matrix products with at most eight activation rows per weight matrix (decode, verify, the T <= 8 routed MoE):
// out[m, n] = sum_k x[m, k] * dec(W[n, k]),  m < 8, on the matrix cores, every weight byte read once.
//
// These products are bound by HBM and, with scalar code, by the dequantisation arithmetic: converting and
// multiplying each weight for each row costs 3+ VALU operations per weight and row. Here the weights go to
// v_mfma_f32_32x32x16_f16 as exact integer factors (see mfma_quant.hpp: ~1.4 operations per weight, independent
// of the number of rows), the block scales are applied in f32 once per 256-column super-block, and the eight
// activation rows occupy 8 of the 32 rows of the MFMA A operand (the matrix cores have capacity to spare).
//
// f32 accuracy with f16 operands: the rows are scaled by a power of two so that their largest magnitude lands
// near 2^14 and split as hi + lo halves (22 significant bits); both halves multiply the same integer weight
// fragment and accumulate into the same f32 accumulator. Nothing else is rounded before the f32 scaling.
//
// Two kernels. Rows of 1, 2, 4 or 8 super-blocks (every shape the engine's models have) take flat_kernel further down: one
// super-block per wave, no loop. The looped skinny_kernel serves the other row lengths:
// one workgroup = one task (a weight matrix and up to 8 rows) x 256 weight rows (128 hidden units for gate/up).
// The rows are staged once, for all of K, in LDS (hi and lo planes, 16-byte chunks XOR-swizzled by row so the
// eight rows of a fragment read fall in different banks); after that the four waves run independently, with no
// barrier in the K loop, each streaming its own 64 weight rows with one super-block of loads in flight.
#include "skinny.hpp"

#include <type_traits>

#include "mfma_quant.hpp"

using namespace tsp;

namespace {

constexpr int kRows = 8;
constexpr uint32_t kMaxColumns = 2048;  // 2 planes x 8 rows x 2048 halfs = 64 KB of LDS

enum Source : int { SRC_DENSE = 0, SRC_RECORD_TOKENS = 1, SRC_RECORD_ROUTES = 2 };
enum Output : int { OUT_ROWS = 0, OUT_SWIGLU = 1 };

struct SkinnyArgs {
    const float* x;        // activation rows, x_stride bytes apart
    uint64_t x_stride;
    const uint8_t* w0;     // dense matrix / pair_lo / down experts
    const uint8_t* w1;     // pair_hi
    tsp_planar_spec spec;
    uint32_t experts, selected, tokens;
    const uint32_t* ids;   // routes when there is no union block
    const uint32_t* meta;  // union records
    uint32_t m, n, k;      // dense: rows of x; weight rows (hidden units for SwiGLU); columns
    float* out;            // rows out_stride bytes apart
    uint64_t out_stride;
    uint32_t* error_word;
    // an always-on expert riding in the same launch: the workgroups of task index `shared_index` take every token as a
    // row, these weights (gate / up, or down in shared_w0), these input rows and these output rows
    const uint8_t* shared_w0;
    const uint8_t* shared_w1;
    const float* shared_x;
    uint64_t shared_x_stride;
    float* shared_out;
    uint64_t shared_out_stride;
    uint32_t shared_index;
};

// The always-on expert's task: row k is token k.
__device__ __forceinline__ bool is_shared_task(const SkinnyArgs& a, uint32_t index) { return a.shared_w0 != nullptr && index == a.shared_index; }

struct Task { uint32_t expert, count, src[kRows], dst[kRows]; };

// Task `index`: the dense rows, a union record, or a single route when there is no union block.
template <int SRC>
__device__ __forceinline__ bool load_task(const SkinnyArgs& a, uint32_t index, Task& t) {
    if (is_shared_task(a, index)) {
        t.expert = 0; t.count = a.tokens;
#pragma unroll
        for (int k = 0; k < kRows; ++k) t.src[k] = t.dst[k] = uint32_t(k) < a.tokens ? k : 0;
        return a.tokens <= kRows;
    } else if constexpr (SRC == SRC_DENSE) {
        t.expert = 0; t.count = a.m;
#pragma unroll
        for (int k = 0; k < kRows; ++k) t.src[k] = t.dst[k] = k;
        return index == 0;
    } else if (a.meta) {
        // every word is read before the record count is looked at (index < 128 always lies inside the block): one round trip, not two
        const uint32_t live = a.meta[6];
        t.expert = a.meta[8 + index];
        t.count = a.meta[136 + index];
#pragma unroll
        for (int k = 0; k < kRows; ++k) {
            const uint32_t token = a.meta[264 + index * 8 + k], route = a.meta[1288 + index * 8 + k];
            t.src[k] = SRC == SRC_RECORD_TOKENS ? token : route;
            t.dst[k] = route;
        }
        return index < live;
    } else {
        if (index >= a.tokens * a.selected) return false;
        t.expert = a.ids[index];
        t.count = 1;
#pragma unroll
        for (int k = 0; k < kRows; ++k) { t.src[k] = SRC == SRC_RECORD_TOKENS ? index / a.selected : index; t.dst[k] = index; }
        return true;
    }
}

// KS = number of K slices: a workgroup has 4 * KS waves, wave w owns weight-row group w % 4 and K slice w / 4; the
// slices' partial sums meet in LDS at the end (fixed order, so results do not depend on timing). With about one task
// tile per compute unit, slicing K is what puts more than one wave on each SIMD.
template <int BKIND, int OUT, int SRC, int KS>
__global__ __launch_bounds__(256 * KS, 2) void skinny_kernel(SkinnyArgs args) {
    SkinnyArgs a = args;
    const bool shared = is_shared_task(a, blockIdx.y);
    if (shared) { a.x = a.shared_x; a.x_stride = a.shared_x_stride; a.out = a.shared_out; a.out_stride = a.shared_out_stride; }
    constexpr bool Q6 = BKIND == B_Q6K_PLANAR;
    constexpr uint32_t THREADS = 256 * KS;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // [hi plane][lo plane][activation sums]
    __shared__ float wave_max[4 * KS];

    const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = (tid / kWave) % 4, slice = tid / (4 * kWave);
    const uint32_t col = lane % 32, khalf = lane / 32;
    Task task;
    if (!load_task<SRC>(a, blockIdx.y, task)) return;
    if (task.expert >= a.experts || task.count == 0 || task.count > kRows) {
        if (tid == 0 && blockIdx.x == 0 && (task.expert >= a.experts || task.count > kRows)) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
        return;
    }
    const uint32_t K = a.k, bpr = K / 256, chunks = K / 8;  // 16-byte chunks per row and plane
    _Float16* const a_hi = reinterpret_cast<_Float16*>(lds);
    _Float16* const a_lo = a_hi + kRows * K;
    _Float16* const sums = a_lo + kRows * K;  // [row][super-block][8 hi, 8 lo] of (sub-block sum / 32), Q4_K only

    // ---- stage the rows: largest magnitude -> power-of-two scale -> hi/lo halves (+ sub-block sums)
    uint32_t bad = 0;
    float biggest = 0;
    for (uint32_t i = tid; i < kRows * K / 4; i += THREADS) {
        const uint32_t r = i / (K / 4), c4 = i % (K / 4);
        if (r < task.count) {
            const float4 v = *reinterpret_cast<const float4*>(reinterpret_cast<const uint8_t*>(a.x) + uint64_t(task.src[r]) * a.x_stride + c4 * 16);
            if (nonfinite(v.x) || nonfinite(v.y) || nonfinite(v.z) || nonfinite(v.w)) bad = TSP_ERRBIT_NONFINITE;
            biggest = fmaxf(biggest, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        }
    }
    biggest = wave_largest(biggest);
    if (lane == 0) wave_max[tid / kWave] = biggest;
    __syncthreads();
    biggest = wave_max[0];
#pragma unroll
    for (int w = 1; w < 4 * KS; ++w) biggest = fmaxf(biggest, wave_max[w]);
    // scale = 2^(13 - exponent(biggest)): the largest |x * scale| is below 2^15, the sub-block sums / 32 below 2^15 too
    float scale = 1.0f, inv_scale = 1.0f;
    if (biggest > 0 && !nonfinite(biggest)) {
        const int e = int((__float_as_uint(biggest) >> 23) & 0xffu) - 127;
        int shift = 13 - e;
        shift = shift > 100 ? 100 : shift < -100 ? -100 : shift;
        scale = __uint_as_float(uint32_t(127 + shift) << 23);
        inv_scale = __uint_as_float(uint32_t(127 - shift) << 23);
    }
    for (uint32_t i = tid; i < kRows * chunks; i += THREADS) {
        const uint32_t r = i / chunks, c = i % chunks;
        f16x8 hi{}, lo{};
        float sum = 0;
        if (r < task.count) {
            const float4* src = reinterpret_cast<const float4*>(reinterpret_cast<const uint8_t*>(a.x) + uint64_t(task.src[r]) * a.x_stride + c * 32);
            const float4 v0 = src[0], v1 = src[1];
            const float v[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float s = v[e] * scale;
                hi[e] = _Float16(s);
                lo[e] = _Float16(s - float(hi[e]));
                sum += s;
            }
        }
        const uint32_t at = (r * chunks + (c ^ r)) * 8;
        *reinterpret_cast<f16x8*>(a_hi + at) = hi;
        *reinterpret_cast<f16x8*>(a_lo + at) = lo;
        if constexpr (!Q6) {
            // four neighbouring lanes hold the four chunks of one 32-column sub-block (chunks is a multiple of 32)
            sum = dpp_add<0xB1>(sum);
            sum = dpp_add<0x4E>(sum);
            if ((c & 3) == 0) {
                const float s32 = sum * 0.03125f;
                const _Float16 h = _Float16(s32);
                const uint32_t sub = c / 4;
                _Float16* o = sums + (r * bpr + sub / 8) * 16 + sub % 8;
                o[0] = h;
                o[8] = _Float16(s32 - float(h));
            }
        }
    }
    __syncthreads();

    // ---- weight rows of this wave
    const uint8_t* wbase[2];
    uint32_t wrow[2], out_col[2];
    bool col_live[2];
    if constexpr (OUT == OUT_SWIGLU) {
        const uint32_t unit = blockIdx.x * 128 + wave * 32 + col;
        const uint32_t half_e = a.experts / 2;
        const uint8_t* pair = (task.expert < half_e ? a.w0 : a.w1) + uint64_t(task.expert < half_e ? task.expert : task.expert - half_e) * 2 * a.spec.planar_expert_bytes;
        wbase[0] = shared ? a.shared_w0 : pair;
        wbase[1] = shared ? a.shared_w1 : pair + a.spec.planar_expert_bytes;
        col_live[0] = col_live[1] = unit < a.n;
        wrow[0] = wrow[1] = col_live[0] ? unit : a.n - 1;
        out_col[0] = out_col[1] = unit;
    } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t n = blockIdx.x * 256 + wave * 64 + j * 32 + col;
            col_live[j] = n < a.n;
            wrow[j] = col_live[j] ? n : a.n - 1;
            out_col[j] = n;
            wbase[j] = shared ? a.shared_w0 : BKIND == B_Q4K_RAW ? a.w0 : a.w0 + uint64_t(task.expert) * a.spec.planar_expert_bytes;
        }
    }

    const uint32_t b_begin = slice * (bpr / KS), b_end = b_begin + bpr / KS;  // the host picks KS so that it divides bpr
    f32x16 acc[2], blk[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[j][v] = 0.0f;

    // A fragment of the 16-column step whose first column is 8 * chunk: rows 8..31 of the operand repeat rows 0..7
    const uint32_t arow = col & 7;
    auto a_frag = [&](const _Float16* plane, uint32_t chunk) {
        return *reinterpret_cast<const f16x8*>(plane + (arow * chunks + (chunk ^ arow)) * 8);
    };
    // both halves of the rows against the same weight fragments; `first` starts the super-block accumulator from zero
    auto mfma = [&](uint32_t chunk, const f16x8& b0, const f16x8& b1, bool first) {
        const f16x8 ah = a_frag(a_hi, chunk), al = a_frag(a_lo, chunk);
        if (first) {
            const f32x16 zero{};
            blk[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, b0, zero, 0, 0, 0);
            blk[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, b1, zero, 0, 0, 0);
        } else {
            blk[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, b0, blk[0], 0, 0, 0);
            blk[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, b1, blk[1], 0, 0, 0);
        }
        blk[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, b0, blk[0], 0, 0, 0);
        blk[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, b1, blk[1], 0, 0, 0);
    };
    // only accumulator registers 0..3 hold rows 0..7 (row = 4 * khalf + v)
    auto fold = [&](float d0, float d1) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            acc[0][v] = __builtin_fmaf(d0, blk[0][v], acc[0][v]);
            acc[1][v] = __builtin_fmaf(d1, blk[1][v], acc[1][v]);
        }
    };

    if constexpr (Q6) {
        struct BlockQ6 { u32x4 la[2], lb[2], qh[2]; uint32_t sc[4]; float d; };
        auto load_block = [&](uint32_t b, int j) {
            b = b < bpr ? b : bpr - 1;
            const uint64_t at = uint64_t(wrow[j]) * bpr + b;
            const uint8_t* ql = wbase[j] + a.spec.qs_offset + at * 128 + khalf * 16;
            const uint8_t* qh = wbase[j] + a.spec.qh_offset + at * 64 + khalf * 16;
            BlockQ6 r;
#pragma unroll
            for (int sec = 0; sec < 2; ++sec) {
                r.la[sec] = *reinterpret_cast<const u32x4*>(ql + sec * 64);
                r.lb[sec] = *reinterpret_cast<const u32x4*>(ql + sec * 64 + 32);
                r.qh[sec] = *reinterpret_cast<const u32x4*>(qh + sec * 32);
            }
            const uint4 sc16 = *reinterpret_cast<const uint4*>(wbase[j] + a.spec.sm_offset + at * 16);
            r.sc[0] = sc16.x; r.sc[1] = sc16.y; r.sc[2] = sc16.z; r.sc[3] = sc16.w;
            r.d = half_bits_to_float(*reinterpret_cast<const uint16_t*>(wbase[j] + a.spec.dm_offset + at * 2));
            return r;
        };
        BlockQ6 cur[2] = {load_block(b_begin, 0), load_block(b_begin, 1)};
        for (uint32_t b = b_begin; b < b_end; ++b) {
            const BlockQ6 nxt[2] = {load_block(b + 1, 0), load_block(b + 1, 1)};
            auto section = [&](auto sec_tag) {
                constexpr int SEC = decltype(sec_tag)::value;
                RawQ6 raw[2];
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    raw[j].la = cur[j].la[SEC]; raw[j].lb = cur[j].lb[SEC]; raw[j].qh = cur[j].qh[SEC];
                    raw[j].sc[0] = cur[j].sc[SEC * 2]; raw[j].sc[1] = cur[j].sc[SEC * 2 + 1];
                }
                auto quarter = [&](auto q_tag) {
                    constexpr int Q = decltype(q_tag)::value;
                    f16x8 f0[2], f1[2];
                    frags_q6k<Q>(raw[0], khalf, f0);
                    frags_q6k<Q>(raw[1], khalf, f1);
                    const uint32_t chunk = b * 32 + SEC * 16 + Q * 4 + khalf * 2;  // columns b*256 + SEC*128 + Q*32 + 16h
                    mfma(chunk, f0[0], f1[0], SEC == 0 && Q == 0);
                    mfma(chunk + 1, f0[1], f1[1], false);
                };
                quarter(std::integral_constant<int, 0>{});
                quarter(std::integral_constant<int, 1>{});
                quarter(std::integral_constant<int, 2>{});
                quarter(std::integral_constant<int, 3>{});
            };
            section(std::integral_constant<int, 0>{});
            section(std::integral_constant<int, 1>{});
            fold(cur[0].d, cur[1].d);
            cur[0] = nxt[0]; cur[1] = nxt[1];
        }
    } else {
        constexpr uint32_t BLK = BKIND == B_Q4K_PLANAR ? 128 : 144, QS_AT = BKIND == B_Q4K_PLANAR ? 0 : 16;
        struct BlockQ4 { u32x4 pair[4]; HdrQ4 hdr; };
        auto load_block = [&](uint32_t b, int j) {
            b = b < bpr ? b : bpr - 1;
            const uint8_t* qs = wbase[j] + (BKIND == B_Q4K_PLANAR ? a.spec.qs_offset : 0) + (uint64_t(wrow[j]) * bpr + b) * BLK + QS_AT + khalf * 16;
            BlockQ4 r;
#pragma unroll
            for (int p = 0; p < 4; ++p) r.pair[p] = *reinterpret_cast<const u32x4*>(qs + p * 32);
            r.hdr = load_hdr_q4k<BKIND>(wbase[j], a.spec, wrow[j], bpr, b);
            return r;
        };
        BlockQ4 cur[2] = {load_block(b_begin, 0), load_block(b_begin, 1)};
        for (uint32_t b = b_begin; b < b_end; ++b) {
            const BlockQ4 nxt[2] = {load_block(b + 1, 0), load_block(b + 1, 1)};
            auto pair_step = [&](auto p_tag) {
                constexpr int P = decltype(p_tag)::value;
                f16x8 f0[2], f1[2];
                const uint32_t chunk = b * 32 + P * 8 + khalf * 2;  // columns b*256 + P*64 + 16h
                frags_q4k<P, 0>(cur[0].pair[P], cur[0].hdr, f0);
                frags_q4k<P, 0>(cur[1].pair[P], cur[1].hdr, f1);
                mfma(chunk, f0[0], f1[0], P == 0);
                mfma(chunk + 1, f0[1], f1[1], false);
                frags_q4k<P, 1>(cur[0].pair[P], cur[0].hdr, f0);
                frags_q4k<P, 1>(cur[1].pair[P], cur[1].hdr, f1);
                mfma(chunk + 4, f0[0], f1[0], false);
                mfma(chunk + 5, f0[1], f1[1], false);
            };
            pair_step(std::integral_constant<int, 0>{});
            pair_step(std::integral_constant<int, 1>{});
            pair_step(std::integral_constant<int, 2>{});
            pair_step(std::integral_constant<int, 3>{});
            fold(cur[0].hdr.d, cur[1].hdr.d);
            // minima: acc -= 32 * dmin * sum_s (Sx / 32)(hi + lo)[m, s] * mn[n, s]
            const f16x8 m0 = minima_frag(cur[0].hdr), m1 = minima_frag(cur[1].hdr);
            const f16x8 sf = *reinterpret_cast<const f16x8*>(sums + (arow * bpr + b) * 16 + khalf * 8);
            const f32x16 zero{};
            blk[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sf, m0, zero, 0, 0, 0);
            blk[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sf, m1, zero, 0, 0, 0);
            fold(-32.0f * cur[0].hdr.dmin, -32.0f * cur[1].hdr.dmin);
            cur[0] = nxt[0]; cur[1] = nxt[1];
        }
    }

    // ---- partial sums of slices 1.. are added into slice 0 in slice order; the activation planes are free by then
    if constexpr (KS > 1) {
        float* const partial = reinterpret_cast<float*>(lds);  // [slice - 1][wave][tile][v][lane]
        __syncthreads();
        if (slice > 0) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v) partial[((((slice - 1) * 4 + wave) * 2 + j) * 4 + v) * kWave + lane] = acc[j][v];
        }
        __syncthreads();
        if (slice > 0) { publish_error(bad, a.error_word); return; }
#pragma unroll
        for (int s = 1; s < KS; ++s)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[j][v] += partial[((((s - 1) * 4 + wave) * 2 + j) * 4 + v) * kWave + lane];
    }
    // ---- epilogue: accumulator v of tile j is row 4 * khalf + v, weight row `col`
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const uint32_t r = 4 * khalf + v;
        if (r >= task.count) continue;
        uint8_t* orow = reinterpret_cast<uint8_t*>(a.out) + uint64_t(task.dst[r]) * a.out_stride;
        if constexpr (OUT == OUT_SWIGLU) {
            if (!col_live[0]) continue;
            const float g = acc[0][v] * inv_scale, u = acc[1][v] * inv_scale;
            const float sg = sigmoid_stable(g);
            const float h = (g * sg) * u;
            if (nonfinite(g) || nonfinite(u) || nonfinite(h)) bad = TSP_ERRBIT_NONFINITE;
            reinterpret_cast<float*>(orow)[out_col[0]] = h;
        } else {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if (!col_live[j]) continue;
                const float val = acc[j][v] * inv_scale;
                if (nonfinite(val)) bad = TSP_ERRBIT_NONFINITE;
                reinterpret_cast<float*>(orow)[out_col[j]] = val;
            }
        }
    }
    publish_error(bad, a.error_word);
}

// ---------------------------------------------------------------- one super-block per wave
// When a row has 1, 2, 4 or 8 super-blocks, a wave takes ONE super-block (256 columns) of 64 weight rows and nothing is
// looped: its weight bytes are requested first, and while they travel the wave stages its own 256 columns of the
// activation rows in a private corner of LDS (its own power-of-two scale: the partial sums are brought back to true
// units before they meet), so no wave waits for another until the slices of a unit column add up at the end, in slice
// order. A workgroup is the slices of one unit column (four or more waves: more unit columns when a row has fewer than
// four super-blocks). Many short waves with every load in flight from the first instruction fill the chip better than
// a few long pipelines here: these products move ~1 MB per expert and have about one expert per three compute units.
constexpr uint32_t kSlice = 256;                                       // columns per wave
constexpr uint32_t kWaveLds = 2 * kRows * kSlice * 2 + kRows * 32;      // hi plane, lo plane, sub-block sums: 8 448 B

template <int BKIND, int OUT, int SRC>
__global__ __launch_bounds__(512, 4) void flat_kernel(SkinnyArgs args) {  // four waves per SIMD: <= 128 registers per lane
    SkinnyArgs a = args;
    const bool shared = is_shared_task(a, blockIdx.y);
    if (shared) { a.x = a.shared_x; a.x_stride = a.shared_x_stride; a.out = a.shared_out; a.out_stride = a.shared_out_stride; }
    static_assert(BKIND != B_Q6K_PLANAR, "Q6_K planes take flat16_kernel");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // [wave][hi plane][lo plane][sums]; partial sums over it at the end

    const uint32_t tid = threadIdx.x, lane = tid % kWave, wv = tid / kWave;
    const uint32_t col = lane % 32, khalf = lane / 32;
    const uint32_t bpr = a.k / 256, ucols = blockDim.x / kWave / bpr;  // the host launches ucols * bpr waves
    const uint32_t slice = wv % bpr, ucol = wv / bpr;
    Task task;
    if (!load_task<SRC>(a, blockIdx.y, task)) return;
    if (task.expert >= a.experts || task.count == 0 || task.count > kRows) {
        if (tid == 0 && blockIdx.x == 0 && (task.expert >= a.experts || task.count > kRows)) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
        return;
    }

    // ---- this wave's 256 columns of the activation rows (lane l: columns 4l .. 4l+3 of each row), requested first: loads
    // come back in the order they were asked for, and these few cached bytes must not queue behind the weight bytes
    uint32_t bad = 0;
    float4 v[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        // a record rarely fills its eight rows: the rows past its count are neither read nor staged. Their places in LDS keep
        // whatever was there; a token row of the product depends on its own operand row only, and those rows are never stored.
        v[r] = float4{0, 0, 0, 0};
        if (uint32_t(r) < task.count)  // uniform
            v[r] = *reinterpret_cast<const float4*>(reinterpret_cast<const uint8_t*>(a.x) + uint64_t(task.src[r]) * a.x_stride + (slice * kSlice + lane * 4) * 4);
    }

    // ---- weight rows of this wave, and their bytes: requested before any arithmetic
    const uint8_t* wbase[2];
    uint32_t wrow[2], out_col[2];
    bool col_live[2];
    if constexpr (OUT == OUT_SWIGLU) {
        const uint32_t unit = (blockIdx.x * ucols + ucol) * 32 + col;
        const uint32_t half_e = a.experts / 2;
        const uint8_t* pair = (task.expert < half_e ? a.w0 : a.w1) + uint64_t(task.expert < half_e ? task.expert : task.expert - half_e) * 2 * a.spec.planar_expert_bytes;
        wbase[0] = shared ? a.shared_w0 : pair;
        wbase[1] = shared ? a.shared_w1 : pair + a.spec.planar_expert_bytes;
        col_live[0] = col_live[1] = unit < a.n;
        wrow[0] = wrow[1] = col_live[0] ? unit : a.n - 1;
        out_col[0] = out_col[1] = unit;
    } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t n = (blockIdx.x * ucols + ucol) * 64 + j * 32 + col;
            col_live[j] = n < a.n;
            wrow[j] = col_live[j] ? n : a.n - 1;
            out_col[j] = n;
            wbase[j] = shared ? a.shared_w0 : a.w0 + uint64_t(task.expert) * a.spec.planar_expert_bytes;
        }
    }
    struct Block { u32x4 pair[4]; HdrQ4 hdr; };
    Block cur[2];
    auto load_tile = [&](auto j_tag) {
        constexpr int j = decltype(j_tag)::value;
        const uint64_t at = uint64_t(wrow[j]) * bpr + slice;
        constexpr uint32_t BLK = BKIND == B_Q4K_PLANAR ? 128 : 144, QS_AT = BKIND == B_Q4K_PLANAR ? 0 : 16;
        const uint8_t* qs = wbase[j] + (BKIND == B_Q4K_PLANAR ? a.spec.qs_offset : 0) + at * BLK + QS_AT + khalf * 16;
#pragma unroll
        for (int p = 0; p < 4; ++p) cur[j].pair[p] = *reinterpret_cast<const u32x4*>(qs + p * 32);
        cur[j].hdr = load_hdr_q4k<BKIND>(wbase[j], a.spec, wrow[j], bpr, slice);
    };
    load_tile(std::integral_constant<int, 0>{});
    load_tile(std::integral_constant<int, 1>{});
    __builtin_amdgcn_sched_barrier(0);  // every request above is out before the first wait below

    // ---- stage the activation rows while the weight bytes travel
    uint8_t* const mine = lds + wv * kWaveLds;
    _Float16* const a_hi = reinterpret_cast<_Float16*>(mine);
    _Float16* const a_lo = a_hi + kRows * kSlice;
    _Float16* const sums = a_lo + kRows * kSlice;  // [row][8 hi, 8 lo] of (sub-block sum / 32)
    float biggest = 0;
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        if (nonfinite(v[r].x) || nonfinite(v[r].y) || nonfinite(v[r].z) || nonfinite(v[r].w)) bad = TSP_ERRBIT_NONFINITE;
        biggest = fmaxf(biggest, fmaxf(fmaxf(fabsf(v[r].x), fabsf(v[r].y)), fmaxf(fabsf(v[r].z), fabsf(v[r].w))));
    }
    biggest = wave_largest(biggest);
    // scale = 2^(13 - exponent(biggest)): the largest |x * scale| is below 2^15, the sub-block sums / 32 below 2^15 too
    float scale = 1.0f, inv_scale = 1.0f;
    if (biggest > 0 && !nonfinite(biggest)) {
        const int e = int((__float_as_uint(biggest) >> 23) & 0xffu) - 127;
        int shift = 13 - e;
        shift = shift > 100 ? 100 : shift < -100 ? -100 : shift;
        scale = __uint_as_float(uint32_t(127 + shift) << 23);
        inv_scale = __uint_as_float(uint32_t(127 - shift) << 23);
    }
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        if (uint32_t(r) >= task.count) continue;
        const float s4[4] = {v[r].x * scale, v[r].y * scale, v[r].z * scale, v[r].w * scale};
        f16x4 hi, lo;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            hi[e] = _Float16(s4[e]);
            lo[e] = _Float16(s4[e] - float(hi[e]));
        }
        // 16-byte chunk c = l / 2 of row r sits at position c ^ r; this lane owns half of it
        const uint32_t at = (r * 32 + ((lane / 2) ^ r)) * 8 + (lane % 2) * 4;
        *reinterpret_cast<f16x4*>(a_hi + at) = hi;
        *reinterpret_cast<f16x4*>(a_lo + at) = lo;
        float sum = (s4[0] + s4[1]) + (s4[2] + s4[3]);  // eight neighbouring lanes hold one 32-column sub-block
        sum = octet_sum(sum);
        if (lane % 8 == 0) {
            const float s32 = sum * 0.03125f;
            const _Float16 h = _Float16(s32);
            sums[r * 16 + lane / 8] = h;
            sums[r * 16 + 8 + lane / 8] = _Float16(s32 - float(h));
        }
    }
    // the planes are read back by other lanes of this same wave only: LDS serves a wave's requests in order
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    f32x16 blk[2];
    float acc[2][4] = {{0, 0, 0, 0}, {0, 0, 0, 0}};  // rows 4 * khalf + v of tile j
    const uint32_t arow = col & 7;
    auto a_frag = [&](const _Float16* plane, uint32_t chunk) {
        return *reinterpret_cast<const f16x8*>(plane + (arow * 32 + (chunk ^ arow)) * 8);
    };
    auto mfma = [&](uint32_t chunk, const f16x8& b0, const f16x8& b1, bool first) {
        const f16x8 ah = a_frag(a_hi, chunk), al = a_frag(a_lo, chunk);
        if (first) {
            const f32x16 zero{};
            blk[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, b0, zero, 0, 0, 0);
            blk[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, b1, zero, 0, 0, 0);
        } else {
            blk[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, b0, blk[0], 0, 0, 0);
            blk[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, b1, blk[1], 0, 0, 0);
        }
        blk[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, b0, blk[0], 0, 0, 0);
        blk[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, b1, blk[1], 0, 0, 0);
    };
    auto fold = [&](float d0, float d1) {
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) {
            acc[0][v4] = __builtin_fmaf(d0, blk[0][v4], acc[0][v4]);
            acc[1][v4] = __builtin_fmaf(d1, blk[1][v4], acc[1][v4]);
        }
    };
    auto pair_step = [&](auto p_tag) {
        constexpr int P = decltype(p_tag)::value;
        f16x8 f0[2], f1[2];
        const uint32_t chunk = P * 8 + khalf * 2;  // columns P*64 + 16h of the slice
        frags_q4k<P, 0>(cur[0].pair[P], cur[0].hdr, f0);
        frags_q4k<P, 0>(cur[1].pair[P], cur[1].hdr, f1);
        mfma(chunk, f0[0], f1[0], P == 0);
        mfma(chunk + 1, f0[1], f1[1], false);
        frags_q4k<P, 1>(cur[0].pair[P], cur[0].hdr, f0);
        frags_q4k<P, 1>(cur[1].pair[P], cur[1].hdr, f1);
        mfma(chunk + 4, f0[0], f1[0], false);
        mfma(chunk + 5, f0[1], f1[1], false);
    };
    pair_step(std::integral_constant<int, 0>{});
    pair_step(std::integral_constant<int, 1>{});
    pair_step(std::integral_constant<int, 2>{});
    pair_step(std::integral_constant<int, 3>{});
    fold(cur[0].hdr.d, cur[1].hdr.d);
    // minima: acc -= 32 * dmin * sum_s (Sx / 32)(hi + lo)[m, s] * mn[n, s]
    const f16x8 m0 = minima_frag(cur[0].hdr), m1 = minima_frag(cur[1].hdr);
    const f16x8 sf = *reinterpret_cast<const f16x8*>(sums + arow * 16 + khalf * 8);
    const f32x16 zero{};
    blk[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sf, m0, zero, 0, 0, 0);
    blk[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sf, m1, zero, 0, 0, 0);
    fold(-32.0f * cur[0].hdr.dmin, -32.0f * cur[1].hdr.dmin);
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) acc[j][v4] *= inv_scale;  // exact: a power of two

    // ---- the slices of a unit column meet in LDS, added in slice order; the planes are free once every wave is here
    if (bpr > 1) {
        float* const partial = reinterpret_cast<float*>(lds);  // [slice - 1][unit column][tile][v][lane]
        __syncthreads();
        if (slice > 0) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v4 = 0; v4 < 4; ++v4) partial[((((slice - 1) * ucols + ucol) * 2 + j) * 4 + v4) * kWave + lane] = acc[j][v4];
        }
        __syncthreads();
        if (slice > 0) { publish_error(bad, a.error_word); return; }
        for (uint32_t s = 1; s < bpr; ++s)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v4 = 0; v4 < 4; ++v4) acc[j][v4] += partial[((((s - 1) * ucols + ucol) * 2 + j) * 4 + v4) * kWave + lane];
    }
    // ---- epilogue: accumulator v of tile j is row 4 * khalf + v, weight row `col`
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
        const uint32_t r = 4 * khalf + v4;
        if (r >= task.count) continue;
        const uint32_t dst = khalf ? task.dst[4 + v4] : task.dst[v4];
        uint8_t* orow = reinterpret_cast<uint8_t*>(a.out) + uint64_t(dst) * a.out_stride;
        if constexpr (OUT == OUT_SWIGLU) {
            if (!col_live[0]) continue;
            const float g = acc[0][v4], u = acc[1][v4];
            const float sg = sigmoid_stable(g);
            const float h = (g * sg) * u;
            if (nonfinite(g) || nonfinite(u) || nonfinite(h)) bad = TSP_ERRBIT_NONFINITE;
            reinterpret_cast<float*>(orow)[out_col[0]] = h;
        } else {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if (!col_live[j]) continue;
                const float val = acc[j][v4];
                if (nonfinite(val)) bad = TSP_ERRBIT_NONFINITE;
                reinterpret_cast<float*>(orow)[out_col[j]] = val;
            }
        }
    }
    publish_error(bad, a.error_word);
}

// The same kernel for Q6_K planes on 16x16x32 MFMA tiles: sixteen operand rows hold the (at most eight) token rows with
// half the idle rows of the 32x32x16 tile, an instruction covers 32 columns, and a wave's 64 weight rows are four tiles
// of 16. Lane (n, kq) of a tile owns weight row n and a quarter of the super-block: section s = kq / 2 (128 columns) and
// the 16-byte half h = kq % 2 of each of its 32-byte groups, i.e. the same 16-byte pieces the 32x32x16 layout gives a
// lane, for one section instead of two. Eight instructions (times hi and lo) per tile and super-block, half the
// matrix-pipe time of the wider tile, and the result registers shrink from 16 to 4 per tile: the whole block fits the
// 128 registers of four waves per SIMD without spilling (the Q4_K form of this layout did not: its four headers and
// per-position scales cost more than the tile saves, 56 us against 37 for config 2's gate/up).
template <int BKIND, int OUT, int SRC>
__global__ __launch_bounds__(512, 4) void flat16_kernel(SkinnyArgs args) {  // four waves per SIMD: <= 128 registers per lane
    SkinnyArgs a = args;
    const bool shared = is_shared_task(a, blockIdx.y);
    if (shared) { a.x = a.shared_x; a.x_stride = a.shared_x_stride; a.out = a.shared_out; a.out_stride = a.shared_out_stride; }
    static_assert(BKIND == B_Q6K_PLANAR, "Q6_K planes only");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // [wave][hi plane][lo plane][sums]; partial sums over it at the end

    const uint32_t tid = threadIdx.x, lane = tid % kWave, wv = tid / kWave;
    const uint32_t n16 = lane % 16, kq = lane / 16, sec = kq / 2, half = kq % 2;
    const uint32_t bpr = a.k / 256, ucols = blockDim.x / kWave / bpr;  // the host launches ucols * bpr waves
    const uint32_t slice = wv % bpr, ucol = wv / bpr;
    Task task;
    if (!load_task<SRC>(a, blockIdx.y, task)) return;
    if (task.expert >= a.experts || task.count == 0 || task.count > kRows) {
        if (tid == 0 && blockIdx.x == 0 && (task.expert >= a.experts || task.count > kRows)) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
        return;
    }

    // ---- this wave's 256 columns of the activation rows (lane l: columns 4l .. 4l+3 of each row), requested first: loads
    // come back in the order they were asked for, and these few cached bytes must not queue behind the weight bytes
    uint32_t bad = 0;
    float4 v[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        // a record rarely fills its eight rows: the rows past its count are neither read nor staged. Their places in LDS keep
        // whatever was there; a token row of the product depends on its own operand row only, and those rows are never stored.
        v[r] = float4{0, 0, 0, 0};
        if (uint32_t(r) < task.count)  // uniform
            v[r] = *reinterpret_cast<const float4*>(reinterpret_cast<const uint8_t*>(a.x) + uint64_t(task.src[r]) * a.x_stride + (slice * kSlice + lane * 4) * 4);
    }

    // ---- weight rows of this wave (tiles 0, 1: gate units, tiles 2, 3: the same units of up; or 64 rows of down)
    const uint8_t* wbase[4];
    uint32_t wrow[4], out_col[4];
    bool col_live[4];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
        if constexpr (OUT == OUT_SWIGLU) {
            const uint32_t unit = (blockIdx.x * ucols + ucol) * 32 + (nt % 2) * 16 + n16;
            const uint32_t half_e = a.experts / 2;
            const uint8_t* pair = (task.expert < half_e ? a.w0 : a.w1) + uint64_t(task.expert < half_e ? task.expert : task.expert - half_e) * 2 * a.spec.planar_expert_bytes;
            wbase[nt] = nt < 2 ? (shared ? a.shared_w0 : pair) : (shared ? a.shared_w1 : pair + a.spec.planar_expert_bytes);
            col_live[nt] = unit < a.n;
            wrow[nt] = col_live[nt] ? unit : a.n - 1;
            out_col[nt] = unit;
        } else {
            const uint32_t n = (blockIdx.x * ucols + ucol) * 64 + nt * 16 + n16;
            col_live[nt] = n < a.n;
            wrow[nt] = col_live[nt] ? n : a.n - 1;
            out_col[nt] = n;
            wbase[nt] = shared ? a.shared_w0 : a.w0 + uint64_t(task.expert) * a.spec.planar_expert_bytes;
        }
    }
    struct Tile { RawQ6 raw; float d; };  // the lane's pieces of section sec
    Tile cur[4];
    auto load_tile = [&](auto nt_tag) {
        constexpr int nt = decltype(nt_tag)::value;
        const uint64_t at = uint64_t(wrow[nt]) * bpr + slice;
        const uint8_t* ql = wbase[nt] + a.spec.qs_offset + at * 128 + sec * 64 + half * 16;
        cur[nt].raw.la = *reinterpret_cast<const u32x4*>(ql);
        cur[nt].raw.lb = *reinterpret_cast<const u32x4*>(ql + 32);
        cur[nt].raw.qh = *reinterpret_cast<const u32x4*>(wbase[nt] + a.spec.qh_offset + at * 64 + sec * 32 + half * 16);
        const uint2 sc8 = *reinterpret_cast<const uint2*>(wbase[nt] + a.spec.sm_offset + at * 16 + sec * 8);
        cur[nt].raw.sc[0] = sc8.x; cur[nt].raw.sc[1] = sc8.y;
        cur[nt].d = half_bits_to_float(*reinterpret_cast<const uint16_t*>(wbase[nt] + a.spec.dm_offset + at * 2));
    };
    load_tile(std::integral_constant<int, 0>{});
    load_tile(std::integral_constant<int, 1>{});
    load_tile(std::integral_constant<int, 2>{});
    load_tile(std::integral_constant<int, 3>{});
    __builtin_amdgcn_sched_barrier(0);  // every request above is out before the first wait below

    // ---- stage the activation rows while the weight bytes travel
    uint8_t* const mine = lds + wv * kWaveLds;
    _Float16* const a_hi = reinterpret_cast<_Float16*>(mine);
    _Float16* const a_lo = a_hi + kRows * kSlice;
    float biggest = 0;
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        if (nonfinite(v[r].x) || nonfinite(v[r].y) || nonfinite(v[r].z) || nonfinite(v[r].w)) bad = TSP_ERRBIT_NONFINITE;
        biggest = fmaxf(biggest, fmaxf(fmaxf(fabsf(v[r].x), fabsf(v[r].y)), fmaxf(fabsf(v[r].z), fabsf(v[r].w))));
    }
    biggest = wave_largest(biggest);
    // scale = 2^(13 - exponent(biggest)): the largest |x * scale| is below 2^15, the sub-block sums / 32 below 2^15 too
    float scale = 1.0f, inv_scale = 1.0f;
    if (biggest > 0 && !nonfinite(biggest)) {
        const int e = int((__float_as_uint(biggest) >> 23) & 0xffu) - 127;
        int shift = 13 - e;
        shift = shift > 100 ? 100 : shift < -100 ? -100 : shift;
        scale = __uint_as_float(uint32_t(127 + shift) << 23);
        inv_scale = __uint_as_float(uint32_t(127 - shift) << 23);
    }
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        if (uint32_t(r) >= task.count) continue;
        const float s4[4] = {v[r].x * scale, v[r].y * scale, v[r].z * scale, v[r].w * scale};
        f16x4 hi, lo;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            hi[e] = _Float16(s4[e]);
            lo[e] = _Float16(s4[e] - float(hi[e]));
        }
        // 16-byte chunk c = l / 2 of row r sits at position c ^ r; this lane owns half of it
        const uint32_t at = (r * 32 + ((lane / 2) ^ r)) * 8 + (lane % 2) * 4;
        *reinterpret_cast<f16x4*>(a_hi + at) = hi;
        *reinterpret_cast<f16x4*>(a_lo + at) = lo;
    }
    // the planes are read back by other lanes of this same wave only: LDS serves a wave's requests in order
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // ---- one super-block: operand row lane % 16 is token row (lane % 16) % 8; result register v of a lane is token row 4 kq + v
    const uint32_t arow = n16 & 7;
    auto a_frag = [&](const _Float16* plane, uint32_t chunk) {
        return *reinterpret_cast<const f16x8*>(plane + (arow * 32 + (chunk ^ arow)) * 8);
    };
    f32x4 blk[4];
    // quarter Q of section sec: two 8-column fragments per tile (f = 0, 1) at chunk base + f
    auto quarter = [&](auto q_tag, bool first) {
        constexpr int Q = decltype(q_tag)::value;
        const uint32_t chunk = sec * 16 + Q * 4 + half * 2;  // columns sec*128 + Q*32 + 16 half (+ 8 f)
        const f16x8 ah0 = a_frag(a_hi, chunk), al0 = a_frag(a_lo, chunk), ah1 = a_frag(a_hi, chunk + 1), al1 = a_frag(a_lo, chunk + 1);
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) {
            f16x8 f[2];
            frags_q6k<Q>(cur[nt].raw, half, f);
            if (first) {
                const f32x4 zero{};
                blk[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah0, f[0], zero, 0, 0, 0);
            } else {
                blk[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah0, f[0], blk[nt], 0, 0, 0);
            }
            blk[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(al0, f[0], blk[nt], 0, 0, 0);
            blk[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah1, f[1], blk[nt], 0, 0, 0);
            blk[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(al1, f[1], blk[nt], 0, 0, 0);
        }
    };
    quarter(std::integral_constant<int, 0>{}, true);
    quarter(std::integral_constant<int, 1>{}, false);
    quarter(std::integral_constant<int, 2>{}, false);
    quarter(std::integral_constant<int, 3>{}, false);
    float acc[4][4];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) acc[nt][v4] = cur[nt].d * blk[nt][v4];
    }
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) acc[nt][v4] *= inv_scale;  // exact: a power of two

    // ---- the slices of a unit column meet in LDS, added in slice order; the planes are free once every wave is here
    if (bpr > 1) {
        float* const partial = reinterpret_cast<float*>(lds);  // [slice - 1][unit column][tile][v][lane]
        __syncthreads();
        if (slice > 0) {
#pragma unroll
            for (int nt = 0; nt < 4; ++nt)
#pragma unroll
                for (int v4 = 0; v4 < 4; ++v4) partial[((((slice - 1) * ucols + ucol) * 4 + nt) * 4 + v4) * kWave + lane] = acc[nt][v4];
        }
        __syncthreads();
        if (slice > 0) { publish_error(bad, a.error_word); return; }
        for (uint32_t s = 1; s < bpr; ++s)
#pragma unroll
            for (int nt = 0; nt < 4; ++nt)
#pragma unroll
                for (int v4 = 0; v4 < 4; ++v4) acc[nt][v4] += partial[((((s - 1) * ucols + ucol) * 4 + nt) * 4 + v4) * kWave + lane];
    }
    // ---- epilogue: register v of tile nt is token row 4 kq + v (lanes kq >= 2 hold repeats), weight row n16 of the tile
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
        const uint32_t r = 4 * kq + v4;
        if (kq >= 2 || r >= task.count) continue;
        const uint32_t dst = kq ? task.dst[4 + v4] : task.dst[v4];
        uint8_t* orow = reinterpret_cast<uint8_t*>(a.out) + uint64_t(dst) * a.out_stride;
        if constexpr (OUT == OUT_SWIGLU) {
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                if (!col_live[u]) continue;
                const float g = acc[u][v4], up = acc[2 + u][v4];
                const float sg = sigmoid_stable(g);
                const float h = (g * sg) * up;
                if (nonfinite(g) || nonfinite(up) || nonfinite(h)) bad = TSP_ERRBIT_NONFINITE;
                reinterpret_cast<float*>(orow)[out_col[u]] = h;
            }
        } else {
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) {
                if (!col_live[nt]) continue;
                const float val = acc[nt][v4];
                if (nonfinite(val)) bad = TSP_ERRBIT_NONFINITE;
                reinterpret_cast<float*>(orow)[out_col[nt]] = val;
            }
        }
    }
    publish_error(bad, a.error_word);
}

template <int BKIND, int OUT, int SRC>
int launch_flat(const char* name, const SkinnyArgs& a, uint32_t tasks, hipStream_t s) {
    const uint32_t bpr = a.k / 256, waves = bpr < 4 ? 4 : bpr, ucols = waves / bpr;
    const uint32_t per_group = ucols * (OUT == OUT_SWIGLU ? 32 : 64), col_tiles = (a.n + per_group - 1) / per_group;
    static std::atomic<uint64_t> raised{0};
    int device = 0;
    if (setup_pending(raised, &device)) {
        if constexpr (BKIND == B_Q6K_PLANAR)
            TSP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&flat16_kernel<BKIND, OUT, SRC>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        int(8 * kWaveLds)));
        else
            TSP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&flat_kernel<BKIND, OUT, SRC>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        int(8 * kWaveLds)));
        setup_done(raised, device);
    }
    if constexpr (BKIND == B_Q6K_PLANAR) TSP_LAUNCH(name, s, flat16_kernel<BKIND, OUT, SRC><<<dim3(col_tiles, tasks), waves * kWave, waves * kWaveLds, s>>>(a));
    else TSP_LAUNCH(name, s, flat_kernel<BKIND, OUT, SRC><<<dim3(col_tiles, tasks), waves * kWave, waves * kWaveLds, s>>>(a));
    return launch_status(name);
}

uint32_t lds_bytes(uint32_t columns, bool sums) { return 2 * kRows * columns * 2 + (sums ? kRows * (columns / 256) * 32 : 0); }

template <int BKIND, int OUT, int SRC, int KS>
int launch_sliced(const char* name, const SkinnyArgs& a, uint32_t col_tiles, uint32_t tasks, hipStream_t s) {
    const uint32_t bytes = lds_bytes(a.k, BKIND != B_Q6K_PLANAR);
    static std::atomic<uint64_t> raised{0};
    int device = 0;
    if (setup_pending(raised, &device)) {
        TSP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&skinny_kernel<BKIND, OUT, SRC, KS>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    int(lds_bytes(kMaxColumns, true))));
        setup_done(raised, device);
    }
    TSP_LAUNCH(name, s, skinny_kernel<BKIND, OUT, SRC, KS><<<dim3(col_tiles, tasks), 256 * KS, bytes, s>>>(a));
    return launch_status(name);
}

// Two K slices whenever the super-blocks split evenly: the task tiles of these products number about one per compute unit.
template <int BKIND, int OUT, int SRC>
int launch(const char* name, const SkinnyArgs& a, uint32_t col_tiles, uint32_t tasks, hipStream_t s) {
    const uint32_t bpr = a.k / 256;
    if (bpr == 1 || bpr == 2 || bpr == 4 || bpr == 8) return launch_flat<BKIND, OUT, SRC>(name, a, tasks, s);
    if ((a.k / 256) % 2 == 0) return launch_sliced<BKIND, OUT, SRC, 2>(name, a, col_tiles, tasks, s);
    return launch_sliced<BKIND, OUT, SRC, 1>(name, a, col_tiles, tasks, s);
}

bool aligned16(const void* p, uint64_t stride) { return reinterpret_cast<uintptr_t>(p) % 16 == 0 && stride % 16 == 0; }

}  // namespace

namespace tsp {

bool skinny_moe_supported(uint32_t gate_up_type, uint32_t down_type, uint32_t channels, uint32_t hidden, const void* x, uint64_t x_stride,
                          const void* h, uint64_t h_stride, bool with_down) {
    if (gate_up_type != 12 || channels % 256 || channels > kMaxColumns || !aligned16(x, x_stride)) return false;
    if (with_down && (down_type != 14 || hidden % 256 || hidden > kMaxColumns || !aligned16(h, h_stride))) return false;
    return true;
}

int skinny_moe_gate_up(const SkinnyMoe& m, hipStream_t s) {
    SkinnyArgs a{};
    a.x = m.x; a.x_stride = m.x_stride; a.w0 = m.pair_lo; a.w1 = m.pair_hi; a.spec = m.gu; a.experts = m.experts; a.selected = m.selected;
    a.tokens = m.tokens; a.ids = m.ids; a.meta = m.meta; a.n = m.hidden; a.k = m.channels; a.out = m.h; a.out_stride = m.h_stride;
    a.error_word = m.error_word;
    if (m.shared_gate) {
        a.shared_w0 = m.shared_gate; a.shared_w1 = m.shared_up; a.shared_x = m.x; a.shared_x_stride = m.x_stride;
        a.shared_out = m.shared_h; a.shared_out_stride = m.shared_h_stride; a.shared_index = m.records;
    }
    return launch<B_Q4K_PLANAR, OUT_SWIGLU, SRC_RECORD_TOKENS>("skinny_gate_up_swiglu", a, (m.hidden + 127) / 128, m.records + (m.shared_gate ? 1 : 0), s);
}

int skinny_moe_down(const SkinnyMoe& m, hipStream_t s) {
    SkinnyArgs a{};
    a.x = m.h; a.x_stride = m.h_stride; a.w0 = m.down; a.spec = m.dn; a.experts = m.experts; a.selected = m.selected;
    a.tokens = m.tokens; a.ids = m.ids; a.meta = m.meta; a.n = m.channels; a.k = m.hidden; a.out = m.y; a.out_stride = m.y_stride;
    a.error_word = m.error_word;
    if (m.shared_down) {
        a.shared_w0 = m.shared_down; a.shared_x = m.shared_h; a.shared_x_stride = m.shared_h_stride;
        a.shared_out = m.shared_y; a.shared_out_stride = m.shared_y_stride; a.shared_index = m.records;
    }
    return launch<B_Q6K_PLANAR, OUT_ROWS, SRC_RECORD_ROUTES>("skinny_down", a, (m.channels + 255) / 256, m.records + (m.shared_down ? 1 : 0), s);
}

}  // namespace tsp
