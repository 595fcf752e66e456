// Prefill dequant-GEMM on the matrix cores: out[m, n] = sum_k x[m, k] * dec(W[n, k]).
//
// Operands follow the engine's declared precision for this path: weights are dequantised in f32
// ((d*sc)*q - dmin*mn, d*sc*(q-32)) and rounded once to f16, activations are bf16 values carried
// as f16 (exact for every bf16 inside the f16 range), products accumulate in f32 inside
// v_mfma_f32_32x32x16_f16.
//
// One workgroup = 4 waves = one task (<= 128 activation rows of one expert, or one 128-row slab of a
// dense matrix) x 256 weight rows. Each wave owns 64 weight rows (two 32-wide MFMA column tiles) and
// all 128 activation rows (four row tiles): 8 accumulator tiles = 128 VGPRs.
//   * Weights never touch LDS: a lane loads the 8-byte nibble runs of ITS weight row straight into
//     the MFMA B-fragment layout (lane = (row % 32, k-half)), so every weight is dequantised exactly
//     once per task and there is no cross-wave traffic for B.
//   * Activations are shared by the four waves: staged global -> LDS (padded rows, conflict-free
//     16-byte reads), double buffered, one barrier per K step.
//   * For gate/up the two column tiles of a wave are the gate rows and the up rows of the same 32
//     hidden units, so SwiGLU is an element-wise epilogue on accumulator registers.
#include "decode.hpp"

using namespace tsp;

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

enum BKind : int { B_Q4K_RAW = 0, B_Q4K_PLANAR = 1, B_Q6K_PLANAR = 2 };
enum Epilogue : int { EPI_F32 = 0, EPI_BF16 = 1, EPI_SWIGLU = 2 };
enum Rows : int { ROWS_DENSE = 0, ROWS_GATHER_TOKENS = 1, ROWS_TASK_SLOTS = 2 };

constexpr int kTaskRows = 128;

struct GemmArgs {
    const _Float16* a;        // activation rows, a_stride halfs apart
    uint64_t a_stride;
    const uint8_t* w0;        // dense matrix / pair_lo / down experts
    const uint8_t* w1;        // pair_hi
    tsp_planar_spec spec;     // planar layouts (per expert); raw: columns/rows only
    uint32_t experts;
    const uint32_t* tasks;    // grouped: [2 + 2*bound] with 128-row tiles
    const uint32_t* counts;
    const uint32_t* token_map;
    const uint32_t* ids;
    uint32_t tokens, selected;
    uint32_t m, n, k;         // dense rows; weight rows (or hidden units for SwiGLU); columns
    void* out;
    uint64_t out_stride;      // bytes
    float out_scale;
    uint32_t* error_word;
};

__device__ __forceinline__ f16x2 pack2(float a, float b) {
    const f32x2 v = {a, b};
    return __builtin_convertvector(v, f16x2);  // RNE
}

__device__ __forceinline__ f16x8 pack8(const float* w) {
    const f16x2 p0 = pack2(w[0], w[1]), p1 = pack2(w[2], w[3]), p2 = pack2(w[4], w[5]), p3 = pack2(w[6], w[7]);
    return f16x8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
}

__device__ __forceinline__ float ubq(uint32_t w, int i) { return float((w >> (8 * i)) & 0xffu); }

// Eight weights dl*q - ml from the byte-wise codes of two dwords.
__device__ __forceinline__ f16x8 affine8(uint32_t c0, uint32_t c1, float dl, float neg_ml) {
    float w[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) { w[i] = __builtin_fmaf(ubq(c0, i), dl, neg_ml); w[4 + i] = __builtin_fmaf(ubq(c1, i), dl, neg_ml); }
    return pack8(w);
}

// ---------------------------------------------------------------- B fragments, one K step, one weight row
// Q4_K: K step = 64 (one nibble pair = sub-blocks 2p and 2p+1); four k16 fragments.
template <int BKIND>
__device__ __forceinline__ void load_b_q4k(const uint8_t* base, const tsp_planar_spec& s, uint64_t row, uint32_t bpr, uint32_t step,
                                           uint32_t khalf, uint2& lo8, uint2& hi8, float& dl_a, float& nml_a, float& dl_b, float& nml_b) {
    const uint32_t b = step / 4, p = step % 4;
    const uint64_t blk = row * bpr + b;
    float d, dmin;
    uint32_t sc_a, sc_b, mn_a, mn_b;
    if constexpr (BKIND == B_Q4K_PLANAR) {
        const uint8_t* qs = base + s.qs_offset + blk * 128 + p * 32 + khalf * 8;
        lo8 = *reinterpret_cast<const uint2*>(qs);
        hi8 = *reinterpret_cast<const uint2*>(qs + 16);
        const uint8_t* sm = base + s.sm_offset + blk * 16 + p * 2;
        const uint32_t sc = *reinterpret_cast<const uint16_t*>(sm), mn = *reinterpret_cast<const uint16_t*>(sm + 8);
        const uint32_t dm = *reinterpret_cast<const uint32_t*>(base + s.dm_offset + blk * 4);
        sc_a = sc & 0xffu; sc_b = sc >> 8; mn_a = mn & 0xffu; mn_b = mn >> 8;
        d = half_bits_to_float(dm & 0xffffu); dmin = half_bits_to_float(dm >> 16);
    } else {
        const uint8_t* block = base + blk * 144;
        const uint4 hdr = *reinterpret_cast<const uint4*>(block);
        lo8 = *reinterpret_cast<const uint2*>(block + 16 + p * 32 + khalf * 8);
        hi8 = *reinterpret_cast<const uint2*>(block + 32 + p * 32 + khalf * 8);
        d = half_bits_to_float(hdr.x & 0xffffu); dmin = half_bits_to_float(hdr.x >> 16);
        const uint32_t sh = (p & 1u) * 16u;
        const uint32_t s2 = (hdr.y >> sh) & 0xffffu, m2 = (hdr.z >> sh) & 0xffffu, e2 = (hdr.w >> sh) & 0xffffu;
        if (p < 2) {
            sc_a = s2 & 63u; sc_b = (s2 >> 8) & 63u; mn_a = m2 & 63u; mn_b = (m2 >> 8) & 63u;
        } else {
            sc_a = (e2 & 15u) | (((s2 >> 6) & 3u) << 4);
            sc_b = ((e2 >> 8) & 15u) | (((s2 >> 14) & 3u) << 4);
            mn_a = ((e2 >> 4) & 15u) | (((m2 >> 6) & 3u) << 4);
            mn_b = ((e2 >> 12) & 15u) | (((m2 >> 14) & 3u) << 4);
        }
    }
    dl_a = d * float(sc_a); dl_b = d * float(sc_b);
    nml_a = -(dmin * float(mn_a)); nml_b = -(dmin * float(mn_b));
}

__device__ __forceinline__ void frags_q4k(uint2 lo8, uint2 hi8, float dl_a, float nml_a, float dl_b, float nml_b, f16x8 frag[4]) {
    constexpr uint32_t M4 = 0x0f0f0f0fu;
    frag[0] = affine8(lo8.x & M4, lo8.y & M4, dl_a, nml_a);
    frag[1] = affine8(hi8.x & M4, hi8.y & M4, dl_a, nml_a);
    frag[2] = affine8((lo8.x >> 4) & M4, (lo8.y >> 4) & M4, dl_b, nml_b);
    frag[3] = affine8((hi8.x >> 4) & M4, (hi8.y >> 4) & M4, dl_b, nml_b);
}

// Q6_K planes: K step = 128 (one section); eight k16 fragments. For k16 step s the eight weights of a
// lane are elements q*32 + j .. +7 of the section with q = s/2, j = (s%2)*16 + khalf*8.
struct RawQ6 { uint2 la[2], lb[2], qh[2]; float d; const uint8_t* sc; };

__device__ __forceinline__ void load_b_q6k(const uint8_t* base, const tsp_planar_spec& s, uint64_t row, uint32_t bpr, uint32_t step,
                                           uint32_t khalf, RawQ6& r) {
    const uint32_t b = step / 2, sec = step % 2;
    const uint64_t blk = row * bpr + b;
#pragma unroll
    for (int par = 0; par < 2; ++par) {
        const uint32_t j = par * 16 + khalf * 8;
        const uint8_t* ql = base + s.qs_offset + blk * 128 + sec * 64 + j;
        r.la[par] = *reinterpret_cast<const uint2*>(ql);
        r.lb[par] = *reinterpret_cast<const uint2*>(ql + 32);
        r.qh[par] = *reinterpret_cast<const uint2*>(base + s.qh_offset + blk * 64 + sec * 32 + j);
    }
    r.d = half_bits_to_float(*reinterpret_cast<const uint16_t*>(base + s.dm_offset + blk * 2));
    r.sc = base + s.sm_offset + blk * 16 + sec * 8;
}

__device__ __forceinline__ void frags_q6k(const RawQ6& r, f16x8 frag[8]) {
    constexpr uint32_t M4 = 0x0f0f0f0fu, M2 = 0x30303030u;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int par = 0; par < 2; ++par) {
            const uint2 l = (q & 1) ? r.lb[par] : r.la[par];
            const uint2 h = r.qh[par];
            uint32_t c0, c1;
            if (q < 2) { c0 = l.x & M4; c1 = l.y & M4; } else { c0 = (l.x >> 4) & M4; c1 = (l.y >> 4) & M4; }
            const int shift = 4 - 2 * q;  // bits 2q..2q+1 of qh move to bits 4..5
            c0 |= (shift >= 0 ? h.x << shift : h.x >> -shift) & M2;
            c1 |= (shift >= 0 ? h.y << shift : h.y >> -shift) & M2;
            // sub-scale of the 16-weight group: element / 16 = q*2 + par within the section
            const float ds = r.d * float(int(int8_t(r.sc[q * 2 + par])));
            frag[q * 2 + par] = affine8(c0, c1, ds, -32.0f * ds);
        }
    }
}

// ---------------------------------------------------------------- the kernel
template <int BKIND, int EPI, int ROWS>
__global__ __launch_bounds__(256) void gemm_kernel(GemmArgs a) {
    constexpr int KSTEP = BKIND == B_Q6K_PLANAR ? 128 : 64;
    constexpr int NFRAG = KSTEP / 16;
    constexpr int LDA = KSTEP + 8;  // halfs per staged row: 16 bytes of padding keeps 16-byte reads conflict free
    __shared__ __attribute__((aligned(16))) _Float16 lds_a[2][kTaskRows * LDA];
    __shared__ uint32_t row_src[kTaskRows];
    __shared__ uint32_t row_dst[kTaskRows];
    __shared__ uint32_t task_bad;

    const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const uint32_t col = lane % 32, khalf = lane / 32;
    const uint32_t task = blockIdx.y;

    // ---- task resolution
    uint32_t expert = 0, nrows = 0;
    if (tid == 0) task_bad = 0;
    __syncthreads();
    if constexpr (ROWS == ROWS_DENSE) {
        const uint32_t row0 = task * kTaskRows;
        if (row0 >= a.m) return;
        nrows = a.m - row0 < kTaskRows ? a.m - row0 : kTaskRows;
        if (tid < kTaskRows) { row_src[tid] = row0 + tid; row_dst[tid] = row0 + tid; }
    } else {
        const uint32_t bound = a.tokens * a.selected / kTaskRows + a.experts;
        const uint32_t live = a.tasks[0];
        if (live > bound || a.tasks[1] != a.tokens * a.selected) {
            if (tid == 0 && blockIdx.x == 0 && task == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
            return;
        }
        if (task >= live) return;
        expert = a.tasks[2 + 2 * task];
        const uint32_t start = a.tasks[3 + 2 * task];
        const uint32_t count = expert < a.experts ? a.counts[expert] : 0;
        if (expert >= a.experts || count > a.tokens || start >= count) {
            if (tid == 0 && blockIdx.x == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
            return;
        }
        nrows = count - start < kTaskRows ? count - start : kTaskRows;
        if (tid < kTaskRows) {
            uint32_t rid = 0xffffffffu;
            if (tid < nrows) {
                rid = a.token_map[uint64_t(expert) * a.tokens + start + tid];
                if (rid >= a.tokens * a.selected || a.ids[rid] != expert) { rid = 0xffffffffu; task_bad = 1; }
            }
            row_src[tid] = ROWS == ROWS_GATHER_TOKENS ? (rid == 0xffffffffu ? 0xffffffffu : rid / a.selected) : task * kTaskRows + tid;
            row_dst[tid] = ROWS == ROWS_GATHER_TOKENS ? task * kTaskRows + tid : rid;
        }
    }
    __syncthreads();
    if (task_bad && tid == 0 && blockIdx.x == 0) atomicOr(a.error_word, TSP_ERRBIT_INDEX);
    const int mt_live = (nrows + 31) / 32;

    // ---- weight rows of this wave
    const uint8_t* wbase[2];
    uint64_t wrow[2];
    uint32_t out_col[2];
    bool col_live[2];
    if constexpr (EPI == EPI_SWIGLU) {
        const uint32_t unit = blockIdx.x * 128 + wave * 32 + col;
        const uint32_t half_e = a.experts / 2;
        const uint8_t* pair = (expert < half_e ? a.w0 : a.w1) + uint64_t(expert < half_e ? expert : expert - half_e) * 2 * a.spec.planar_expert_bytes;
        wbase[0] = pair; wbase[1] = pair + a.spec.planar_expert_bytes;
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
            wbase[j] = BKIND == B_Q4K_RAW ? a.w0 : a.w0 + uint64_t(expert) * a.spec.planar_expert_bytes;
        }
    }
    const uint32_t bpr = a.k / 256;
    const uint32_t ksteps = a.k / KSTEP;

    f32x16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // ---- activation staging: thread t copies (KSTEP*2/2) bytes of row t/2
    constexpr int SEG = KSTEP / 2;  // halfs per thread per step
    const uint32_t st_row = tid / 2, st_seg = tid % 2;
    const uint32_t src_row = row_src[st_row];
    const bool st_live = st_row < nrows && src_row != 0xffffffffu;
    const _Float16* st_src = a.a + uint64_t(st_live ? src_row : 0) * a.a_stride + st_seg * SEG;
    uint4 stage[SEG / 8];
    auto fetch_a = [&](uint32_t step) {
#pragma unroll
        for (int i = 0; i < SEG / 8; ++i)
            stage[i] = st_live ? *reinterpret_cast<const uint4*>(st_src + uint64_t(step) * KSTEP + i * 8) : uint4{0, 0, 0, 0};
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int i = 0; i < SEG / 8; ++i) *reinterpret_cast<uint4*>(&lds_a[buf][st_row * LDA + st_seg * SEG + i * 8]) = stage[i];
    };

    fetch_a(0);
    store_a(0);
    for (uint32_t step = 0; step < ksteps; ++step) {
        const int buf = step & 1;
        if (step + 1 < ksteps) fetch_a(step + 1);
        f16x8 bfrag[2][NFRAG];
        if constexpr (BKIND == B_Q6K_PLANAR) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                RawQ6 raw;
                load_b_q6k(wbase[j], a.spec, wrow[j], bpr, step, khalf, raw);
                frags_q6k(raw, bfrag[j]);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                uint2 lo8, hi8;
                float dl_a, nml_a, dl_b, nml_b;
                load_b_q4k<BKIND>(wbase[j], a.spec, wrow[j], bpr, step, khalf, lo8, hi8, dl_a, nml_a, dl_b, nml_b);
                frags_q4k(lo8, hi8, dl_a, nml_a, dl_b, nml_b, bfrag[j]);
            }
        }
        __syncthreads();  // lds_a[buf] is complete; every wave has left lds_a[buf ^ 1]
#pragma unroll
        for (int f = 0; f < NFRAG; ++f) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (i < mt_live) {
                    const f16x8 afrag = *reinterpret_cast<const f16x8*>(&lds_a[buf][(i * 32 + col) * LDA + f * 16 + khalf * 8]);
                    acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afrag, bfrag[0][f], acc[i][0], 0, 0, 0);
                    acc[i][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afrag, bfrag[1][f], acc[i][1], 0, 0, 0);
                }
            }
        }
        if (step + 1 < ksteps) store_a(buf ^ 1);
    }

    // ---- epilogue. Accumulator v of tile (i, j): row = i*32 + 8*(v/4) + 4*khalf + v%4, column = col.
    uint32_t bad = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
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
                const float sg = g >= 0 ? 1.0f / (1.0f + expf(-g)) : expf(g) / (1.0f + expf(g));
                const float h = (g * sg) * u;
                // h is carried between the two GEMMs as bf16 (RNE) and fed to the f16 matrix core as h * 2^-8
                const uint32_t hb = __float_as_uint(h);
                const uint32_t rounded = (hb + 0x7fffu + ((hb >> 16) & 1u)) & 0xffff0000u;
                if (nonfinite(g) || nonfinite(u) || nonfinite(h) || (rounded & 0x7f800000u) == 0x7f800000u) bad = TSP_ERRBIT_NONFINITE;
                reinterpret_cast<_Float16*>(a.out)[uint64_t(dst) * a.n + out_col[0]] = _Float16(__uint_as_float(rounded) * 0.00390625f);
            } else {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    if (!col_live[j]) continue;
                    const float val = acc[i][j][v] * a.out_scale;
                    if (nonfinite(val)) bad = TSP_ERRBIT_NONFINITE;
                    uint8_t* orow = static_cast<uint8_t*>(a.out) + uint64_t(dst) * a.out_stride;
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

// f32 rows -> bf16 (RNE) -> f16, or bf16 rows -> f16. Values outside the f16 range are flagged.
template <bool FROM_BF16>
__global__ __launch_bounds__(256) void to_f16_rows(const void* __restrict__ src, uint64_t src_stride_bytes, _Float16* __restrict__ dst,
                                                   uint32_t rows, uint32_t columns, uint32_t* error_word) {
    uint32_t bad = 0;
    const uint64_t total = uint64_t(rows) * columns;
    for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < total; i += uint64_t(gridDim.x) * blockDim.x) {
        const uint64_t r = i / columns, c = i % columns;
        const uint8_t* row = static_cast<const uint8_t*>(src) + r * src_stride_bytes;
        uint32_t bits;
        if constexpr (FROM_BF16) {
            bits = uint32_t(reinterpret_cast<const uint16_t*>(row)[c]) << 16;
        } else {
            const uint32_t fb = __float_as_uint(reinterpret_cast<const float*>(row)[c]);
            bits = (fb + 0x7fffu + ((fb >> 16) & 1u)) & 0xffff0000u;
            if ((fb & 0x7f800000u) == 0x7f800000u) bits = fb;
        }
        const _Float16 h = _Float16(__uint_as_float(bits));
        if ((bits & 0x7f800000u) == 0x7f800000u || (__builtin_bit_cast(uint16_t, h) & 0x7c00u) == 0x7c00u) bad = TSP_ERRBIT_NONFINITE;
        dst[i] = h;
    }
    publish_error(bad, error_word);
}

template <int BKIND, int EPI, int ROWS>
int launch(const GemmArgs& a, uint32_t col_tiles, uint32_t tasks, hipStream_t s) {
    constexpr const char* name = EPI == EPI_SWIGLU ? "gemm_gate_up_swiglu" : ROWS == ROWS_TASK_SLOTS ? "gemm_down" : "gemm_dense";
    TSP_LAUNCH(name, s, gemm_kernel<BKIND, EPI, ROWS><<<dim3(col_tiles, tasks), 256, 0, s>>>(a));
    return launch_status("dequant_gemm");
}

int convert_rows(const void* src, uint64_t stride, int from_bf16, _Float16* dst, uint32_t rows, uint32_t columns, uint32_t* err, hipStream_t s) {
    const uint64_t total = uint64_t(rows) * columns;
    const uint32_t grid = uint32_t((total + 255) / 256 > 8192 ? 8192 : (total + 255) / 256);
    if (from_bf16) TSP_LAUNCH("to_f16_rows", s, to_f16_rows<true><<<grid, 256, 0, s>>>(src, stride, dst, rows, columns, err));
    else TSP_LAUNCH("to_f16_rows", s, to_f16_rows<false><<<grid, 256, 0, s>>>(src, stride, dst, rows, columns, err));
    return launch_status("to_f16_rows");
}

uint64_t align256(uint64_t v) { return (v + 255) / 256 * 256; }

}  // namespace

extern "C" uint64_t tsp_dense_mm_workspace_bytes(uint32_t tokens, uint32_t columns) { return align256(uint64_t(tokens) * columns * 2); }

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
    const uint64_t in_span = uint64_t(tokens - 1) * input_stride_bytes + uint64_t(columns) * in_elem;
    const uint64_t out_span = uint64_t(tokens - 1) * output_stride_bytes + uint64_t(rows) * out_elem;
    TSP_REQUIRE(!ranges_overlap(output, out_span, matrix, matrix_bytes) && !ranges_overlap(output, out_span, input, in_span) &&
                    !ranges_overlap(output, out_span, workspace, workspace_bytes) &&
                    !ranges_overlap(workspace, workspace_bytes, matrix, matrix_bytes) && !ranges_overlap(workspace, workspace_bytes, input, in_span),
                "dense dequant-GEMM buffers overlap");
    const auto s = static_cast<hipStream_t>(stream);
    auto* xh = static_cast<_Float16*>(workspace);
    int rc = convert_rows(input, input_stride_bytes, input_is_bf16, xh, tokens, columns, error_word, s);
    if (rc != TSP_OK) return rc;
    a.a = xh; a.a_stride = columns; a.w0 = static_cast<const uint8_t*>(matrix); a.experts = 1;
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

// ---------------------------------------------------------------- grouped MoE
namespace {
struct NaxLayout { uint64_t xh, tasks128, hbuf, total; uint32_t bound128; };
NaxLayout nax_layout(uint32_t tokens, uint32_t selected, uint32_t experts, uint32_t channels, uint32_t hidden) {
    NaxLayout l{};
    l.bound128 = tokens * selected / kTaskRows + experts;
    l.xh = 0;
    l.tasks128 = align256(uint64_t(tokens) * channels * 2);
    l.hbuf = l.tasks128 + align256((2 + 2 * uint64_t(l.bound128)) * 4);
    l.total = l.hbuf + align256(uint64_t(l.bound128) * kTaskRows * hidden * 2);
    return l;
}
}  // namespace

extern "C" uint64_t tsp_planar_nax_workspace_bytes(uint32_t tokens, uint32_t selected, uint32_t experts, uint32_t channels, uint32_t hidden) {
    return nax_layout(tokens, selected, experts, channels, hidden).total;
}

extern "C" int tsp_planar_nax_grouped_moe(const tsp_grouped_moe* m, void* stream) {
    TSP_REQUIRE(m, "null grouped MoE description");
    TSP_REQUIRE(m->gate_kind == TSP_KIND_Q4K_COLOC_GATE && m->up_kind == TSP_KIND_Q4K_COLOC_UP && m->down_kind == TSP_KIND_Q6K_PLANAR_X,
                "planar v3 grouped MoE on the matrix cores takes Q4_K co-located gate/up and Q6_K planes for down");
    TSP_REQUIRE(m->tokens >= 1 && m->tokens <= 2048 && m->selected >= 1 && m->selected <= 16 && m->selected <= m->experts &&
                    m->experts >= 2 && m->experts <= 512 && m->experts % 2 == 0 && m->channels % 256 == 0 && m->hidden % 256 == 0 &&
                    m->channels <= 65536 && m->hidden <= 65536,
                "planar v3 NAX grouped MoE shape or stride mismatch");
    TSP_REQUIRE(m->x_stride_bytes >= uint64_t(m->channels) * 4 && m->x_stride_bytes % 4 == 0 &&
                    m->y_stride_bytes >= uint64_t(m->channels) * 4 && m->y_stride_bytes % 4 == 0,
                "planar v3 NAX grouped MoE shape or stride mismatch");
    TSP_REQUIRE(m->pair_lo && m->pair_hi && m->down && m->ids && m->x && m->y && m->token_map && m->counts && m->tasks &&
                    m->workspace && m->error_word,
                "null device pointer");
    tsp_planar_spec gu, dn;
    int rc = tsp_make_expert_spec(12, m->channels, m->hidden, &gu);
    if (rc == TSP_OK) rc = tsp_make_expert_spec(14, m->hidden, m->channels, &dn);
    if (rc != TSP_OK) return rc;
    const NaxLayout l = nax_layout(m->tokens, m->selected, m->experts, m->channels, m->hidden);
    TSP_REQUIRE(m->workspace_bytes >= l.total, "planar v3 NAX scratch too small for requested batch");
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
    auto* tasks128 = reinterpret_cast<uint32_t*>(ws + l.tasks128);
    auto* hbuf = reinterpret_cast<_Float16*>(ws + l.hbuf);

    rc = tsp_grouped_routes(m->ids, m->token_map, m->counts, m->experts, m->selected, m->tokens, m->error_word, stream);
    if (rc == TSP_OK) rc = tsp_grouped_tasks(m->counts, m->tasks, m->experts, m->selected, m->tokens, 32, m->error_word, stream);
    if (rc == TSP_OK) rc = tsp_grouped_tasks(m->counts, tasks128, m->experts, m->selected, m->tokens, kTaskRows, m->error_word, stream);
    if (rc == TSP_OK) rc = convert_rows(m->x, m->x_stride_bytes, 0, xh, m->tokens, m->channels, m->error_word, s);
    if (rc != TSP_OK) return rc;

    GemmArgs g{};
    g.a = xh; g.a_stride = m->channels; g.w0 = static_cast<const uint8_t*>(m->pair_lo); g.w1 = static_cast<const uint8_t*>(m->pair_hi);
    g.spec = gu; g.experts = m->experts; g.tasks = tasks128; g.counts = m->counts; g.token_map = m->token_map; g.ids = m->ids;
    g.tokens = m->tokens; g.selected = m->selected; g.n = m->hidden; g.k = m->channels; g.out = hbuf; g.out_scale = 1.0f;
    g.error_word = m->error_word;
    rc = launch<B_Q4K_PLANAR, EPI_SWIGLU, ROWS_GATHER_TOKENS>(g, (m->hidden + 127) / 128, l.bound128, s);
    if (rc != TSP_OK) return rc;

    GemmArgs d{};
    d.a = hbuf; d.a_stride = m->hidden; d.w0 = static_cast<const uint8_t*>(m->down); d.spec = dn; d.experts = m->experts;
    d.tasks = tasks128; d.counts = m->counts; d.token_map = m->token_map; d.ids = m->ids; d.tokens = m->tokens; d.selected = m->selected;
    d.n = m->channels; d.k = m->hidden; d.out = m->y; d.out_stride = m->y_stride_bytes; d.out_scale = 256.0f;  // undo the 2^-8 carried by h
    d.error_word = m->error_word;
    return launch<B_Q6K_PLANAR, EPI_F32, ROWS_TASK_SLOTS>(d, (m->channels + 255) / 256, l.bound128, s);
}
