// Dense Q4_K dequant-GEMM for few activation rows (include/tokspur/graph.hpp:753 `grouped_mm` with one expert; the prefill
// product of a short chunk): raw GGUF rows, out[m, n] = sum_k x[m, k] * w[n, k] for fewer rows than the many-row kernel takes.
//
// With 64-row tiles a product of 128 rows x 8192 weight rows has 64 workgroup tiles of 64 x 256 for 256 compute units, and
// each of them walks all of K alone. Here a workgroup owns a 64 x 64 output tile (256 of them at that shape) and its waves
// split K: wave w takes super-block w (256 columns) of the tile's 64 activation rows and 64 weight rows, everything it needs
// is requested at once (no loop: one round trip to memory), the waves' partial tiles meet in LDS and are added up in wave
// order, the order of a sequential pass over K. The activation rows are asked for the cheap way, as whole 512-byte row
// pieces (a request = two rows), and turned into MFMA fragments through the wave's own part of LDS: a lane fetching the
// sixteen columns of its own row instead touches 32 lines per request where this touches 8, and the address unit, not
// memory, then sets the pace (18 us against 14 at 128 rows x 8192 weight rows). The arithmetic is the integer-factor scheme of the other Q4_K matrix-core
// kernels: the products sc * q as exact halves against the activations (bf16 values carried as halves), d applied in f32 per
// super-block, the minima as one more MFMA against the activations' sub-block sums.
#include "dense_ksplit.hpp"
#include "mfma_quant.hpp"

#include <type_traits>

using namespace tsp;

namespace {

constexpr int kTile = 64;                    // activation rows and weight rows of a workgroup's tile
constexpr int kQuarterBytes = 4096;          // a wave's 32 x 32 f32 partial of one quarter of the tile
constexpr int kWaveBytes = 4 * kQuarterBytes;

template <int WAVES>
__global__ __launch_bounds__(WAVES * kWave) void dense_ksplit_kernel(DenseKsplitArgs a) {
    __shared__ __attribute__((aligned(16))) uint8_t partials[WAVES * kWaveBytes];  // [wave][weight-row half j][activation-row half i][32 x 32 f32]
    const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const uint32_t n = lane % 32, khalf = lane / 32;
    constexpr uint32_t bpr = WAVES;  // super-blocks per row = waves
    const uint32_t n0 = blockIdx.x * kTile, m0 = blockIdx.y * kTile;

    // ---- everything the wave multiplies, requested at once: its super-block of the tile's activation rows (a row past the
    // end repeats the last row and is never stored) and of the tile's weight rows (the same for a row past the matrix)
    f16x8 A[2][16], sxA[2];
    u32x4 piece[2][16];  // request q of row tile i: the 512 bytes of rows 2q and 2q + 1 of the tile, lane l chunk l % 32 of row 2q + l / 32
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const uint32_t r = m0 + i * 32 + 2 * q + khalf < a.m ? m0 + i * 32 + 2 * q + khalf : a.m - 1;
            piece[i][q] = *reinterpret_cast<const u32x4*>(a.a + uint64_t(r) * a.k + wave * 256 + n * 8);
        }
        const uint32_t r = m0 + i * 32 + n < a.m ? m0 + i * 32 + n : a.m - 1;
        sxA[i] = *reinterpret_cast<const f16x8*>(a.sx + (uint64_t(r) * bpr + wave) * 16 + khalf * 8);
    }
    u32x4 raw[2][4];
    uint4 header[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t c = n0 + j * 32 + n < a.n ? n0 + j * 32 + n : a.n - 1;
        const uint8_t* block = a.w + (uint64_t(c) * bpr + wave) * 144;
        header[j] = *reinterpret_cast<const uint4*>(block);
#pragma unroll
        for (int p = 0; p < 4; ++p) raw[j][p] = *reinterpret_cast<const u32x4*>(block + 16 + p * 32 + khalf * 16);
    }
    const Q4Consts q4c = q4_consts();
    const Q4ScaleConsts q4s = q4_scale_consts();

    // ---- rows to fragments through the wave's own 16 KB (its partial tile's place later on): 32 rows of 512 bytes, chunk c of
    // row r at position c ^ (r % 16), so that sixteen lanes writing a row's chunks or reading one chunk of sixteen rows touch
    // every bank once. LDS serves a wave's requests in order: the second tile's writes come after the first tile's reads.
    uint8_t* const turn = partials + wave * kWaveBytes;
    auto to_fragments = [&](auto i_tag) {
        constexpr int i = decltype(i_tag)::value;
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const uint32_t r = 2 * q + khalf;
            *reinterpret_cast<u32x4*>(turn + r * 512 + ((n ^ (r % 16)) * 16)) = piece[i][q];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            // fragment t: the eight columns at khalf * 16 + (t / 4) * 64 + ((t / 2) % 2) * 32 + (t % 2) * 8 of the lane's row: one chunk
            const uint32_t c = khalf * 2 + (t / 4) * 8 + ((t / 2) % 2) * 4 + (t % 2);
            A[i][t] = *reinterpret_cast<const f16x8*>(turn + n * 512 + ((c ^ (n % 16)) * 16));
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    to_fragments(std::integral_constant<int, 0>{});
    to_fragments(std::integral_constant<int, 1>{});

    // ---- the wave's partial tile, a quarter at a time: weight rows j * 32 .. + 31 against activation rows i * 32 .. + 31
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const HdrQ4 hdr = decode_hdr_q4k<B_Q4K_RAW>(RawHdrQ4{header[j], 0});
        float d = hdr.d, dmin = hdr.dmin;
        asm volatile("" : "+v"(d), "+v"(dmin));  // as floats in registers: folded in as halves they make every multiply-add a mixed-precision one
        f32x16 blk[2];
        auto steps = [&](auto p_tag) {
            constexpr int P = decltype(p_tag)::value;
            const Q4PairScale sc = q4_pair_scale<P>(hdr.sc[0], hdr.sc[1], q4s);  // sub-blocks 2P (low nibbles) and 2P + 1 (high nibbles)
#pragma unroll
            for (int hi = 0; hi < 2; ++hi) {
                f16x8 f[2];
                frags_q4k_pair(raw[j][P], sc, hi, q4c, f);
#pragma unroll
                for (int ff = 0; ff < 2; ++ff)
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
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
        const f16x8 mn = minima_frag(hdr);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            // partial = d * sum(x * sc * q) - dmin * sum_s Sx(hi + lo)[m, s] * mn[n, s]
            const f32x16 zero{};
            const f32x16 mblk = __builtin_amdgcn_mfma_f32_32x32x16_f16(sxA[i], mn, zero, 0, 0, 0);
            uint8_t* out = partials + wave * kWaveBytes + (j * 2 + i) * kQuarterBytes + lane * 16;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                f32x4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaf(-dmin, mblk[4 * c + e], d * blk[i][4 * c + e]);
                *reinterpret_cast<f32x4*>(out + c * 1024) = v;
            }
        }
    }
    __syncthreads();

    // ---- the super-blocks' partials added up in order. Float f of a quarter is accumulator 4 (f / 256) + f % 4 of fragment
    // lane (f % 256) / 4: activation row 8 (f / 256) + 4 (lane / 32) + f % 4, weight row lane % 32 of the quarter.
    uint32_t bad = 0;
    for (uint32_t pair = tid; pair < 4 * 512; pair += WAVES * kWave) {  // a pair of neighbouring floats: the same weight row, two rows
        const uint32_t quarter = pair / 512, f = (pair % 512) * 2, j = quarter / 2, i = quarter % 2;
        const uint8_t* in = partials + quarter * kQuarterBytes + f * 4;
        float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float2 p2 = *reinterpret_cast<const float2*>(in + w * kWaveBytes);
            s0 += p2.x; s1 += p2.y;
        }
        const uint32_t from = (f % 256) / 4, col = n0 + j * 32 + from % 32;
        const uint32_t row = m0 + i * 32 + 8 * (f / 256) + 4 * (from / 32) + f % 4;
        if (col >= a.n) continue;
        const float sums[2] = {s0, s1};
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            if (row + e >= a.m) continue;
            const float val = sums[e];
            if (nonfinite(val)) bad = TSP_ERRBIT_NONFINITE;
            uint8_t* orow = static_cast<uint8_t*>(a.out) + uint64_t(row + e) * a.out_stride;
            if (a.out_bf16) {
                const uint32_t vb = __float_as_uint(val);
                reinterpret_cast<uint16_t*>(orow)[col] = uint16_t((vb + 0x7fffu + ((vb >> 16) & 1u)) >> 16);
            } else {
                reinterpret_cast<float*>(orow)[col] = val;
            }
        }
    }
    publish_error(bad, a.error_word);
}

}  // namespace

namespace tsp {

// Up to 384 rows: a round of tiles takes about 10 us whatever the rows (8192 weight rows: 128 tiles per 64 activation rows, so
// two rounds fill 256 compute units), and from 385 rows on the 64 x 256 tiles of the general kernel are the faster ones
// (measured at 2048 x 8192: 14 against 34 us at 128 rows, 25 against 36 at 256, 34.5 against 38 at 384, 42.5 against 39.6 at 448).
bool dense_ksplit_takes(uint32_t tokens, uint32_t rows, uint32_t columns) {
    return tokens >= 1 && tokens <= 384 && rows >= 1 && (columns == 512 || columns == 1024 || columns == 2048);
}

int launch_dense_ksplit(const DenseKsplitArgs& a, hipStream_t s) {
    const dim3 grid((a.n + kTile - 1) / kTile, (a.m + kTile - 1) / kTile);
    switch (a.k / 256) {
        case 2: TSP_LAUNCH("gemm_dense_ksplit", s, dense_ksplit_kernel<2><<<grid, 2 * kWave, 0, s>>>(a)); break;
        case 4: TSP_LAUNCH("gemm_dense_ksplit", s, dense_ksplit_kernel<4><<<grid, 4 * kWave, 0, s>>>(a)); break;
        default: TSP_LAUNCH("gemm_dense_ksplit", s, dense_ksplit_kernel<8><<<grid, 8 * kWave, 0, s>>>(a)); break;
    }
    return launch_status("dense_ksplit");
}

}  // namespace tsp
