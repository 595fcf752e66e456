// Q8_0 GEMV for up to sixteen token rows on the matrix cores (LM head, verify): y[m, r] = sum_k d[r, k/32] * q[r, k] * x[m, k].
//
// A Q8_0 row is a run of 34-byte blocks (f16 scale + 32 int8). The int8 quants are exact halves, so a block is one
// 16x16x32 MFMA step per 16 weight rows: the block's 32 columns are the instruction's whole K, a lane (n, kq) supplies the
// eight quants 8 kq .. 8 kq + 7 of weight row n, and the sixteen operand rows on the other side are the token rows (eight
// of them repeated when there are only eight). The block's scale multiplies the f32 result once (4 fused multiply-adds per
// lane and 16 weight rows). The activations are scaled by a power of two and split into hi + lo halves, staged once in
// LDS for all of K, so the result carries 22 significant bits of x: this is the f32 GEMV of the engine to within f32
// accumulation error, at ~1.3 VALU operations per weight byte whatever the number of token rows.
//
// Raw rows are only 2-byte aligned inside, so the bytes travel global -> registers -> LDS -> registers: a wave reads
// its 32 weight rows x 8 blocks (272 contiguous bytes per row, 16-byte aligned because 8 blocks = 17 x 16 bytes) with
// whole-chunk loads by consecutive lanes, parks them in a wave-private LDS tile whose row stride (272 bytes: unpadded) spreads
// the rows over all banks, and each lane then picks its 8 quants of a block (for each half of the tile's 32 rows) with
// aligned dword reads and a byte funnel shift. The next group of 8 blocks is in flight while the current one is multiplied.
//
// Workgroups are persistent (one per compute unit, 8 waves): the activations are staged once per workgroup, which owns
// every n-th of the matrix's 32-row tiles (n workgroups: at any moment the grid reads one stretch of the matrix, 1 us
// faster at 151 936 x 2048 than a contiguous share per workgroup); its waves take the workgroup's tiles through a counter in LDS. A
// lane asks for its share of the token rows first and for its wave's first weight bytes second, and stages the rows
// while the weights travel. Every address inside the loop is a uniform base plus a lane offset fixed before the loop.
//
// Nine to sixteen token rows do not fit LDS for all of K beside the weight tiles, so that variant splits K in two:
// even workgroups take the first half of the columns, odd ones the second, each over its share of the tiles, and both
// add their f32 partial sums into an output the host cleared before the launch (two addends onto zero: the sum does
// not depend on which arrives first). The matrix is still read once.
#include "q8_mfma.hpp"

#include <type_traits>

#include "mfma_quant.hpp"

using namespace tsp;

namespace {

constexpr uint32_t kWaves = 8, kThreads = kWaves * kWave;
constexpr uint32_t kGroupBlocks = 8, kGroupBytes = kGroupBlocks * 34, kGroupChunks = kGroupBytes / 16;  // 272 B = 17 chunks
// Bytes between rows of the LDS weight tile: 68 dwords = 4 mod 64 banks, so the sixteen rows times two column quarters that a
// half-wave reads one dword of land in 32 different banks, and the tile is written as the contiguous run of chunks it is.
constexpr uint32_t kTileStride = kGroupBytes;
constexpr uint32_t kTileBytes = 32 * kTileStride;         // 8 704 B per wave
constexpr uint32_t kStageLoads = (32 * kGroupChunks + kWave - 1) / kWave;  // 9 chunk loads per lane and group (the last half used)

struct Q8MfmaArgs {
    const uint8_t* matrix;
    const float* x;   // token-major [M, columns]
    float* y;         // token-major [M, rows]
    uint32_t columns, rows, m;
    uint32_t* error_word;
};

__global__ void clear_rows(float4* out, uint64_t count4) {
    const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < count4) out[i] = float4{0, 0, 0, 0};
}

// The token rows of a workgroup, [kRows, K] from column k0 on, in chunks of eight columns: chunk i = tid + j * kThreads is columns
// 8 (i % (K / 8)) .. + 7 of row i / (K / 8). kRows * K / 8 <= 2048 = kMine * kThreads for K <= 2048 (8 rows) or 1024 (16 rows).
constexpr uint32_t kMine = 4;

template <int kRows>
__device__ __forceinline__ void request_token_rows(const Q8MfmaArgs& a, uint32_t K, uint32_t k0, float4 (&xv)[kMine][2]) {
    const uint32_t chunks = K / 8;
#pragma unroll
    for (uint32_t j = 0; j < kMine; ++j) {
        const uint32_t i = threadIdx.x + j * kThreads, r = i / chunks, c = i % chunks;
        xv[j][0] = xv[j][1] = float4{0, 0, 0, 0};
        if (i < kRows * chunks && r < a.m) {
            const float4* src = reinterpret_cast<const float4*>(a.x + uint64_t(r) * a.columns + k0 + c * 8);
            xv[j][0] = src[0];
            xv[j][1] = src[1];
        }
    }
}

// Largest magnitude of the workgroup's rows -> power-of-two scale -> hi + lo halves in LDS, the 16-byte chunks of a row swizzled
// by the row's index (chunk c of row r sits at c ^ r). Returns the factor that undoes the scale; ends with a barrier.
template <int kRows>
__device__ __forceinline__ float stage_token_rows(const float4 (&xv)[kMine][2], uint32_t K, _Float16* a_hi, _Float16* a_lo, float* wave_max,
                                                  uint32_t& bad) {
    const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave, chunks = K / 8;
    float biggest = 0;
#pragma unroll
    for (uint32_t j = 0; j < kMine; ++j) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const float4 v = xv[j][h];
            if (nonfinite(v.x) || nonfinite(v.y) || nonfinite(v.z) || nonfinite(v.w)) bad = TSP_ERRBIT_NONFINITE;
            biggest = fmaxf(biggest, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        }
    }
    biggest = wave_largest(biggest);
    if (lane == 0) wave_max[wave] = biggest;
    __syncthreads();
    biggest = wave_max[0];
#pragma unroll
    for (uint32_t w = 1; w < kWaves; ++w) biggest = fmaxf(biggest, wave_max[w]);
    float scale = 1.0f, inv_scale = 1.0f;
    if (biggest > 0 && !nonfinite(biggest)) {
        const int e = int((__float_as_uint(biggest) >> 23) & 0xffu) - 127;
        int shift = 13 - e;
        shift = shift > 100 ? 100 : shift < -100 ? -100 : shift;
        scale = __uint_as_float(uint32_t(127 + shift) << 23);
        inv_scale = __uint_as_float(uint32_t(127 - shift) << 23);
    }
#pragma unroll
    for (uint32_t j = 0; j < kMine; ++j) {
        const uint32_t i = tid + j * kThreads, r = i / chunks, c = i % chunks;
        if (i >= kRows * chunks) break;
        const float v[8] = {xv[j][0].x, xv[j][0].y, xv[j][0].z, xv[j][0].w, xv[j][1].x, xv[j][1].y, xv[j][1].z, xv[j][1].w};
        f16x8 hi, lo;  // zeros for the rows past a.m
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float sv = v[e] * scale;
            hi[e] = _Float16(sv);
            lo[e] = _Float16(sv - float(hi[e]));
        }
        const uint32_t at = (r * chunks + (c ^ r)) * 8;
        *reinterpret_cast<f16x8*>(a_hi + at) = hi;
        *reinterpret_cast<f16x8*>(a_lo + at) = lo;
    }
    __syncthreads();
    return inv_scale;
}

// DEPTH = (tile, group) items whose bytes are on their way while one is multiplied (1, 2 or 4; it divides the number of groups
// of a workgroup). ROWS = token rows staged (8: all of K per workgroup; 16: half of K per workgroup, sums added into y).
template <int DEPTH, int ROWS>
__global__ __launch_bounds__(kThreads, 1) void q8_mfma_kernel(Q8MfmaArgs a) {
    constexpr int kRows = ROWS;
    constexpr uint32_t KSPLIT = ROWS / 8;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // [hi plane][lo plane][8 weight tiles]
    __shared__ float wave_max[kWaves];
    __shared__ uint32_t next_tile;

    const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const uint32_t n16 = lane % 16, kq = lane / 16;  // 16x16x32 MFMA: operand row / column lane % 16, columns 8 kq .. 8 kq + 7 of the block
    // K: the columns this workgroup multiplies, starting at column k0 (group g0 of the rows)
    const uint32_t K = a.columns / KSPLIT, chunks = K / 8, groups = K / 256, row_bytes = a.columns / 32 * 34;
    const uint32_t k0 = (blockIdx.x % KSPLIT) * K, g0 = k0 / 256;
    const uint32_t sharer = blockIdx.x / KSPLIT, sharers = gridDim.x / KSPLIT;  // the host launches a multiple of KSPLIT
    if (tid == 0) next_tile = 0;
    __syncthreads();  // the tile counter is set before any wave takes from it
    _Float16* const a_hi = reinterpret_cast<_Float16*>(lds);
    _Float16* const a_lo = a_hi + kRows * K;
    uint8_t* const tile = lds + 2 * kRows * K * 2 + wave * kTileBytes;

    // ---- the token rows: this lane's 16-byte chunks are requested first (they come from cache and return first), then the
    // wave's first weight bytes, and only then the arithmetic. The weights travel while the rows are staged.
    uint32_t bad = 0;
    float4 xv[kMine][2];
    request_token_rows<kRows>(a, K, k0, xv);
    // chunk `id` of a group tile: row id / 17 of the wave's 32, bytes (id % 17) * 16 of that row's 272. The byte offsets from
    // the tile's first row and the group's first byte never change, so a request is a uniform address plus a lane offset.
    uint32_t chunk_at[kStageLoads];
#pragma unroll
    for (uint32_t t = 0; t < kStageLoads; ++t) {
        uint32_t id = t * kWave + lane;
        id = id < 32 * kGroupChunks ? id : 32 * kGroupChunks - 1;  // the tail lanes repeat the last chunk
        chunk_at[t] = (id / kGroupChunks) * row_bytes + (id % kGroupChunks) * 16;
    }
    uint2 stage[DEPTH][kStageLoads][2];
    auto fetch_group = [&](uint32_t row0, uint32_t group, auto set_tag) {
        constexpr int SET = decltype(set_tag)::value;
        const uint8_t* from = a.matrix + uint64_t(row0) * row_bytes + uint64_t(g0 + group) * kGroupBytes;  // uniform
        const bool whole = row0 + 32 <= a.rows;                                                           // uniform
#pragma unroll
        for (uint32_t t = 0; t < kStageLoads; ++t) {
            uint32_t at = chunk_at[t];
            if (!whole) {  // the matrix's last tile: rows past the end repeat the last row
                uint32_t id = t * kWave + lane;
                id = id < 32 * kGroupChunks ? id : 32 * kGroupChunks - 1;
                const uint32_t row = row0 + id / kGroupChunks < a.rows ? id / kGroupChunks : a.rows - 1 - row0;
                at = row * row_bytes + (id % kGroupChunks) * 16;
            }
            const uint4 v = *reinterpret_cast<const uint4*>(from + at);
            stage[SET][t][0] = uint2{v.x, v.y};
            stage[SET][t][1] = uint2{v.z, v.w};
        }
    };
    // Workgroup b of n owns tiles b, b + n, b + 2 n, ... and its waves take the next free one of them from
    // a counter in LDS (which wave computes a tile does not change the result). The bytes of the next (tile, group) item
    // are requested before the current one is multiplied, so a wave always holds its next tile index one step ahead.
    const uint32_t share_end = (a.rows + 31) / 32;
    auto take_tile = [&]() {
        uint32_t t = 0;
        if (lane == 0) t = atomicAdd(&next_tile, 1u);
        return uint32_t(__builtin_amdgcn_readfirstlane(int(t))) * sharers + sharer;
    };
    uint32_t t = take_tile(), t_next = take_tile();
    if (t < share_end) {
        fetch_group(t * 32, 0, std::integral_constant<int, 0>{});
        if constexpr (DEPTH >= 2) fetch_group(t * 32, 1, std::integral_constant<int, 1 % DEPTH>{});
        if constexpr (DEPTH >= 4) {
            fetch_group(t * 32, 2, std::integral_constant<int, 2 % DEPTH>{});
            fetch_group(t * 32, 3, std::integral_constant<int, 3 % DEPTH>{});
        }
    }
    __builtin_amdgcn_sched_barrier(0);  // every request above is out before the first wait below
    const float inv_scale = stage_token_rows<kRows>(xv, K, a_hi, a_lo, wave_max, bad);

    // The activation chunk of block B of group g, columns 8 kq .. 8 kq + 7, is chunk g * 32 + B * 4 + kq of row `arow`, kept at
    // position chunk ^ arow. arow < kRows only flips the low bits, which B % kVariants and kq decide: the lane keeps one
    // address per variant and the rest of the chunk index is an offset known when the code is compiled (B) or uniform (g).
    const uint32_t arow = n16 & (kRows - 1);
    constexpr uint32_t kVariants = kRows / 4;
    uint32_t a_at[kVariants];  // in halves, from the start of a plane
#pragma unroll
    for (uint32_t v = 0; v < kVariants; ++v) a_at[v] = (arow * chunks + ((v * 4 + kq) ^ arow)) * 8;
    auto store_group = [&](auto set_tag) {
        constexpr int SET = decltype(set_tag)::value;
#pragma unroll
        for (uint32_t t = 0; t < kStageLoads; ++t) {
            uint32_t id = t * kWave + lane;
            id = id < 32 * kGroupChunks ? id : 32 * kGroupChunks - 1;
            uint8_t* at = tile + (id / kGroupChunks) * kTileStride + (id % kGroupChunks) * 16;
            *reinterpret_cast<uint4*>(at) = uint4{stage[SET][t][0].x, stage[SET][t][0].y, stage[SET][t][1].x, stage[SET][t][1].y};
        }
    };

    for (; t < share_end; t = t_next, t_next = take_tile()) {
        const uint32_t row0 = t * 32;
        float acc[2][4] = {{0, 0, 0, 0}, {0, 0, 0, 0}};  // [16-row half of the tile][token row 4 kq + v]
        // one item: its bytes go registers -> LDS tile, the item DEPTH ahead is requested into the freed registers, then the
        // tile is multiplied.
        auto item = [&](uint32_t g, auto set_tag) {
            store_group(set_tag);  // the previous item's reads were issued before this point; LDS serves a wave in order
            const uint32_t ahead = g + DEPTH;
            const bool wraps = ahead >= groups;
            // past the workgroup's share: ask again for the group at hand (its lines are in cache), nothing new comes from memory
            const bool more = t_next < share_end;
            const uint32_t following = wraps && more ? t_next : t;
            const uint32_t group = !wraps ? ahead : more ? ahead - groups : g;
            fetch_group(following * 32, group, set_tag);
            const uint8_t* mine = tile + n16 * kTileStride + kq * 8;
            auto block = [&](auto b_tag) {
                constexpr int B = decltype(b_tag)::value;
                // the lane's eight quants of the block, for rows n16 and n16 + 16 of the tile: bytes 34 B + 2 + 8 kq .. + 8 of the
                // row, dword aligned for odd B, 2 bytes past a dword for even B
                constexpr uint32_t Q_AT = 34 * B + 2, ALIGNED = Q_AT & ~3u;
                f16x8 b_frag[2];
                float scale_d[2];
#pragma unroll
                for (int nt = 0; nt < 2; ++nt) {
                    const uint8_t* row = mine + nt * 16 * kTileStride;
                    uint32_t w[2];
                    if constexpr (Q_AT % 4 == 0) {
                        w[0] = *reinterpret_cast<const uint32_t*>(row + ALIGNED);
                        w[1] = *reinterpret_cast<const uint32_t*>(row + ALIGNED + 4);
                    } else {
                        uint32_t d[3];
#pragma unroll
                        for (int i = 0; i < 3; ++i) d[i] = *reinterpret_cast<const uint32_t*>(row + ALIGNED + 4 * i);
                        w[0] = __builtin_amdgcn_alignbyte(d[1], d[0], 2);
                        w[1] = __builtin_amdgcn_alignbyte(d[2], d[1], 2);
                    }
                    b_frag[nt] = quants8(w[0], w[1]);
                    scale_d[nt] = half_bits_to_float(*reinterpret_cast<const uint16_t*>(tile + (nt * 16 + n16) * kTileStride + 34 * B));
                }
                // columns g * 256 + B * 32 + 8 kq of the lane's token row
                const uint32_t at = a_at[B % kVariants] + (g * 32 + (B / kVariants) * kVariants * 4) * 8;
                const f16x8 ah = *reinterpret_cast<const f16x8*>(a_hi + at), al = *reinterpret_cast<const f16x8*>(a_lo + at);
                const f32x4 zero{};
#pragma unroll
                for (int nt = 0; nt < 2; ++nt) {
                    // the lo halves of the rows first, the hi halves on top of them: one f32 result per block to scale
                    const f32x4 part_lo = __builtin_amdgcn_mfma_f32_16x16x32_f16(al, b_frag[nt], zero, 0, 0, 0);
                    const f32x4 part = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, b_frag[nt], part_lo, 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[nt][v] = __builtin_fmaf(scale_d[nt], part[v], acc[nt][v]);  // rows 4 kq + v
                }
            };
            block(std::integral_constant<int, 0>{});
            block(std::integral_constant<int, 1>{});
            block(std::integral_constant<int, 2>{});
            block(std::integral_constant<int, 3>{});
            block(std::integral_constant<int, 4>{});
            block(std::integral_constant<int, 5>{});
            block(std::integral_constant<int, 6>{});
            block(std::integral_constant<int, 7>{});
        };
        for (uint32_t g = 0; g < groups; g += DEPTH) {  // the host picks a DEPTH that divides the number of groups
            item(g, std::integral_constant<int, 0>{});
            if constexpr (DEPTH >= 2) item(g + 1, std::integral_constant<int, 1 % DEPTH>{});
            if constexpr (DEPTH >= 4) {
                item(g + 2, std::integral_constant<int, 2 % DEPTH>{});
                item(g + 3, std::integral_constant<int, 3 % DEPTH>{});
            }
        }
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
            const uint32_t r = row0 + nt * 16 + n16;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t m = 4 * kq + v;  // lanes with 4 kq >= kRows hold repeats of rows 0 .. kRows - 1
                if (m < kRows && m < a.m && r < a.rows) {
                    const float val = acc[nt][v] * inv_scale;
                    if (nonfinite(val)) bad = TSP_ERRBIT_NONFINITE;
                    if constexpr (KSPLIT == 1) a.y[uint64_t(m) * a.rows + r] = val;
                    else unsafeAtomicAdd(a.y + uint64_t(m) * a.rows + r, val);
                }
            }
        }
    }
    publish_error(bad, a.error_word);
}

// ---- q8_lanes_v1 rows: [f16 scale x blocks][runs of 16 blocks x 512 B: quant i of the run's sixteen blocks side by side].
// The unit of work is 16 weight rows x one run (512 columns): per row 32 bytes of scales and 512 bytes of quants, both whole
// 16-byte chunks at 16-byte aligned offsets when the row has a multiple of 16 blocks. A wave parks the 34 chunks of each row
// in its LDS tile at a row stride of 560 bytes (140 dwords = 12 mod 64 banks: the sixteen rows that a quarter-wave reads one
// 16-byte chunk of land in 64 different banks). A lane (n, kq) then reads the eight chunks of quants 8 kq .. 8 kq + 7 of row n,
// which hold those quants for all sixteen blocks, and turns each 4 x 4 byte square (4 quants x 4 blocks) into the four dwords
// "4 quants of one block" with two rounds of byte permutes: four permutes per block and lane. From there on a block is what it
// is for raw rows: exact halves, one 16x16x32 MFMA step for the lo and one for the hi halves of the token rows, and the
// block's scale times the f32 result.
constexpr uint32_t kRunBlocks = 16, kRunChunks = 2 + 32;  // 32 B of scales + 512 B of quants per row and run
constexpr uint32_t kLaneRows = 16, kLaneStride = 560, kLaneTileBytes = kLaneRows * kLaneStride;  // 8 960 B per wave
constexpr uint32_t kLaneLoads = (kLaneRows * kRunChunks + kWave - 1) / kWave;  // 9 chunk loads per lane and run (the last half used)

// ROWS = token rows staged: 8 (all of K per workgroup) or 16 (even workgroups the first half of a row's runs, odd ones the second,
// each pair over its share of the tiles, both adding their f32 sums into an output the host cleared: the matrix is read once).
template <int DEPTH, int ROWS>
__global__ __launch_bounds__(kThreads, 1) void q8_lanes_mfma_kernel(Q8MfmaArgs a) {
    constexpr int kRows = ROWS;
    constexpr uint32_t KSPLIT = ROWS / 8;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // [hi plane][lo plane][8 weight tiles]
    __shared__ float wave_max[kWaves];
    __shared__ uint32_t next_tile;

    const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const uint32_t n16 = lane % 16, kq = lane / 16;
    // K: the columns this workgroup multiplies, runs run0 .. run0 + runs - 1 of every row
    const uint32_t K = a.columns / KSPLIT, chunks = K / 8, blocks = a.columns / 32, runs = blocks / kRunBlocks / KSPLIT, row_bytes = blocks * 34;
    const uint32_t run0 = (blockIdx.x % KSPLIT) * runs;
    const uint32_t sharer = blockIdx.x / KSPLIT, sharers = gridDim.x / KSPLIT;  // the host launches a multiple of KSPLIT
    const uint32_t tiles = (a.rows + kLaneRows - 1) / kLaneRows;
    if (tid == 0) next_tile = 0;
    __syncthreads();
    _Float16* const a_hi = reinterpret_cast<_Float16*>(lds);
    _Float16* const a_lo = a_hi + kRows * K;
    uint8_t* const tile = lds + 2 * kRows * K * 2 + wave * kLaneTileBytes;

    uint32_t bad = 0;
    float4 xv[kMine][2];
    request_token_rows<kRows>(a, K, run0 * (kRunBlocks * 32), xv);

    // chunk `id` of a tile: row id / 34 of the wave's 16, piece id % 34 of that row's run: pieces 0 and 1 are the run's scales
    // (32 bytes per run from the row's start), pieces 2 .. 33 its quants (512 bytes per run after all the scales).
    auto piece_at = [&](uint32_t row, uint32_t piece, uint32_t run) {
        return row * row_bytes + (piece < 2 ? run * 32 + piece * 16 : 2 * blocks + run * 512 + (piece - 2) * 16);
    };
    uint32_t chunk_at[kLaneLoads], chunk_step[kLaneLoads];  // byte offset at run 0 and bytes per run
#pragma unroll
    for (uint32_t t = 0; t < kLaneLoads; ++t) {
        uint32_t id = t * kWave + lane;
        id = id < kLaneRows * kRunChunks ? id : kLaneRows * kRunChunks - 1;  // the tail lanes repeat the last chunk
        chunk_at[t] = piece_at(id / kRunChunks, id % kRunChunks, run0);
        chunk_step[t] = id % kRunChunks < 2 ? 32 : 512;
    }
    uint2 stage[DEPTH][kLaneLoads][2];
    auto fetch_run = [&](uint32_t row0, uint32_t run, auto set_tag) {
        constexpr int SET = decltype(set_tag)::value;
        const uint8_t* from = a.matrix + uint64_t(row0) * row_bytes;  // uniform
        const bool whole = row0 + kLaneRows <= a.rows;               // uniform
#pragma unroll
        for (uint32_t t = 0; t < kLaneLoads; ++t) {
            uint32_t at = chunk_at[t] + run * chunk_step[t];
            if (!whole) {  // the matrix's last tile: rows past the end repeat the last row
                uint32_t id = t * kWave + lane;
                id = id < kLaneRows * kRunChunks ? id : kLaneRows * kRunChunks - 1;
                const uint32_t row = row0 + id / kRunChunks < a.rows ? id / kRunChunks : a.rows - 1 - row0;
                at = piece_at(row, id % kRunChunks, run0 + run);
            }
            const uint4 v = *reinterpret_cast<const uint4*>(from + at);
            stage[SET][t][0] = uint2{v.x, v.y};
            stage[SET][t][1] = uint2{v.z, v.w};
        }
    };
    const uint32_t share_end = tiles;
    auto take_tile = [&]() {
        uint32_t t = 0;
        if (lane == 0) t = atomicAdd(&next_tile, 1u);
        return uint32_t(__builtin_amdgcn_readfirstlane(int(t))) * sharers + sharer;
    };
    uint32_t t = take_tile(), t_next = take_tile();
    if (t < share_end) {
        fetch_run(t * kLaneRows, 0, std::integral_constant<int, 0>{});
        if constexpr (DEPTH >= 2) fetch_run(t * kLaneRows, 1, std::integral_constant<int, 1 % DEPTH>{});
    }
    __builtin_amdgcn_sched_barrier(0);  // every request above is out before the first wait below
    const float inv_scale = stage_token_rows<kRows>(xv, K, a_hi, a_lo, wave_max, bad);

    // the activation chunk of block B of run g, columns 8 kq .. 8 kq + 7: chunk g * 64 + B * 4 + kq of row `arow`, kept at
    // chunk ^ arow; arow < kRows flips the three or four low bits, which B % kVariants and kq decide
    const uint32_t arow = n16 & (kRows - 1);
    constexpr uint32_t kVariants = kRows / 4;
    uint32_t a_at[kVariants];
#pragma unroll
    for (uint32_t v = 0; v < kVariants; ++v) a_at[v] = (arow * chunks + ((v * 4 + kq) ^ arow)) * 8;
    auto store_run = [&](auto set_tag) {
        constexpr int SET = decltype(set_tag)::value;
#pragma unroll
        for (uint32_t t = 0; t < kLaneLoads; ++t) {
            uint32_t id = t * kWave + lane;
            id = id < kLaneRows * kRunChunks ? id : kLaneRows * kRunChunks - 1;
            uint8_t* at = tile + (id / kRunChunks) * kLaneStride + (id % kRunChunks) * 16;
            *reinterpret_cast<uint4*>(at) = uint4{stage[SET][t][0].x, stage[SET][t][0].y, stage[SET][t][1].x, stage[SET][t][1].y};
        }
    };

    for (; t < share_end; t = t_next, t_next = take_tile()) {
        const uint32_t row0 = t * kLaneRows;
        float acc[4] = {0, 0, 0, 0};  // token row 4 kq + v
        auto item = [&](uint32_t g, auto set_tag) {
            store_run(set_tag);  // the previous item's reads were issued before this point; LDS serves a wave in order
            const uint32_t ahead = g + DEPTH;
            const bool wraps = ahead >= runs;
            // past the workgroup's share: ask again for the run at hand (its lines are in cache), nothing new comes from memory
            const bool more = t_next < share_end;
            const uint32_t following = wraps && more ? t_next : t;
            const uint32_t run = !wraps ? ahead : more ? ahead - runs : g;
            fetch_run(following * kLaneRows, run, set_tag);
            const uint8_t* mine = tile + n16 * kLaneStride;
            const uint4 s0 = *reinterpret_cast<const uint4*>(mine), s1 = *reinterpret_cast<const uint4*>(mine + 16);
            const uint32_t scales[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};  // two f16 scales per dword
            uint4 q[8];  // q[j]: quant 8 kq + j of the run's sixteen blocks, one byte per block
#pragma unroll
            for (int j = 0; j < 8; ++j) q[j] = *reinterpret_cast<const uint4*>(mine + 32 + (8 * kq + j) * 16);
            auto quad = [&](auto m_tag) {  // blocks 4 M .. 4 M + 3 of the run
                constexpr int M = decltype(m_tag)::value;
                uint32_t d[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) d[j] = M == 0 ? q[j].x : M == 1 ? q[j].y : M == 2 ? q[j].z : q[j].w;
                // byte b of d[j] = quant j of block 4 M + b. First round: pairs of quants interleaved, for blocks 0, 1 (lo) and 2, 3 (hi)
                uint32_t lo[4], hi[4];
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    lo[p] = __builtin_amdgcn_perm(d[2 * p + 1], d[2 * p], 0x05010400u);
                    hi[p] = __builtin_amdgcn_perm(d[2 * p + 1], d[2 * p], 0x07030602u);
                }
                // second round: w[b][0] = quants 0 .. 3 and w[b][1] = quants 4 .. 7 of block 4 M + b
                uint32_t w[4][2];
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    w[0][half] = __builtin_amdgcn_perm(lo[2 * half + 1], lo[2 * half], 0x05040100u);
                    w[1][half] = __builtin_amdgcn_perm(lo[2 * half + 1], lo[2 * half], 0x07060302u);
                    w[2][half] = __builtin_amdgcn_perm(hi[2 * half + 1], hi[2 * half], 0x05040100u);
                    w[3][half] = __builtin_amdgcn_perm(hi[2 * half + 1], hi[2 * half], 0x07060302u);
                }
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    constexpr int kBase = 4 * M;
                    const int B = kBase + b;
                    const f16x8 b_frag = quants8(w[b][0], w[b][1]);
                    const float scale_d = half_bits_to_float((scales[B / 2] >> (16 * (B % 2))) & 0xffffu);
                    const uint32_t at = a_at[B % kVariants] + (g * 64 + (B / kVariants) * kVariants * 4) * 8;  // columns g * 512 + B * 32 + 8 kq of the lane's token row
                    const f16x8 ah = *reinterpret_cast<const f16x8*>(a_hi + at), al = *reinterpret_cast<const f16x8*>(a_lo + at);
                    const f32x4 zero{};
                    const f32x4 part_lo = __builtin_amdgcn_mfma_f32_16x16x32_f16(al, b_frag, zero, 0, 0, 0);
                    const f32x4 part = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, b_frag, part_lo, 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[v] = __builtin_fmaf(scale_d, part[v], acc[v]);
                }
            };
            quad(std::integral_constant<int, 0>{});
            quad(std::integral_constant<int, 1>{});
            quad(std::integral_constant<int, 2>{});
            quad(std::integral_constant<int, 3>{});
        };
        for (uint32_t g = 0; g < runs; g += DEPTH) {  // the host picks a DEPTH that divides the number of runs
            item(g, std::integral_constant<int, 0>{});
            if constexpr (DEPTH >= 2) item(g + 1, std::integral_constant<int, 1 % DEPTH>{});
        }
        const uint32_t r = row0 + n16;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const uint32_t m = 4 * kq + v;  // with eight token rows the lanes with kq >= 2 hold repeats of rows 0 .. 7
            if (m < kRows && m < a.m && r < a.rows) {
                const float val = acc[v] * inv_scale;
                if (nonfinite(val)) bad = TSP_ERRBIT_NONFINITE;
                if constexpr (KSPLIT == 1) a.y[uint64_t(m) * a.rows + r] = val;
                else unsafeAtomicAdd(a.y + uint64_t(m) * a.rows + r, val);
            }
        }
    }
    publish_error(bad, a.error_word);
}

}  // namespace

namespace tsp {

bool q8_mfma_supported(const void* matrix, const float* x, uint32_t columns, uint32_t rows) {
    return columns % 256 == 0 && columns <= 2048 && rows >= 32 && reinterpret_cast<uintptr_t>(matrix) % 16 == 0 &&
           reinterpret_cast<uintptr_t>(x) % 16 == 0;
}

bool q8_mfma_supported_16(const void* matrix, const float* x, const float* y, uint32_t columns, uint32_t rows) {
    return q8_mfma_supported(matrix, x, columns, rows) && columns % 1024 == 0 && rows >= 64 && rows % 4 == 0 &&
           reinterpret_cast<uintptr_t>(y) % 16 == 0;
}

int q8_mfma(const void* matrix, const float* x, float* y, uint32_t columns, uint32_t rows, uint32_t width, uint32_t* error_word, hipStream_t s) {
    const Q8MfmaArgs a{static_cast<const uint8_t*>(matrix), x, y, columns, rows, width, error_word};
    // 8 rows x all columns and 16 rows x half the columns stage the same number of bytes
    const uint32_t lds_bytes = 2 * 8 * columns * 2 + kWaves * kTileBytes;
    static std::atomic<uint64_t> raised{0};
    static int units_of[64] = {};
    int device = 0;
    if (setup_pending(raised, &device)) {
        const int most = int(2 * 8 * 2048 * 2 + kWaves * kTileBytes);
        TSP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&q8_mfma_kernel<1, 8>), hipFuncAttributeMaxDynamicSharedMemorySize, most));
        TSP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&q8_mfma_kernel<2, 8>), hipFuncAttributeMaxDynamicSharedMemorySize, most));
        TSP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&q8_mfma_kernel<2, 16>), hipFuncAttributeMaxDynamicSharedMemorySize, most));
        TSP_HIP(hipDeviceGetAttribute(&units_of[device], hipDeviceAttributeMultiprocessorCount, device));
        setup_done(raised, device);
    }
    const int compute_units = units_of[device];
    const uint32_t tiles = (rows + 31) / 32;
    uint32_t grid = uint32_t(compute_units > 0 ? compute_units : 256);
    if (width > 8) {
        // two workgroups (one per half of the columns) share each run of tiles; the output starts at zero
        uint32_t pairs = grid / 2 ? grid / 2 : 1;
        if (pairs * kWaves > tiles) pairs = (tiles + kWaves - 1) / kWaves;
        const uint64_t count4 = uint64_t(width) * rows / 4;
        TSP_LAUNCH("clear_rows", s, clear_rows<<<uint32_t((count4 + 255) / 256), 256, 0, s>>>(reinterpret_cast<float4*>(y), count4));
        TSP_LAUNCH("q8_mfma", s, q8_mfma_kernel<2, 16><<<2 * pairs, kThreads, lds_bytes, s>>>(a));
        return launch_status("q8_mfma");
    }
    if (grid * kWaves > tiles) grid = (tiles + kWaves - 1) / kWaves;
    // two items in flight measured best on MI355X (one: 72 us, two: 69 us, four: 75 us at 151 936 x 2048)
    if ((columns / 256) % 2 == 0) TSP_LAUNCH("q8_mfma", s, q8_mfma_kernel<2, 8><<<grid, kThreads, lds_bytes, s>>>(a));
    else TSP_LAUNCH("q8_mfma", s, q8_mfma_kernel<1, 8><<<grid, kThreads, lds_bytes, s>>>(a));
    return launch_status("q8_mfma");
}

bool q8_lanes_mfma_supported(const void* matrix, const float* x, uint32_t columns, uint32_t rows) {
    return columns % 512 == 0 && columns <= 2048 && rows >= 16 && reinterpret_cast<uintptr_t>(matrix) % 16 == 0 &&
           reinterpret_cast<uintptr_t>(x) % 16 == 0;
}

bool q8_lanes_mfma_supported_16(const void* matrix, const float* x, const float* y, uint32_t columns, uint32_t rows) {
    return q8_lanes_mfma_supported(matrix, x, columns, rows) && columns % 1024 == 0 && rows >= 32 && rows % 4 == 0 &&
           reinterpret_cast<uintptr_t>(y) % 16 == 0;
}

int q8_lanes_mfma(const void* matrix, const float* x, float* y, uint32_t columns, uint32_t rows, uint32_t width, uint32_t* error_word,
                  hipStream_t s) {
    const Q8MfmaArgs a{static_cast<const uint8_t*>(matrix), x, y, columns, rows, width, error_word};
    const uint32_t lds_bytes = 2 * 8 * columns * 2 + kWaves * kLaneTileBytes;
    static std::atomic<uint64_t> raised{0};
    static int units_of[64] = {};
    int device = 0;
    if (setup_pending(raised, &device)) {
        const int most = int(2 * 8 * 2048 * 2 + kWaves * kLaneTileBytes);
        TSP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&q8_lanes_mfma_kernel<1, 8>), hipFuncAttributeMaxDynamicSharedMemorySize, most));
        TSP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&q8_lanes_mfma_kernel<2, 8>), hipFuncAttributeMaxDynamicSharedMemorySize, most));
        TSP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&q8_lanes_mfma_kernel<1, 16>), hipFuncAttributeMaxDynamicSharedMemorySize, most));
        TSP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&q8_lanes_mfma_kernel<2, 16>), hipFuncAttributeMaxDynamicSharedMemorySize, most));
        TSP_HIP(hipDeviceGetAttribute(&units_of[device], hipDeviceAttributeMultiprocessorCount, device));
        setup_done(raised, device);
    }
    const int compute_units = units_of[device];
    const uint32_t tiles = (rows + kLaneRows - 1) / kLaneRows;
    uint32_t grid = uint32_t(compute_units > 0 ? compute_units : 256);
    if (width > 8) {
        // two workgroups (one per half of a row's runs) share each stretch of tiles; the output starts at zero
        uint32_t pairs = grid / 2 ? grid / 2 : 1;
        if (pairs * kWaves > tiles) pairs = (tiles + kWaves - 1) / kWaves;
        const uint64_t count4 = uint64_t(width) * rows / 4;
        TSP_LAUNCH("clear_rows", s, clear_rows<<<uint32_t((count4 + 255) / 256), 256, 0, s>>>(reinterpret_cast<float4*>(y), count4));
        if ((columns / 1024) % 2 == 0) TSP_LAUNCH("q8_lanes_mfma", s, q8_lanes_mfma_kernel<2, 16><<<2 * pairs, kThreads, lds_bytes, s>>>(a));
        else TSP_LAUNCH("q8_lanes_mfma", s, q8_lanes_mfma_kernel<1, 16><<<2 * pairs, kThreads, lds_bytes, s>>>(a));
        return launch_status("q8_lanes_mfma");
    }
    if (grid * kWaves > tiles) grid = (tiles + kWaves - 1) / kWaves;
    if ((columns / 512) % 2 == 0) TSP_LAUNCH("q8_lanes_mfma", s, q8_lanes_mfma_kernel<2, 8><<<grid, kThreads, lds_bytes, s>>>(a));
    else TSP_LAUNCH("q8_lanes_mfma", s, q8_lanes_mfma_kernel<1, 8><<<grid, kThreads, lds_bytes, s>>>(a));
    return launch_status("q8_lanes_mfma");
}

}  // namespace tsp
