// Dense Q4_K GEMM for a thousand and more activation rows: out[m, n] = sum_k x[m, k] * half(dec(W[n, k])), f32 accumulation.
//
// With this many rows the weights must not be unpacked over and over: the 64-row tiles of the general kernel (gemm.hip)
// unpack every weight once per 64 activation rows, and at 2048 rows spend eight vector instructions per MFMA doing so. Here
// a workgroup owns a 128 x 256 output tile (four waves, each 128 activation rows x 64 weight rows) or a 256 x 256 tile (eight
// waves, each 256 x 32): 128 accumulator registers per lane either way, two waves per SIMD, and a weight is unpacked once
// per 128 or 256 rows. What bounds the loop is the rate at which a SIMD issues instructions next to its MFMAs (measured:
// one wave issues one every ~8 cycles, two waves together one every ~4.6, a mixed-precision multiply-add counts about
// double, a 16-byte LDS read from one wave every 17), not the matrix pipe (about half busy), LDS bandwidth (240-307 bytes
// per cycle measured, a quarter of it used, no bank conflicts) or memory.
//
//   * Arithmetic: the engine's for this path. A weight is its f32 value d * sc * q - dmin * mn rounded once to half: the
//     code q, masked out where it sits, is a subnormal half q * 2^-24, and one mixed-precision fused multiply-add per
//     weight evaluates (d * sc * 2^24) * that - dmin * mn in f32 and rounds it to half; activations are the bf16 values
//     carried as halves; products accumulate in f32 on v_mfma_f32_32x32x16_f16.
//   * Activations: the tile's rows x 128 bytes per step go global -> LDS directly, two steps ahead, into a ring of three
//     slabs shared by the waves. 16-byte chunk c of row r sits at position c ^ ((r / 2) % 8): a 16-byte read by sixteen
//     consecutive lanes (rows) then covers all 64 banks once (with c ^ (r % 8), rows r and r + 8 met in the same banks).
//   * Weights: the step's 32 bytes of nibbles of the tile's 256 rows (8 KB, ring of three) and, once per super-block, the
//     rows' 16 header bytes (d, dmin, packed scales and minima; ring of two) travel the same way. Every request in the
//     loop is unconditional and issued by every thread (rows past the matrix's end repeat its last row), so each wave
//     waits with an exact count.
//   * One barrier per step, before the step's last group of MFMAs rather than between steps (see step_fn).
//   * Workgroups are dealt to the XCDs in runs of consecutive tiles, column tiles fastest: the workgroups of one XCD
//     share a slab of activation rows in its L2 and read every weight byte once.
#include "dense_tall.hpp"

#include <atomic>
#include <type_traits>
#include <utility>

#include "mfma_quant.hpp"

using namespace tsp;

namespace {

// A pointer that is the same in every lane, moved to scalar registers (the base operand of a direct-to-LDS request has to be one).
__device__ __forceinline__ const uint8_t* uniform_pointer(const uint8_t* p) {
    const uint64_t bits = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(bits))), hi = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(bits >> 32)));
    return reinterpret_cast<const uint8_t*>(uint64_t(hi) << 32 | lo);
}

// Byte N of a word as a float: one v_cvt_f32_ubyteN.
template <int N>
__device__ __forceinline__ float byte_as_float(uint32_t word) { return float((word >> (8 * N)) & 0xffu); }

// Two weights from two codes sitting in the mantissas of two halves (`codes`: q or q << 4 per half, everything else zero: the
// subnormal halves q * 2^-24 resp. q * 2^-20): each is scale * code + offset evaluated as one f32 fused multiply-add whose
// result is rounded to half (v_fma_mix widens the half operand to f32 inside the instruction, subnormals included), one
// instruction per weight and no separate conversion of the code to a float. With scale = d * sc * 2^24 (2^20) and offset =
// -dmin * mn this is the f32 value d * sc * q - dmin * mn exactly, then rounded once.
__device__ __forceinline__ uint32_t two_weights(uint32_t codes, float scale, float offset) {
    const f16x2 c = as_h2(codes);
    const _Float16 lo = _Float16(__builtin_fmaf(float(c[0]), scale, offset)), hi = _Float16(__builtin_fmaf(float(c[1]), scale, offset));
    return as_u32(f16x2{lo, hi});
}

constexpr int kStepK = 64, kRing = 3, kHdrStages = 2;

// waves per SIMD: 128-row tiles leave room for two workgroups per compute unit, 256-row tiles for one
constexpr int tall_waves_per_simd(int rt, int ct, int waves, int tn) { return ((waves * ct * 32 / tn) * rt * 32 == 128 ? 2 : 1) * waves / 4; }

// RT x CT: the row tiles (32 activation rows each) and column tiles (32 weight rows each) of a wave, 16 accumulator registers
// apiece; WAVES waves stand 8 / CT wide across the tile's 256 weight rows and WAVES CT / 8 high. Two forms are launched:
//   4 x 2, four waves: a 128 x 256 tile; two workgroups share a compute unit.
//   8 x 1, eight waves: a 256 x 256 tile; a weight is unpacked once per 256 rows, at the price of an LDS read per MFMA.
// (8 x 2 with four waves, a wave alone on its SIMD with 256 accumulator registers, compiles too and measured in between.)
// TN = weight rows of a tile: 256, or 128 for
//   4 x 1, four waves: a 128 x 128 tile, for 512 to 1023 activation rows, where 256 weight rows per tile would leave half of
//     the compute units without a tile (512 x 8192 results are 256 such tiles); 64 accumulator registers per lane.
template <int RT, int CT, int WAVES, int TN = 256, int PER_SIMD = tall_waves_per_simd(RT, CT, WAVES, TN)>
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(PER_SIMD, PER_SIMD))) void dense_tall_kernel(DenseTallArgs a) {
    constexpr int kTileN = TN, kQsBytes = kTileN * 32, kHdrBytes = kTileN * 16;
    constexpr int kThreadsT = 64 * WAVES, WN = TN / 32 / CT, WM = WAVES / WN, kTileM = WM * RT * 32;
    static_assert(WM >= 1 && WN * WM == WAVES && kQsBytes % (kThreadsT * 16) == 0);
    constexpr int kSlabBytes = kTileM * kStepK * 2, kSlabPieces = kSlabBytes / (kThreadsT * 16);
    constexpr int kQsAt = kRing * kSlabBytes, kHdrAt = kQsAt + kRing * kQsBytes;
    __shared__ __attribute__((aligned(16))) uint8_t lds_raw[kHdrAt + kHdrStages * kHdrBytes];
    static_assert(sizeof(lds_raw) * (kTileM == 128 ? 2 : 1) <= 160 * 1024, "the workgroups of a compute unit share 160 KB");

    const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const uint32_t col = lane % 32, khalf = (lane / 32) & 1;
    const uint32_t wm = wave / WN, wn = wave % WN;  // the wave's RT x 32 activation rows and CT x 32 weight rows of the tile

    // ---- the workgroup's tile: XCD x (workgroup id % 8) takes the x-th run of consecutive tiles
    const uint32_t n_tiles = (a.n + kTileN - 1) / kTileN, m_tiles = (a.m + kTileM - 1) / kTileM;
    const uint32_t tiles = n_tiles * m_tiles, per_xcd = (tiles + 7) / 8;
    const uint32_t logical = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (blockIdx.x / 8 >= per_xcd || logical >= tiles) return;
    const uint32_t m0 = (logical / n_tiles) * kTileM, n0 = (logical % n_tiles) * kTileN;
    const uint32_t bpr = a.k / 256, steps = a.k / kStepK;
    const uint32_t row_bytes = bpr * 144;

    // ---- per-thread parts of the request addresses (the per-step parts are uniform)
    // activations: request i of thread t fills 16-byte position t + T i of the slab (T threads) = slot t % 8 of row (t + T i) / 8,
    // with chunk (t % 8) ^ ((row / 2) % 8) of that row
    uint32_t a_lane[kSlabPieces];
#pragma unroll
    for (int i = 0; i < kSlabPieces; ++i) {
        const uint32_t r = (tid + kThreadsT * i) / 8, row = m0 + r < a.m ? m0 + r : a.m - 1;
        a_lane[i] = (row * a.a_stride + (((tid % 8) ^ ((r >> 1) & 7)) * 8)) * 2;
    }
    // nibbles: request q of thread t fills position u = t + T q of the stage = slot u % 2 of weight row u / 2, with chunk
    // (u % 2) ^ ((row / 8) % 2) of the step's 32 bytes of that row; headers: position t % 256 = weight row t % 256 (with eight
    // waves the two halves of the workgroup fetch the same bytes to the same place: every wave's count of requests is the same)
    constexpr int QN = kQsBytes / (kThreadsT * 16);
    uint32_t q_lane[QN];
#pragma unroll
    for (int q = 0; q < QN; ++q) {
        const uint32_t u = tid + kThreadsT * q, q_r = u / 2, q_row = n0 + q_r < a.n ? n0 + q_r : a.n - 1;
        q_lane[q] = q_row * row_bytes + (((u % 2) ^ ((q_r >> 3) & 1)) * 16);
    }
    const uint32_t h_r = tid % kTileN, h_row = n0 + h_r < a.n ? n0 + h_r : a.n - 1;
    const uint32_t h_lane = h_row * row_bytes;
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane(lds_address(lds_raw));
    const uint32_t my_slab = lds0 + wave * 1024, my_qs = lds0 + kQsAt + wave * 1024, my_hdr = lds0 + kHdrAt + (wave % (kTileN / 64)) * 1024;
    // Step `step`'s bytes into ring slot step % 3. Steps past the end ask for the last step's bytes again (read by the front of a step that never runs), and
    // ask for headers where a real step would: the number of requests per step must not depend on where the matrix ends,
    // the waits below count them.
    auto request = [&](uint32_t step) {
        const uint32_t slot = step % kRing, hdr_slot = (step / 4) % kHdrStages;
        const bool with_headers = step % 4 == 0;
        step = step < steps ? step : steps - 1;
        const uint32_t b = step / 4, pair = step % 4;
        const uint8_t* a_base = uniform_pointer(reinterpret_cast<const uint8_t*>(a.a) + uint64_t(step) * (kStepK * 2));
        const uint32_t slab = my_slab + slot * kSlabBytes;
#pragma unroll
        for (int i = 0; i < kSlabPieces; ++i) load_to_lds_16(a_base, a_lane[i], slab + i * (kThreadsT * 16));
#pragma unroll
        for (int q = 0; q < QN; ++q) load_to_lds_16(a.w + uint64_t(b) * 144 + 16 + pair * 32, q_lane[q], my_qs + slot * kQsBytes + q * (kThreadsT * 16));
        if (with_headers) load_to_lds_16(a.w + uint64_t(b) * 144, h_lane, my_hdr + hdr_slot * kHdrBytes);
    };

    f32x16 acc[RT][CT];
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int j = 0; j < CT; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // fragment reads: lane (col, khalf) takes chunk 4 hi + 2 khalf + ff of activation row col (+ 32 i) and the k-half's 16 bytes of
    // the nibbles of weight row col (+ 32 j)
    const uint32_t a_row_at = (wm * (RT * 32) + col) * 128, a_swz = (col >> 1) & 7;
    uint32_t q_at[CT], hdr_at[CT];
#pragma unroll
    for (int j = 0; j < CT; ++j) {
        const uint32_t r = wn * (CT * 32) + j * 32 + col;
        q_at[j] = kQsAt + r * 32 + ((khalf ^ ((r >> 3) & 1)) * 16);
        hdr_at[j] = kHdrAt + r * 16;
    }

    struct { uint32_t low, high; } kc{0x000f000fu, 0x00f000f0u};  // kept in registers: as literals they would double the size of every mask instruction
    asm volatile("" : "+s"(kc.low), "+s"(kc.high));
    float d[CT], dmin[CT];
    uint32_t sc[CT][2], mn[CT][2];  // eight scales and eight minima per weight row, one per byte
    u32x4 raw[CT];                  // the lane's 16 bytes of the step's pair of sub-blocks, per column tile: low nibbles are sub-block 2 P, high nibbles 2 P + 1
    // activation fragments of the k16 group at work and of the one after it; with one column tile per wave a fragment serves
    // one MFMA only, and its register is refilled for the next group right behind that MFMA instead (half the registers)
    constexpr bool kRolling = CT == 1;
    f16x8 af[kRolling ? 1 : 2][RT];

    // The four k16 groups of a step are (low, high nibbles) x (first, second eight columns of the lane's sixteen).
    auto read_a = [&](uint32_t step, int g, f16x8 (&to)[RT]) {
        const uint8_t* slab = lds_raw + (step % kRing) * kSlabBytes;
        const uint32_t chunk = ((4 * (g / 2) + 2 * khalf + (g % 2)) ^ a_swz) * 16;
#pragma unroll
        for (int i = 0; i < RT; ++i) to[i] = *reinterpret_cast<const f16x8*>(slab + a_row_at + i * (32 * 128) + chunk);
    };
    // The lane's byte position of row tile 0 of a group's fragments, as one opaque register per group: the row tiles then are
    // immediate offsets of the read. Left to fold the slot's offset (up to 64 KB) and the row tile's into one constant, the
    // compiler overflows the 16-bit offset field and keeps a separate address register for every fragment of a step.
    auto group_at = [&](uint32_t step, int g) {
        uint32_t at = a_row_at + (((4 * (g / 2) + 2 * khalf + (g % 2)) ^ a_swz) * 16) + (step % kRing) * kSlabBytes;
        asm volatile("" : "+v"(at));
        return at;
    };
    auto read_a_one = [&](uint32_t at, int i) { return *reinterpret_cast<const f16x8*>(lds_raw + at + i * (32 * 128)); };
    // What a step needs before its first MFMA: its nibbles, the activation fragments of its first group, and at the first
    // pair of a super-block the rows' scales and minima.
    auto front = [&](uint32_t step, auto first_pair, u32x4 (&nibbles)[CT]) {
        if constexpr (decltype(first_pair)::value) {
            const uint8_t* hdr = lds_raw + ((step / 4) % kHdrStages) * kHdrBytes;
#pragma unroll
            for (int j = 0; j < CT; ++j) {
                RawHdrQ4 words;
                words.words = *reinterpret_cast<const uint4*>(hdr + hdr_at[j]);
                words.dm = 0;
                const HdrQ4 h = decode_hdr_q4k<B_Q4K_RAW>(words);
                d[j] = h.d; dmin[j] = h.dmin;
                sc[j][0] = h.sc[0]; sc[j][1] = h.sc[1]; mn[j][0] = h.mn[0]; mn[j][1] = h.mn[1];
            }
        }
        const uint8_t* qs = lds_raw + (step % kRing) * kQsBytes;
#pragma unroll
        for (int j = 0; j < CT; ++j) nibbles[j] = *reinterpret_cast<const u32x4*>(qs + q_at[j]);
        if constexpr (!kRolling) read_a(step, 0, af[0]);
    };

    // One step. The workgroup's barrier does not sit between two steps but before a step's last group: by then a wave has
    // every byte of the step in registers, so the step's ring slot can be given to the requests of step + 3, and the bytes of
    // step + 1, asked for two steps ago, have landed in every wave's view after the barrier. The last group's MFMAs then
    // cover the barrier, the requests and the next step's front; at the boundary between two steps nothing waits.
    auto step_fn = [&](uint32_t step, auto p_tag) {
        constexpr int P = decltype(p_tag)::value;  // the pair of sub-blocks of the super-block: step % 4
        float scale[CT], offset[CT];
        u32x4 next_raw[CT];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int hi = g / 2, ff = g % 2;
            // the activation fragments of a group are read one group ahead: their LDS latency passes behind the unpacking
            if (!kRolling && g < 3) read_a(step, g + 1, af[(g + 1) % 2]);
            if (g == 3) {
                // Younger than the requests of step + 1 are those of step + 2: the slab's pieces, the nibbles, and the headers
                // when step + 2 begins a super-block.
                lds_barrier_after_loads<kSlabPieces + QN + (P == 2 ? 1 : 0)>();
                request(step + 3);
                if constexpr (!kRolling) front(step + 1, std::bool_constant<P == 3>{}, next_raw);
            }
            if (ff == 0) {
                // sub-block 2 P + hi; weight = half(d * sc * q - dmin * mn), the f32 value rounded once
#pragma unroll
                for (int j = 0; j < CT; ++j) {
                    const uint32_t s4 = sc[j][P / 2], m4 = mn[j][P / 2];
                    constexpr int B = (P % 2) * 2;
                    const float s8 = hi == 0 ? byte_as_float<B>(s4) : byte_as_float<B + 1>(s4);
                    const float m8 = hi == 0 ? byte_as_float<B>(m4) : byte_as_float<B + 1>(m4);
                    scale[j] = (d[j] * s8) * (hi == 0 ? 16777216.0f : 1048576.0f);  // a power of two: no rounding
                    offset[j] = -(dmin[j] * m8);
                }
            }
            // A word holds four codes, one nibble of each byte; bytes (0, 2), then (1, 3), are masked out where they are: two halves
            // whose only set bits are a code's. Eight columns come out in the order (0, 2, 1, 3, 4, 6, 5, 7), the activations' order.
            // At most two column tiles at a time, so that only two weight fragments are alive at once.
            constexpr int JB = CT >= 2 ? 2 : 1;
#pragma unroll
            for (int j0 = 0; j0 < CT; j0 += JB) {
                f16x8 b[JB];
#pragma unroll
                for (int jj = 0; jj < JB; ++jj) {
                    const int j = j0 + jj;
                    u32x4 packed;
#pragma unroll
                    for (int w = 0; w < 2; ++w) {
                        const uint32_t word = raw[j][2 * ff + w], mask = hi == 0 ? kc.low : kc.high;
                        packed[2 * w] = two_weights(word & mask, scale[j], offset[j]);
                        packed[2 * w + 1] = two_weights((word >> 8) & mask, scale[j], offset[j]);
                    }
                    b[jj] = __builtin_bit_cast(f16x8, packed);
                }
                // with one column tile the step's last unpacking has just freed the nibbles' registers: the next step's go there
                if constexpr (kRolling) if (g == 3) front(step + 1, std::bool_constant<P == 3>{}, raw);
                uint32_t next_at = 0;
                if constexpr (kRolling) next_at = g < 3 ? group_at(step, g + 1) : group_at(step + 1, 0);
#pragma unroll
                for (int i = 0; i < RT; ++i) {
#pragma unroll
                    for (int jj = 0; jj < JB; ++jj)
                        acc[i][j0 + jj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[kRolling ? 0 : g % 2][i], b[jj], acc[i][j0 + jj], 0, 0, 0);
                    // the next group's fragment into the register this MFMA has read (after the barrier of the last group:
                    // the next step's first group)
                    if constexpr (kRolling) af[0][i] = read_a_one(next_at, i);
                }
            }
        }
        if constexpr (!kRolling) {
#pragma unroll
            for (int j = 0; j < CT; ++j) raw[j] = next_raw[j];
        }
        // A wave issues in order: eight MFMAs in a row hold it for eight times the matrix pipe's 32 cycles, with its own
        // unpacking waiting behind them. Interleaved, one MFMA then four vector instructions (and an LDS read every other
        // time), the unpacking of the next group runs in the shadow of this group's MFMAs.
#pragma unroll
        for (int k = 0; k < 4 * RT * CT; ++k) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, CT == 1 ? 2 : RT * CT > 8 ? 3 : 4, 0);
            if (CT == 1 || k % 2 == 0) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
    };

    request(0);
    request(1);
    request(2);
    lds_barrier_after_loads<2 * (kSlabPieces + QN)>();  // step 0 has landed; the requests of steps 1 and 2 are the younger ones
    front(0, std::true_type{}, raw);
    if constexpr (kRolling) {
        const uint32_t at = group_at(0, 0);
#pragma unroll
        for (int i = 0; i < RT; ++i) af[0][i] = read_a_one(at, i);
    }
    for (uint32_t b = 0; b < bpr; ++b) {
        step_fn(b * 4 + 0, std::integral_constant<int, 0>{});
        step_fn(b * 4 + 1, std::integral_constant<int, 1>{});
        step_fn(b * 4 + 2, std::integral_constant<int, 2>{});
        step_fn(b * 4 + 3, std::integral_constant<int, 3>{});
    }
    wait_all_loads();  // the last steps requested buffers that nobody reads: they must have landed before the LDS is given away

    // ---- epilogue. Accumulator v of tile (i, j): row 32 i + 8 (v / 4) + 4 khalf + v % 4 of the wave's rows, weight row col of column tile j
    uint32_t biggest = 0;  // the largest result's bits without the sign: anything not finite shows at the end
    const uint32_t wave_m0 = m0 + wm * (RT * 32), wave_n0 = n0 + wn * (CT * 32);
    const bool whole = wave_n0 + CT * 32 <= a.n && reinterpret_cast<uintptr_t>(a.out) % 16 == 0 && a.out_stride % 16 == 0;  // uniform
    __syncthreads();  // every wave has left the rings, and every request into them has landed: the LDS is the epilogue's
    if (whole) {
        // The wave's results go out as whole 16-byte pieces, neighbouring lanes along a row, after a turn through LDS that the
        // wave has to itself (16 or 18 KB: a few row tiles at a time; a row pitch of 16 bytes
        // more than the row keeps the column-wise writes and the row-wise reads off each other's banks). A lane storing
        // its own 2- or 4-byte results one by one, 128 stores, took a fifth of the kernel's time.
        constexpr int kRegion = CT == 1 && WAVES == 4 ? 12 * 1024 : WAVES == 8 ? 16 * 1024 : 16 * 1024 + 2048;
        uint8_t* const mine = lds_raw + wave * kRegion;
        static_assert(WAVES * kRegion <= int(sizeof(lds_raw)));
        auto pass = [&](auto bf16_tag, auto first_tag) {
            constexpr bool BF16 = decltype(bf16_tag)::value;
            constexpr int first_tile = decltype(first_tag)::value;
            constexpr int kTiles = CT == 1 ? (BF16 ? 4 : 2) : (BF16 ? 8 : 4) / CT, kElem = BF16 ? 2 : 4, kPitch = CT * 32 * kElem + 16;
            static_assert(kTiles * 32 * kPitch <= kRegion && first_tile + kTiles <= RT);
#pragma unroll
            for (int t = 0; t < kTiles; ++t) {
                const int i = first_tile + t;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const uint32_t r = t * 32 + 8 * (v / 4) + 4 * khalf + (v % 4);
#pragma unroll
                    for (int j = 0; j < CT; ++j) {
                        const float val = acc[i][j][v];
                        const uint32_t vb = __float_as_uint(val), magnitude = vb & 0x7fffffffu;
                        biggest = biggest > magnitude ? biggest : magnitude;
                        uint8_t* at = mine + r * kPitch + (j * 32 + col) * kElem;
                        if constexpr (BF16) *reinterpret_cast<uint16_t*>(at) = uint16_t((vb + 0x7fffu + ((vb >> 16) & 1u)) >> 16);
                        else *reinterpret_cast<float*>(at) = val;
                    }
                }
            }
            // written and read back by this wave only: LDS serves a wave's requests in order
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            constexpr int kPieces = CT * 32 * kElem / 16;                    // 16-byte pieces per row
            constexpr int kRounds = kTiles * 32 * kPieces / kWave;      // pieces per lane
#pragma unroll
            for (int q = 0; q < kRounds; ++q) {
                const uint32_t c = q * kWave + lane, r = c / kPieces, piece = c % kPieces;
                const uint4 data = *reinterpret_cast<const uint4*>(mine + r * kPitch + piece * 16);
                const uint32_t row = wave_m0 + first_tile * 32 + r;
                if (row < a.m)
                    *reinterpret_cast<uint4*>(static_cast<uint8_t*>(a.out) + uint64_t(row) * a.out_stride + uint64_t(wave_n0) * kElem + piece * 16) = data;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        };
        // four row tiles at a time as bf16, two as f32 (with two column tiles per wave; twice that with four, and four and two with one)
        constexpr int kTilesB = CT == 1 ? 4 : 8 / CT, kTilesF = CT == 1 ? 2 : 4 / CT;
        auto passes = [&]<int... I>(auto bf16_tag, std::integer_sequence<int, I...>) {
            (pass(bf16_tag, std::integral_constant<int, I * (decltype(bf16_tag)::value ? kTilesB : kTilesF)>{}), ...);
        };
        if (a.out_bf16) passes(std::true_type{}, std::make_integer_sequence<int, RT / kTilesB>{});
        else passes(std::false_type{}, std::make_integer_sequence<int, RT / kTilesF>{});
    } else {
        // a ragged column tile or rows that 16 bytes do not align: element by element
#pragma unroll
        for (int i = 0; i < RT; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t row = wave_m0 + i * 32 + 8 * (v / 4) + 4 * khalf + (v % 4);
                if (row >= a.m) continue;
                uint8_t* orow = static_cast<uint8_t*>(a.out) + uint64_t(row) * a.out_stride;
#pragma unroll
                for (int j = 0; j < CT; ++j) {
                    const uint32_t n = wave_n0 + j * 32 + col;
                    if (n >= a.n) continue;
                    const float val = acc[i][j][v];
                    const uint32_t vb = __float_as_uint(val), magnitude = vb & 0x7fffffffu;
                    biggest = biggest > magnitude ? biggest : magnitude;
                    if (a.out_bf16) reinterpret_cast<uint16_t*>(orow)[n] = uint16_t((vb + 0x7fffu + ((vb >> 16) & 1u)) >> 16);
                    else reinterpret_cast<float*>(orow)[n] = val;
                }
            }
        }
    }
    publish_error(biggest >= 0x7f800000u ? uint32_t(TSP_ERRBIT_NONFINITE) : 0u, a.error_word);
}

}  // namespace

namespace tsp {

bool dense_tall_takes(uint32_t tokens, uint32_t rows, uint32_t columns, uint64_t matrix_bytes) {
    return tokens >= 512 && rows >= 256 && columns % 256 == 0 && columns >= 256 && matrix_bytes < (1ull << 32) &&
           uint64_t(tokens) * columns * 2 < (1ull << 32);
}

int launch_dense_tall(const DenseTallArgs& a, hipStream_t s) {
    static std::atomic<uint64_t> seen{0};
    static int units[64];
    int device = 0;
    if (setup_pending(seen, &device)) {
        int n = 0;
        TSP_HIP(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device));
        units[device] = n >= 1 ? n : 1;
        setup_done(seen, device);
    }
    // 256-row tiles only where one round of them keeps nearly every compute unit busy (2048 x 8192 results on 256 units): there
    // they are a few percent faster. Elsewhere 128-row tiles, two workgroups to a unit, lose less to the last, partly filled
    // round, and a second round of 256-row tiles cannot start behind the first one's epilogue as a second workgroup can.
    const uint32_t n_tiles = (a.n + 255) / 256, cus = uint32_t(units[device]);
    const uint32_t tall = n_tiles * ((a.m + 255) / 256), low = n_tiles * ((a.m + 127) / 128);
    const uint32_t narrow = ((a.n + 127) / 128) * ((a.m + 127) / 128);
    if (a.m < 1024 && low < cus) {
        // too few 128 x 256 tiles for the chip: 128 x 128 tiles, one workgroup of four waves each
        TSP_LAUNCH("gemm_dense_tall", s, (dense_tall_kernel<4, 1, 4, 128><<<(narrow + 7) / 8 * 8, 256, 0, s>>>(a)));
    } else if (tall <= cus && uint64_t(tall) * 10 >= uint64_t(cus) * 9) {
        TSP_LAUNCH("gemm_dense_tall", s, (dense_tall_kernel<8, 1, 8><<<(tall + 7) / 8 * 8, 512, 0, s>>>(a)));
    } else {
        TSP_LAUNCH("gemm_dense_tall", s, (dense_tall_kernel<4, 2, 4><<<(low + 7) / 8 * 8, 256, 0, s>>>(a)));
    }
    return launch_status("dense_tall");
}

}  // namespace tsp
