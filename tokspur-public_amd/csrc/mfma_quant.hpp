// Shared pieces of the matrix-core kernels: vector types, the LDS-only barrier, and the unpacking of K-quant blocks
// into MFMA B fragments of exact integer products (sc * q for Q4_K, sc * (q - 32) for Q6_K) as packed halves.
#pragma once
#include "decode.hpp"

namespace tsp {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

enum BKind : int { B_Q4K_RAW = 0, B_Q4K_PLANAR = 1, B_Q6K_PLANAR = 2 };

// Workgroup barrier that waits for this wave's LDS traffic only. __syncthreads() also drains every outstanding
// global load, which would serialise the prefetch of the next K step behind the barrier.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
// The same, after all but the YOUNGEST vector-memory operations of this wave have completed (they complete in issue
// order): for data that a direct global -> LDS load is bringing in, which no register dependency waits for.
template <int YOUNGEST>
__device__ __forceinline__ void lds_barrier_after_loads() {
    static_assert(YOUNGEST >= 0 && YOUNGEST < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(YOUNGEST) : "memory");
}
// 16 bytes per lane from global memory straight into LDS at lds_base + 16 * lane (lds_base uniform over the wave).
// The compiler does not know this load: it counts in vmcnt like any other, so waits the compiler places for its own
// loads are only ever longer than needed, and whoever reads the bytes waits for them with lds_barrier_after_loads.
__device__ __forceinline__ void load_to_lds_16(const void* src, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(src) : "memory", "m0");
}
// The same with the global address as a uniform base (scalar registers) plus a 32-bit byte offset per lane.
__device__ __forceinline__ void load_to_lds_16(const void* uniform_base, uint32_t lane_offset, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(lane_offset), "s"(uniform_base) : "memory", "m0");
}
__device__ __forceinline__ uint32_t lds_address(const void* p) {
    return uint32_t(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)p));
}
__device__ __forceinline__ void wait_all_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

__device__ __forceinline__ f16x2 as_h2(uint32_t bits) { return __builtin_bit_cast(f16x2, bits); }
__device__ __forceinline__ uint32_t as_u32(f16x2 v) { return __builtin_bit_cast(uint32_t, v); }
__device__ __forceinline__ f16x2 splat(float v) { const _Float16 h = _Float16(v); return f16x2{h, h}; }
// one rounding per lane: the products below are only exact as fused multiply-adds
__device__ __forceinline__ f16x2 fma2(f16x2 a, f16x2 b, f16x2 c) { return __builtin_elementwise_fma(a, b, c); }

// Bytes (b0, b1) resp. (b2, b3) of `codes` into the low bytes of two f16 lanes whose high bytes are `hi`.
__device__ __forceinline__ uint32_t spread01(uint32_t codes, uint32_t hi) { return __builtin_amdgcn_perm(hi, codes, 0x04010400u); }
__device__ __forceinline__ uint32_t spread23(uint32_t codes, uint32_t hi) { return __builtin_amdgcn_perm(hi, codes, 0x04030402u); }

// Eight codes 0..15 (one per byte of c0, c1) times the integer scale: (1024 + q) * sc - 1024 * sc, exact in f16.
__device__ __forceinline__ f16x8 scaled8_q4(uint32_t c0, uint32_t c1, f16x2 sc, f16x2 bias) {
    constexpr uint32_t K = 0x64646464u;  // 0x64xx = 1024 + xx
    const f16x2 p0 = fma2(as_h2(spread01(c0, K)), sc, bias), p1 = fma2(as_h2(spread23(c0, K)), sc, bias);
    const f16x2 p2 = fma2(as_h2(spread01(c1, K)), sc, bias), p3 = fma2(as_h2(spread23(c1, K)), sc, bias);
    return f16x8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
}

// Eight int8 quants (two dwords) as exact halves: q ^ 0x80 = q + 128 in 0..255, 0x6400 | u = 1024 + u, minus 1152.
__device__ __forceinline__ f16x8 quants8(uint32_t w0, uint32_t w1) {
    constexpr uint32_t K = 0x64646464u;
    const uint32_t u0 = w0 ^ 0x80808080u, u1 = w1 ^ 0x80808080u;
    const f16x2 off = splat(-1152.0f);
    const f16x2 p0 = as_h2(spread01(u0, K)) + off, p1 = as_h2(spread23(u0, K)) + off;
    const f16x2 p2 = as_h2(spread01(u1, K)) + off, p3 = as_h2(spread23(u1, K)) + off;
    return f16x8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
}

// ---------------------------------------------------------------- Q4_K operands
struct HdrQ4 { uint32_t sc[2], mn[2]; float d, dmin; };  // eight 6-bit scales and minima, one per byte

// The header of super-block b of a row, as loaded: for planes the 16 bytes of scales and minima and the word holding d and dmin,
// for GGUF rows the block's first 16 bytes (d, dmin, the 12 packed bytes). Kept apart from its decoding so that a kernel
// can request a header a step ahead and touch the bytes only when it needs them: any arithmetic on a loaded register makes
// the compiler wait for the load on the spot, and with it for every request issued before it.
struct RawHdrQ4 { uint4 words; uint32_t dm; };

template <int BKIND>
__device__ __forceinline__ RawHdrQ4 fetch_hdr_q4k(const uint8_t* base, const tsp_planar_spec& s, uint64_t row, uint32_t bpr, uint32_t b) {
    const uint64_t blk = row * bpr + b;
    RawHdrQ4 r;
    if constexpr (BKIND == B_Q4K_PLANAR) {
        r.words = *reinterpret_cast<const uint4*>(base + s.sm_offset + blk * 16);
        r.dm = *reinterpret_cast<const uint32_t*>(base + s.dm_offset + blk * 4);
    } else {
        r.words = *reinterpret_cast<const uint4*>(base + blk * 144);
        r.dm = 0;
    }
    return r;
}

template <int BKIND>
__device__ __forceinline__ HdrQ4 decode_hdr_q4k(const RawHdrQ4& r) {
    HdrQ4 h;
    if constexpr (BKIND == B_Q4K_PLANAR) {
        h.sc[0] = r.words.x; h.sc[1] = r.words.y; h.mn[0] = r.words.z; h.mn[1] = r.words.w;
        h.d = half_bits_to_float(r.dm & 0xffffu); h.dmin = half_bits_to_float(r.dm >> 16);
    } else {
        const uint4 g = r.words;
        h.d = half_bits_to_float(g.x & 0xffffu); h.dmin = half_bits_to_float(g.x >> 16);
        // 12 packed bytes -> one byte per value: sub-blocks 0..3 are the low six bits of bytes 0..7, sub-blocks
        // 4..7 take four bits from bytes 8..11 and two from the top of bytes 0..7
        h.sc[0] = g.y & 0x3f3f3f3fu;
        h.mn[0] = g.z & 0x3f3f3f3fu;
        h.sc[1] = (g.w & 0x0f0f0f0fu) | ((g.y >> 2) & 0x30303030u);
        h.mn[1] = ((g.w >> 4) & 0x0f0f0f0fu) | ((g.z >> 2) & 0x30303030u);
    }
    return h;
}

template <int BKIND>
__device__ __forceinline__ HdrQ4 load_hdr_q4k(const uint8_t* base, const tsp_planar_spec& s, uint64_t row, uint32_t bpr, uint32_t b) {
    return decode_hdr_q4k<BKIND>(fetch_hdr_q4k<BKIND>(base, s, row, bpr, b));
}

// Fragments of pair P: bytes 16h..16h+15 of the 32-byte pair; low nibbles (HI = 0) are sub-block 2P, high nibbles
// sub-block 2P+1. Fragment f of a half covers activation columns HI*32 + 16h + f*8 .. +8 of the 64-column slab.
template <int P, int HI>
__device__ __forceinline__ void frags_q4k(const u32x4& raw, const HdrQ4& h, f16x8 frag[2]) {
    constexpr uint32_t M4 = 0x0f0f0f0fu;
    const uint32_t sc = (h.sc[P >> 1] >> ((P & 1) * 16 + HI * 8)) & 0xffu;
    const f16x2 s2 = splat(float(sc)), bias = s2 * splat(-1024.0f);
    frag[0] = scaled8_q4((raw[0] >> (4 * HI)) & M4, (raw[1] >> (4 * HI)) & M4, s2, bias);
    frag[1] = scaled8_q4((raw[2] >> (4 * HI)) & M4, (raw[3] >> (4 * HI)) & M4, s2, bias);
}

// The same fragments with the columns of every eight in the order (0, 2, 1, 3, 4, 6, 5, 7), for activations stored in
// that order: one mask-or per pair of weights instead of a mask and two byte permutes per four. Low nibbles become
// 1024 + q, high nibbles stay in place as 1024 + 16 q and take the scale sc / 16 (exact: sc < 64).
// (w & mask) | bits is one instruction (v_and_or_b32) only when the constants sit in registers: a VOP3 instruction of
// this target takes no literal, and with two literals the compiler emits an and plus an or. The kernel therefore pins
// the three constants to registers once and hands them to the unpacking.
struct Q4Consts { uint32_t lo_mask, hi_mask, bits; };
__device__ __forceinline__ Q4Consts q4_consts() {
    Q4Consts c{0x000f000fu, 0x00f000f0u, 0x64006400u};
    asm volatile("" : "+s"(c.lo_mask), "+s"(c.hi_mask), "+v"(c.bits));
    return c;
}
template <int HI>
__device__ __forceinline__ f16x8 scaled8_q4_swapped(uint32_t w0, uint32_t w1, f16x2 sc, f16x2 bias, const Q4Consts& c) {
    const uint32_t m = HI ? c.hi_mask : c.lo_mask;
    const f16x2 p0 = fma2(as_h2((w0 & m) | c.bits), sc, bias), p1 = fma2(as_h2(((w0 >> 8) & m) | c.bits), sc, bias);
    const f16x2 p2 = fma2(as_h2((w1 & m) | c.bits), sc, bias), p3 = fma2(as_h2(((w1 >> 8) & m) | c.bits), sc, bias);
    return f16x8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
}
template <int P, int HI>
__device__ __forceinline__ void frags_q4k_swapped(const u32x4& raw, const HdrQ4& h, const Q4Consts& c, f16x8 frag[2]) {
    const uint32_t sc = (h.sc[P >> 1] >> ((P & 1) * 16 + HI * 8)) & 0xffu;
    const f16x2 s2 = splat(float(sc) * (HI ? 0.0625f : 1.0f)), bias = splat(float(sc) * (HI ? -64.0f : -1024.0f));
    frag[0] = scaled8_q4_swapped<HI>(raw[0], raw[1], s2, bias, c);
    frag[1] = scaled8_q4_swapped<HI>(raw[2], raw[3], s2, bias, c);
}

// The same unpacking with the scale set-up shared by a pair of sub-blocks: the six-bit scales of sub-blocks 2P and 2P + 1 sit
// in neighbouring bytes of the header; one byte permute puts them under 0x64 (1024 + sc as halves, side by side), one packed
// add takes the 1024 off, and two packed multiplies make (sc, sc / 16) and (-1024 sc, -64 sc): the factors and the
// offsets of the low-nibble and the high-nibble products. Four instructions per pair instead of ten per sub-block.
struct Q4ScaleConsts { uint32_t sel[2]; uint32_t k64; f16x2 off, mul, bias; };
__device__ __forceinline__ Q4ScaleConsts q4_scale_consts() {
    // selector bytes: 0..3 pick a byte of the header word, 4..7 a byte of the constant 0x64646464
    Q4ScaleConsts c{{0x04010400u, 0x04030402u}, 0x64646464u, f16x2{_Float16(-1024.0f), _Float16(-1024.0f)},
                    f16x2{_Float16(1.0f), _Float16(0.0625f)}, f16x2{_Float16(-1024.0f), _Float16(-64.0f)}};
    asm volatile("" : "+s"(c.sel[0]), "+s"(c.sel[1]), "+v"(c.k64));
    return c;
}
struct Q4PairScale { f16x2 mul, bias; };  // [0]: low nibbles (sub-block 2P), [1]: high nibbles (sub-block 2P + 1)
template <int P>
__device__ __forceinline__ Q4PairScale q4_pair_scale(uint32_t sc_lo4, uint32_t sc_hi4, const Q4ScaleConsts& c) {
    const uint32_t word = P < 2 ? sc_lo4 : sc_hi4;  // scales 0..3 | 4..7, one per byte
    const f16x2 sc = as_h2(__builtin_amdgcn_perm(c.k64, word, c.sel[P & 1])) + c.off;  // (sc[2P], sc[2P + 1])
    return Q4PairScale{sc * c.mul, sc * c.bias};
}
__device__ __forceinline__ void frags_q4k_pair(const u32x4& raw, const Q4PairScale& s, int hi, const Q4Consts& c, f16x8 frag[2]) {
    const f16x2 s2 = hi ? f16x2{s.mul[1], s.mul[1]} : f16x2{s.mul[0], s.mul[0]};
    const f16x2 bias = hi ? f16x2{s.bias[1], s.bias[1]} : f16x2{s.bias[0], s.bias[0]};
    if (hi) {
        frag[0] = scaled8_q4_swapped<1>(raw[0], raw[1], s2, bias, c);
        frag[1] = scaled8_q4_swapped<1>(raw[2], raw[3], s2, bias, c);
    } else {
        frag[0] = scaled8_q4_swapped<0>(raw[0], raw[1], s2, bias, c);
        frag[1] = scaled8_q4_swapped<0>(raw[2], raw[3], s2, bias, c);
    }
}

// B operand of the minima term: the eight integer minima, the same in both k-halves (hi and lo sums).
__device__ __forceinline__ f16x8 minima_frag(const HdrQ4& h) {
    constexpr uint32_t K = 0x64646464u;
    const f16x2 one = splat(1.0f), off = splat(-1024.0f);
    const f16x2 p0 = fma2(as_h2(spread01(h.mn[0], K)), one, off), p1 = fma2(as_h2(spread23(h.mn[0], K)), one, off);
    const f16x2 p2 = fma2(as_h2(spread01(h.mn[1], K)), one, off), p3 = fma2(as_h2(spread23(h.mn[1], K)), one, off);
    return f16x8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
}

// ---------------------------------------------------------------- Q6_K operands (planes ql / qh / sc / d)
struct RawQ6 { u32x4 la, lb, qh; uint32_t sc[2]; };  // one section: low nibbles of quarters 0/2 and 1/3, high bit pairs, 8 sub-scales

// Quarter Q of the section (elements Q*32 .. Q*32+31): this lane's 16 bytes are elements Q*32 + 16h + 0..15, all in
// the 16-weight group 2Q + h. Fragment f covers activation columns Q*32 + 16h + f*8 .. +8 of the section.
template <int Q>
__device__ __forceinline__ void frags_q6k(const RawQ6& r, uint32_t khalf, f16x8 frag[2]) {
    // A code c = low nibble | two high bits << 4 becomes the half 0x5400 | c << 4 = 64 + c, and (64 + c) * sc - 96 * sc =
    // (c - 32) * sc in one fused multiply-add. The half is put together from its two bytes, four weights at a time: the low
    // byte is the nibble << 4, the high byte 0x54 | the two high bits, and a byte permute pairs them up; the six-bit code
    // itself is never formed (that took a shift and an or per pair of weights more).
    constexpr uint32_t MH = 0xf0f0f0f0u, M2 = 0x03030303u;
    uint32_t K = 0x54545454u;
    asm("" : "+v"(K));  // in a vector register: with two scalar constants (x & M2) | K is two instructions, not one v_and_or_b32
    const u32x4& l = (Q & 1) ? r.lb : r.la;
    const uint32_t g = 2 * Q + khalf;
    const int sc = int(int8_t((r.sc[g >> 2] >> ((g & 3) * 8)) & 0xffu));
    const f16x2 s2 = splat(float(sc)), bias = s2 * splat(-96.0f);
    f16x2 p[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t low = Q < 2 ? (l[i] << 4) & MH : l[i] & MH;
        const uint32_t high = ((Q == 0 ? r.qh[i] : r.qh[i] >> (2 * Q)) & M2) | K;  // bits 2Q..2Q+1 of every byte of qh
        p[2 * i] = fma2(as_h2(__builtin_amdgcn_perm(high, low, 0x05010400u)), s2, bias);      // weights 0, 1 of the four
        p[2 * i + 1] = fma2(as_h2(__builtin_amdgcn_perm(high, low, 0x07030602u)), s2, bias);  // weights 2, 3
    }
    frag[0] = f16x8{p[0][0], p[0][1], p[1][0], p[1][1], p[2][0], p[2][1], p[3][0], p[3][1]};
    frag[1] = f16x8{p[4][0], p[4][1], p[5][0], p[5][1], p[6][0], p[6][1], p[7][0], p[7][1]};
}


}  // namespace tsp
