// Device-side block decoders: one weight of one block, in f32, with the arithmetic order
// (d*sc)*q - dmin*mn etc. fixed so that the result equals the engine's double-then-one-cast value
// whenever that double arithmetic is exact (every product below is exact in f32: 11-bit f16
// significands times 6/7/8-bit integers; only the final subtraction/addition rounds, once).
#pragma once

#include "tsp_common.hpp"

namespace tsp {

#if defined(__HIPCC__)

__device__ __forceinline__ uint32_t ld16(const uint8_t* p) { return uint32_t(p[0]) | (uint32_t(p[1]) << 8); }
__device__ __forceinline__ uint32_t ld32(const uint8_t* p) { return ld16(p) | (ld16(p + 2) << 16); }

// 6-bit scale and minimum of sub-block g from the 12 packed bytes of a Q4_K/Q5_K header.
__device__ __forceinline__ void k4_scale_min(const uint8_t* s12, uint32_t g, uint32_t& sc, uint32_t& mn) {
    if (g < 4) {
        sc = s12[g] & 63u;
        mn = s12[4 + g] & 63u;
    } else {
        const uint32_t j = g - 4, packed = s12[8 + j];
        sc = (packed & 15u) | ((uint32_t(s12[j]) >> 6) << 4);
        mn = (packed >> 4) | ((uint32_t(s12[4 + j]) >> 6) << 4);
    }
}

// Element `i` of one raw GGUF block of encoding T.
template <uint32_t T>
__device__ __forceinline__ float decode_element(const uint8_t* block, uint32_t i) {
    if constexpr (T == 0) {
        return __uint_as_float(ld32(block));
    } else if constexpr (T == 1) {
        return half_bits_to_float(ld16(block));
    } else if constexpr (T == 30) {
        return __uint_as_float(ld16(block) << 16);
    } else if constexpr (T == 7) {
        const uint32_t low = (uint32_t(block[8 + i % 16]) >> (4 * (i / 16))) & 15u;
        const uint32_t q = low | (((ld32(block + 4) >> i) & 1u) << 4);
        return half_bits_to_float(ld16(block)) * float(q) + half_bits_to_float(ld16(block + 2));
    } else if constexpr (T == 8) {
        return half_bits_to_float(ld16(block)) * float(int(int8_t(block[2 + i])));
    } else if constexpr (T == 12 || T == 13) {
        uint32_t sc, mn;
        k4_scale_min(block + 4, i / 32, sc, mn);
        constexpr uint32_t payload = T == 12 ? 16 : 48;
        uint32_t q = (uint32_t(block[payload + (i / 64) * 32 + i % 32]) >> (4 * ((i % 64) / 32))) & 15u;
        if constexpr (T == 13) q |= ((uint32_t(block[16 + i % 32]) >> (i / 32)) & 1u) << 4;
        const float dl = half_bits_to_float(ld16(block)) * float(sc);
        const float ml = half_bits_to_float(ld16(block + 2)) * float(mn);
        return dl * float(q) - ml;
    } else if constexpr (T == 14) {
        const uint32_t sec = i / 128, t = i % 128;
        const uint32_t low = (uint32_t(block[sec * 64 + t % 64]) >> (4 * (t / 64))) & 15u;
        const uint32_t high = (uint32_t(block[128 + sec * 32 + t % 32]) >> (2 * (t / 32))) & 3u;
        const float ds = half_bits_to_float(ld16(block + 208)) * float(int(int8_t(block[192 + i / 16])));
        return ds * float(int(low | (high << 4)) - 32);
    } else {
        static_assert(T == 20, "no decoder for this encoding");
        constexpr int alphabet[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
        const uint32_t code = (uint32_t(block[2 + i % 16]) >> (4 * (i / 16))) & 15u;
        int v = 0;
#pragma unroll
        for (int k = 0; k < 16; ++k) v = code == uint32_t(k) ? alphabet[k] : v;
        return half_bits_to_float(ld16(block)) * float(v);
    }
}

template <uint32_t T> struct BlockGeometry;
template <> struct BlockGeometry<0> { static constexpr uint32_t elements = 1, bytes = 4; };
template <> struct BlockGeometry<1> { static constexpr uint32_t elements = 1, bytes = 2; };
template <> struct BlockGeometry<30> { static constexpr uint32_t elements = 1, bytes = 2; };
template <> struct BlockGeometry<7> { static constexpr uint32_t elements = 32, bytes = 24; };
template <> struct BlockGeometry<8> { static constexpr uint32_t elements = 32, bytes = 34; };
template <> struct BlockGeometry<12> { static constexpr uint32_t elements = 256, bytes = 144; };
template <> struct BlockGeometry<13> { static constexpr uint32_t elements = 256, bytes = 176; };
template <> struct BlockGeometry<14> { static constexpr uint32_t elements = 256, bytes = 210; };
template <> struct BlockGeometry<20> { static constexpr uint32_t elements = 32, bytes = 18; };

#endif

// Calls f.template operator()<T>() for the decodable encoding `type`; false if there is none.
template <class F>
bool dispatch_encoding(uint32_t type, F&& f) {
    switch (type) {
    case 0: f.template operator()<0>(); return true;
    case 1: f.template operator()<1>(); return true;
    case 7: f.template operator()<7>(); return true;
    case 8: f.template operator()<8>(); return true;
    case 12: f.template operator()<12>(); return true;
    case 13: f.template operator()<13>(); return true;
    case 14: f.template operator()<14>(); return true;
    case 20: f.template operator()<20>(); return true;
    case 30: f.template operator()<30>(); return true;
    default: return false;
    }
}

}  // namespace tsp
