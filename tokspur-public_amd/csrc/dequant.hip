// Dequantisation to f32 on the device: the bit-exactness witness for every weight format.
// One thread per output element; consecutive threads read neighbouring bytes of one block.
#include "decode.hpp"

using namespace tsp;

namespace {

template <uint32_t T>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ blocks, float* __restrict__ out,
                                                      uint64_t nelem, uint32_t* error_word) {
    constexpr uint32_t E = BlockGeometry<T>::elements, B = BlockGeometry<T>::bytes;
    uint32_t bad = 0;
    for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < nelem; i += uint64_t(gridDim.x) * blockDim.x) {
        const float v = decode_element<T>(blocks + (i / E) * B, uint32_t(i % E));
        bad |= nonfinite(v) ? TSP_ERRBIT_NONFINITE : 0u;
        out[i] = v;
    }
    publish_error(bad, error_word);
}

// Planar v3 expert: planes of one field each, blocks in (row, block) order.
template <uint32_t T>
__global__ __launch_bounds__(256) void dequant_planar_kernel(const uint8_t* __restrict__ base, tsp_planar_spec s,
                                                             float* __restrict__ out, uint64_t nelem, uint32_t* error_word) {
    uint32_t bad = 0;
    for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < nelem; i += uint64_t(gridDim.x) * blockDim.x) {
        float v;
        if constexpr (T == 12 || T == 13) {
            const uint64_t blk = i / 256;
            const uint32_t e = uint32_t(i % 256), grp = e / 32, l = e % 32;
            uint32_t q = (uint32_t(base[s.qs_offset + blk * 128 + (grp >> 1) * 32 + l]) >> ((grp & 1u) * 4u)) & 15u;
            if constexpr (T == 13) q |= ((uint32_t(base[s.qh_offset + blk * 32 + l]) >> grp) & 1u) << 4;
            const uint8_t* sm = base + s.sm_offset + blk * 16;
            const uint8_t* dm = base + s.dm_offset + blk * 4;
            const float dl = half_bits_to_float(ld16(dm)) * float(sm[grp]);
            const float ml = half_bits_to_float(ld16(dm + 2)) * float(sm[8 + grp]);
            v = dl * float(q) - ml;
        } else if constexpr (T == 14) {
            const uint64_t blk = i / 256;
            const uint32_t e = uint32_t(i % 256), sec = e / 128, t = e % 128;
            const uint32_t low = (uint32_t(base[s.qs_offset + blk * 128 + sec * 64 + t % 64]) >> (4 * (t / 64))) & 15u;
            const uint32_t high = (uint32_t(base[s.qh_offset + blk * 64 + sec * 32 + t % 32]) >> (2 * (t / 32))) & 3u;
            const float ds = half_bits_to_float(ld16(base + s.dm_offset + blk * 2)) *
                             float(int(int8_t(base[s.sm_offset + blk * 16 + e / 16])));
            v = ds * float(int(low | (high << 4)) - 32);
        } else if constexpr (T == 7) {
            const uint64_t blk = i / 32;
            const uint32_t e = uint32_t(i % 32);
            const uint32_t low = (uint32_t(base[s.qs_offset + blk * 16 + e % 16]) >> (4 * (e / 16))) & 15u;
            const uint32_t q = low | (((ld32(base + s.qh_offset + blk * 4) >> e) & 1u) << 4);
            const uint8_t* dm = base + s.dm_offset + blk * 4;
            v = half_bits_to_float(ld16(dm)) * float(q) + half_bits_to_float(ld16(dm + 2));
        } else {
            static_assert(T == 8);
            const uint64_t blk = i / 32;
            v = half_bits_to_float(ld16(base + s.dm_offset + blk * 2)) * float(int(int8_t(base[s.qs_offset + i])));
        }
        bad |= nonfinite(v) ? TSP_ERRBIT_NONFINITE : 0u;
        out[i] = v;
    }
    publish_error(bad, error_word);
}

uint32_t grid_for(uint64_t nelem) {
    const uint64_t want = (nelem + 255) / 256;
    return uint32_t(want < 1 ? 1 : want > 65536 ? 65536 : want);
}

}  // namespace

extern "C" int tsp_dequantize(uint32_t type, const void* blocks, uint64_t nbytes, float* out, uint64_t nelem,
                              uint32_t* error_word, void* stream) {
    TSP_REQUIRE(tsp_can_decode(type), "no owned numerical decoder for this encoding");
    const auto* enc = find_encoding(type);
    TSP_REQUIRE(nelem && nelem % enc->elements == 0 && !mul_overflows(nelem / enc->elements, enc->bytes) &&
                    (nelem / enc->elements) * enc->bytes == nbytes,
                "quantized input/output size mismatch");
    TSP_REQUIRE(blocks && out && error_word, "null device pointer");
    TSP_REQUIRE(!ranges_overlap(blocks, nbytes, out, nelem * 4), "dequantize output overlaps its input");
    dispatch_encoding(type, [&]<uint32_t T>() {
        TSP_LAUNCH("dequant", static_cast<hipStream_t>(stream), dequant_kernel<T><<<grid_for(nelem), 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<const uint8_t*>(blocks), out, nelem, error_word));
    });
    return launch_status("dequantize");
}

extern "C" int tsp_dequantize_planar(const tsp_planar_spec* spec, const void* planar, float* out, uint32_t* error_word,
                                     void* stream) {
    TSP_REQUIRE(spec && planar && out && error_word, "null pointer");
    tsp_planar_spec check;
    const int rc = tsp_make_expert_spec(spec->source_type, spec->columns, spec->rows, &check);
    if (rc != TSP_OK) return rc;
    TSP_REQUIRE(std::memcmp(&check, spec, sizeof check) == 0, "planar spec does not match its own geometry");
    TSP_REQUIRE(reinterpret_cast<uintptr_t>(planar) % 16 == 0, "planar v3 experts are 16-byte aligned");
    const uint64_t nelem = uint64_t(spec->rows) * spec->columns;
    const auto* base = static_cast<const uint8_t*>(planar);
    const auto s = static_cast<hipStream_t>(stream);
    switch (spec->source_type) {
    case 12: TSP_LAUNCH("dequant_planar", s, dequant_planar_kernel<12><<<grid_for(nelem), 256, 0, s>>>(base, *spec, out, nelem, error_word)); break;
    case 13: TSP_LAUNCH("dequant_planar", s, dequant_planar_kernel<13><<<grid_for(nelem), 256, 0, s>>>(base, *spec, out, nelem, error_word)); break;
    case 14: TSP_LAUNCH("dequant_planar", s, dequant_planar_kernel<14><<<grid_for(nelem), 256, 0, s>>>(base, *spec, out, nelem, error_word)); break;
    case 7: TSP_LAUNCH("dequant_planar", s, dequant_planar_kernel<7><<<grid_for(nelem), 256, 0, s>>>(base, *spec, out, nelem, error_word)); break;
    default: TSP_LAUNCH("dequant_planar", s, dequant_planar_kernel<8><<<grid_for(nelem), 256, 0, s>>>(base, *spec, out, nelem, error_word)); break;
    }
    return launch_status("dequantize_planar");
}
