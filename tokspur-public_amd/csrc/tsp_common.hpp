// Shared host/device helpers for the gfx950 kernels. Wave size is 64 throughout.
#pragma once

#include "../../include/tokspur_hip.h"

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>

namespace tsp {

// ---------------------------------------------------------------- host-side refusals
void set_error(const char* fmt, ...);

#define TSP_REQUIRE(cond, ...)                                   \
    do {                                                         \
        if (!(cond)) { ::tsp::set_error(__VA_ARGS__); return TSP_ERR_FORMAT; } \
    } while (0)

#define TSP_HIP(call)                                                                         \
    do {                                                                                      \
        hipError_t e_ = (call);                                                               \
        if (e_ != hipSuccess) { ::tsp::set_error("%s: %s", #call, hipGetErrorString(e_)); return TSP_ERR_HIP; } \
    } while (0)

inline bool mul_overflows(uint64_t a, uint64_t b) { return a && b > UINT64_MAX / a; }

// Per-device set-up (a kernel's dynamic LDS limit is raised on the device that is current, its compute units are counted):
// `done` has one bit per device ordinal, set by setup_done() only AFTER the set-up has run. Two threads that race both run
// it, which is harmless (the calls are idempotent), and neither launches before it has run.
inline bool setup_pending(const std::atomic<uint64_t>& done, int* ordinal = nullptr) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device > 63) device = 0;
    if (ordinal) *ordinal = device;
    return (done.load(std::memory_order_acquire) & (1ull << device)) == 0;
}
inline void setup_done(std::atomic<uint64_t>& done, int device) { done.fetch_or(1ull << device, std::memory_order_release); }

inline bool ranges_overlap(const void* a, uint64_t an, const void* b, uint64_t bn) {
    const auto x = reinterpret_cast<uintptr_t>(a), y = reinterpret_cast<uintptr_t>(b);
    return an && bn && x < y + bn && y < x + an;
}

int launch_status(const char* what);

// Per-kernel timing (the engine's GraphProfile / KernelTiming, include/tokspur/graph.hpp:353-400): while a
// profile window is open every launch is bracketed by a pair of events on its own stream.
struct KernelTimer {
    KernelTimer(const char* name, hipStream_t stream);
    ~KernelTimer();
    int slot;
    hipStream_t stream;
};
extern bool g_profiling;
#define TSP_LAUNCH(name, stream, ...)                                  \
    do {                                                               \
        if (::tsp::g_profiling) {                                      \
            ::tsp::KernelTimer timer_(name, stream);                   \
            __VA_ARGS__;                                               \
        } else {                                                       \
            __VA_ARGS__;                                               \
        }                                                              \
    } while (0)

struct Encoding { uint32_t id, elements, bytes; };
const Encoding* find_encoding(uint32_t type);

// ---------------------------------------------------------------- device helpers
#if defined(__HIPCC__)

constexpr int kWave = 64;

__device__ __forceinline__ float half_bits_to_float(uint32_t bits) {
    // v_cvt_f32_f16: exact for every pattern, subnormals included (f16 denormals are always honoured).
    return __half2float(__ushort_as_half(static_cast<unsigned short>(bits)));
}

__device__ __forceinline__ bool nonfinite(float v) { return (__float_as_uint(v) & 0x7f800000u) == 0x7f800000u; }

template <int Ctrl>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), Ctrl, 0xf, 0xf, true);
    return v + __int_as_float(moved);
}

// Sum over the 64 lanes of a wave; the result is uniform (returned from scalar registers).
__device__ __forceinline__ float wave_sum(float v) {
    v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v);  // row_half_mirror
    v = dpp_add<0x140>(v);  // row_mirror -> every lane of a 16-lane row holds the row's sum
    const int bits = __float_as_int(v);
    const float a = __int_as_float(__builtin_amdgcn_readlane(bits, 0)), b = __int_as_float(__builtin_amdgcn_readlane(bits, 16));
    const float c = __int_as_float(__builtin_amdgcn_readlane(bits, 32)), d = __int_as_float(__builtin_amdgcn_readlane(bits, 48));
    return (a + b) + (c + d);
}

// 1 / (1 + e^-g) with a single exponential that never overflows: e = e^-|g| is the small one of e^g and e^-g.
__device__ __forceinline__ float sigmoid_stable(float g) {
    const float e = expf(-fabsf(g));
    return (g >= 0 ? 1.0f : e) / (1.0f + e);
}

// The same with the hardware's exponential and reciprocal (each good to about one unit in the last place): a handful of
// instructions instead of the several dozen of expf and an IEEE division, for kernels bound by their instruction count.
__device__ __forceinline__ float sigmoid_fast(float g) {
    const float e = __builtin_amdgcn_exp2f(-fabsf(g) * 1.44269504088896340736f);
    return (g >= 0 ? 1.0f : e) * __builtin_amdgcn_rcpf(1.0f + e);
}

// Largest of the wave's 64 values (NaNs are passed over, as fmaxf does); the result is uniform.
template <int Ctrl>
__device__ __forceinline__ float dpp_max(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), Ctrl, 0xf, 0xf, true);
    return fmaxf(v, __int_as_float(moved));
}
__device__ __forceinline__ float wave_largest(float v) {
    v = dpp_max<0xB1>(v);
    v = dpp_max<0x4E>(v);
    v = dpp_max<0x141>(v);
    v = dpp_max<0x140>(v);
    const int bits = __float_as_int(v);
    const float a = __int_as_float(__builtin_amdgcn_readlane(bits, 0)), b = __int_as_float(__builtin_amdgcn_readlane(bits, 16));
    const float c = __int_as_float(__builtin_amdgcn_readlane(bits, 32)), d = __int_as_float(__builtin_amdgcn_readlane(bits, 48));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

// Sum over aligned groups of 8 lanes; every lane of a group receives the group's sum.
__device__ __forceinline__ float octet_sum(float v) {
    v = dpp_add<0xB1>(v);
    v = dpp_add<0x4E>(v);
    v = dpp_add<0x141>(v);
    return v;
}

__device__ __forceinline__ uint32_t wave_or(uint32_t v) {
    for (int m = 1; m < kWave; m <<= 1) v |= __shfl_xor(v, m, kWave);
    return v;
}

// One atomic per wave, and only when some lane saw a problem.
__device__ __forceinline__ void publish_error(uint32_t bad, uint32_t* error_word) {
    if (__builtin_amdgcn_ballot_w64(bad != 0) != 0) {
        const uint32_t all = wave_or(bad);
        if (__lane_id() == 0) atomicOr(error_word, all);
    }
}

#endif  // __HIPCC__

}  // namespace tsp
