// Per-kernel event timing behind tsp_profile_begin / tsp_profile_end.
#include "tsp_common.hpp"

#include <mutex>
#include <string>
#include <vector>

namespace tsp {

bool g_profiling = false;

namespace {
struct Sample { const char* name; hipEvent_t begin, end; };
std::mutex g_mutex;
std::vector<Sample> g_samples;          // events are created once and reused across windows
size_t g_used = 0;
constexpr size_t kMaxSamples = 16384;
}  // namespace

KernelTimer::KernelTimer(const char* name, hipStream_t s) : slot(-1), stream(s) {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_used >= kMaxSamples) return;
    if (g_used == g_samples.size()) {
        Sample fresh{name, nullptr, nullptr};
        if (hipEventCreate(&fresh.begin) != hipSuccess || hipEventCreate(&fresh.end) != hipSuccess) return;
        g_samples.push_back(fresh);
    }
    g_samples[g_used].name = name;
    slot = int(g_used++);
    (void)hipEventRecord(g_samples[size_t(slot)].begin, stream);
}

KernelTimer::~KernelTimer() {
    if (slot < 0) return;
    std::lock_guard<std::mutex> lock(g_mutex);
    (void)hipEventRecord(g_samples[size_t(slot)].end, stream);
}

}  // namespace tsp

using namespace tsp;

extern "C" int tsp_profile_begin(void) {
    std::lock_guard<std::mutex> lock(g_mutex);
    g_used = 0;
    g_profiling = true;
    return TSP_OK;
}

extern "C" int tsp_profile_end(tsp_kernel_time* out, uint32_t capacity, uint32_t* count) {
    std::lock_guard<std::mutex> lock(g_mutex);
    g_profiling = false;
    std::vector<tsp_kernel_time> rows;
    for (size_t i = 0; i < g_used; ++i) {
        TSP_HIP(hipEventSynchronize(g_samples[i].end));
        float ms = 0;
        TSP_HIP(hipEventElapsedTime(&ms, g_samples[i].begin, g_samples[i].end));
        size_t at = 0;
        while (at < rows.size() && std::string(rows[at].name) != g_samples[i].name) ++at;
        if (at == rows.size()) {
            tsp_kernel_time fresh{};
            snprintf(fresh.name, sizeof fresh.name, "%s", g_samples[i].name);
            fresh.min_ms = ms;
            rows.push_back(fresh);
        }
        rows[at].launches += 1;
        rows[at].total_ms += ms;
        if (ms < rows[at].min_ms) rows[at].min_ms = ms;
    }
    g_used = 0;
    if (count) *count = uint32_t(rows.size());
    for (size_t i = 0; i < rows.size() && i < capacity; ++i) out[i] = rows[i];
    return TSP_OK;
}
