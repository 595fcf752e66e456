// tokspur::HipGraph over the C ABI of include/tokspur_hip.h. See hip_graph.hpp for the contract.
#include "hip_graph.hpp"

#include <cmath>

#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cstring>
#include <limits>
#include <thread>

#include "tokspur_hip.h"

namespace tokspur {
namespace {

void require(bool condition, const char* message) {
    if (!condition) throw FormatError(message);
}
void hip(hipError_t status, const char* what) {
    if (status != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(status));
}
// host-side refusals of the C ABI keep the engine's exception type
void check(int status) {
    if (status == TSP_OK) return;
    if (status == TSP_ERR_FORMAT) throw FormatError(tsp_last_error());
    throw std::runtime_error(tsp_last_error());
}
uint64_t checked_mul(uint64_t a, uint64_t b) {
    require(b == 0 || a <= UINT64_MAX / b, "size overflow");
    return a * b;
}
uint64_t next_owner() {
    static uint64_t counter = 0x746f6b73;
    return ++counter;
}

struct Allocation {
    void* device = nullptr;
    uint64_t bytes = 0;
    bool live = false, immutable = false;
    std::string label;
};
struct PlanarEntry {
    size_t slot;
    uint64_t offset, bytes;
    PlanarMatrixShape shape;
};

}  // namespace

struct HipGraph::Impl {
    uint64_t owner = next_owner();
    uint64_t budget = 0, live_bytes = 0, peak_bytes = 0, allocations = 0;
    std::vector<Allocation> slots;  // never recycled
    std::vector<PlanarEntry> planar;
    std::vector<PlanarEntry> q8;  // registered dense Q8_0 matrices: shape.kind holds the row layout
    std::thread::id thread = std::this_thread::get_id();
    hipStream_t stream = nullptr;
    hipEvent_t started = nullptr, finished = nullptr;
    uint32_t* error_word = nullptr;
    bool encoding = false, locked = false, topk_prepared = false;
    uint64_t dispatches = 0;
    std::chrono::steady_clock::time_point wall_start;
    // scratch sized while idle by the prepare_* calls
    void* union_meta = nullptr;
    void* nax_workspace = nullptr;
    uint64_t nax_workspace_bytes = 0;
    void* dense_workspace = nullptr;
    uint64_t dense_workspace_bytes = 0;
    void* grouped_workspace = nullptr;
    uint64_t grouped_workspace_bytes = 0;
    void* q8_workspace = nullptr;
    uint64_t q8_workspace_bytes = 0;
    uint32_t prepared_gate_up = 0, prepared_down = 0;
    bool router_batch = false, router_batch_prepared = false;
    // per-operator timing: boundary b is recorded on the stream before operator b; the batch's end closes the last one
    struct Mark { const char* kernel; uint32_t encoding; std::array<uint32_t, 4> shape; };
    uint32_t profile_capacity = 0;
    uint64_t profile_payload = 0;
    std::vector<hipEvent_t> boundaries;  // profile_capacity + 1 once configured
    std::vector<Mark> marks;
    GraphProfile profile;

    void same_thread() const { require(std::this_thread::get_id() == thread, "GPU graph used from another thread"); }
    void idle() const {
        same_thread();
        require(!encoding, "GPU graph operation requires an idle graph");
    }
    void active(const char* kernel, uint32_t type = uint32_t(-1), std::array<uint32_t, 4> shape = {}) {
        same_thread();
        require(encoding, "GPU graph operator outside begin/submit");
        if (profile_capacity) {
            require(dispatches < profile_capacity && marks.size() == dispatches, "GPU profiler dispatch bookkeeping failed");
            marks.push_back({kernel, type, shape});  // reserved while idle: no allocation here
            hip(hipEventRecord(boundaries[dispatches], stream), "hipEventRecord");
        }
        ++dispatches;
    }
    void drop_profile() {
        profile.mode = ProfileMode::disabled;
        profile.timings_valid = profile.cpu_clock_is_mach = false;
        profile.gpu_tick_nanoseconds = profile.cpu_clock_mismatch_fraction = profile.sampled_milliseconds = 0;
        profile.kernels.clear();  // keeps its reserved capacity
        marks.clear();
    }
    void collect_profile(double gpu_ms, double wall_ms) {
        require(marks.size() == dispatches, "GPU counter mark/dispatch bookkeeping differs");
        const double unavailable = std::numeric_limits<double>::quiet_NaN();
        const bool spans = gpu_ms > 0 && wall_ms > 0;
        const double mismatch = spans ? std::abs(gpu_ms - wall_ms) / wall_ms : unavailable;
        profile.mode = ProfileMode::dispatch_boundary;
        profile.timings_valid = profile_calibration_valid(1.0, mismatch);
        profile.gpu_tick_nanoseconds = profile.timings_valid ? 1.0 : unavailable;
        profile.cpu_clock_mismatch_fraction = mismatch;
        profile.sampled_milliseconds = profile.timings_valid ? 0 : unavailable;
        uint64_t previous = 1;
        for (size_t i = 0; i < marks.size(); ++i) {
            float to_end = 0;  // boundary i + 1, or the batch's end for the last operator
            hip(hipEventElapsedTime(&to_end, started, i + 1 < marks.size() ? boundaries[i + 1] : finished), "hipEventElapsedTime");
            const uint64_t end = std::max(previous, uint64_t(1) + uint64_t(std::llround(std::max(0.0, double(to_end)) * 1e6)));
            if (i == 0) {
                float to_start = 0;
                hip(hipEventElapsedTime(&to_start, started, boundaries[0]), "hipEventElapsedTime");
                previous = uint64_t(1) + uint64_t(std::llround(std::max(0.0, double(to_start)) * 1e6));
            }
            const uint64_t start = std::min(previous, end);
            const double ms = profile.timings_valid ? double(end - start) / 1e6 : unavailable;
            profile.kernels.push_back({marks[i].kernel, marks[i].encoding, marks[i].shape, start, end, ms});
            profile.sampled_milliseconds += ms;
            previous = end;
        }
    }
    const Allocation& allocation(const GpuView& v, bool writable = false) const {
        require(v.owner == owner && v.slot < slots.size() && slots[v.slot].live, "released or foreign GPU view");
        const Allocation& a = slots[v.slot];
        require(v.offset <= a.bytes && v.bytes <= a.bytes - v.offset, "GPU view out of bounds");
        require(!writable || !a.immutable, "immutable GPU view used as a destination");
        return a;
    }
    uint8_t* device(const GpuView& v, bool writable = false) const { return static_cast<uint8_t*>(allocation(v, writable).device) + v.offset; }
    void charge(uint64_t bytes) {
        require(bytes > 0 && bytes <= budget - std::min(budget, live_bytes), "GPU graph byte budget exceeded");
        live_bytes += bytes;
        peak_bytes = std::max(peak_bytes, live_bytes);
    }
    GpuView make(uint64_t bytes, std::string label, bool immutable) {
        charge(bytes);
        void* p = nullptr;
        const hipError_t status = hipMalloc(&p, bytes);
        if (status != hipSuccess) { live_bytes -= bytes; hip(status, "hipMalloc"); }
        slots.push_back({p, bytes, true, immutable, std::move(label)});
        ++allocations;
        return {owner, slots.size() - 1, 0, bytes};
    }
    void* raw(uint64_t bytes) {  // internal scratch: charged like any other allocation
        charge(bytes);
        void* p = nullptr;
        const hipError_t status = hipMalloc(&p, bytes);
        if (status != hipSuccess) { live_bytes -= bytes; hip(status, "hipMalloc"); }
        ++allocations;
        return p;
    }
    // internal scratch kept or grown while idle (nothing in flight reads it): preparing twice, or for a second layer of
    // another shape, is as harmless as it is in the engine, whose prepare_* calls only build pipelines (graph.mm:4468)
    void grow(void*& scratch, uint64_t& have, uint64_t need) {
        if (need <= have) return;
        if (scratch) {
            hip(hipFree(scratch), "hipFree");
            live_bytes -= have;
            scratch = nullptr;
            have = 0;
        }
        scratch = raw(need);
        have = need;
    }
    static bool overlaps(const GpuView& a, const GpuView& b) {
        return a.slot == b.slot && a.offset < b.offset + b.bytes && b.offset < a.offset + a.bytes;
    }
    const PlanarEntry* planar_of(const GpuView& v) const {
        for (const auto& e : planar)
            if (e.slot == v.slot && e.offset == v.offset && e.bytes == v.bytes) return &e;
        return nullptr;
    }
    // rows of `columns` floats, `stride` bytes apart, inside the view
    void rows_fit(const GpuRowsF32& r, const char* message) const {
        require(r.rows >= 1 && r.columns >= 1 && r.stride_bytes >= uint64_t(r.columns) * 4 && r.stride_bytes % 4 == 0 &&
                    r.view.bytes >= uint64_t(r.rows - 1) * r.stride_bytes + uint64_t(r.columns) * 4,
                message);
    }
};

// include/tokspur/graph.hpp:433 `MetalGraph(library_path, byte_budget)`: the engine loads its compiled kernels from that
// path. Here they are linked into libtokspur_hip.so, so the path is not opened; a caller's construction code runs unchanged.
HipGraph::HipGraph(const std::string& library_path, uint64_t byte_budget) : HipGraph(byte_budget) { (void)library_path; }

HipGraph::HipGraph(uint64_t byte_budget) : impl_(std::make_unique<Impl>()) {
    require(byte_budget > 0, "GPU graph byte budget must be positive");
    require(tsp_abi_version() >= 1, "tokspur HIP library too old");
    impl_->budget = byte_budget;
    hip(hipStreamCreate(&impl_->stream), "hipStreamCreate");
    hip(hipEventCreate(&impl_->started), "hipEventCreate");
    hip(hipEventCreate(&impl_->finished), "hipEventCreate");
    hip(hipMalloc(reinterpret_cast<void**>(&impl_->error_word), 256), "hipMalloc");
    hip(hipMemset(impl_->error_word, 0, 256), "hipMemset");
}

HipGraph::~HipGraph() {
    if (!impl_) return;
    (void)hipStreamSynchronize(impl_->stream);
    for (auto& a : impl_->slots)
        if (a.live) (void)hipFree(a.device);
    for (void* p : {impl_->union_meta, impl_->nax_workspace, impl_->dense_workspace, impl_->grouped_workspace, impl_->q8_workspace, static_cast<void*>(impl_->error_word)})
        if (p) (void)hipFree(p);
    for (hipEvent_t e : impl_->boundaries) (void)hipEventDestroy(e);
    (void)hipEventDestroy(impl_->started);
    (void)hipEventDestroy(impl_->finished);
    (void)hipStreamDestroy(impl_->stream);
}

// ------------------------------------------------------------------ storage
GpuView HipGraph::zeros(uint64_t bytes, std::string label) {
    impl_->idle();
    const GpuView v = impl_->make(bytes, std::move(label), false);
    hip(hipMemset(impl_->device(v), 0, bytes), "hipMemset");
    return v;
}

GpuView HipGraph::upload(std::span<const std::byte> data, std::string label, bool immutable) {
    impl_->idle();
    require(!data.empty(), "empty GPU upload");
    const GpuView v = impl_->make(data.size(), std::move(label), immutable);
    hip(hipMemcpy(impl_->slots[v.slot].device, data.data(), data.size(), hipMemcpyHostToDevice), "hipMemcpy");
    return v;
}

GpuView HipGraph::slice(GpuView buffer, uint64_t offset, uint64_t bytes) const {
    (void)impl_->allocation(buffer);
    require(bytes > 0 && offset <= buffer.bytes && bytes <= buffer.bytes - offset, "GPU slice out of bounds");
    return {buffer.owner, buffer.slot, buffer.offset + offset, bytes};
}

void HipGraph::write(GpuView destination, std::span<const std::byte> data) {
    impl_->idle();
    require(data.size() == destination.bytes, "GPU write size mismatch");
    hip(hipMemcpy(impl_->device(destination, true), data.data(), data.size(), hipMemcpyHostToDevice), "hipMemcpy");
}

std::vector<std::byte> HipGraph::read(GpuView source) const {
    std::vector<std::byte> out(source.bytes);
    read(source, out);
    return out;
}

void HipGraph::read(GpuView source, std::span<std::byte> destination) const {
    impl_->idle();
    require(destination.size() == source.bytes, "GPU read size mismatch");
    hip(hipMemcpy(destination.data(), impl_->device(source), source.bytes, hipMemcpyDeviceToHost), "hipMemcpy");
}

void HipGraph::release(GpuView full_buffer) {
    impl_->idle();
    const Allocation& a = impl_->allocation(full_buffer);
    require(full_buffer.offset == 0 && full_buffer.bytes == a.bytes, "release requires the full buffer view");
    for (const auto& e : impl_->planar) require(e.slot != full_buffer.slot, "registered planar matrices stay resident");
    for (const auto& e : impl_->q8) require(e.slot != full_buffer.slot, "registered Q8_0 matrices stay resident");
    hip(hipFree(a.device), "hipFree");
    Allocation& slot = impl_->slots[full_buffer.slot];
    impl_->live_bytes -= slot.bytes;
    slot.live = false;
    slot.device = nullptr;
}

GraphMemory HipGraph::memory() const { return {impl_->budget, impl_->live_bytes, impl_->peak_bytes, impl_->allocations, impl_->profile_payload}; }

// include/tokspur/graph.hpp:503 (src/graph.mm:2669-2750)
ProfileMode HipGraph::configure_profiling(uint32_t capacity) {
    auto& p = *impl_; p.idle();
    require(capacity <= 16384, "GPU profiling capacity limit");
    const auto release = [&p] {
        for (hipEvent_t e : p.boundaries) (void)hipEventDestroy(e);
        p.boundaries.clear();
        p.live_bytes -= p.profile_payload;
        p.profile_payload = 0;
        p.profile_capacity = 0;
        p.drop_profile();
    };
    if (!capacity) { release(); return ProfileMode::disabled; }
    constexpr uint32_t chunk = 2048;  // the engine sizes its sample buffers per 2048 dispatches, whole pages each
    uint64_t payload = 0;
    for (uint32_t first = 0; first < capacity; first += chunk) payload += (uint64_t(std::min(chunk, capacity - first)) * 16 + 4095) / 4096 * 4096;
    require(payload <= p.budget - std::min(p.budget, p.live_bytes) + p.profile_payload, "GPU counter payload exceeds graph budget");
    release();
    std::vector<hipEvent_t> fresh;
    fresh.reserve(size_t(capacity) + 1);
    for (uint32_t i = 0; i <= capacity; ++i) {
        hipEvent_t e = nullptr;
        const hipError_t status = hipEventCreate(&e);
        if (status != hipSuccess) {
            for (hipEvent_t made : fresh) (void)hipEventDestroy(made);
            hip(status, "hipEventCreate");
        }
        fresh.push_back(e);
    }
    p.boundaries = std::move(fresh);
    p.marks.reserve(capacity);
    p.profile.kernels.reserve(capacity);
    p.profile_capacity = capacity;
    p.profile_payload = payload;
    p.live_bytes += payload;
    p.peak_bytes = std::max(p.peak_bytes, p.live_bytes);
    ++p.allocations;
    return ProfileMode::dispatch_boundary;
}
const GraphProfile& HipGraph::last_profile() const { impl_->idle(); return impl_->profile; }

std::string HipGraph::device_name() const {
    int device = 0;
    hip(hipGetDevice(&device), "hipGetDevice");
    hipDeviceProp_t props{};
    hip(hipGetDeviceProperties(&props, device), "hipGetDeviceProperties");
    return props.name[0] ? std::string(props.name) : std::string(props.gcnArchName);
}

void HipGraph::validate_disjoint(std::span<const GpuView> inputs, std::span<const GpuView> destinations) const {
    for (const auto& d : destinations) {
        (void)impl_->allocation(d, true);
        for (const auto& i : inputs) {
            (void)impl_->allocation(i);
            require(!Impl::overlaps(d, i), "unsupported GPU buffer alias");
        }
    }
    for (size_t a = 0; a < destinations.size(); ++a)
        for (size_t b = a + 1; b < destinations.size(); ++b) require(!Impl::overlaps(destinations[a], destinations[b]), "unsupported GPU buffer alias");
}

// ------------------------------------------------------------------ planners of grouped_mm / dense_mm_q8
namespace {
GroupedMmPlan plan_from(const tsp_grouped_mm_plan_t& c, const char* kernel) {
    GroupedMmPlan plan;
    static_assert(sizeof(GroupedMmArgs) == sizeof(tsp_grouped_mm_args_t), "argument blocks differ");
    std::memcpy(&plan.args, &c.args, sizeof plan.args);
    plan.matrix_bytes = c.matrix_bytes;
    plan.indices_bytes = c.indices_bytes;
    plan.input_bytes = c.input_bytes;
    plan.output_bytes = c.output_bytes;
    plan.token_map_bytes = c.token_map_bytes;
    plan.counts_bytes = c.counts_bytes;
    plan.tasks_bytes = c.tasks_bytes;
    plan.grid_x = c.grid_x;
    plan.grid_y = c.grid_y;
    plan.kernel = kernel;
    return plan;
}
}  // namespace

const char* grouped_mm_kernel(uint32_t encoding, PrefillWeightLayout layout) {
    require(grouped_mm_takes(encoding, layout) && layout != PrefillWeightLayout::planar_v3,
            encoding == 7 || encoding == 8 || encoding == 12 || encoding == 13 ? "grouped mm layout/encoding mismatch" : "grouped mm encoding");
    return "graph_grouped_mm";
}
const char* dense_mm_q8_kernel(PrefillWeightLayout layout) {
    (void)grouped_mm_kernel(8, layout);
    return "graph_dense_mm_q8";
}
GroupedMmPlan grouped_mm_plan(uint32_t encoding, PrefillWeightLayout layout, uint32_t columns, uint32_t rows, uint32_t experts, uint32_t selected,
                              uint32_t tokens, uint64_t input_stride_bytes, uint64_t output_stride_bytes, bool broadcast, bool allow_nax_2k) {
    tsp_grouped_mm_plan_t c{};
    check(tsp_grouped_mm_plan(encoding, uint32_t(layout), columns, rows, experts, selected, tokens, input_stride_bytes, output_stride_bytes, broadcast,
                              allow_nax_2k, &c));
    return plan_from(c, grouped_mm_kernel(encoding, layout));
}
GroupedMmPlan dense_mm_q8_plan(PrefillWeightLayout layout, uint32_t columns, uint32_t rows, uint32_t tokens, uint64_t input_stride_bytes,
                               uint64_t output_stride_bytes, bool allow_nax_2k) {
    tsp_grouped_mm_plan_t c{};
    check(tsp_dense_mm_q8_plan(uint32_t(layout), columns, rows, tokens, input_stride_bytes, output_stride_bytes, allow_nax_2k, &c));
    return plan_from(c, dense_mm_q8_kernel(layout));
}

// ------------------------------------------------------------------ Pack v3 registration
void HipGraph::register_planar_matrix(GpuView matrix, PlanarMatrixShape shape) {
    impl_->idle();
    require(!impl_->locked, "planar matrices are registered before the first batch");
    const Allocation& a = impl_->allocation(matrix);
    require(a.immutable, "planar matrix must be an immutable view");
    require(reinterpret_cast<uintptr_t>(impl_->device(matrix)) % 16 == 0, "planar matrix requires 16-byte alignment");
    require(shape.experts >= 1 && shape.experts <= 4096 && shape.kind >= 2 && shape.kind <= TSP_KIND_Q6K_PLANAR_X, "planar matrix kind mismatch");
    const bool coloc = shape.kind >= 2 && shape.kind <= 7;
    const uint32_t expected = shape.kind <= 3 ? 12u : shape.kind <= 5 ? 13u : shape.kind <= 7 ? 8u : shape.kind == 8 ? 7u : shape.kind == 9 ? 8u : 14u;
    require(shape.source_type == expected, "planar matrix kind does not match its source type");
    tsp_planar_spec spec{};
    check(tsp_make_expert_spec(shape.source_type, shape.columns, shape.rows, &spec));
    // a co-located tensor holds half of the experts as [gate_e, up_e] pairs
    require(!coloc || shape.experts % 2 == 0, "co-located gate/up tensors hold an even number of experts");
    const uint64_t want = coloc ? checked_mul(checked_mul(shape.experts / 2, 2), spec.planar_expert_bytes) : checked_mul(shape.experts, spec.planar_expert_bytes);
    require(matrix.bytes == want, "planar matrix byte span mismatch");
    for (const auto& e : impl_->planar)
        require(!Impl::overlaps(matrix, {impl_->owner, e.slot, e.offset, e.bytes}), "planar matrix overlaps a registered matrix");
    impl_->planar.push_back({matrix.slot, matrix.offset, matrix.bytes, shape});
}

// include/tokspur/graph.hpp:468 `register_q8_matrix` (src/graph.mm:9001-9019): a dense Q8_0 matrix announced before the first
// batch, in GGUF rows or q8_lanes_v1 rows (the two have the same byte span). The checks are the engine's: immutable view,
// whole rows of 34-byte blocks, no overlap with a registered matrix.
void HipGraph::register_q8_matrix(GpuView matrix, uint32_t columns, uint32_t rows, PrefillWeightLayout layout) {
    impl_->idle();
    require(!impl_->locked, "Q8_0 matrices are registered before the first batch");
    const Allocation& a = impl_->allocation(matrix);
    require(a.immutable, "Q8_0 matrix must be an immutable view");
    require(layout == PrefillWeightLayout::gguf || layout == PrefillWeightLayout::q8_lanes_v1, "dense Q8_0 GEMM layout");
    require(columns >= 32 && columns % 32 == 0 && columns <= 65536 && rows >= 1 && rows <= 1000000, "Q8_0 matrix geometry mismatch");
    require(matrix.bytes == checked_mul(checked_mul(rows, columns / 32), 34), "Q8_0 matrix byte span mismatch");
    for (const auto& e : impl_->q8) require(!Impl::overlaps(matrix, {impl_->owner, e.slot, e.offset, e.bytes}), "Q8_0 matrix overlaps a registered matrix");
    impl_->q8.push_back({matrix.slot, matrix.offset, matrix.bytes, {8, uint32_t(layout), columns, rows, 1}});
}
uint64_t HipGraph::q8_matrix_count() const { return impl_->q8.size(); }

uint64_t HipGraph::planar_matrix_count() const { return impl_->planar.size(); }

std::optional<PlanarMatrixShape> HipGraph::planar_matrix_shape(GpuView matrix) const {
    const PlanarEntry* e = impl_->planar_of(matrix);
    return e ? std::optional<PlanarMatrixShape>(e->shape) : std::nullopt;
}

void HipGraph::prepare_planar_moe_v3(uint32_t gate_up_encoding, uint32_t down_encoding, bool prepare_nax, uint32_t max_nax_tokens,
                                     uint32_t max_experts, uint32_t max_selected, uint32_t max_channels, uint32_t max_hidden) {
    impl_->idle();
    require((gate_up_encoding == 12 || gate_up_encoding == 13 || gate_up_encoding == 8) && (down_encoding == 7 || down_encoding == 8 || down_encoding == 14),
            "unsupported planar v3 MoE encodings");
    require(max_nax_tokens >= 1 && max_nax_tokens <= 2048 && max_experts >= 2 && max_experts <= 512 && max_selected >= 1 && max_selected <= 16 &&
                max_channels >= 256 && max_hidden >= 256,
            "planar v3 MoE preparation bounds mismatch");
    if (!impl_->union_meta) impl_->union_meta = impl_->raw(9280);
    if (prepare_nax) {
        const uint32_t channels = (max_channels + 255) / 256 * 256, hidden = (max_hidden + 255) / 256 * 256;
        const uint64_t bytes = tsp_planar_nax_shared_workspace_bytes(max_nax_tokens, max_selected, max_experts, channels, hidden);  // room for an always-on expert's rows too
        impl_->grow(impl_->nax_workspace, impl_->nax_workspace_bytes, bytes);
    }
    impl_->prepared_gate_up = gate_up_encoding;
    impl_->prepared_down = down_encoding;
}

void HipGraph::prepare_dense_mm(uint32_t max_tokens, uint32_t max_columns) {
    impl_->idle();
    require(max_tokens >= 1 && max_tokens <= 65536 && max_columns >= 256 && max_columns <= 65536, "dense dequant-GEMM preparation bounds mismatch");
    const uint64_t bytes = tsp_dense_mm_workspace_bytes(max_tokens, (max_columns + 255) / 256 * 256);
    impl_->grow(impl_->dense_workspace, impl_->dense_workspace_bytes, bytes);
}

// ------------------------------------------------------------------ batches
void HipGraph::begin() {
    impl_->idle();
    impl_->locked = true;
    impl_->encoding = true;
    impl_->dispatches = 0;
    impl_->drop_profile();
    hip(hipEventRecord(impl_->started, impl_->stream), "hipEventRecord");
    // with a profile asked for, the GPU's clock and the host's start the batch together: the stream is idle here, so the wait is short
    if (impl_->profile_capacity) hip(hipEventSynchronize(impl_->started), "hipEventSynchronize");
    impl_->wall_start = std::chrono::steady_clock::now();
}

void HipGraph::abort() {
    impl_->same_thread();
    require(impl_->encoding, "no GPU batch to abort");
    // launches already enqueued cannot be recalled: drain them, then drop whatever they flagged
    hip(hipStreamSynchronize(impl_->stream), "hipStreamSynchronize");
    hip(hipMemset(impl_->error_word, 0, 4), "hipMemset");
    impl_->encoding = false;
    impl_->drop_profile();
}

BatchResult HipGraph::submit() {
    impl_->same_thread();
    require(impl_->encoding, "no GPU batch to submit");
    hip(hipEventRecord(impl_->finished, impl_->stream), "hipEventRecord");
    hip(hipStreamSynchronize(impl_->stream), "hipStreamSynchronize");
    const double wall_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - impl_->wall_start).count();
    impl_->encoding = false;
    uint32_t word = 0;
    hip(hipMemcpy(&word, impl_->error_word, 4, hipMemcpyDeviceToHost), "hipMemcpy");
    if (word) {
        hip(hipMemset(impl_->error_word, 0, 4), "hipMemset");  // later batches are unaffected
        impl_->drop_profile();
        throw FormatError("GPU graph produced nonfinite values or invalid gates");
    }
    float gpu_ms = 0;
    hip(hipEventElapsedTime(&gpu_ms, impl_->started, impl_->finished), "hipEventElapsedTime");
    if (impl_->profile_capacity) impl_->collect_profile(gpu_ms, wall_ms);
    return {impl_->dispatches, wall_ms, gpu_ms};
}

// ------------------------------------------------------------------ operators
void HipGraph::gemv(uint32_t encoding, GpuView matrix, GpuView input, GpuView output, uint32_t columns, uint32_t rows) {
    auto& p = *impl_; p.active("graph_quantized_gemv", encoding, {columns, rows, 0, 0});
    require(input.bytes == uint64_t(columns) * 4 && output.bytes == uint64_t(rows) * 4, "GEMV vector byte span mismatch");
    const std::array in{matrix, input};
    validate_disjoint(in, std::array{output});
    const PlanarEntry* planar = p.planar_of(matrix);
    check(tsp_gemv(encoding, planar ? TSP_LAYOUT_PLANAR_V3 : TSP_LAYOUT_GGUF, p.device(matrix), matrix.bytes, reinterpret_cast<const float*>(p.device(input)),
                   reinterpret_cast<float*>(p.device(output, true)), columns, rows, p.error_word, p.stream));
}

void HipGraph::gemv_rows(uint32_t encoding, GpuView matrix, GpuRowsF32 input, GpuRowsF32 output) {
    auto& p = *impl_; p.active("graph_quantized_gemv_rows", encoding, {input.columns, output.columns, input.rows, 0});
    p.rows_fit(input, "GEMV rows geometry mismatch");
    p.rows_fit(output, "GEMV rows geometry mismatch");
    require(input.rows == output.rows, "GEMV rows geometry mismatch");
    validate_disjoint(std::array{matrix, input.view}, std::array{output.view});
    check(tsp_gemv_rows(encoding, TSP_LAYOUT_GGUF, p.device(matrix), matrix.bytes, reinterpret_cast<const float*>(p.device(input.view)), input.stride_bytes,
                        reinterpret_cast<float*>(p.device(output.view, true)), output.stride_bytes, input.rows, input.columns, output.columns,
                        p.error_word, p.stream));
}

namespace {
uint64_t floats(const GpuView& v) {
    require(v.bytes % 4 == 0 && v.bytes / 4 <= 0xffffffffull, "graph float view byte span");
    return v.bytes / 4;
}
}  // namespace

bool HipGraph::commit_partial() {
    auto& p = *impl_;
    p.same_thread();
    require(p.encoding, "GPU graph operator outside begin/submit");
    return p.dispatches != 0;
}

void HipGraph::rms(GpuView input, GpuView gains, GpuView output, uint32_t group_width, float epsilon) {
    auto& p = *impl_; p.active("graph_rms");
    const uint64_t count = floats(input);
    require(group_width && count % group_width == 0 && group_width <= 65536 && floats(output) == count &&
                (floats(gains) == count || floats(gains) == group_width) && std::isfinite(epsilon) && epsilon > 0,
            "graph RMS shape/epsilon mismatch");
    validate_disjoint(std::array{input, gains}, std::array{output});
    check(tsp_rms(reinterpret_cast<const float*>(p.device(input)), reinterpret_cast<const float*>(p.device(gains)), reinterpret_cast<float*>(p.device(output, true)),
                  count, group_width, gains.bytes == uint64_t(group_width) * 4 && count != group_width, epsilon, p.error_word, p.stream));
}
void HipGraph::rms_sigmoid_gate(GpuView input, GpuView gains, GpuView gate, GpuView output, uint32_t group_width, float epsilon) {
    auto& p = *impl_; p.active("graph_rms_sigmoid_gate");
    const uint64_t count = floats(input);
    require(group_width && count % group_width == 0 && group_width <= 65536 && floats(gate) == count && floats(output) == count &&
                (floats(gains) == count || floats(gains) == group_width) && std::isfinite(epsilon) && epsilon > 0,
            "graph RMS sigmoid gate shape/epsilon mismatch");
    validate_disjoint(std::array{input, gains, gate}, std::array{output});
    check(tsp_rms_sigmoid_gate(reinterpret_cast<const float*>(p.device(input)), reinterpret_cast<const float*>(p.device(gains)),
                               reinterpret_cast<const float*>(p.device(gate)), reinterpret_cast<float*>(p.device(output, true)), count, group_width,
                               gains.bytes == uint64_t(group_width) * 4 && count != group_width, epsilon, p.error_word, p.stream));
}
void HipGraph::activate(GpuView input, GpuView output, Activation kind, float scale) {
    auto& p = *impl_; p.active("graph_activate");
    const uint64_t count = floats(input);
    require(floats(output) == count && uint32_t(kind) <= 3 && std::isfinite(scale), "graph activation shape/mode mismatch");
    // the output may be the input itself, not a view that merely overlaps it: the C ABI refuses that
    check(tsp_activate(reinterpret_cast<const float*>(p.device(input)), reinterpret_cast<float*>(p.device(output, true)), count, uint32_t(kind), scale,
                       p.error_word, p.stream));
}
void HipGraph::multiply(GpuView input, GpuView gate, GpuView output, bool sigmoid_gate) {
    auto& p = *impl_; p.active("graph_multiply");
    const uint64_t count = floats(input);
    require(floats(gate) == count && floats(output) == count, "graph multiplication shape mismatch");
    check(tsp_multiply(reinterpret_cast<const float*>(p.device(input)), reinterpret_cast<const float*>(p.device(gate)),
                       reinterpret_cast<float*>(p.device(output, true)), count, sigmoid_gate, p.error_word, p.stream));
}
void HipGraph::residual_read(GpuView normalized, GpuView scores, GpuView inject, GpuView output, GpuView scales, uint32_t branches, uint32_t channels) {
    auto& p = *impl_; p.active("graph_residual_read");
    require(branches && branches <= 64 && channels && channels <= 65536 && floats(normalized) == checked_mul(branches, channels) &&
                floats(scores) == floats(normalized) && floats(inject) == branches && floats(output) == channels && floats(scales) == branches,
            "graph residual-read shape mismatch");
    validate_disjoint(std::array{normalized, scores, inject}, std::array{output, scales});
    check(tsp_residual_read(reinterpret_cast<const float*>(p.device(normalized)), reinterpret_cast<const float*>(p.device(scores)),
                            reinterpret_cast<const float*>(p.device(inject)), reinterpret_cast<float*>(p.device(output, true)),
                            reinterpret_cast<float*>(p.device(scales, true)), branches, channels, p.error_word, p.stream));
}
void HipGraph::residual_write(GpuView streams, GpuView input, GpuView scales, GpuView destination) {
    auto& p = *impl_; p.active("graph_residual_write");
    const uint64_t channels = floats(input), branches = floats(scales);
    require(branches && branches <= 64 && channels && channels <= 65536 && floats(streams) == checked_mul(branches, channels) && floats(destination) == floats(streams),
            "graph residual-write shape mismatch");
    validate_disjoint(std::array{input, scales}, std::array{destination});
    check(tsp_residual_write(reinterpret_cast<const float*>(p.device(streams)), reinterpret_cast<const float*>(p.device(input)),
                             reinterpret_cast<const float*>(p.device(scales)), reinterpret_cast<float*>(p.device(destination, true)), uint32_t(branches),
                             uint32_t(channels), p.error_word, p.stream));
}

void HipGraph::configure_moe_router_f32_batch(bool enabled) {
    auto& p = *impl_; p.idle();
    require(!p.router_batch_prepared && !p.locked, "router FP32 batch selection is fixed before preparation or any batch");
    p.router_batch = enabled;
}
bool HipGraph::moe_router_f32_batch_enabled() const { impl_->same_thread(); return impl_->router_batch; }
const char* HipGraph::moe_router_f32_projection_kernel() const {
    impl_->same_thread();
    return impl_->router_batch ? moe_router_f32_kernel : "graph_quantized_gemv";
}
void HipGraph::prepare_moe_router_f32_batch() {
    auto& p = *impl_; p.idle();
    p.router_batch_prepared = true;
}
void HipGraph::moe_router_f32_batch(GpuView matrix, GpuRowsF32 input, GpuRowsF32 output) {
    auto& p = *impl_; p.active(moe_router_f32_kernel, uint32_t(-1), {input.columns, output.columns, input.rows, 0});
    require(p.router_batch && p.router_batch_prepared, "router FP32 batch requires explicit idle selection/preparation and direct batches");
    require(input.rows == output.rows, "router FP32 batch row count mismatch");
    const auto plan = moe_router_f32_plan(input.columns, output.columns, input.rows, input.stride_bytes, output.stride_bytes, false);
    require(matrix.bytes == plan.matrix_bytes && input.view.bytes >= plan.input_bytes && output.view.bytes >= plan.output_bytes &&
                matrix.offset % 4 == 0 && input.view.offset % 4 == 0 && output.view.offset % 4 == 0,
            "router FP32 batch view extent/alignment");
    validate_disjoint(std::array{matrix, input.view}, std::array{output.view});
    check(tsp_router_f32_batch(reinterpret_cast<const float*>(p.device(matrix)), reinterpret_cast<const float*>(p.device(input.view)),
                               input.stride_bytes, reinterpret_cast<float*>(p.device(output.view, true)), output.stride_bytes, input.columns,
                               output.columns, input.rows, p.error_word, p.stream));
}

void HipGraph::prepare_q8_matvec_many(uint32_t width) {
    impl_->idle();
    require(width == 1 || width == 2 || width == 4 || width == 8, "unsupported Q8-many pipeline width");
}

void HipGraph::q8_matvec_many(GpuView matrix, GpuView input, GpuView output, uint32_t columns, uint32_t rows, uint32_t width) {
    auto& p = *impl_; p.active("graph_q8_matvec_many", uint32_t(-1), {columns, rows, width, 0});
    require(input.bytes == uint64_t(columns) * width * 4 && output.bytes == uint64_t(rows) * width * 4, "Q8-many vector byte span mismatch");
    validate_disjoint(std::array{matrix, input}, std::array{output});
    check(tsp_q8_matvec_many(TSP_LAYOUT_GGUF, p.device(matrix), matrix.bytes, reinterpret_cast<const float*>(p.device(input)),
                             reinterpret_cast<float*>(p.device(output, true)), columns, rows, width, p.error_word, p.stream));
}

void HipGraph::route(GpuView logits, GpuView indices, GpuView weights, uint32_t selected, RouterMode mode, bool normalize_selected) {
    auto& p = *impl_; p.active("graph_route");
    require(logits.bytes % 4 == 0 && logits.bytes / 4 <= 4096 && indices.bytes == uint64_t(selected) * 4 && weights.bytes == uint64_t(selected) * 4,
            "graph router shape/mode mismatch");
    validate_disjoint(std::array{logits}, std::array{indices, weights});
    check(tsp_route(reinterpret_cast<const float*>(p.device(logits)), reinterpret_cast<uint32_t*>(p.device(indices, true)),
                    reinterpret_cast<float*>(p.device(weights, true)), uint32_t(logits.bytes / 4), selected, uint32_t(mode), normalize_selected,
                    p.error_word, p.stream));
}

void HipGraph::prefill_route_batch(GpuView logits, GpuView indices, GpuView weights, uint32_t experts, uint32_t selected, uint32_t tokens,
                                   RouterMode mode, bool normalize_selected) {
    auto& p = *impl_; p.active("graph_route_batch", uint32_t(-1), {experts, selected, tokens, uint32_t(mode)});
    require(logits.bytes == checked_mul(checked_mul(tokens, experts), 4) && indices.bytes == checked_mul(checked_mul(tokens, selected), 4) &&
                weights.bytes == indices.bytes,
            "prefill route batch geometry/mode mismatch");
    validate_disjoint(std::array{logits}, std::array{indices, weights});
    check(tsp_route_batch(reinterpret_cast<const float*>(p.device(logits)), reinterpret_cast<uint32_t*>(p.device(indices, true)),
                          reinterpret_cast<float*>(p.device(weights, true)), experts, selected, tokens, uint32_t(mode), normalize_selected,
                          p.error_word, p.stream));
}

void HipGraph::routed_gemv(uint32_t encoding, GpuView matrices, GpuView indices, GpuView input, GpuView output, uint32_t columns, uint32_t rows,
                           uint32_t experts, bool broadcast_input) {
    auto& p = *impl_; p.active("graph_routed_gemv", encoding, {columns, rows, experts, 0});
    require(indices.bytes % 4 == 0 && indices.bytes >= 4, "routed GEMV index span mismatch");
    const uint32_t selected = uint32_t(indices.bytes / 4);
    require(input.bytes == uint64_t(columns) * 4 * (broadcast_input ? 1 : selected) && output.bytes == uint64_t(rows) * 4 * selected,
            "routed GEMV vector byte span mismatch");
    validate_disjoint(std::array{matrices, indices, input}, std::array{output});
    check(tsp_routed_gemv(encoding, p.device(matrices), matrices.bytes, reinterpret_cast<const uint32_t*>(p.device(indices)),
                          reinterpret_cast<const float*>(p.device(input)), reinterpret_cast<float*>(p.device(output, true)), columns, rows, experts,
                          selected, broadcast_input, p.error_word, p.stream));
}

void HipGraph::swiglu(GpuView gate, GpuView up, GpuView output, float scale) {
    auto& p = *impl_; p.active("graph_swiglu", uint32_t(-1), {uint32_t(gate.bytes / 4), 0, 0, 0});
    require(gate.bytes == up.bytes && gate.bytes == output.bytes && gate.bytes % 4 == 0 && gate.bytes > 0, "graph SwiGLU shape/scale mismatch");
    (void)p.allocation(gate); (void)p.allocation(up);
    check(tsp_swiglu(reinterpret_cast<const float*>(p.device(gate)), reinterpret_cast<const float*>(p.device(up)),
                     reinterpret_cast<float*>(p.device(output, true)), gate.bytes / 4, scale, p.error_word, p.stream));
}

void HipGraph::mixture(GpuView expert_outputs, GpuView weights, GpuView shared_output, GpuView shared_logit, GpuView output) {
    auto& p = *impl_; p.active("graph_mixture");
    require(output.bytes % 4 == 0 && output.bytes > 0 && weights.bytes % 4 == 0 && weights.bytes > 0 && shared_output.bytes == output.bytes &&
                shared_logit.bytes == 4 && expert_outputs.bytes == checked_mul(output.bytes, weights.bytes / 4),
            "mixture shape mismatch");
    validate_disjoint(std::array{expert_outputs, weights, shared_output, shared_logit}, std::array{output});
    check(tsp_mixture(reinterpret_cast<const float*>(p.device(expert_outputs)), reinterpret_cast<const float*>(p.device(weights)),
                      reinterpret_cast<const float*>(p.device(shared_output)), reinterpret_cast<const float*>(p.device(shared_logit)),
                      reinterpret_cast<float*>(p.device(output, true)), uint32_t(output.bytes / 4), uint32_t(weights.bytes / 4), p.error_word, p.stream));
}

void HipGraph::prefill_mixture_batch(GpuView experts, GpuView weights, GpuView shared, GpuView shared_logit, GpuRowsF32 output, uint32_t selected) {
    auto& p = *impl_; p.active("graph_mixture_batch", uint32_t(-1), {output.columns, selected, output.rows, 0});
    p.rows_fit(output, "mixture shape mismatch");
    const uint64_t tokens = output.rows, channels = output.columns;
    require(selected >= 1 && experts.bytes == checked_mul(checked_mul(tokens * selected, channels), 4) && weights.bytes == tokens * selected * 4 &&
                shared.bytes == tokens * channels * 4 && shared_logit.bytes == tokens * 4,
            "mixture shape mismatch");
    validate_disjoint(std::array{experts, weights, shared, shared_logit}, std::array{output.view});
    check(tsp_mixture_batch(reinterpret_cast<const float*>(p.device(experts)), reinterpret_cast<const float*>(p.device(weights)),
                            reinterpret_cast<const float*>(p.device(shared)), reinterpret_cast<const float*>(p.device(shared_logit)),
                            reinterpret_cast<float*>(p.device(output.view, true)), output.stride_bytes, output.columns, selected, output.rows,
                            p.error_word, p.stream));
}

namespace {
struct PlanarTriple { PlanarMatrixShape lo, hi, dn; };
}

void HipGraph::planar_moe_gate_up_swiglu_m8(GpuView pair_lo, GpuView pair_hi, GpuView indices, GpuRowsF32 input, GpuRowsF32 expert_hidden,
                                            uint32_t experts, uint32_t selected) {
    auto& p = *impl_; p.active("planar_moe_gate_up_swiglu_m8", uint32_t(-1), {input.columns, expert_hidden.columns, experts, input.rows});
    const PlanarEntry* lo = p.planar_of(pair_lo);
    const PlanarEntry* hi = p.planar_of(pair_hi);
    require(lo && hi && p.union_meta, "planar v3 MoE requires registered matrices and prepare_planar_moe_v3");
    p.rows_fit(input, "planar v3 MoE shape or stride mismatch");
    p.rows_fit(expert_hidden, "planar v3 MoE shape or stride mismatch");
    require(lo->shape.experts == experts && hi->shape.experts == experts && input.rows >= 1 && input.rows <= 8 &&
                expert_hidden.rows == input.rows * selected && indices.bytes == uint64_t(expert_hidden.rows) * 4 &&
                input.columns == lo->shape.columns && expert_hidden.columns == lo->shape.rows,
            "planar v3 MoE shape or stride mismatch");
    validate_disjoint(std::array{pair_lo, pair_hi, indices, input.view}, std::array{expert_hidden.view});
    tsp_small_moe m{};
    m.pair_lo = p.device(pair_lo); m.pair_hi = p.device(pair_hi);
    m.gate_kind = lo->shape.kind; m.up_kind = hi->shape.kind; m.down_kind = TSP_KIND_Q8_PLANAR;
    m.channels = input.columns; m.hidden = expert_hidden.columns; m.experts = experts; m.selected = selected; m.tokens = input.rows;
    m.ids = reinterpret_cast<const uint32_t*>(p.device(indices));
    m.x = reinterpret_cast<const float*>(p.device(input.view)); m.x_stride_bytes = input.stride_bytes;
    m.h = reinterpret_cast<float*>(p.device(expert_hidden.view, true)); m.h_stride_bytes = expert_hidden.stride_bytes;
    m.union_meta = static_cast<uint32_t*>(p.union_meta); m.error_word = p.error_word;
    check(tsp_planar_moe_gate_up_swiglu_m8(&m, p.stream));
}

void HipGraph::planar_moe_routed_m8(GpuView pair_lo, GpuView pair_hi, GpuView down_weights, GpuView indices, GpuRowsF32 input,
                                    GpuRowsF32 expert_hidden, GpuRowsF32 expert_down, uint32_t experts, uint32_t selected) {
    auto& p = *impl_; p.active("planar_moe_routed_m8", uint32_t(-1), {input.columns, expert_down.columns, experts, input.rows});
    const PlanarEntry* lo = p.planar_of(pair_lo);
    const PlanarEntry* hi = p.planar_of(pair_hi);
    const PlanarEntry* dn = p.planar_of(down_weights);
    require(lo && hi && dn && p.union_meta, "planar v3 MoE requires registered matrices and prepare_planar_moe_v3");
    p.rows_fit(input, "planar v3 MoE shape or stride mismatch");
    p.rows_fit(expert_hidden, "planar v3 MoE shape or stride mismatch");
    p.rows_fit(expert_down, "planar v3 MoE shape or stride mismatch");
    require(lo->shape.experts == experts && hi->shape.experts == experts && dn->shape.experts == experts && input.rows >= 1 && input.rows <= 8 &&
                expert_hidden.rows == input.rows * selected && expert_down.rows == expert_hidden.rows &&
                indices.bytes == uint64_t(expert_hidden.rows) * 4 && input.columns == lo->shape.columns &&
                expert_hidden.columns == lo->shape.rows && dn->shape.columns == expert_hidden.columns && dn->shape.rows == expert_down.columns &&
                expert_down.columns == input.columns,
            "planar v3 MoE shape or stride mismatch");
    validate_disjoint(std::array{pair_lo, pair_hi, down_weights, indices, input.view}, std::array{expert_hidden.view, expert_down.view});
    tsp_small_moe m{};
    m.pair_lo = p.device(pair_lo); m.pair_hi = p.device(pair_hi); m.down = p.device(down_weights);
    m.gate_kind = lo->shape.kind; m.up_kind = hi->shape.kind; m.down_kind = dn->shape.kind;
    m.channels = input.columns; m.hidden = expert_hidden.columns; m.experts = experts; m.selected = selected; m.tokens = input.rows;
    m.ids = reinterpret_cast<const uint32_t*>(p.device(indices));
    m.x = reinterpret_cast<const float*>(p.device(input.view)); m.x_stride_bytes = input.stride_bytes;
    m.h = reinterpret_cast<float*>(p.device(expert_hidden.view, true)); m.h_stride_bytes = expert_hidden.stride_bytes;
    m.y = reinterpret_cast<float*>(p.device(expert_down.view, true)); m.y_stride_bytes = expert_down.stride_bytes;
    m.union_meta = static_cast<uint32_t*>(p.union_meta); m.error_word = p.error_word;
    check(tsp_planar_moe_routed_m8(&m, p.stream));
}

void HipGraph::planar_nax_grouped_moe(GpuView pair_lo, GpuView pair_hi, GpuView down_weights, GpuView indices, GpuRowsF32 input,
                                      GpuRowsF32 expert_down, GpuView token_map, GpuView counts, GpuView tasks, uint32_t experts,
                                      uint32_t selected, const SharedPlanarExpert* shared) {
    auto& p = *impl_; p.active("planar_nax_grouped_moe", uint32_t(-1), {input.columns, expert_down.columns, experts, input.rows});
    const PlanarEntry* lo = p.planar_of(pair_lo);
    const PlanarEntry* hi = p.planar_of(pair_hi);
    const PlanarEntry* dn = p.planar_of(down_weights);
    require(lo && hi && dn && p.nax_workspace, "planar v3 NAX grouped MoE requires registered matrices and prepared scratch");
    p.rows_fit(input, "planar v3 NAX grouped MoE shape or stride mismatch");
    p.rows_fit(expert_down, "planar v3 NAX grouped MoE shape or stride mismatch");
    const uint32_t tokens = input.rows;
    require(lo->shape.experts == experts && hi->shape.experts == experts && dn->shape.experts == experts && expert_down.rows == tokens * selected &&
                indices.bytes == uint64_t(tokens) * selected * 4 && input.columns == lo->shape.columns && expert_down.columns == input.columns &&
                dn->shape.columns == lo->shape.rows && dn->shape.rows == input.columns,
            "planar v3 NAX grouped MoE shape or stride mismatch");
    require(token_map.bytes >= checked_mul(checked_mul(experts, tokens), 4) && counts.bytes >= uint64_t(experts) * 4 &&
                tasks.bytes >= (2 + 2 * (uint64_t(tokens) * selected / 32 + experts)) * 4,
            "planar v3 NAX grouped MoE routing scratch too small");
    const uint64_t need = shared ? tsp_planar_nax_shared_workspace_bytes(tokens, selected, experts, input.columns, lo->shape.rows)
                                 : tsp_planar_nax_workspace_bytes(tokens, selected, experts, input.columns, lo->shape.rows);
    require(need <= p.nax_workspace_bytes, "planar v3 NAX scratch too small for requested batch");
    validate_disjoint(std::array{pair_lo, pair_hi, down_weights, indices, input.view}, std::array{expert_down.view, token_map, counts, tasks});
    tsp_grouped_moe m{};
    m.pair_lo = p.device(pair_lo); m.pair_hi = p.device(pair_hi); m.down = p.device(down_weights);
    m.gate_kind = lo->shape.kind; m.up_kind = hi->shape.kind; m.down_kind = dn->shape.kind;
    m.channels = input.columns; m.hidden = lo->shape.rows; m.experts = experts; m.selected = selected; m.tokens = tokens;
    m.ids = reinterpret_cast<const uint32_t*>(p.device(indices));
    m.x = reinterpret_cast<const float*>(p.device(input.view)); m.x_stride_bytes = input.stride_bytes;
    m.y = reinterpret_cast<float*>(p.device(expert_down.view, true)); m.y_stride_bytes = expert_down.stride_bytes;
    m.token_map = reinterpret_cast<uint32_t*>(p.device(token_map, true));
    m.counts = reinterpret_cast<uint32_t*>(p.device(counts, true));
    m.tasks = reinterpret_cast<uint32_t*>(p.device(tasks, true));
    m.workspace = p.nax_workspace; m.workspace_bytes = p.nax_workspace_bytes; m.error_word = p.error_word;
    if (!shared) {
        check(tsp_planar_nax_grouped_moe(&m, p.stream));
        return;
    }
    const PlanarEntry* sp = p.planar_of(shared->pair);
    const PlanarEntry* sd = p.planar_of(shared->down);
    require(sp && sd, "planar v3 NAX grouped MoE requires registered matrices and prepared scratch");
    p.rows_fit(shared->rows, "planar v3 NAX grouped MoE shape or stride mismatch");
    require(sp->shape.kind == lo->shape.kind && sd->shape.kind == dn->shape.kind && sp->shape.columns == lo->shape.columns &&
                sp->shape.rows == lo->shape.rows && sd->shape.columns == dn->shape.columns && sd->shape.rows == dn->shape.rows &&
                shared->rows.rows == tokens && shared->rows.columns == input.columns,
            "planar v3 NAX grouped MoE shape or stride mismatch");
    validate_disjoint(std::array{pair_lo, pair_hi, down_weights, indices, input.view, shared->pair, shared->down},
                      std::array{expert_down.view, token_map, counts, tasks, shared->rows.view});
    tsp_planar_spec gu{};
    check(tsp_make_expert_spec(12, input.columns, lo->shape.rows, &gu));
    tsp_shared_expert e{};
    e.gate = p.device(shared->pair);                                             // a co-located pair tensor holds [gate_0, up_0, gate_1, ...]
    e.up = static_cast<const uint8_t*>(e.gate) + gu.planar_expert_bytes;
    e.down = p.device(shared->down);
    e.y = reinterpret_cast<float*>(p.device(shared->rows.view, true)); e.y_stride_bytes = shared->rows.stride_bytes;
    check(tsp_planar_nax_grouped_moe_shared(&m, &e, p.stream));
}

void HipGraph::prepare_grouped_mm(uint32_t encoding, PrefillWeightLayout layout, uint32_t max_tokens, uint32_t max_selected, uint32_t max_experts,
                                  uint32_t max_columns) {
    impl_->idle();
    require(grouped_mm_takes(encoding, layout), "grouped prefill requires idle preparation and direct batches");
    require(max_tokens >= 1 && max_tokens <= 2048 && max_selected >= 1 && max_selected <= 16 && max_experts >= 1 && max_experts <= 512 &&
                max_columns >= 32 && max_columns <= 65536,
            "grouped prefill geometry mismatch");
    const uint64_t bytes = tsp_grouped_mm_workspace_bytes(max_tokens, max_selected, max_experts, (max_columns + 255) / 256 * 256, 0);
    impl_->grow(impl_->grouped_workspace, impl_->grouped_workspace_bytes, bytes);
}

void HipGraph::grouped_mm(uint32_t encoding, PrefillWeightLayout layout, GpuView matrices, GpuView indices, GpuRowsF32 input, GpuRowsF32 output,
                          GpuView token_map, GpuView counts, GpuView tasks, uint32_t experts, uint32_t selected, bool broadcast) {
    auto& p = *impl_; p.active("graph_grouped_mm", encoding, {input.columns, output.columns, experts, input.rows});
    require(p.grouped_workspace, "grouped prefill requires idle preparation and direct batches");
    require(selected && output.rows % selected == 0, "grouped prefill route-row count mismatch");
    const uint32_t tokens = output.rows / selected;
    require(input.rows == (broadcast ? tokens : output.rows), "grouped prefill input-row count mismatch");
    p.rows_fit(input, "grouped prefill buffer span or alignment is invalid");
    p.rows_fit(output, "grouped prefill buffer span or alignment is invalid");
    require(indices.bytes == uint64_t(output.rows) * 4 && token_map.bytes >= checked_mul(checked_mul(experts, tokens), 4) && counts.bytes >= uint64_t(experts) * 4 &&
                tasks.bytes >= (2 + 2 * (uint64_t(output.rows) / 32 + experts)) * 4,
            "grouped prefill buffer span or alignment is invalid");
    require(tsp_grouped_mm_workspace_bytes(tokens, selected, experts, input.columns, broadcast) <= p.grouped_workspace_bytes,
            "grouped prefill scratch too small for requested batch");
    validate_disjoint(std::array{matrices, input.view, indices}, std::array{output.view, token_map, counts, tasks});
    check(tsp_grouped_mm(encoding, uint32_t(layout), p.device(matrices), matrices.bytes, reinterpret_cast<const uint32_t*>(p.device(indices)),
                         reinterpret_cast<const float*>(p.device(input.view)), input.stride_bytes, reinterpret_cast<float*>(p.device(output.view, true)),
                         output.stride_bytes, reinterpret_cast<uint32_t*>(p.device(token_map, true)), reinterpret_cast<uint32_t*>(p.device(counts, true)),
                         reinterpret_cast<uint32_t*>(p.device(tasks, true)), input.columns, output.columns, experts, selected, tokens, broadcast,
                         p.grouped_workspace, p.grouped_workspace_bytes, p.error_word, p.stream));
}

void HipGraph::dense_mm(uint32_t encoding, PrefillWeightLayout layout, GpuView matrix, GpuRowsF32 input, GpuRowsF32 output) {
    auto& p = *impl_; p.active("graph_dense_mm", encoding, {input.columns, output.columns, 1, input.rows});
    require(p.dense_workspace, "dense dequant-GEMM requires prepare_dense_mm");
    p.rows_fit(input, "dense dequant-GEMM geometry");
    p.rows_fit(output, "dense dequant-GEMM geometry");
    require(input.rows == output.rows, "dense dequant-GEMM geometry");
    require(tsp_dense_mm_workspace_bytes(input.rows, input.columns) <= p.dense_workspace_bytes, "dense dequant-GEMM workspace too small");
    validate_disjoint(std::array{matrix, input.view}, std::array{output.view});
    check(tsp_dense_mm(encoding, uint32_t(layout), p.device(matrix), matrix.bytes, p.device(input.view), input.stride_bytes, 0,
                       p.device(output.view, true), output.stride_bytes, 0, input.rows, input.columns, output.columns, p.dense_workspace,
                       p.dense_workspace_bytes, p.error_word, p.stream));
}

void HipGraph::prepare_dense_mm_q8(PrefillWeightLayout layout, uint32_t max_tokens, uint32_t max_columns, uint32_t max_rows) {
    impl_->idle();
    require(layout == PrefillWeightLayout::gguf || layout == PrefillWeightLayout::q8_lanes_v1, "dense Q8_0 GEMM layout");
    if (max_tokens == 0 && max_columns == 0 && max_rows == 0) return;
    require(max_tokens >= 1 && max_tokens <= 65536 && max_columns >= 32 && max_columns <= 65536 && max_rows >= 1 && max_rows <= 1000000,
            "dense Q8_0 GEMM preparation bounds mismatch");
    const uint64_t bytes = tsp_dense_mm_q8_workspace_bytes(max_tokens, max_columns, max_rows);
    impl_->grow(impl_->q8_workspace, impl_->q8_workspace_bytes, bytes);
}

void HipGraph::dense_mm_q8(PrefillWeightLayout layout, GpuView matrix, GpuRowsF32 input, GpuRowsF32 output, bool) {
    auto& p = *impl_; p.active("graph_dense_mm_q8", 8, {input.columns, output.columns, input.rows, uint32_t(layout)});
    require(layout == PrefillWeightLayout::gguf || layout == PrefillWeightLayout::q8_lanes_v1, "dense Q8_0 GEMM layout");
    p.rows_fit(input, "dense Q8_0 GEMM geometry");
    p.rows_fit(output, "dense Q8_0 GEMM geometry");
    require(input.rows == output.rows && input.rows >= 1, "dense Q8_0 GEMM geometry");
    validate_disjoint(std::array{matrix, input.view}, std::array{output.view});
    if (input.rows >= 32 && input.columns % 64 == 0 && p.q8_workspace &&
        tsp_dense_mm_q8_workspace_bytes(input.rows, input.columns, output.columns) <= p.q8_workspace_bytes) {
        check(tsp_dense_mm_q8_staged(uint32_t(layout), p.device(matrix), matrix.bytes, reinterpret_cast<const float*>(p.device(input.view)),
                                     input.stride_bytes, reinterpret_cast<float*>(p.device(output.view, true)), output.stride_bytes, input.rows,
                                     input.columns, output.columns, p.q8_workspace, p.q8_workspace_bytes, p.error_word, p.stream));
        return;
    }
    check(tsp_dense_mm_q8(uint32_t(layout), p.device(matrix), matrix.bytes, reinterpret_cast<const float*>(p.device(input.view)), input.stride_bytes,
                          reinterpret_cast<float*>(p.device(output.view, true)), output.stride_bytes, input.rows, input.columns, output.columns,
                          p.error_word, p.stream));
}

void HipGraph::configure_small_gemv(uint32_t column_splits) {
    impl_->idle();
    require(column_splits == 0 || column_splits == 1 || column_splits == 4 || column_splits == 8 || column_splits == 16 || column_splits == 32,
            "small GEMV column split count");
}

void HipGraph::configure_block_gemv(uint32_t formats) {
    impl_->idle();
    require(formats <= 3, "block GEMV format mask");
}

uint64_t HipGraph::logit_topk_scratch_bytes(uint32_t max_rows, uint32_t max_vocabulary) {
    const uint64_t bytes = tsp_logit_topk_scratch_bytes(max_rows, max_vocabulary);
    require(bytes > 0, "GPU logit top-k scratch bounds mismatch");
    return bytes;
}

uint64_t HipGraph::logit_topk_output_bytes(uint32_t max_rows) {
    const uint64_t bytes = tsp_logit_topk_output_bytes(max_rows);
    require(bytes > 0, "GPU logit top-k output row count out of bounds");
    return bytes;
}

void HipGraph::prepare_logit_topk() {
    impl_->idle();
    impl_->topk_prepared = true;
}

void HipGraph::logit_topk(GpuRowsF32 logits, GpuView partial_scratch, GpuView out_rows) {
    auto& p = *impl_; p.active("logit_topk", uint32_t(-1), {logits.rows, logits.columns, 0, 64});
    require(p.topk_prepared, "GPU logit top-k requires prepared direct batches");
    p.rows_fit(logits, "GPU logit top-k geometry mismatch");
    validate_disjoint(std::array{logits.view}, std::array{partial_scratch, out_rows});
    check(tsp_logit_topk(reinterpret_cast<const float*>(p.device(logits.view)), logits.stride_bytes, logits.rows, logits.columns,
                         p.device(partial_scratch, true), partial_scratch.bytes, p.device(out_rows, true), out_rows.bytes, p.stream));
}

// ------------------------------------------------------------------ MoE compositions
namespace {
void shape_check(MoeShape s) {  // src/moe.cpp:9-12
    require(s.channels >= 1 && s.hidden >= 1 && s.experts >= 1 && s.selected >= 1 && s.selected <= s.experts && s.selected <= 64,
            "mixture sublayer shape mismatch");
}
}  // namespace

MoeScratch allocate_moe_scratch(HipGraph& graph, MoeShape shape) {
    shape_check(shape);
    const std::array<uint64_t, 10> counts{shape.experts, shape.selected, shape.selected, checked_mul(shape.hidden, shape.selected),
                                          checked_mul(shape.hidden, shape.selected), checked_mul(shape.channels, shape.selected), shape.hidden,
                                          shape.hidden, shape.channels, 1};
    std::array<GpuView, 10> views{};
    size_t made = 0;
    try {
        for (; made < counts.size(); ++made) views[made] = graph.zeros(checked_mul(counts[made], 4), "mixture scratch");
    } catch (...) {
        for (size_t i = 0; i < made; ++i) graph.release(views[i]);
        throw;
    }
    return {views[0], views[1], views[2], views[3], views[4], views[5], views[6], views[7], views[8], views[9]};
}

void release_moe_scratch(HipGraph& graph, const MoeScratch& scratch) {
    for (const auto view : scratch.views()) graph.release(view);
}

// src/grouped_mm.cpp:8-12 `layout_check`
bool grouped_mm_takes(uint32_t encoding, PrefillWeightLayout layout) {
    if (layout == PrefillWeightLayout::gguf) return encoding == 7 || encoding == 8 || encoding == 12 || encoding == 13;
    return (layout == PrefillWeightLayout::q8_lanes_v1 && encoding == 8) || (layout == PrefillWeightLayout::q51_lanes_v1 && encoding == 7);
}

bool is_planar_moe(const HipGraph& g, const MoeWeights& w, MoeShape s) {
    const auto lo = g.planar_matrix_shape(w.gate.view);
    const auto hi = g.planar_matrix_shape(w.up.view);
    const auto dn = g.planar_matrix_shape(w.down.view);
    if (!lo || !hi || !dn) return false;
    return (lo->kind == 2u || lo->kind == 4u || lo->kind == 6u) && (hi->kind == 3u || hi->kind == 5u || hi->kind == 7u) &&
           (dn->kind == 8u || dn->kind == 9u || dn->kind == 10u) && lo->source_type == w.gate.encoding && hi->source_type == w.up.encoding &&
           dn->source_type == w.down.encoding && lo->source_type == hi->source_type && lo->columns == s.channels && lo->rows == s.hidden &&
           lo->experts == s.experts && hi->columns == s.channels && hi->rows == s.hidden && hi->experts == s.experts && dn->columns == s.hidden &&
           dn->rows == s.channels && dn->experts == s.experts;
}

void encode_moe(HipGraph& graph, const MoeWeights& w, const MoeScratch& s, GpuView input, GpuView output, MoeShape shape, RouterMode mode,
                bool normalize_selected) {
    shape_check(shape);
    graph.gemv(w.router.encoding, w.router.view, input, s.logits, shape.channels, shape.experts);
    graph.route(s.logits, s.indices, s.weights, shape.selected, mode, normalize_selected);
    if (is_planar_moe(graph, w, shape)) {
        graph.planar_moe_routed_m8(w.gate.view, w.up.view, w.down.view, s.indices, {input, 1, shape.channels, uint64_t(shape.channels) * 4},
                                   {s.gate, shape.selected, shape.hidden, uint64_t(shape.hidden) * 4},
                                   {s.down, shape.selected, shape.channels, uint64_t(shape.channels) * 4}, shape.experts, shape.selected);
    } else {
        graph.routed_gemv(w.gate.encoding, w.gate.view, s.indices, input, s.gate, shape.channels, shape.hidden, shape.experts, true);
        graph.routed_gemv(w.up.encoding, w.up.view, s.indices, input, s.up, shape.channels, shape.hidden, shape.experts, true);
        graph.swiglu(s.gate, s.up, s.gate);
        graph.routed_gemv(w.down.encoding, w.down.view, s.indices, s.gate, s.down, shape.hidden, shape.channels, shape.experts, false);
    }
    graph.gemv(w.shared_gate.encoding, w.shared_gate.view, input, s.shared_gate, shape.channels, shape.hidden);
    graph.gemv(w.shared_up.encoding, w.shared_up.view, input, s.shared_up, shape.channels, shape.hidden);
    graph.swiglu(s.shared_gate, s.shared_up, s.shared_gate);
    graph.gemv(w.shared_down.encoding, w.shared_down.view, s.shared_gate, s.shared_down, shape.hidden, shape.channels);
    graph.gemv(w.shared_router.encoding, w.shared_router.view, input, s.shared_logit, shape.channels, 1);
    graph.mixture(s.down, s.weights, s.shared_down, s.shared_logit, output);
}

MoeBatchScratch allocate_moe_batch_scratch(HipGraph& graph, MoeShape shape, uint32_t tokens) {
    shape_check(shape);
    require(tokens >= 1 && tokens <= 2048, "prefill MoE token count out of bounds");
    const uint64_t routes = uint64_t(tokens) * shape.selected;
    const auto tasks_bytes = [&](uint64_t r, uint64_t experts) { return (2 + 2 * (r / 32 + experts)) * 4; };
    const std::array<uint64_t, 12> bytes{routes * 4, routes * 4, checked_mul(routes * shape.channels, 4), checked_mul(uint64_t(shape.experts) * tokens, 4),
                                         uint64_t(shape.experts) * 4, tasks_bytes(routes, shape.experts), uint64_t(tokens) * 4,
                                         checked_mul(uint64_t(tokens) * shape.channels, 4), uint64_t(2) * tokens * 4, 2 * 4, tasks_bytes(tokens, 2),
                                         uint64_t(tokens) * 4};
    std::array<GpuView, 12> v{};
    size_t made = 0;
    try {
        for (; made < bytes.size(); ++made) v[made] = graph.zeros(bytes[made], "prefill mixture scratch");
    } catch (...) {
        for (size_t i = 0; i < made; ++i) graph.release(v[i]);
        throw;
    }
    return {v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8], v[9], v[10], v[11]};
}

void release_moe_batch_scratch(HipGraph& graph, const MoeBatchScratch& s) {
    for (const auto view : {s.indices, s.weights, s.expert_down, s.token_map, s.counts, s.tasks, s.shared_indices, s.shared_down, s.shared_token_map,
                            s.shared_counts, s.shared_tasks, s.shared_logit})
        graph.release(view);
}

void encode_moe_batch(HipGraph& graph, const MoeWeights& w, const MoeBatchScratch& s, GpuView logits, GpuRowsF32 input, GpuRowsF32 output,
                      MoeShape shape, RouterMode mode, bool normalize_selected) {
    shape_check(shape);
    const uint32_t tokens = input.rows;
    graph.prefill_route_batch(logits, s.indices, s.weights, shape.experts, shape.selected, tokens, mode, normalize_selected);
    // The shared expert is expert 0 of a two-expert planar stack. Beside Q4_K / Q6_K routed experts of the same kinds it rides in
    // their two GEMM launches; otherwise it is a grouped product of its own in which every token selects expert 0
    // (shared_indices stay zero).
    const auto routed = graph.planar_matrix_shape(w.gate.view), routed_down = graph.planar_matrix_shape(w.down.view);
    const auto own = graph.planar_matrix_shape(w.shared_gate.view), own_down = graph.planar_matrix_shape(w.shared_down.view);
    const bool rides = routed && routed_down && own && own_down && routed->kind == TSP_KIND_Q4K_COLOC_GATE && own->kind == routed->kind &&
                       routed_down->kind == TSP_KIND_Q6K_PLANAR_X && own_down->kind == routed_down->kind;
    const GpuRowsF32 expert_down{s.expert_down, tokens * shape.selected, shape.channels, uint64_t(shape.channels) * 4};
    const GpuRowsF32 shared_rows{s.shared_down, tokens, shape.channels, uint64_t(shape.channels) * 4};
    if (rides) {
        const HipGraph::SharedPlanarExpert shared{w.shared_gate.view, w.shared_down.view, shared_rows};
        graph.planar_nax_grouped_moe(w.gate.view, w.up.view, w.down.view, s.indices, input, expert_down, s.token_map, s.counts, s.tasks,
                                     shape.experts, shape.selected, &shared);
    } else {
        graph.planar_nax_grouped_moe(w.gate.view, w.up.view, w.down.view, s.indices, input, expert_down, s.token_map, s.counts, s.tasks,
                                     shape.experts, shape.selected);
        graph.planar_nax_grouped_moe(w.shared_gate.view, w.shared_up.view, w.shared_down.view, s.shared_indices, input, shared_rows,
                                     s.shared_token_map, s.shared_counts, s.shared_tasks, 2, 1);
    }
    graph.gemv_rows(w.shared_router.encoding, w.shared_router.view, input, {s.shared_logit, tokens, 1, 4});
    graph.prefill_mixture_batch(s.expert_down, s.weights, s.shared_down, s.shared_logit, output, shape.selected);
}

// ------------------------------------------------------------------ encode_moe_mm_many
MoeRouterF32Plan moe_router_f32_plan(uint32_t columns, uint32_t experts, uint32_t tokens, uint64_t input_stride_bytes,
                                     uint64_t output_stride_bytes, bool engine_bounds) {
    const bool shape_ok = engine_bounds ? (columns == 2560 && experts == 512 && tokens && tokens <= 512)
                                        : (columns && columns % 32 == 0 && columns <= 65536 && experts && experts <= 65536 && tokens && tokens <= 65536);
    if (!shape_ok || input_stride_bytes < uint64_t(columns) * 4 || output_stride_bytes < uint64_t(experts) * 4 || input_stride_bytes % 16 ||
        output_stride_bytes % 16)
        throw FormatError("bounded raw FP32 router batch geometry/stride");
    const auto span = [](uint32_t rows, uint64_t stride, uint64_t last) {
        if (rows > 1 && stride > (UINT64_MAX - last) / (rows - 1)) throw FormatError("bounded raw FP32 router batch span");
        return uint64_t(rows - 1) * stride + last;
    };
    const uint64_t input = span(tokens, input_stride_bytes, uint64_t(columns) * 4), output = span(tokens, output_stride_bytes, uint64_t(experts) * 4);
    if (input > (256ull << 20) || output > (256ull << 20)) throw FormatError("bounded raw FP32 router batch span");
    return {{columns, experts, tokens, 0, input_stride_bytes, output_stride_bytes}, uint64_t(columns) * experts * 4, input, output,
            (experts + 31) / 32, (tokens + 31) / 32};
}

MoeMmManyBytes moe_mm_many_bytes(MoeShape shape, uint32_t capacity, bool allow_nax_2k) {
    shape_check(shape);
    MoeMmManyBytes b;
    check(tsp_moe_mm_many_bytes(shape.channels, shape.hidden, shape.experts, shape.selected, capacity, allow_nax_2k ? 1 : 0, b.views.data(), &b.total));
    return b;
}

MoeMmManyScratch allocate_moe_mm_many_scratch(HipGraph& graph, MoeShape shape, uint32_t capacity, bool allow_nax_2k) {
    const MoeMmManyBytes b = moe_mm_many_bytes(shape, capacity, allow_nax_2k);
    std::array<GpuView, 13> v{};
    size_t made = 0;
    try {
        for (; made < v.size(); ++made) v[made] = graph.zeros(b.views[made], "tiled mixture scratch");
    } catch (...) {
        for (size_t i = 0; i < made; ++i) graph.release(v[i]);
        throw;
    }
    return {{v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8], v[9]}, v[10], v[11], v[12], capacity};
}

void release_moe_mm_many_scratch(HipGraph& graph, const MoeMmManyScratch& scratch) {
    for (const auto view : scratch.views()) graph.release(view);
}

namespace {
// The raw-GGUF arm runs three grouped products: each takes what `grouped_mm` takes (Q4_K, Q5_K, Q5_1, Q8_0 rows and the two lane layouts).
void raw_arm_check(const MoeWeights& w, const MoeMmLayouts& l) {
    for (const auto& [matrix, layout] : {std::pair{w.gate, l.gate}, std::pair{w.up, l.up}, std::pair{w.down, l.down}})
        require(grouped_mm_takes(matrix.encoding, layout), "grouped mm layout/encoding mismatch");
}
}  // namespace

void prepare_moe_mm_many(HipGraph& graph, const MoeWeights& w, MoeShape shape, uint32_t capacity, MoeMmLayouts l) {
    shape_check(shape);
    require(capacity >= 1, "tiled MoE capacity");
    const uint32_t rows = capacity < 2048 ? capacity : 2048;
    if (is_planar_moe(graph, w, shape)) {
        graph.prepare_planar_moe_v3(w.gate.encoding, w.down.encoding, true, rows, shape.experts, shape.selected, shape.channels, shape.hidden);
    } else {
        raw_arm_check(w, l);  // refused here, while idle, rather than in the middle of a batch
        graph.prepare_grouped_mm(w.gate.encoding, l.gate, rows, shape.selected, shape.experts, shape.channels > shape.hidden ? shape.channels : shape.hidden);
    }
    graph.prepare_moe_router_f32_batch();  // src/moe_mm_many.cpp:50
    const uint32_t widest = shape.channels > shape.hidden ? shape.channels : shape.hidden;
    for (const auto layout : {l.shared_gate, l.shared_up, l.shared_down}) graph.prepare_dense_mm_q8(layout, rows, widest, widest);
}

void encode_moe_mm_many(HipGraph& g, const MoeWeights& w, const MoeMmManyScratch& s, GpuRowsF32 input, GpuRowsF32 output, MoeShape shape,
                        RouterMode mode, bool normalize_selected, MoeMmLayouts l) {
    shape_check(shape);
    const uint32_t chunk = s.capacity < 2048 ? s.capacity : 2048;
    require(chunk > 0 && input.rows >= 1 && input.rows == output.rows && input.columns == shape.channels && output.columns == shape.channels,
            "tiled MoE active rows/router mode");
    if (input.rows > chunk) {  // src/moe_mm_many.cpp:134-143
        for (uint32_t at = 0; at < input.rows; at += chunk) {
            const uint32_t n = input.rows - at < chunk ? input.rows - at : chunk;
            const GpuView in = g.slice(input.view, uint64_t(at) * input.stride_bytes, uint64_t(n - 1) * input.stride_bytes + uint64_t(input.columns) * 4);
            const GpuView out = g.slice(output.view, uint64_t(at) * output.stride_bytes, uint64_t(n - 1) * output.stride_bytes + uint64_t(output.columns) * 4);
            encode_moe_mm_many(g, w, s, {in, n, input.columns, input.stride_bytes}, {out, n, output.columns, output.stride_bytes}, shape, mode,
                               normalize_selected, l);
        }
        return;
    }
    const bool planar = is_planar_moe(g, w, shape);
    if (!planar) raw_arm_check(w, l);  // before anything is enqueued
    const MoeMmManyBytes b = moe_mm_many_bytes(shape, s.capacity, true);
    const auto all = s.views();
    for (size_t i = 0; i < all.size(); ++i) require(all[i].bytes == b.views[i], "tiled MoE scratch capacity extent");
    const uint32_t n = input.rows;
    for (const auto& r : {input, output})
        require(r.stride_bytes >= uint64_t(shape.channels) * 4 && r.stride_bytes % 16 == 0 &&
                    r.view.bytes >= uint64_t(n - 1) * r.stride_bytes + uint64_t(shape.channels) * 4,
                "tiled MoE strided row extent");
    const std::array<GpuView, 9> read{input.view, w.router.view, w.gate.view, w.up.view, w.down.view, w.shared_gate.view, w.shared_up.view,
                                      w.shared_down.view, w.shared_router.view};
    std::array<GpuView, 14> write{output.view};
    std::copy(all.begin(), all.end(), write.begin() + 1);
    g.validate_disjoint(read, write);
    // the first `per_row * n` floats of a scratch view, flat or as n rows
    try {
    const auto active = [&](GpuView v, uint64_t per_row) { return g.slice(v, 0, per_row * n * 4); };
    const auto rows = [&](GpuView v, uint32_t count, uint32_t columns) { return GpuRowsF32{g.slice(v, 0, uint64_t(count) * columns * 4), count, columns, uint64_t(columns) * 4}; };
    const GpuView logits = active(s.rows.logits, shape.experts), ids = active(s.rows.indices, shape.selected), weights = active(s.rows.weights, shape.selected);
    // src/moe_mm_many.cpp:170-177: one f32 GEMM for the chunk when selected, else one GEMV per row
    if (g.moe_router_f32_batch_enabled() && w.router.encoding == 0 && n > 1)
        g.moe_router_f32_batch(w.router.view, input, {logits, n, shape.experts, uint64_t(shape.experts) * 4});
    else
        g.gemv_rows(w.router.encoding, w.router.view, input, {logits, n, shape.experts, uint64_t(shape.experts) * 4});
    g.prefill_route_batch(logits, ids, weights, shape.experts, shape.selected, n, mode, normalize_selected);
    const GpuRowsF32 gate = rows(s.rows.gate, n * shape.selected, shape.hidden), down_rows = rows(s.rows.down, n * shape.selected, shape.channels);
    if (planar) {
        if (n <= 8) g.planar_moe_routed_m8(w.gate.view, w.up.view, w.down.view, ids, input, gate, down_rows, shape.experts, shape.selected);
        else g.planar_nax_grouped_moe(w.gate.view, w.up.view, w.down.view, ids, input, down_rows, s.token_map, s.counts, s.tasks, shape.experts, shape.selected);
    } else {
        const GpuRowsF32 up = rows(s.rows.up, n * shape.selected, shape.hidden);
        g.grouped_mm(w.gate.encoding, l.gate, w.gate.view, ids, input, gate, s.token_map, s.counts, s.tasks, shape.experts, shape.selected, true);
        g.grouped_mm(w.up.encoding, l.up, w.up.view, ids, input, up, s.token_map, s.counts, s.tasks, shape.experts, shape.selected, true);
        g.swiglu(gate.view, up.view, gate.view);
        g.grouped_mm(w.down.encoding, l.down, w.down.view, ids, gate, down_rows, s.token_map, s.counts, s.tasks, shape.experts, shape.selected, false);
    }
    const GpuRowsF32 sg = rows(s.rows.shared_gate, n, shape.hidden), su = rows(s.rows.shared_up, n, shape.hidden);
    g.dense_mm_q8(l.shared_gate, w.shared_gate.view, input, sg);
    g.dense_mm_q8(l.shared_up, w.shared_up.view, input, su);
    g.swiglu(sg.view, su.view, sg.view);
    g.dense_mm_q8(l.shared_down, w.shared_down.view, sg, rows(s.rows.shared_down, n, shape.channels));
    const GpuView shared_logit = active(s.rows.shared_logit, 1);
    g.gemv_rows(w.shared_router.encoding, w.shared_router.view, input, {shared_logit, n, 1, 4});
    g.prefill_mixture_batch(active(s.rows.down, uint64_t(shape.selected) * shape.channels), weights, active(s.rows.shared_down, shape.channels),
                            shared_logit, output, shape.selected);
    } catch (...) {  // src/moe_mm_many.cpp:282: a refusal part-way leaves no half-encoded batch behind
        g.abort();
        throw;
    }
}

}  // namespace tokspur
