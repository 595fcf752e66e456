// tokspur::HipGraph — the host side of the quantized-matmul / MoE path on one MI355X, with the operator
// interface of the engine's graph class (include/tokspur/graph.hpp:431-1168 `MetalGraph`) for this path:
// same handle types, same operator names and argument meaning, same lifecycle and error behaviour.
//
//   * buffers are `GpuView` capabilities issued by this graph (zeros / upload / slice), charged to a byte
//     budget and checked on every use; a released or foreign view is refused, never rebound
//     (graph.hpp:94-101, ledger graph.mm:1866-1893);
//   * allocation, upload, read-back and registration are legal only while the graph is idle; operators are
//     legal only between begin() and submit() / abort() (graph.mm:991-992); nothing is allocated while encoding;
//   * host-side refusals throw FormatError before anything is enqueued; device-side conditions (non-finite
//     values, bad expert ids) set a sticky word that submit() reads and turns into
//     FormatError("GPU graph produced nonfinite values or invalid gates") (graph.mm:3977-3978);
//   * one host thread and one in-order HIP stream per graph.
//
// Every operator forwards to one entry point of the C ABI in include/tokspur_hip.h.
#pragma once

#include <array>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <memory>
#include <optional>
#include <span>
#include <stdexcept>
#include <string>
#include <vector>

namespace tokspur {

// include/tokspur/gguf.hpp:16-19
class FormatError : public std::runtime_error {
public:
    using std::runtime_error::runtime_error;
};

// include/tokspur/graph.hpp:96-108
struct GpuView {
    uint64_t owner = 0;
    size_t slot = 0;
    uint64_t offset = 0;
    uint64_t bytes = 0;
};
struct GpuRowsF32 {
    GpuView view;
    uint32_t rows = 0;
    uint32_t columns = 0;
    uint64_t stride_bytes = 0;
};
// include/tokspur/graph.hpp:123-129; kind 10 (Q6_K planes) is this library's extension
struct PlanarMatrixShape {
    uint32_t source_type = 0;
    uint32_t kind = 0;
    uint32_t columns = 0;
    uint32_t rows = 0;
    uint32_t experts = 0;
};
// include/tokspur/graph.hpp:140-146 (the fields that exist without Metal)
struct GraphMemory {
    uint64_t budget = 0;
    uint64_t live_bytes = 0;
    uint64_t peak_bytes = 0;
    uint64_t allocations = 0;
    uint64_t profile_counter_payload_bytes = 0;  // what configure_profiling holds, part of live_bytes
};
// include/tokspur/graph.hpp:337-344,353-359,386-400: opt-in timing of every operator of a batch. A row of `kernels` is one
// operator call, in encoding order: the label the engine gives that operator's kernel where it has a single one, the
// operator's own name where it launches several, and the engine's encoding / shape metadata. `start` and `end` are
// nanoseconds on the GPU's event clock counted from the batch's first boundary (+ 1, so that a sample is never zero), hence
// gpu_tick_nanoseconds is 1 in a calibrated profile. Calibration compares the GPU's span of the batch with steady_clock's
// between begin() and the return of submit(): a short batch can miss the 3 % tolerance through submission latency alone;
// its raw samples are kept, its milliseconds are NaN, and the batch itself never fails on that account.
enum class ProfileMode { disabled, dispatch_boundary, encoder_boundary };
inline bool profile_calibration_valid(double tick_nanoseconds, double mismatch_fraction) {
    return std::isfinite(tick_nanoseconds) && tick_nanoseconds > 0 && std::isfinite(mismatch_fraction) && mismatch_fraction >= 0 &&
           mismatch_fraction <= 0.03;
}
struct KernelTiming {
    std::string kernel;
    uint32_t encoding;
    std::array<uint32_t, 4> shape;
    uint64_t start, end;
    double milliseconds;
};
struct GraphProfile {
    ProfileMode mode = ProfileMode::disabled;
    bool timings_valid = false;
    bool cpu_clock_is_mach = false;
    double gpu_tick_nanoseconds = 0;
    double cpu_clock_mismatch_fraction = 0;
    double sampled_milliseconds = 0;
    std::vector<KernelTiming> kernels;
};
// include/tokspur/graph.hpp:270-275
struct BatchResult {
    uint64_t dispatches = 0;
    double wall_ms = 0;
    double gpu_ms = 0;
};
// include/tokspur/routing.hpp:10, include/tokspur/grouped_mm.hpp:6 (+ the Pack v3 planes as layout 3)
enum class Activation : uint32_t { identity, silu, sigmoid, softplus };  // include/tokspur/graph.hpp:134
enum class RouterMode : uint32_t { softmax, sigmoid };
enum class PrefillWeightLayout : uint32_t { gguf = 0, q8_lanes_v1 = 1, q51_lanes_v1 = 2, planar_v3 = 3 };
// include/tokspur/sampling.hpp:21-29
struct GpuLogitTopKRow {
    uint32_t vocabulary = 0;
    uint32_t count = 0;
    uint32_t first_nonfinite_col = 0xffffffffu;
    uint32_t first_subnormal_col = 0xffffffffu;
    std::array<uint32_t, 64> ids{};
    std::array<float, 64> logits{};
};
static_assert(sizeof(GpuLogitTopKRow) == 528, "GpuLogitTopKRow ABI");

class HipGraph {
public:
    explicit HipGraph(uint64_t byte_budget);
    HipGraph(const std::string& library_path, uint64_t byte_budget);  // graph.hpp:433; the kernels are linked in, the path is not opened
    ~HipGraph();
    HipGraph(const HipGraph&) = delete;
    HipGraph& operator=(const HipGraph&) = delete;

    // ---- storage (idle only), graph.hpp:438-496
    [[nodiscard]] GpuView zeros(uint64_t bytes, std::string label);
    [[nodiscard]] GpuView upload(std::span<const std::byte> data, std::string label, bool immutable = true);
    [[nodiscard]] GpuView slice(GpuView buffer, uint64_t offset, uint64_t bytes) const;
    void write(GpuView destination, std::span<const std::byte> data);
    [[nodiscard]] std::vector<std::byte> read(GpuView source) const;
    void read(GpuView source, std::span<std::byte> destination) const;
    void release(GpuView full_buffer);
    [[nodiscard]] GraphMemory memory() const;
    // graph.hpp:503,528. Idle only; zero disables; at most 16384 operators per batch. The boundary events are charged to the
    // byte budget (16 bytes per operator in whole pages per 2048 operators, the engine's accounting) and a request beyond the
    // budget is refused with nothing changed. An operator past the capacity is refused while encoding. last_profile() is the
    // last successfully submitted batch's; begin(), abort() and a batch refused for a device error leave it empty.
    ProfileMode configure_profiling(uint32_t max_dispatches);
    [[nodiscard]] const GraphProfile& last_profile() const;
    [[nodiscard]] std::string device_name() const;
    void validate_disjoint(std::span<const GpuView> inputs, std::span<const GpuView> destinations) const;  // graph.hpp:671

    // ---- Pack v3 registration (idle only, before the first batch), graph.hpp:465-471
    void register_planar_matrix(GpuView matrix, PlanarMatrixShape shape);
    [[nodiscard]] uint64_t planar_matrix_count() const;
    void register_q8_matrix(GpuView matrix, uint32_t columns, uint32_t rows, PrefillWeightLayout layout = PrefillWeightLayout::gguf);  // graph.hpp:468
    [[nodiscard]] uint64_t q8_matrix_count() const;
    [[nodiscard]] std::optional<PlanarMatrixShape> planar_matrix_shape(GpuView matrix) const;
    void prepare_planar_moe_v3(uint32_t gate_up_encoding, uint32_t down_encoding, bool prepare_nax = true,
                               uint32_t max_nax_tokens = 2048, uint32_t max_experts = 512, uint32_t max_selected = 10,
                               uint32_t max_channels = 2560, uint32_t max_hidden = 640);
    void prepare_dense_mm(uint32_t max_tokens, uint32_t max_columns);  // workspace of dense_mm, sized while idle

    // ---- batches, graph.hpp:709-714
    void begin();
    void abort();
    [[nodiscard]] BatchResult submit();
    // graph.hpp:715-716: hands what is encoded so far to the GPU without waiting and continues the same batch. Operators are
    // launched on the graph's stream as they are encoded, so there is nothing left to hand over: true for a batch with
    // operators in it, false (and no change) for an empty one. submit() and abort() wait for every part.
    bool commit_partial();

    // ---- operators (between begin and submit)
    void gemv(uint32_t encoding, GpuView matrix, GpuView input, GpuView output, uint32_t columns, uint32_t rows);  // graph.hpp:730
    void gemv_rows(uint32_t encoding, GpuView matrix, GpuRowsF32 input, GpuRowsF32 output);                         // graph.hpp:733
    // graph.hpp:821-825: the router projection of a whole chunk as one f32 GEMM instead of one GEMV per row. Off until
    // selected; selection and preparation happen while idle, before the first use (src/graph.mm:5701-5746).
    void configure_moe_router_f32_batch(bool enabled);
    [[nodiscard]] bool moe_router_f32_batch_enabled() const;
    [[nodiscard]] const char* moe_router_f32_projection_kernel() const;
    void prepare_moe_router_f32_batch();
    void moe_router_f32_batch(GpuView matrix, GpuRowsF32 input, GpuRowsF32 output);
    void prepare_q8_matvec_many(uint32_t width);                                                                    // graph.hpp:744
    void q8_matvec_many(GpuView matrix, GpuView input, GpuView output, uint32_t columns, uint32_t rows, uint32_t width);
    void route(GpuView logits, GpuView indices, GpuView weights, uint32_t selected, RouterMode mode, bool normalize_selected);  // 1091
    void prefill_route_batch(GpuView logits, GpuView indices, GpuView weights, uint32_t experts, uint32_t selected,
                             uint32_t tokens, RouterMode mode, bool normalize_selected);                             // graph.hpp:852
    void routed_gemv(uint32_t encoding, GpuView matrices, GpuView indices, GpuView input, GpuView output, uint32_t columns,
                     uint32_t rows, uint32_t experts, bool broadcast_input);                                         // graph.hpp:1093
    // the f32 operators either side of the sublayer, graph.hpp:983-986 and src/graph.mm:7715-7734
    void rms(GpuView input, GpuView effective_gains, GpuView output, uint32_t group_width, float epsilon);
    void rms_sigmoid_gate(GpuView input, GpuView effective_gains, GpuView gate, GpuView output, uint32_t group_width, float epsilon);
    void activate(GpuView input, GpuView output, Activation kind, float scale = 1);
    void multiply(GpuView input, GpuView gate, GpuView output, bool sigmoid_gate = false);
    void residual_read(GpuView normalized, GpuView scores, GpuView inject, GpuView output, GpuView scales, uint32_t branches, uint32_t channels);
    void residual_write(GpuView streams, GpuView input, GpuView scales, GpuView destination);
    void swiglu(GpuView gate, GpuView up, GpuView output, float scale = 1);                                          // graph.hpp:990
    void mixture(GpuView expert_outputs, GpuView weights, GpuView shared_output, GpuView shared_logit, GpuView output);  // 1102
    void prefill_mixture_batch(GpuView experts, GpuView weights, GpuView shared, GpuView shared_logit, GpuRowsF32 output,
                               uint32_t selected);                                                                  // graph.hpp:853
    void planar_moe_gate_up_swiglu_m8(GpuView pair_lo, GpuView pair_hi, GpuView indices, GpuRowsF32 input,
                                      GpuRowsF32 expert_hidden, uint32_t experts, uint32_t selected);               // graph.hpp:472
    void planar_moe_routed_m8(GpuView pair_lo, GpuView pair_hi, GpuView down_weights, GpuView indices, GpuRowsF32 input,
                              GpuRowsF32 expert_hidden, GpuRowsF32 expert_down, uint32_t experts, uint32_t selected);  // 475
    // `shared` (not in the engine's signature): an always-on expert kept in the routed experts' formats rides in the two GEMM
    // launches, every token one of its rows. Its gate and up are expert 0 of a registered co-located pair tensor, its down
    // expert 0 of a registered Q6_K planes tensor; `rows` [tokens, channels] receives down(silu(gate x) * up x).
    struct SharedPlanarExpert { GpuView pair; GpuView down; GpuRowsF32 rows; };
    void planar_nax_grouped_moe(GpuView pair_lo, GpuView pair_hi, GpuView down_weights, GpuView indices, GpuRowsF32 input,
                                GpuRowsF32 expert_down, GpuView token_map, GpuView counts, GpuView tasks, uint32_t experts,
                                uint32_t selected, const SharedPlanarExpert* shared = nullptr);                      // graph.hpp:478
    // graph.hpp:750-753 `prepare_grouped_mm` / `grouped_mm`: raw GGUF Q4_K expert stacks, one output row per route
    void prepare_grouped_mm(uint32_t encoding, PrefillWeightLayout layout, uint32_t max_tokens = 2048, uint32_t max_selected = 10,
                            uint32_t max_experts = 512, uint32_t max_columns = 2560);
    void grouped_mm(uint32_t encoding, PrefillWeightLayout layout, GpuView matrices, GpuView indices, GpuRowsF32 input, GpuRowsF32 output,
                    GpuView token_map, GpuView counts, GpuView tasks, uint32_t experts, uint32_t selected, bool broadcast);
    // the same with experts = 1, selected = 1, broadcast: the dense dequant-GEMM (Q4_K rows or planes, Q6_K planes)
    void dense_mm(uint32_t encoding, PrefillWeightLayout layout, GpuView matrix, GpuRowsF32 input, GpuRowsF32 output);
    // graph.hpp:859-860 `prepare_dense_mm_q8` / `dense_mm_q8`: out[m, :] = W x[m, :] for a dense Q8_0 matrix in GGUF rows or
    // q8_lanes_v1 rows, f32 rows in and out (decoded and accumulated in f32, each weight read once per eight rows).
    // Preparing with bounds (not in the engine's signature) sizes a scratch for the many-row form: from 32 rows on, with
    // columns in multiples of 64 and within the bounds, matrix and rows are staged as halves and one matrix-core GEMM
    // multiplies them (the engine's kernel stages halves too); the bounds may grow by preparing again.
    void prepare_dense_mm_q8(PrefillWeightLayout layout, uint32_t max_tokens = 0, uint32_t max_columns = 0, uint32_t max_rows = 0);
    void dense_mm_q8(PrefillWeightLayout layout, GpuView matrix, GpuRowsF32 input, GpuRowsF32 output, bool reuse_bf16 = false);
    // graph.hpp:548-553 selectors of the engine's GEMV variants: same arithmetic here whatever they say, kept so that
    // callers' set-up code runs unchanged (idle only, same accepted values)
    void configure_small_gemv(uint32_t column_splits);
    void configure_block_gemv(uint32_t formats);
    static uint64_t logit_topk_scratch_bytes(uint32_t max_rows, uint32_t max_vocabulary = 1u << 20);                 // graph.hpp:1030
    static uint64_t logit_topk_output_bytes(uint32_t max_rows);
    void prepare_logit_topk();
    void logit_topk(GpuRowsF32 logits, GpuView partial_scratch, GpuView out_rows);                                    // graph.hpp:1033

private:
    struct Impl;
    std::unique_ptr<Impl> impl_;
};

// ---- include/tokspur/grouped_mm.hpp:8-26: the argument block (56 bytes, as the engine's kernels take it) and the pure
// geometry / byte-bound planners of grouped_mm and dense_mm_q8. They refuse what the engine refuses, with FormatError and the
// engine's wording; `threads` / `threadgroup_bytes` are the engine's launch constants, kept so that callers that print a plan
// compile unchanged.
struct GroupedMmArgs {
    uint32_t columns, rows, row_bytes, experts;
    uint32_t selected, tokens, broadcast, maximum_tasks;
    uint64_t expert_stride_bytes, input_stride_bytes, output_stride_bytes;
};
static_assert(sizeof(GroupedMmArgs) == 56, "GroupedMmArgs ABI");
struct GroupedMmPlan {
    GroupedMmArgs args{};
    uint64_t matrix_bytes = 0, indices_bytes = 0, input_bytes = 0, output_bytes = 0;
    uint64_t token_map_bytes = 0, counts_bytes = 0, tasks_bytes = 0;
    uint32_t grid_x = 0, grid_y = 0, threads = 128, threadgroup_bytes = 8192;
    const char* kernel = nullptr;
};
GroupedMmPlan grouped_mm_plan(uint32_t encoding, PrefillWeightLayout layout, uint32_t columns, uint32_t rows, uint32_t experts,
                              uint32_t selected, uint32_t tokens, uint64_t input_stride_bytes, uint64_t output_stride_bytes, bool broadcast,
                              bool allow_nax_2k = false);
GroupedMmPlan dense_mm_q8_plan(PrefillWeightLayout layout, uint32_t columns, uint32_t rows, uint32_t tokens, uint64_t input_stride_bytes,
                               uint64_t output_stride_bytes, bool allow_nax_2k = false);
const char* grouped_mm_kernel(uint32_t encoding, PrefillWeightLayout layout);
const char* dense_mm_q8_kernel(PrefillWeightLayout layout);

// ---- the MoE sublayer for one token, include/tokspur/moe.hpp:9-45, src/moe.cpp:13-83
struct GpuMatrix { GpuView view; uint32_t encoding; };
struct MoeShape { uint32_t channels, hidden, experts, selected; };
struct MoeWeights { GpuMatrix router, gate, up, down, shared_gate, shared_up, shared_down, shared_router; };
struct MoeScratch {
    GpuView logits, indices, weights, gate, up, down, shared_gate, shared_up, shared_down, shared_logit;
    [[nodiscard]] std::array<GpuView, 10> views() const { return {logits, indices, weights, gate, up, down, shared_gate, shared_up, shared_down, shared_logit}; }
};
MoeScratch allocate_moe_scratch(HipGraph& graph, MoeShape shape);
void release_moe_scratch(HipGraph& graph, const MoeScratch& scratch);
[[nodiscard]] bool is_planar_moe(const HipGraph& graph, const MoeWeights& weights, MoeShape shape);
// what `grouped_mm` multiplies (src/grouped_mm.cpp:9): an encoding and a row layout
[[nodiscard]] bool grouped_mm_takes(uint32_t encoding, PrefillWeightLayout layout);
// Encodes router GEMV -> top-k -> routed experts -> shared expert -> mixture into the caller's current batch; allocates,
// reads and commits nothing.
void encode_moe(HipGraph& graph, const MoeWeights& weights, const MoeScratch& scratch, GpuView input, GpuView output,
                MoeShape shape, RouterMode mode, bool normalize_selected);

// ---- the prefill MoE sublayer for a batch of tokens (the routed half of src/moe_mm_many.cpp:126-283): batch router top-k ->
// grouped planar MoE -> shared expert through the same grouped path -> batch mixture. Logits are an input (the router
// projection is outside this path).
struct MoeBatchScratch {
    GpuView indices, weights, expert_down, token_map, counts, tasks, shared_indices, shared_down, shared_token_map, shared_counts,
        shared_tasks, shared_logit;
};
MoeBatchScratch allocate_moe_batch_scratch(HipGraph& graph, MoeShape shape, uint32_t tokens);
void release_moe_batch_scratch(HipGraph& graph, const MoeBatchScratch& scratch);
void encode_moe_batch(HipGraph& graph, const MoeWeights& weights, const MoeBatchScratch& scratch, GpuView logits, GpuRowsF32 input,
                      GpuRowsF32 output, MoeShape shape, RouterMode mode, bool normalize_selected);

// ---- the whole prefill MoE sublayer for up to `capacity` token rows, include/tokspur/moe_mm_many.hpp:7-63 and
// src/moe_mm_many.cpp:126-283 (default arm): router projection (F32 rows) -> batch top-k -> routed experts (planar: at most
// eight rows through the routed kernels, more through the grouped GEMM; raw GGUF: grouped_mm x 2 + SwiGLU + grouped_mm) ->
// shared expert as dense Q8_0 products -> shared router -> batch mixture. Rows beyond 2048 are worked off in chunks.
struct MoeMmLayouts {
    PrefillWeightLayout gate = PrefillWeightLayout::gguf, up = PrefillWeightLayout::gguf, down = PrefillWeightLayout::gguf;
    PrefillWeightLayout shared_gate = PrefillWeightLayout::gguf, shared_up = PrefillWeightLayout::gguf, shared_down = PrefillWeightLayout::gguf;
};
// include/tokspur/moe_mm_many.hpp:11-25 and src/moe_mm_many_plan.cpp:6-14. With `engine_bounds` the plan refuses what the
// engine refuses (2560 columns, 512 experts, at most 512 rows); without, what the device kernel cannot take (columns not in
// multiples of 32, more than 65536 either way). Strides are byte counts, multiples of 16.
struct MoeRouterF32Args {
    uint32_t columns, experts, tokens, reserved;
    uint64_t input_stride_bytes, output_stride_bytes;
};
static_assert(sizeof(MoeRouterF32Args) == 32, "router FP32 argument ABI");
struct MoeRouterF32Plan {
    MoeRouterF32Args args;
    uint64_t matrix_bytes, input_bytes, output_bytes;
    uint32_t grid_x, grid_y;  // 32-wide tiles of experts and of rows, as the engine counts them
};
inline constexpr const char* moe_router_f32_kernel = "graph_moe_router_f32_batch";
MoeRouterF32Plan moe_router_f32_plan(uint32_t columns, uint32_t experts, uint32_t tokens, uint64_t input_stride_bytes,
                                     uint64_t output_stride_bytes, bool engine_bounds = true);
struct MoeMmManyBytes {
    std::array<uint64_t, 13> views{};
    uint64_t total = 0;
};
struct MoeMmManyScratch {
    MoeScratch rows;
    GpuView token_map, counts, tasks;
    uint32_t capacity = 0;
    [[nodiscard]] std::array<GpuView, 13> views() const {
        const auto r = rows.views();
        return {r[0], r[1], r[2], r[3], r[4], r[5], r[6], r[7], r[8], r[9], token_map, counts, tasks};
    }
};
MoeMmManyBytes moe_mm_many_bytes(MoeShape shape, uint32_t capacity, bool allow_nax_2k = true);
MoeMmManyScratch allocate_moe_mm_many_scratch(HipGraph& graph, MoeShape shape, uint32_t capacity, bool allow_nax_2k = true);
void release_moe_mm_many_scratch(HipGraph& graph, const MoeMmManyScratch& scratch);
// idle only: sizes the workspaces the routed and shared products need for `capacity` rows
void prepare_moe_mm_many(HipGraph& graph, const MoeWeights& weights, MoeShape shape, uint32_t capacity, MoeMmLayouts layouts = {});
void encode_moe_mm_many(HipGraph& graph, const MoeWeights& weights, const MoeMmManyScratch& scratch, GpuRowsF32 input, GpuRowsF32 output,
                        MoeShape shape, RouterMode mode, bool normalize_selected, MoeMmLayouts layouts = {});

}  // namespace tokspur
