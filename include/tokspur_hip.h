/*
 * tokspur_hip — C ABI of the MI355X (gfx950) quantized-matmul / MoE kernels.
 *
 * This is the layer a tokspur maintainer binds underneath the native engine's graph executor:
 * every device entry point below replaces one `tokspur::MetalGraph` operator encoder (cited per
 * function, paths relative to the reference tree's native/ directory) and every host entry point
 * replaces one pure planner / layout routine. The reference has no C ABI of its own; its boundary
 * is the C++ class in include/tokspur/graph.hpp:431-1168, which the host class in
 * tokspur-public_amd/host/hip_graph.hpp mirrors on top of these functions.
 *
 * Conventions
 *  - Plain pointers and sizes only. Device pointers are HIP device addresses; `stream` is a
 *    hipStream_t passed as void* (NULL = the default stream). Calls enqueue and return; nothing
 *    here synchronises or allocates device memory unless its comment says so.
 *  - Return value: TSP_OK, or a refusal made on the host BEFORE anything was enqueued
 *    (TSP_ERR_FORMAT = what the reference reports as tokspur::FormatError; TSP_ERR_HIP = a HIP
 *    runtime error). tsp_last_error() returns the message for the calling thread.
 *  - `error_word` is the device-side sticky error word of the reference's kernels (buffer index 7,
 *    e.g. kernels/gemv.metal:114,213): kernels OR in TSP_ERRBIT_NONFINITE (1) when an output is
 *    not finite and TSP_ERRBIT_INDEX (4) on a bad expert id or grouping geometry. The caller zeroes
 *    it, reads it once per batch and refuses the batch when it is non-zero (src/graph.mm:3977-3978).
 *  - Outputs must not overlap inputs; padding beyond `columns` of a strided row is never written.
 */
#ifndef TOKSPUR_HIP_H
#define TOKSPUR_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TSP_OK 0
#define TSP_ERR_FORMAT 1
#define TSP_ERR_HIP 2

#define TSP_ERRBIT_NONFINITE 1u
#define TSP_ERRBIT_INDEX 4u

/* GGUF tensor encodings the path decodes (src/gguf.cpp:21-32, src/numeric.cpp:93-95). */
#define TSP_F32 0u
#define TSP_F16 1u
#define TSP_Q5_1 7u
#define TSP_Q8_0 8u
#define TSP_Q4_K 12u
#define TSP_Q5_K 13u
#define TSP_Q6_K 14u
#define TSP_IQ4_NL 20u
#define TSP_BF16 30u

/* Row layouts of a dense matrix (include/tokspur/grouped_mm.hpp:6; planar = one Pack v3 expert). */
#define TSP_LAYOUT_GGUF 0u
#define TSP_LAYOUT_Q8_LANES_V1 1u
#define TSP_LAYOUT_Q51_LANES_V1 2u
#define TSP_LAYOUT_PLANAR_V3 3u

/* Pack v3 planar kinds (include/tokspur/planar_pack_v3.hpp:29-40). Kind 10 is this library's
 * extension: Q6_K experts in planes [ql 128][qh 64][sc 16][d 2] per block, for down projections. */
#define TSP_KIND_PLAIN 0u
#define TSP_KIND_Q8_LANES_V1 1u
#define TSP_KIND_Q4K_COLOC_GATE 2u
#define TSP_KIND_Q4K_COLOC_UP 3u
#define TSP_KIND_Q5K_COLOC_GATE 4u
#define TSP_KIND_Q5K_COLOC_UP 5u
#define TSP_KIND_Q8_COLOC_GATE 6u
#define TSP_KIND_Q8_COLOC_UP 7u
#define TSP_KIND_Q51_PLANAR 8u
#define TSP_KIND_Q8_PLANAR 9u
#define TSP_KIND_Q6K_PLANAR_X 10u

const char* tsp_last_error(void);
/* ABI revision of this header; bumped on any incompatible change. */
uint32_t tsp_abi_version(void);

/* Per-kernel timing, the engine's `configure_profiling` / `GraphProfile{KernelTiming}`
 * (include/tokspur/graph.hpp:353-400; src/graph.mm:2669): between begin and end every kernel launched
 * through this library is bracketed by a pair of events on its stream. tsp_profile_end waits for them,
 * closes the window and returns one row per kernel name. Not for use while other threads launch. */
typedef struct tsp_kernel_time {
    char name[48];
    uint32_t launches;
    float total_ms;
    float min_ms;
} tsp_kernel_time;
int tsp_profile_begin(void);
int tsp_profile_end(tsp_kernel_time* rows, uint32_t capacity, uint32_t* count);
/* Measurement aid with no counterpart in the reference: a plain copy kernel ("calibration_copy") of `bytes`
 * (a multiple of 16) from src to dst. Its HBM traffic is known, so the memory counters of a profiler read for
 * it give the factor by which to scale the same counters read for the other kernels. */
int tsp_calibration_copy(void* dst, const void* src, uint64_t bytes, void* stream);

/* ------------------------------------------------------------------ host: formats and layouts */

/* src/gguf.cpp:21-32, 157-160 `encoding()`: block geometry of a GGUF type. */
int tsp_encoding(uint32_t type, uint32_t* elements_per_block, uint32_t* bytes_per_block);
/* src/numeric.cpp:93-95 `can_decode()`. */
int tsp_can_decode(uint32_t type);

/* include/tokspur/planar_pack_v3.hpp:48-61 `PlanarExpertSpec` (field for field). */
typedef struct tsp_planar_spec {
    uint32_t source_type, columns, rows, blocks_per_row;
    uint64_t source_row_bytes, planar_row_bytes, source_expert_bytes, planar_expert_bytes;
    uint64_t qs_offset, qh_offset, sm_offset, dm_offset;
} tsp_planar_spec;
/* src/planar_pack_v3.cpp:601-650 `make_expert_spec` (+ type 14 for TSP_KIND_Q6K_PLANAR_X:
 * qs = ql plane, qh = qh plane, sm = int8 sub-scale plane, dm = f16 d plane). */
int tsp_make_expert_spec(uint32_t source_type, uint32_t columns, uint32_t rows, tsp_planar_spec* spec);
/* src/planar_pack_v3.cpp:652-674 `pack_sm16` / `unpack_sm16`. */
void tsp_pack_sm16(const uint8_t scales12[12], uint8_t sm16[16]);
int tsp_unpack_sm16(const uint8_t sm16[16], uint8_t scales12[12]);
/* src/planar_pack_v3.cpp:676-758 `pack_expert_planar_v3` / `unpack_expert_planar_v3` (host memory). */
int tsp_pack_expert_planar_v3(const tsp_planar_spec* spec, const uint8_t* gguf_expert, uint64_t gguf_bytes,
                              uint8_t* planar_expert, uint64_t planar_bytes);
int tsp_unpack_expert_planar_v3(const tsp_planar_spec* spec, const uint8_t* planar_expert, uint64_t planar_bytes,
                                uint8_t* gguf_expert, uint64_t gguf_bytes);
/* src/planar_pack_v3.cpp:1061-1123 co-location: half 0 ("pair_lo", stored under the gate tensor's
 * name) holds experts 0..E/2-1 as interleaved [gate_e, up_e]; half 1 ("pair_hi") holds the rest. */
int tsp_pack_coloc_half(const tsp_planar_spec* spec, const uint8_t* gate_gguf, const uint8_t* up_gguf,
                        uint32_t experts, uint32_t half, uint8_t* out, uint64_t out_bytes);
/* src/expert_lanes.cpp:83-119 `packed_quant_offset` / `pack_rows` / `unpack_rows` for Q8_0. */
int tsp_q8_lanes_quant_offset(uint32_t columns, uint32_t block, uint32_t index, uint64_t* offset);
int tsp_q8_lanes_pack_rows(uint32_t columns, const uint8_t* original, uint8_t* packed, uint64_t bytes);
int tsp_q8_lanes_unpack_rows(uint32_t columns, const uint8_t* packed, uint8_t* original, uint64_t bytes);

/* The same for Q5_1 rows (`q51_lanes_v1`): [8-byte block heads d, m, qh x blocks][runs of 16 blocks, 256 B: quant byte i of the
 * run's blocks side by side]; index < 16. */
int tsp_q51_lanes_quant_offset(uint32_t columns, uint32_t block, uint32_t index, uint64_t* offset);
int tsp_q51_lanes_pack_rows(uint32_t columns, const uint8_t* original, uint8_t* packed, uint64_t bytes);
int tsp_q51_lanes_unpack_rows(uint32_t columns, const uint8_t* packed, uint8_t* original, uint64_t bytes);

/* ------------------------------------------------------------------ host: planners */

/* include/tokspur/grouped_mm.hpp:8-21 `GroupedMmArgs` (56 bytes) and `GroupedMmPlan`. */
typedef struct tsp_grouped_mm_args_t {
    uint32_t columns, rows, row_bytes, experts, selected, tokens, broadcast, maximum_tasks;
    uint64_t expert_stride_bytes, input_stride_bytes, output_stride_bytes;
} tsp_grouped_mm_args_t;
typedef struct tsp_grouped_mm_plan_t {
    tsp_grouped_mm_args_t args;
    uint64_t matrix_bytes, indices_bytes, input_bytes, output_bytes, token_map_bytes, counts_bytes, tasks_bytes;
    uint32_t grid_x, grid_y;
} tsp_grouped_mm_plan_t;
/* src/grouped_mm.cpp:24-47 `grouped_mm_plan`; 48-54 `dense_mm_q8_plan`. */
int tsp_grouped_mm_plan(uint32_t encoding, uint32_t layout, uint32_t columns, uint32_t rows, uint32_t experts,
                        uint32_t selected, uint32_t tokens, uint64_t input_stride_bytes, uint64_t output_stride_bytes,
                        int broadcast, int allow_nax_2k, tsp_grouped_mm_plan_t* plan);
int tsp_dense_mm_q8_plan(uint32_t layout, uint32_t columns, uint32_t rows, uint32_t tokens, uint64_t input_stride_bytes,
                         uint64_t output_stride_bytes, int allow_nax_2k, tsp_grouped_mm_plan_t* plan);
/* src/moe_mm_many_plan.cpp:28-52 `moe_mm_many_bytes`: the 13 scratch views and their total. */
int tsp_moe_mm_many_bytes(uint32_t channels, uint32_t hidden, uint32_t experts, uint32_t selected, uint32_t capacity,
                          int allow_nax_2k, uint64_t views[13], uint64_t* total);
/* src/q8_many.cpp:20-35 `q8_many_width` / `q8_many_chunks`. */
int tsp_q8_many_width(uint32_t remaining, uint32_t* width);
int tsp_q8_many_chunks(uint32_t rows, uint32_t* chunks);

/* ------------------------------------------------------------------ device: dequantisation */

/* src/numeric.cpp:97-148 `dequantize` on the device: raw GGUF blocks -> f32, bit-identical to the
 * reference's double-then-one-cast value for every block whose double arithmetic is exact (all
 * blocks with finite f16 fields of ordinary magnitude). Non-finite results set TSP_ERRBIT_NONFINITE. */
int tsp_dequantize(uint32_t type, const void* blocks, uint64_t nbytes, float* out, uint64_t nelem,
                   uint32_t* error_word, void* stream);
/* src/planar_pack_v3.cpp:829-896 `dequantize_expert_planar_v3_f32` on the device, one planar expert. */
int tsp_dequantize_planar(const tsp_planar_spec* spec, const void* planar_expert, float* out,
                          uint32_t* error_word, void* stream);

/* ------------------------------------------------------------------ device: GEMV family */

/* include/tokspur/graph.hpp:730 `MetalGraph::gemv` (src/graph.mm:4182-4270; kernels/gemv.metal:99-117,
 * 232-266): y[r] = sum_c dec(W[r,c]) * x[c], f32 decode and accumulate. `layout` selects raw GGUF
 * rows, q8_lanes_v1 rows (Q8_0 only) or one planar v3 expert (Q4_K, Q8_0, Q6_K planes). */
int tsp_gemv(uint32_t encoding, uint32_t layout, const void* matrix, uint64_t matrix_bytes, const float* x, float* y,
             uint32_t columns, uint32_t rows, uint32_t* error_word, void* stream);
/* include/tokspur/graph.hpp:733 `gemv_rows` (src/graph.mm:4271-4336): gemv once per token row of a
 * strided f32 row set; strides in bytes. */
int tsp_gemv_rows(uint32_t encoding, uint32_t layout, const void* matrix, uint64_t matrix_bytes, const float* x,
                  uint64_t x_stride_bytes, float* y, uint64_t y_stride_bytes, uint32_t count, uint32_t columns,
                  uint32_t rows, uint32_t* error_word, void* stream);
/* include/tokspur/graph.hpp:745 `q8_matvec_many` (kernels/q8_many.metal:7-46): Q8_0 GEMV for
 * width in {1,2,4,8} token rows, x token-major [width, columns], y token-major [width, rows]; each
 * weight is decoded once for all rows. */
int tsp_q8_matvec_many(uint32_t layout, const void* matrix, uint64_t matrix_bytes, const float* x, float* y,
                       uint32_t columns, uint32_t rows, uint32_t width, uint32_t* error_word, void* stream);
/* include/tokspur/graph.hpp:860 `dense_mm_q8` (kernels/grouped_mm.metal:239-243; planner src/grouped_mm.cpp:48-54):
 * out[t, :] = W in[t, :] for a dense Q8_0 matrix in GGUF rows (layout 0) or q8_lanes_v1 rows (layout 1), f32 rows in
 * and out with byte strides. Decoded and accumulated in f32 (the engine stages halves); token rows that lie back to
 * back share each weight read eight at a time, and up to sixteen at a time for rows of 1024 or 2048 columns in either
 * layout (16-byte aligned buffers, at least 64 matrix rows, 32 for the lanes layout, in multiples of 4). */
int tsp_dense_mm_q8(uint32_t layout, const void* matrix, uint64_t matrix_bytes, const float* input, uint64_t input_stride_bytes,
                    float* output, uint64_t output_stride_bytes, uint32_t tokens, uint32_t columns, uint32_t rows,
                    uint32_t* error_word, void* stream);
/* The same product for many token rows at once (a prefill chunk's shared expert), where one pass over the matrix per
 * sixteen rows no longer pays: the matrix is decoded once into halves (d * q rounded to nearest, as the engine's kernel
 * stages them, kernels/grouped_mm.metal:239-243), the rows are rounded to halves, and a matrix-core GEMM with f32
 * accumulation multiplies them. Columns in multiples of 64; `workspace` (16-byte aligned, at least
 * tsp_dense_mm_q8_workspace_bytes) is scratch for the call and must not overlap the other buffers. Results agree with
 * tsp_dense_mm_q8 to the GEMM tolerance (2e-3 of the row scale), not bit for bit. */
uint64_t tsp_dense_mm_q8_workspace_bytes(uint32_t tokens, uint32_t columns, uint32_t rows);
int tsp_dense_mm_q8_staged(uint32_t layout, const void* matrix, uint64_t matrix_bytes, const float* input, uint64_t input_stride_bytes,
                           float* output, uint64_t output_stride_bytes, uint32_t tokens, uint32_t columns, uint32_t rows,
                           void* workspace, uint64_t workspace_bytes, uint32_t* error_word, void* stream);
/* include/tokspur/graph.hpp:1093 `routed_gemv` (kernels/gemv.metal:198-227): per selected expert s,
 * y[s, :] = W[ids[s]] * x (x broadcast, or one x row per route). Raw GGUF expert stacks. */
int tsp_routed_gemv(uint32_t encoding, const void* matrices, uint64_t matrices_bytes, const uint32_t* ids, const float* x,
                    float* y, uint32_t columns, uint32_t rows, uint32_t experts, uint32_t selected, int broadcast_input,
                    uint32_t* error_word, void* stream);

/* ------------------------------------------------------------------ device: router, combine, SwiGLU */

/* include/tokspur/graph.hpp:1091 `route` (kernels/graph.metal:466-526; CPU: src/routing.cpp:11-40):
 * top-`selected` of `experts` f32 logits by (logit desc, id asc); weights = softmax (mode 0) or
 * sigmoid (mode 1), renormalised over the selected when normalize_selected. ids are exact. */
int tsp_route(const float* logits, uint32_t* indices, float* weights, uint32_t experts, uint32_t selected, uint32_t mode,
              int normalize_selected, uint32_t* error_word, void* stream);
/* include/tokspur/graph.hpp:852 `prefill_route_batch` / 837 `moe_route_rows` (kernels/graph.metal:551-638):
 * the same per token row; logits [tokens, experts], outputs [tokens, selected]. */
int tsp_route_batch(const float* logits, uint32_t* indices, float* weights, uint32_t experts, uint32_t selected,
                    uint32_t tokens, uint32_t mode, int normalize_selected, uint32_t* error_word, void* stream);
/* include/tokspur/graph.hpp:825 `moe_router_f32_batch` and :836 `moe_router_f32_window` (kernels/moe_router_f32_batch.metal:13-50;
 * planner src/moe_mm_many_plan.cpp:6-26): the router projection of a whole chunk as one f32 GEMM,
 * output[t, e] = sum_k weights[e, k] * input[t, k], both operands f32 from memory to the accumulator (f32 matrix-core
 * multiply-accumulate, nothing narrowed). weights is [experts, columns] row-major; input and output rows lie
 * `*_stride_bytes` apart (multiples of 16, as the engine's planner demands). Columns in multiples of 32. The engine bounds
 * the shape to 2560 x 512 and 512 (2048 for the window) tokens; this entry point takes any shape within 65536 each way and
 * leaves those bounds to the planner above it. TSP_ERRBIT_NONFINITE when a result is not finite. */
int tsp_router_f32_batch(const float* weights, const float* input, uint64_t input_stride_bytes, float* output,
                         uint64_t output_stride_bytes, uint32_t columns, uint32_t experts, uint32_t tokens,
                         uint32_t* error_word, void* stream);
/* include/tokspur/graph.hpp:1102 `mixture` (kernels/graph.metal:528-544; CPU: src/routing.cpp:42-60):
 * y[c] = sigmoid(shared_logit) * shared[c] + sum_r w[r] * experts[r, c], r in route order. */
int tsp_mixture(const float* expert_outputs, const float* weights, const float* shared_output, const float* shared_logit,
                float* output, uint32_t channels, uint32_t selected, uint32_t* error_word, void* stream);
/* include/tokspur/graph.hpp:853 `prefill_mixture_batch` (kernels/graph.metal:654-691): per token row;
 * expert_outputs [tokens, selected, channels], output rows `output_stride_bytes` apart. */
int tsp_mixture_batch(const float* expert_outputs, const float* weights, const float* shared_output, const float* shared_logit,
                      float* output, uint64_t output_stride_bytes, uint32_t channels, uint32_t selected, uint32_t tokens,
                      uint32_t* error_word, void* stream);
/* include/tokspur/graph.hpp:990 `swiglu` (kernels/graph.metal:312-326): out = silu(gate*scale) * up. */
int tsp_swiglu(const float* gate, const float* up, float* output, uint64_t count, float scale, uint32_t* error_word, void* stream);

/* ------------------------------------------------------------------ device: the f32 operators around the sublayer */

/* What a destination holds after a batch these operators refused is what the engine's holds (kernels/graph.metal:18-21
 * `checked_store`): a non-finite RESULT sets TSP_ERRBIT_NONFINITE and is stored; where an operator tests its operands first
 * (a group's sum of squares in rms, the normalised value and the gate in rms_sigmoid_gate, both factors in multiply, the
 * branch values, scores and inject logits in residual_read) a non-finite operand sets the bit and that element, group or
 * thread stores nothing. */

/* include/tokspur/graph.hpp:983 `rms` (src/graph.mm:7399-7409; kernels/graph.metal:222-247): independent groups of `group_width`
 * values, out = x * rsqrt(mean(x^2) + epsilon) * gain; `gains` holds one gain per element, or `group_width` gains shared by
 * every group (shared_gains). */
int tsp_rms(const float* input, const float* gains, float* output, uint64_t count, uint32_t group_width, int shared_gains, float epsilon,
            uint32_t* error_word, void* stream);
/* include/tokspur/graph.hpp:984 `rms_sigmoid_gate` (kernels/graph.metal:249-282): the same times sigmoid(gate), in one pass. */
int tsp_rms_sigmoid_gate(const float* input, const float* gains, const float* gate, float* output, uint64_t count, uint32_t group_width,
                         int shared_gains, float epsilon, uint32_t* error_word, void* stream);
/* include/tokspur/graph.hpp:985 `activate` (kernels/graph.metal:284-300): out = f(scale * x), kind 0 identity, 1 SiLU, 2 sigmoid,
 * 3 softplus (include/tokspur/graph.hpp:134 `Activation`); may run in place. */
int tsp_activate(const float* input, float* output, uint64_t count, uint32_t kind, float scale, uint32_t* error_word, void* stream);
/* include/tokspur/graph.hpp:986 `multiply` (kernels/graph.metal:302-311): out = x * gate, or x * sigmoid(gate). */
int tsp_multiply(const float* input, const float* gate, float* output, uint64_t count, int sigmoid_gate, uint32_t* error_word, void* stream);
/* `residual_read` (src/graph.mm:7715-7725; kernels/graph.metal:330-351): output[c] = mean over branches of
 * normalized[b, c] * sigmoid(scores[b, c]); scales[b] = 2 sigmoid(inject[b] / branches). At most 64 branches of 65536 channels. */
int tsp_residual_read(const float* normalized, const float* scores, const float* inject, float* output, float* scales, uint32_t branches,
                      uint32_t channels, uint32_t* error_word, void* stream);
/* `residual_write` (src/graph.mm:7726-7734; kernels/graph.metal:353-361): output[b, c] = streams[b, c] + scales[b] * input[c];
 * output may be the streams themselves. */
int tsp_residual_write(const float* streams, const float* input, const float* scales, float* output, uint32_t branches, uint32_t channels,
                       uint32_t* error_word, void* stream);

/* ------------------------------------------------------------------ device: expert permutation */

/* kernels/grouped_mpp.metal:12-37 `graph_grouped_routes` (encoded inside `grouped_mm`, src/graph.mm:4571,
 * and `planar_nax_grouped_moe`, src/graph.mm:9383): token_map[e*tokens + k] = t*selected + slot for the
 * k-th token in ascending order that routes to expert e; counts[e]. Tails of token_map rows are not
 * written. TSP_ERRBIT_INDEX on id >= experts or an expert repeated within one token. */
int tsp_grouped_routes(const uint32_t* ids, uint32_t* token_map, uint32_t* counts, uint32_t experts, uint32_t selected,
                       uint32_t tokens, uint32_t* error_word, void* stream);
/* kernels/grouped_mpp.metal:41-64 `graph_grouped_tasks` / kernels/nax_prefill.metal:4057-4091: tasks[0] =
 * tiles, tasks[1] = routes, tasks[2+2i] = expert, tasks[3+2i] = first row of the tile; unused slots up to
 * tokens*selected/tile + experts are 0xFFFFFFFF. (The Metal indirect-grid words have no HIP counterpart.) */
int tsp_grouped_tasks(const uint32_t* counts, uint32_t* tasks, uint32_t experts, uint32_t selected, uint32_t tokens,
                      uint32_t tile, uint32_t* error_word, void* stream);
/* kernels/planar_moe_v3.metal:413-509 `planar_moe_build_union_m8`: the 9 280-byte union block for
 * tokens <= 8 (layout src/graph.mm:9091, kernels/planar_moe_v3.metal:439-442): [0..7] header,
 * +8 experts[128], +136 counts[128], +264 tokens[128][8], +1288 routes[128][8] (32-bit words). */
int tsp_planar_union_build(const uint32_t* ids, uint32_t* meta, uint32_t experts, uint32_t selected, uint32_t tokens,
                           uint32_t hidden, uint32_t channels, uint32_t* error_word, void* stream);

/* ------------------------------------------------------------------ device: routed MoE, 1..8 token rows */

/* The operands of `planar_moe_gate_up_swiglu_m8` / `planar_moe_routed_m8`
 * (include/tokspur/graph.hpp:472-477; src/graph.mm:9134-9291). pair_lo / pair_hi are the two
 * co-located gate/up tensors (kinds 2/3, 4/5 or 6/7), `down` is [experts] planar experts of kind
 * 8 (Q5_1), 9 (Q8_0) or 10 (Q6_K, this library's extension). x holds `tokens` f32 rows of
 * `channels`; h and y hold tokens*selected rows (route rid = t*selected + slot) of `hidden` and
 * `channels` floats. Strides are bytes. union_meta is the caller's 9 280-byte union block
 * (required when tokens > 1; the entry points rebuild it from ids on every call). */
typedef struct tsp_small_moe {
    const void* pair_lo;
    const void* pair_hi;
    const void* down;
    uint32_t gate_kind, up_kind, down_kind;
    uint32_t channels, hidden, experts, selected, tokens;
    const uint32_t* ids;
    const float* x;
    uint64_t x_stride_bytes;
    float* h;
    uint64_t h_stride_bytes;
    float* y;
    uint64_t y_stride_bytes;
    uint32_t* union_meta;
    uint32_t* error_word;
} tsp_small_moe;
/* include/tokspur/graph.hpp:472 `planar_moe_gate_up_swiglu_m8` (kernels/planar_moe_v3.metal:513-1090):
 * h[rid, r] = silu(Wg[e] x_t)[r] * (Wu[e] x_t)[r], f32 throughout. `down`, `y` are ignored. */
int tsp_planar_moe_gate_up_swiglu_m8(const tsp_small_moe* moe, void* stream);
/* include/tokspur/graph.hpp:475 `planar_moe_routed_m8` (kernels/planar_moe_v3.metal:1572-1803):
 * the above followed by y[rid, :] = Wd[e] h[rid, :]. */
int tsp_planar_moe_routed_m8(const tsp_small_moe* moe, void* stream);
/* The same call with the layer's always-on expert riding in the two launches as one more record whose rows are the
 * tokens (no counterpart: the engine runs the shared expert as GEMVs of its own, src/moe.cpp:71-78). gate, up: one
 * Pack v3 Q4_K expert each; down: one Q6_K planes expert; h [tokens, hidden] and y [tokens, channels] are its rows
 * (h 16-byte aligned). Only with Q4_K co-located gate/up and Q6_K planes down. Rows are bit-identical to a separate
 * call that routes every token to that expert. */
typedef struct tsp_shared_rows {
    const void* gate;
    const void* up;
    const void* down;
    float* h;
    uint64_t h_stride_bytes;
    float* y;
    uint64_t y_stride_bytes;
} tsp_shared_rows;
int tsp_planar_moe_routed_m8_shared(const tsp_small_moe* moe, const tsp_shared_rows* shared, void* stream);

/* ------------------------------------------------------------------ device: prefill dequant-GEMM (matrix cores) */

/* include/tokspur/graph.hpp:750-753 `grouped_mm` with experts = selected = 1, broadcast (the dense case,
 * kernels/grouped_mm.metal:159-243) and 859-860 `dense_mm_q8`: out[t, r] = sum_c x[t, c] * dec(W[r, c]) for
 * `tokens` rows. Activations are used as bf16 values (carried as f16), weights enter the matrix cores as exact integer
 * factors whose block scales are applied in f32, f32 accumulation. The carry is exact for bf16 values of magnitude 2^-14
 * to 65504; smaller ones lose low bits (below 2^-24: zero), and a finite input above 65504 sets TSP_ERRBIT_NONFINITE like an
 * infinity would (the batch is refused rather than computed on a clipped value). The same holds for tsp_grouped_mm and
 * tsp_planar_nax_grouped_moe. One shape differs: Q4_K raw GGUF rows against 512 or more token rows enter the matrix cores as
 * the engine's kernel stages them (test_moe_mm_many_gpu.cpp:54-63), each weight's f32 value d*sc*q - dmin*mn rounded once to
 * half, which is what makes unpacking a weight once per 128 or 256 token rows possible. Input rows are f32 or bf16, output
 * rows f32 or bf16 (RNE); strides in bytes. Q4_K raw GGUF rows or planar planes, Q6_K planes. `workspace` is caller
 * owned scratch of tsp_dense_mm_workspace_bytes(tokens, columns) bytes, 16-byte aligned. */
uint64_t tsp_dense_mm_workspace_bytes(uint32_t tokens, uint32_t columns);
int tsp_dense_mm(uint32_t encoding, uint32_t layout, const void* matrix, uint64_t matrix_bytes, const void* input,
                 uint64_t input_stride_bytes, int input_is_bf16, void* output, uint64_t output_stride_bytes, int output_is_bf16,
                 uint32_t tokens, uint32_t columns, uint32_t rows, void* workspace, uint64_t workspace_bytes,
                 uint32_t* error_word, void* stream);

/* include/tokspur/graph.hpp:750-753 `grouped_mm` (src/graph.mm:4534-4606; kernels/grouped_mm.metal:159-243; route and task
 * preparation kernels/grouped_mpp.metal:12-64): for every route rid = t*selected + slot, output[rid, :] = W[ids[rid]] * x, with x the
 * token's row (broadcast) or row rid of the input. `matrices` is an expert stack [experts][rows][row bytes]; token_map, counts and
 * tasks (tile 32) are outputs with the engine's layouts. Encodings and layouts as src/grouped_mm.cpp:8-12: Q4_K, Q5_K, Q5_1 and
 * Q8_0 in GGUF rows, Q8_0 in q8_lanes_v1 rows, Q5_1 in q51_lanes_v1 rows (640 columns, more than one expert).
 *   Q4_K: activations are used as bf16 values, weights as exact integer factors with f32 block scales, f32 accumulation;
 *   workspace: tsp_grouped_mm_workspace_bytes(...) bytes, 256-byte aligned.
 *   The others: every weight decoded in f32 and rounded once to half, every activation rounded once to half, f32
 *   accumulation on the matrix cores (the engine's staging, kernels/grouped_mm.metal:205-216); strides in multiples of 16
 *   bytes and 16-byte aligned input, as its planner demands; the workspace is not touched. */
uint64_t tsp_grouped_mm_workspace_bytes(uint32_t tokens, uint32_t selected, uint32_t experts, uint32_t columns, int broadcast);
int tsp_grouped_mm(uint32_t encoding, uint32_t layout, const void* matrices, uint64_t matrices_bytes, const uint32_t* ids,
                   const float* input, uint64_t input_stride_bytes, float* output, uint64_t output_stride_bytes, uint32_t* token_map,
                   uint32_t* counts, uint32_t* tasks, uint32_t columns, uint32_t rows, uint32_t experts, uint32_t selected,
                   uint32_t tokens, int broadcast, void* workspace, uint64_t workspace_bytes, uint32_t* error_word, void* stream);

/* The operands of `planar_nax_grouped_moe` (include/tokspur/graph.hpp:478-481; src/graph.mm:9293-9420).
 * x holds `tokens` f32 rows of `channels`; y (the engine's expert_down) holds tokens*selected f32 rows
 * of `channels`, row rid = t*selected + slot. token_map [experts*tokens], counts [experts] and tasks
 * [2 + 2*(tokens*selected/32 + experts)] are outputs with the engine's layouts (tile = 32). workspace is
 * caller-owned scratch (the engine's nax_bf16_scratch, src/graph.mm:9100-9126) of
 * tsp_planar_nax_workspace_bytes(...) bytes, 256-byte aligned. */
typedef struct tsp_grouped_moe {
    const void* pair_lo;
    const void* pair_hi;
    const void* down;
    uint32_t gate_kind, up_kind, down_kind;
    uint32_t channels, hidden, experts, selected, tokens;
    const uint32_t* ids;
    const float* x;
    uint64_t x_stride_bytes;
    float* y;
    uint64_t y_stride_bytes;
    uint32_t* token_map;
    uint32_t* counts;
    uint32_t* tasks;
    void* workspace;
    uint64_t workspace_bytes;
    uint32_t* error_word;
} tsp_grouped_moe;
uint64_t tsp_planar_nax_workspace_bytes(uint32_t tokens, uint32_t selected, uint32_t experts, uint32_t channels, uint32_t hidden);
/* include/tokspur/graph.hpp:478 `planar_nax_grouped_moe` (kernels/planar_moe_v3.metal:2406-2621): expert
 * permutation -> prefix-sum tasks -> gather -> ragged grouped gate/up GEMM with fused SwiGLU (h carried as
 * the half nearest h / 256) -> grouped down GEMM -> scatter of f32 rows to y[rid]. */
int tsp_planar_nax_grouped_moe(const tsp_grouped_moe* moe, void* stream);
/* The same call with the layer's always-on expert riding in the two GEMM launches instead of running as dense GEMMs of
 * its own beside them (src/moe_mm_many.cpp:152-187 runs it as three `dense_mm_q8`; this is for a shared expert kept in
 * the routed experts' formats): `gate` and `up` are one Pack v3 Q4_K expert each (the halves of a co-located pair,
 * src/planar_pack_v3.cpp:1061-1123, need not be adjacent), `down` one Q6_K planes expert; every token is a row of it,
 * and y [tokens, channels] receives down(silu(gate x) * up x), to be handed to `tsp_prefill_mixture_batch` as `shared`.
 * Only with the Q4_K co-located / Q6_K planes kinds; the workspace is tsp_planar_nax_shared_workspace_bytes. */
typedef struct tsp_shared_expert {
    const void* gate;
    const void* up;
    const void* down;
    float* y;
    uint64_t y_stride_bytes;
} tsp_shared_expert;
uint64_t tsp_planar_nax_shared_workspace_bytes(uint32_t tokens, uint32_t selected, uint32_t experts, uint32_t channels, uint32_t hidden);
int tsp_planar_nax_grouped_moe_shared(const tsp_grouped_moe* moe, const tsp_shared_expert* shared, void* stream);

/* ------------------------------------------------------------------ row top-k of the logits */

/* include/tokspur/sampling.hpp:21-29 `GpuLogitTopKRow` == kernels/logit_topk.metal:17-25 `LogitTopKRowOut`, 528 bytes. */
typedef struct tsp_logit_topk_row {
    uint32_t vocabulary;
    uint32_t count;
    uint32_t first_nonfinite_col;
    uint32_t first_subnormal_col;
    uint32_t ids[64];
    float logits[64];
} tsp_logit_topk_row;
/* include/tokspur/graph.hpp:1030-1031, src/graph.mm:9422-9433: bytes of the partial-row scratch and of the output
 * rows; 0 (and tsp_last_error) when the bounds are refused. */
uint64_t tsp_logit_topk_scratch_bytes(uint32_t max_rows, uint32_t max_vocabulary);
uint64_t tsp_logit_topk_output_bytes(uint32_t max_rows);
/* include/tokspur/graph.hpp:1033 `logit_topk`, src/graph.mm:9443-9478, kernels/logit_topk.metal:93-365; ordering of
 * src/sampling.cpp:473-513 `cpu_logit_topk_row`: value descending, column ascending, -0 == +0, non-finite logits
 * skipped and reported, unused slots id 0 / -inf. logits: rows of `vocabulary` floats, stride_bytes apart. */
int tsp_logit_topk(const float* logits, uint64_t stride_bytes, uint32_t rows, uint32_t vocabulary, void* partial_scratch,
                   uint64_t scratch_bytes, void* out_rows, uint64_t out_bytes, void* stream);

/* `tsp_logit_topk` for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid it) and so have no scratch buffer to hand over. No counterpart in the reference. The partial rows
 * live in a device array inside the library (540 672 bytes per device, held until the process ends); the call allocates
 * and frees nothing. At most TSP_LOGIT_TOPK_STATIC_MAX_ROWS rows of at most TSP_LOGIT_TOPK_STATIC_MAX_VOCABULARY
 * columns; larger shapes are refused with TSP_ERR_FORMAT. Results are bit-identical to tsp_logit_topk. Every call on one
 * device shares that device's array: calls that overlap in time on one device (two streams, two threads) race. The
 * first call on a device looks the array's address up, which may not be done under stream capture: make one call
 * before capturing. */
#define TSP_LOGIT_TOPK_STATIC_MAX_ROWS 16u
#define TSP_LOGIT_TOPK_STATIC_MAX_VOCABULARY 262144u
int tsp_logit_topk_static(const float* logits, uint64_t stride_bytes, uint32_t rows, uint32_t vocabulary, void* out_rows,
                          uint64_t out_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif
