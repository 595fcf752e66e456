/*
 * TEST INFRASTRUCTURE ONLY.
 *
 * A scalar CPU restatement of the tokspur native engine's numerical references
 * for the quantized-matmul / MoE path. Only tests, the smoke check and the
 * bench's cpu_baseline leg may link, load or call this library. The product
 * (the HIP library and its host layer) never does.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the reference tree's native/ directory).
 *
 * Parity pins, per function group (see tests/test_oracle_*.py):
 *   binary16            closed form over all 65 536 patterns; oracle/_ref
 *   value/dequantize    hand-encoded single-block fixtures, multi-block Q8
 *                       edge scales, bit-at-a-time independent decoder; _ref
 *   reference_gemv      fixture dot products in double; brute force; _ref
 *   route/mixture       independent probability-sort oracle, tie golden,
 *                       mixture golden; _ref
 *   sigmoid/silu        closed-form points; _ref
 *   pack v3             pack_sm16 vs closed form; round trip; planar dequant
 *                       == GGUF dequant to the bit
 *   q8 / q51 lanes      bijection + closed-form offset; _ref
 *   grouped routes/tasks  brute force on tiny inputs + invariants
 *   union metadata      row-major specification cases (T=1..8 x S=1..16)
 *   logit top-k         sort-based brute force; _ref
 *   plan geometry       byte goldens; _ref
 */
#ifndef TOKSPUR_ORACLE_H
#define TOKSPUR_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_OK 0
#define ORC_FORMAT_ERROR 1 /* the reference would throw tokspur::FormatError */

/* ---- block formats: src/gguf.cpp:21-32, src/numeric.cpp:25-148 ---- */
float orc_binary16(uint16_t bits);
int orc_encoding(uint32_t type, uint32_t* elements_per_block, uint32_t* bytes_per_block);
int orc_can_decode(uint32_t type);
int orc_value(uint32_t type, const uint8_t* block, uint32_t index, double* out);
int orc_dequantize(uint32_t type, const uint8_t* bytes, uint64_t nbytes, float* out, uint64_t nelem);

/* ---- GEMV: src/numeric.cpp:150-184 ---- */
int orc_reference_gemv(uint32_t type, const uint8_t* matrix, uint64_t nbytes, uint32_t columns,
                       uint32_t rows, const float* x, uint64_t nx, double* y);
int orc_reference_gemv_doubleinput(uint32_t type, const uint8_t* matrix, uint64_t nbytes,
                                   uint32_t columns, uint32_t rows, const double* x, uint64_t nx,
                                   double* y);
/* Same arithmetic per row, rows split over `threads` pthreads (timing baseline only). */
int orc_reference_gemv_mt(uint32_t type, const uint8_t* matrix, uint64_t nbytes, uint32_t columns,
                          uint32_t rows, const float* x, uint64_t nx, double* y, uint32_t threads);
/* src/q8_many.cpp:20-49 */
int orc_q8_many_width(uint32_t remaining, uint32_t* width);
int orc_q8_many_chunks(uint32_t rows, uint32_t* chunks);
int orc_reference_q8_many(const uint8_t* matrix, uint64_t nbytes, const float* input,
                          uint32_t columns, uint32_t rows, uint32_t width, double* out);

/* ---- scalar operators: src/operators.cpp:28-40 ---- */
int orc_stable_sigmoid(double v, double* out);
int orc_stable_silu(double v, double* out);
int orc_stable_softplus(double v, double* out);
/* src/operators.cpp:42-96: grouped RMS with effective gains, the gated-residual read (write scales included) and write. */
int orc_group_rms_reference(const double* input, const double* gains, uint64_t count, uint64_t group_width,
                            double epsilon, double* output);
int orc_gated_residual_reference(const double* streams, const double* gains, const double* down, const double* up,
                                 const double* inject, uint64_t branches, uint64_t channels, uint64_t rank, double epsilon,
                                 double* read, double* write_scales);
int orc_residual_write_reference(const double* streams, const double* output, const double* scales, uint64_t branches,
                                 uint64_t channels, double* result);

/* ---- router / mixture: src/routing.cpp:11-60 ---- */
int orc_route_reference(const double* logits, uint64_t count, uint64_t selected, uint32_t mode,
                        int normalize_selected, uint32_t* ids, double* weights);
int orc_mixture_reference(const double* experts, const double* weights, uint64_t nweights,
                          const double* shared, uint64_t channels, double shared_logit,
                          double* out);

/* ---- Pack v3 planar expert layout: src/planar_pack_v3.cpp:601-896 ---- */
typedef struct {
    uint32_t source_type, columns, rows, blocks_per_row;
    uint64_t source_row_bytes, planar_row_bytes, source_expert_bytes, planar_expert_bytes;
    uint64_t qs_offset, qh_offset, sm_offset, dm_offset;
} orc_planar_spec;
int orc_make_expert_spec(uint32_t source_type, uint32_t columns, uint32_t rows, orc_planar_spec* s);
void orc_pack_sm16(const uint8_t s12[12], uint8_t sm[16]);
int orc_unpack_sm16(const uint8_t sm[16], uint8_t s12[12]);
int orc_pack_expert_planar_v3(const orc_planar_spec* s, const uint8_t* gguf, uint64_t gguf_bytes,
                              uint8_t* planar, uint64_t planar_bytes);
int orc_unpack_expert_planar_v3(const orc_planar_spec* s, const uint8_t* planar,
                                uint64_t planar_bytes, uint8_t* gguf, uint64_t gguf_bytes);
int orc_dequantize_expert_planar_v3(const orc_planar_spec* s, const uint8_t* planar,
                                    uint64_t planar_bytes, float* out, uint64_t nelem);
int orc_dequantize_expert_planar_v3_f32(const orc_planar_spec* s, const uint8_t* planar,
                                        uint64_t planar_bytes, float* out, uint64_t nelem);
/* Gate/up co-location, src/planar_pack_v3.cpp:1061-1123: tensor `half` (0 = pair_lo, 1 = pair_hi)
 * holds experts half*E/2 .. half*E/2+E/2-1 as interleaved [gate_e, up_e] planar experts. */
int orc_pack_coloc_half(const orc_planar_spec* s, const uint8_t* gate_gguf, const uint8_t* up_gguf,
                        uint32_t experts, uint32_t half, uint8_t* out, uint64_t out_bytes);

/* ---- q8_lanes_v1 row layout: src/expert_lanes.cpp:60-119 (type 8 only) ---- */
int orc_q8_lanes_quant_offset(uint32_t columns, uint32_t block, uint32_t index, uint64_t* offset);
int orc_q8_lanes_pack_rows(uint32_t columns, const uint8_t* original, uint8_t* packed, uint64_t bytes);
int orc_q8_lanes_unpack_rows(uint32_t columns, const uint8_t* packed, uint8_t* original, uint64_t bytes);
/* ---- q51_lanes_v1 row layout: src/expert_lanes.cpp:60-119 (type 7) ---- */
int orc_q51_lanes_quant_offset(uint32_t columns, uint32_t block, uint32_t index, uint64_t* offset);
int orc_q51_lanes_pack_rows(uint32_t columns, const uint8_t* original, uint8_t* packed, uint64_t bytes);
int orc_q51_lanes_unpack_rows(uint32_t columns, const uint8_t* packed, uint8_t* original, uint64_t bytes);

/* ---- expert permutation + prefix-sum offsets: kernels/grouped_mpp.metal:12-64 ---- */
/* error |= 4 on id >= experts, duplicate expert within one token, off > bound, sum != T*S. */
int orc_grouped_routes(const uint32_t* ids, uint32_t experts, uint32_t selected, uint32_t tokens,
                       uint32_t* token_map, uint32_t* counts, uint32_t* error);
int orc_grouped_tasks(const uint32_t* counts, uint32_t experts, uint32_t selected, uint32_t tokens,
                      uint32_t tile, uint32_t* tasks, uint32_t* error);

/* ---- union records for T <= 8: tests/test_planar_union_metadata.mm:27-55 ---- */
/* meta has 2320 words; only the words the specification touches are written. */
int orc_union_metadata(uint32_t experts, uint32_t selected, uint32_t tokens, uint32_t hidden,
                       uint32_t channels, const uint32_t* ids, uint32_t* meta, uint32_t* error);

/* ---- row top-64: src/sampling.cpp:473-513, include/tokspur/sampling.hpp:21-29 ---- */
typedef struct {
    uint32_t vocabulary, count, first_nonfinite_col, first_subnormal_col;
    uint32_t ids[64];
    float logits[64];
} orc_logit_topk_row;
int orc_logit_topk_row_cpu(const float* logits, uint64_t n, orc_logit_topk_row* out);

/* ---- plan geometry: src/grouped_mm.cpp:24-54, src/moe_mm_many_plan.cpp:28-52 ---- */
typedef struct {
    uint32_t columns, rows, row_bytes, experts, selected, tokens, broadcast, maximum_tasks;
    uint64_t expert_stride_bytes, input_stride_bytes, output_stride_bytes;
} orc_grouped_mm_args; /* 56 bytes, include/tokspur/grouped_mm.hpp:8-13 */
typedef struct {
    orc_grouped_mm_args args;
    uint64_t matrix_bytes, indices_bytes, input_bytes, output_bytes;
    uint64_t token_map_bytes, counts_bytes, tasks_bytes;
    uint32_t grid_x, grid_y;
} orc_grouped_mm_plan;
int orc_grouped_mm_plan_make(uint32_t type, uint32_t layout, uint32_t columns, uint32_t rows,
                             uint32_t experts, uint32_t selected, uint32_t tokens,
                             uint64_t input_stride, uint64_t output_stride, int broadcast,
                             int allow_nax_2k, orc_grouped_mm_plan* plan);
int orc_moe_mm_many_bytes(uint32_t channels, uint32_t hidden, uint32_t experts, uint32_t selected,
                          uint32_t capacity, int allow_nax_2k, uint64_t views[13], uint64_t* total);

/* ---- staging helpers ---- */
/* kernels/planar_moe_v3.metal:82-94: RNE bf16 bits of a finite float; 1 in *bad if non-finite. */
uint16_t orc_round_bf16_bits(float v, uint32_t* bad);
float orc_bf16_to_f32(uint16_t bits);

/* ---- MoE compositions (CPU double reference) ----
 * tests/test_planar_pack_v3.cpp:433-697 and tests/test_moe.cpp:131-163: dequantize -> double dot
 * -> silu -> double dot. gate/up/down are raw GGUF expert stacks [experts][rows][row bytes].
 * hidden_out [routes, hidden] and down_out [routes, channels] are doubles; route r = t*selected+j
 * uses input row t. silu_f32 != 0 evaluates silu(g)*u in float like the planar tests do
 * (test_planar_pack_v3.cpp silu_f32), else in double via stable_silu (src/ffn_check.cpp:117-141). */
int orc_moe_routed_reference(uint32_t gate_up_type, uint32_t down_type, const uint8_t* gate,
                             const uint8_t* up, const uint8_t* down, uint32_t channels,
                             uint32_t hidden, uint32_t experts, const uint32_t* ids,
                             uint32_t tokens, uint32_t selected, const float* input,
                             uint64_t input_stride_floats, int silu_f32, int stage_bf16,
                             double* hidden_out, double* down_out, uint32_t threads);

/* binary32 -> binary16 (RNE) -> binary32: the half staging of kernels/grouped_mm.metal:214-216. */
float orc_round_f16(float v);
/* Declared-precision dense reference, tests/test_moe_mm_many_gpu.cpp:54-63: weights optionally staged,
 * sequential double accumulation; evaluates the weight rows listed in rows_sel (NULL = first nsel).
 * out is [tokens][nsel]. stage_f16: 0 = f32-dequantised weights, 1 = weights rounded to half
 * (kernels/grouped_mm.metal:214-216), 2 = Q6_K rows as d * half(sc * (q - 32)), the staging of a matrix-core
 * kernel that multiplies the integer products as halves and applies d in f32 (no reference counterpart;
 * other types unchanged).
 * `stage` in orc_moe_routed_reference: bit 0 = activations and h as bf16 (kernels/planar_moe_v3.metal:82-94,
 * 2406-2483), bit 1 = weights as half, bit 2 = activations as bf16 and h as 256 * half(h / 256), bit 3 = Q6_K
 * down rows staged as under stage_f16 = 2, bit 4 = gate and up weights as half, bit 5 = down weights as half (bit 1 for one
 * product only). Bits 2 to 5 describe the HIP kernels, not the reference. */
int orc_staged_gemm(uint32_t type, const uint8_t* matrix, uint32_t columns, const uint32_t* rows_sel, uint32_t nsel,
                    const float* x, uint64_t x_stride_floats, uint32_t tokens, int stage_f16, double* out, uint32_t threads);

/* tests/grouped_mm_fixture.hpp:10-19 — the reference tests' LCG weight fixture generator. */
int orc_fixture_weights(uint32_t type, uint32_t k, uint32_t r, uint32_t e, uint8_t* out, uint64_t nbytes);

#ifdef __cplusplus
}
#endif
#endif
