/*
 * TEST INFRASTRUCTURE ONLY — see tokspur_oracle.h.
 *
 * Scalar, double-accumulating CPU restatement of the tokspur native engine's
 * numerical references for the quantized matmul / MoE path. Paths in the
 * citations are relative to the reference tree's native/ directory.
 */
#include "tokspur_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#define REQUIRE(cond) do { if (!(cond)) return ORC_FORMAT_ERROR; } while (0)

static uint32_t f32_bits(float v) { uint32_t b; memcpy(&b, &v, 4); return b; }
static float bits_f32(uint32_t b) { float v; memcpy(&v, &b, 4); return v; }
static uint16_t word_le(const uint8_t* p) { return (uint16_t)(p[0] | ((uint16_t)p[1] << 8)); }
static uint32_t dword_le(const uint8_t* p) { return (uint32_t)word_le(p) | ((uint32_t)word_le(p + 2) << 16); }

static int mul_overflows(uint64_t a, uint64_t b) { return a && b > UINT64_MAX / a; }

/* ------------------------------------------------------------------------- */
/* src/numeric.cpp:81-91 — IEEE binary16 bits to float.                      */
float orc_binary16(uint16_t bits) {
    const uint32_t sign = (uint32_t)(bits & 0x8000u) << 16;
    uint32_t mantissa = bits & 1023u;
    const uint32_t exponent = (bits >> 10) & 31u;
    if (exponent == 31) return bits_f32(sign | 0x7f800000u | (mantissa << 13));
    if (exponent) return bits_f32(sign | ((exponent + 112u) << 23) | (mantissa << 13));
    if (!mantissa) return bits_f32(sign);
    uint32_t e = 113;
    while (!(mantissa & 1024u)) { mantissa <<= 1; --e; }
    return bits_f32(sign | (e << 23) | ((mantissa & 1023u) << 13));
}

/* src/gguf.cpp:21-32 — encoded block geometry table. */
int orc_encoding(uint32_t type, uint32_t* elements, uint32_t* bytes) {
    static const uint32_t table[][3] = {
        {0, 1, 4}, {1, 1, 2}, {2, 32, 18}, {3, 32, 20}, {6, 32, 22}, {7, 32, 24}, {8, 32, 34},
        {10, 256, 84}, {11, 256, 110}, {12, 256, 144}, {13, 256, 176}, {14, 256, 210},
        {20, 32, 18}, {23, 256, 136}, {24, 1, 1}, {25, 1, 2}, {26, 1, 4}, {27, 1, 8}, {28, 1, 8},
        {30, 1, 2},
    };
    for (size_t i = 0; i < sizeof table / sizeof table[0]; ++i)
        if (table[i][0] == type) { *elements = table[i][1]; *bytes = table[i][2]; return ORC_OK; }
    return ORC_FORMAT_ERROR;
}

/* src/numeric.cpp:93-95 */
int orc_can_decode(uint32_t type) {
    return type == 0 || type == 1 || type == 7 || type == 8 || type == 12 || type == 13 ||
           type == 14 || type == 20 || type == 30;
}

/* src/numeric.cpp:25-31 — 6-bit scale/min of Q4_K/Q5_K sub-block `group`. */
static uint32_t group_scale(const uint8_t* block, uint32_t group, int minimum) {
    const uint32_t lane = group % 4;
    if (group < 4) return block[4 + lane + (minimum ? 4 : 0)] & 63u;
    const uint32_t packed = block[12 + lane];
    const uint32_t upper = block[4 + lane + (minimum ? 4 : 0)] >> 6;
    return ((packed >> (minimum ? 4 : 0)) & 15u) | (upper << 4);
}

/* src/numeric.cpp:33-68 — one weight of one block, in double. */
int orc_value(uint32_t type, const uint8_t* block, uint32_t index, double* out) {
    switch (type) {
    case 0: *out = bits_f32(dword_le(block)); return ORC_OK;
    case 1: *out = orc_binary16(word_le(block)); return ORC_OK;
    case 30: *out = bits_f32((uint32_t)word_le(block) << 16); return ORC_OK;
    case 7: {
        const uint32_t low = (block[8 + index % 16] >> (4 * (index / 16))) & 15u;
        const uint32_t high = (dword_le(block + 4) >> index) & 1u;
        *out = (double)orc_binary16(word_le(block)) * (low | (high << 4)) + orc_binary16(word_le(block + 2));
        return ORC_OK;
    }
    case 8:
        *out = (double)orc_binary16(word_le(block)) * (int8_t)block[2 + index];
        return ORC_OK;
    case 12: case 13: {
        const uint32_t low_offset = type == 12 ? 16 : 48;
        uint32_t quant = (block[low_offset + (index / 64) * 32 + index % 32] >> (4 * ((index % 64) / 32))) & 15u;
        if (type == 13) quant |= ((block[16 + index % 32] >> (index / 32)) & 1u) << 4;
        *out = (double)orc_binary16(word_le(block)) * group_scale(block, index / 32, 0) * quant -
               (double)orc_binary16(word_le(block + 2)) * group_scale(block, index / 32, 1);
        return ORC_OK;
    }
    case 14: {
        const uint32_t within = index % 128, section = index / 128;
        const uint32_t low = (block[section * 64 + within % 64] >> (4 * (within / 64))) & 15u;
        const uint32_t high = (block[128 + section * 32 + within % 32] >> (2 * (within / 32))) & 3u;
        const int scale = (int8_t)block[192 + index / 16];
        *out = (double)orc_binary16(word_le(block + 208)) * scale * ((int)(low | (high << 4)) - 32);
        return ORC_OK;
    }
    case 20: {
        static const int alphabet[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
        const uint32_t code = (block[2 + index % 16] >> (4 * (index / 16))) & 15u;
        *out = (double)orc_binary16(word_le(block)) * alphabet[code];
        return ORC_OK;
    }
    default: return ORC_FORMAT_ERROR;
    }
}

/* src/numeric.cpp:70-78 */
static int validate(uint32_t type, uint64_t bytes, uint64_t elements, uint32_t* epb, uint32_t* bpb) {
    REQUIRE(orc_can_decode(type));
    REQUIRE(orc_encoding(type, epb, bpb) == ORC_OK);
    REQUIRE(elements && elements % *epb == 0);
    REQUIRE(!mul_overflows(elements / *epb, *bpb) && (elements / *epb) * *bpb == bytes);
    return ORC_OK;
}

/* src/numeric.cpp:97-148 (general branch) — double value, one cast to float, finite-checked. */
int orc_dequantize(uint32_t type, const uint8_t* bytes, uint64_t nbytes, float* out, uint64_t nelem) {
    uint32_t epb, bpb;
    REQUIRE(validate(type, nbytes, nelem, &epb, &bpb) == ORC_OK);
    for (uint64_t start = 0; start < nelem; start += epb) {
        const uint8_t* block = bytes + (start / epb) * bpb;
        for (uint32_t i = 0; i < epb; ++i) {
            double decoded;
            REQUIRE(orc_value(type, block, i, &decoded) == ORC_OK);
            REQUIRE(isfinite(decoded));
            const float rounded = (float)decoded;
            REQUIRE(isfinite(rounded));
            out[start + i] = rounded;
        }
    }
    return ORC_OK;
}

/* src/numeric.cpp:150-174 — sequential double accumulation, row-major blocks. */
static int gemv_rows(uint32_t type, const uint8_t* matrix, uint32_t columns, uint32_t row_begin,
                     uint32_t row_end, const float* xf, const double* xd, double* y,
                     uint32_t epb, uint32_t bpb) {
    const uint64_t blocks_per_row = columns / epb;
    for (uint32_t row = row_begin; row < row_end; ++row) {
        double sum = 0;
        for (uint64_t group = 0; group < blocks_per_row; ++group) {
            const uint8_t* block = matrix + ((uint64_t)row * blocks_per_row + group) * bpb;
            for (uint32_t i = 0; i < epb; ++i) {
                double weight;
                REQUIRE(orc_value(type, block, i, &weight) == ORC_OK);
                REQUIRE(isfinite(weight));
                const double x = xf ? (double)xf[group * epb + i] : xd[group * epb + i];
                sum += weight * x;
            }
        }
        REQUIRE(isfinite(sum));
        y[row] = sum;
    }
    return ORC_OK;
}

static int gemv_check(uint32_t type, uint64_t nbytes, uint32_t columns, uint32_t rows,
                      const float* xf, const double* xd, uint64_t nx, uint32_t* epb, uint32_t* bpb) {
    REQUIRE(rows && columns == nx);
    REQUIRE(!mul_overflows(columns, rows));
    REQUIRE(validate(type, nbytes, (uint64_t)columns * rows, epb, bpb) == ORC_OK);
    REQUIRE(columns % *epb == 0);
    for (uint64_t i = 0; i < nx; ++i) REQUIRE(isfinite(xf ? (double)xf[i] : xd[i]));
    return ORC_OK;
}

int orc_reference_gemv(uint32_t type, const uint8_t* matrix, uint64_t nbytes, uint32_t columns,
                       uint32_t rows, const float* x, uint64_t nx, double* y) {
    uint32_t epb, bpb;
    REQUIRE(gemv_check(type, nbytes, columns, rows, x, NULL, nx, &epb, &bpb) == ORC_OK);
    return gemv_rows(type, matrix, columns, 0, rows, x, NULL, y, epb, bpb);
}

int orc_reference_gemv_doubleinput(uint32_t type, const uint8_t* matrix, uint64_t nbytes,
                                   uint32_t columns, uint32_t rows, const double* x, uint64_t nx,
                                   double* y) {
    uint32_t epb, bpb;
    REQUIRE(gemv_check(type, nbytes, columns, rows, NULL, x, nx, &epb, &bpb) == ORC_OK);
    return gemv_rows(type, matrix, columns, 0, rows, NULL, x, y, epb, bpb);
}

typedef struct {
    uint32_t type, columns, row_begin, row_end, epb, bpb;
    const uint8_t* matrix; const float* x; double* y; int status;
} gemv_job;

static void* gemv_worker(void* arg) {
    gemv_job* j = (gemv_job*)arg;
    j->status = gemv_rows(j->type, j->matrix, j->columns, j->row_begin, j->row_end, j->x, NULL, j->y, j->epb, j->bpb);
    return NULL;
}

int orc_reference_gemv_mt(uint32_t type, const uint8_t* matrix, uint64_t nbytes, uint32_t columns,
                          uint32_t rows, const float* x, uint64_t nx, double* y, uint32_t threads) {
    uint32_t epb, bpb;
    REQUIRE(gemv_check(type, nbytes, columns, rows, x, NULL, nx, &epb, &bpb) == ORC_OK);
    if (threads < 1) threads = 1;
    if (threads > 256) threads = 256;
    if (threads > rows) threads = rows;
    pthread_t ids[256]; gemv_job jobs[256];
    for (uint32_t t = 0; t < threads; ++t) {
        jobs[t] = (gemv_job){type, columns, (uint32_t)((uint64_t)rows * t / threads),
                             (uint32_t)((uint64_t)rows * (t + 1) / threads), epb, bpb, matrix, x, y, 0};
        if (pthread_create(&ids[t], NULL, gemv_worker, &jobs[t])) { jobs[t].status = -1; gemv_worker(&jobs[t]); ids[t] = 0; }
    }
    int status = ORC_OK;
    for (uint32_t t = 0; t < threads; ++t) { if (ids[t]) pthread_join(ids[t], NULL); if (jobs[t].status) status = ORC_FORMAT_ERROR; }
    return status;
}

/* src/q8_many.cpp:20-29 (ordinary build: no three-row width) */
int orc_q8_many_width(uint32_t remaining, uint32_t* width) {
    REQUIRE(remaining);
    *width = remaining >= 8 ? 8 : remaining >= 4 ? 4 : remaining >= 2 ? 2 : 1;
    return ORC_OK;
}
/* src/q8_many.cpp:30-35 */
int orc_q8_many_chunks(uint32_t rows, uint32_t* chunks) {
    REQUIRE(rows && rows <= 65536);
    uint32_t n = 0, w;
    while (rows) { orc_q8_many_width(rows, &w); rows -= w; ++n; }
    *chunks = n;
    return ORC_OK;
}
/* src/q8_many.cpp:7-19,36-49 — token-major input [width, columns] -> [width, rows]. */
int orc_reference_q8_many(const uint8_t* matrix, uint64_t nbytes, const float* input,
                          uint32_t columns, uint32_t rows, uint32_t width, double* out) {
    REQUIRE(columns && columns <= 65536 && columns % 32 == 0 && rows && rows <= 1000000);
    REQUIRE(width == 1 || width == 2 || width == 4 || width == 8);
    REQUIRE((uint64_t)(columns / 32) * rows * 34 == nbytes);
    for (uint64_t i = 0; i < (uint64_t)columns * width; ++i) REQUIRE(isfinite(input[i]));
    for (uint32_t token = 0; token < width; ++token)
        REQUIRE(orc_reference_gemv(8, matrix, nbytes, columns, rows, input + (uint64_t)token * columns,
                                   columns, out + (uint64_t)token * rows) == ORC_OK);
    return ORC_OK;
}

/* ------------------------------------------------------------------------- */
/* src/operators.cpp:28-40                                                   */
int orc_stable_sigmoid(double v, double* out) {
    REQUIRE(isfinite(v));
    if (v >= 0) { *out = 1 / (1 + exp(-v)); return ORC_OK; }
    const double positive = exp(v);
    *out = positive / (1 + positive);
    return ORC_OK;
}
int orc_stable_silu(double v, double* out) {
    double s;
    REQUIRE(orc_stable_sigmoid(v, &s) == ORC_OK);
    *out = v * s;
    return ORC_OK;
}
int orc_stable_softplus(double v, double* out) {
    REQUIRE(isfinite(v));
    *out = (v > 0 ? v : 0.0) + log1p(exp(-fabs(v)));
    return ORC_OK;
}

/* ------------------------------------------------------------------------- */
/* src/operators.cpp:42-58 — independent groups, double accumulation, gains per element. */
int orc_group_rms_reference(const double* input, const double* gains, uint64_t count, uint64_t group_width,
                            double epsilon, double* output) {
    REQUIRE(group_width && count && count % group_width == 0 && isfinite(epsilon) && epsilon > 0);
    for (uint64_t i = 0; i < count; ++i) REQUIRE(isfinite(input[i]) && isfinite(gains[i]));
    for (uint64_t group = 0; group < count; group += group_width) {
        double squared = 0;
        for (uint64_t i = 0; i < group_width; ++i) squared += input[group + i] * input[group + i];
        REQUIRE(isfinite(squared));
        const double inverse = 1 / sqrt(squared / (double)group_width + epsilon);
        for (uint64_t i = 0; i < group_width; ++i) output[group + i] = input[group + i] * inverse * gains[group + i];
    }
    for (uint64_t i = 0; i < count; ++i) REQUIRE(isfinite(output[i]));
    return ORC_OK;
}

/* src/operators.cpp:60-84 — streams [branch, channel]; down [rank, width], up [width, rank], inject [branches, width],
 * width = branches * channels: normalise, bottleneck = silu(down n / branches), scores = up bottleneck,
 * read[c] = mean_b n[b, c] sigmoid(scores[b, c]), write_scales[b] = 2 sigmoid((inject n)[b] / branches). */
int orc_gated_residual_reference(const double* streams, const double* gains, const double* down, const double* up,
                                 const double* inject, uint64_t branches, uint64_t channels, uint64_t rank, double epsilon,
                                 double* read, double* write_scales) {
    REQUIRE(branches && channels && rank);
    const uint64_t width = branches * channels;
    double* normalized = (double*)malloc(width * sizeof(double));
    double* bottleneck = (double*)malloc(rank * sizeof(double));
    REQUIRE(normalized && bottleneck);
    int rc = orc_group_rms_reference(streams, gains, width, channels, epsilon, normalized);
    if (rc == ORC_OK) {
        for (uint64_t r = 0; r < rank && rc == ORC_OK; ++r) {
            double sum = 0;
            for (uint64_t i = 0; i < width; ++i) sum += down[r * width + i] * normalized[i];
            rc = orc_stable_silu(sum / (double)branches, &bottleneck[r]);
        }
    }
    for (uint64_t c = 0; c < channels; ++c) read[c] = 0;
    for (uint64_t b = 0; b < branches && rc == ORC_OK; ++b) {
        double scale = 0, gate;
        for (uint64_t i = 0; i < width; ++i) scale += inject[b * width + i] * normalized[i];
        rc = orc_stable_sigmoid(scale / (double)branches, &gate);
        write_scales[b] = 2 * gate;
        for (uint64_t c = 0; c < channels && rc == ORC_OK; ++c) {
            const uint64_t at = b * channels + c;
            double score = 0;
            for (uint64_t r = 0; r < rank; ++r) score += up[at * rank + r] * bottleneck[r];
            rc = orc_stable_sigmoid(score, &gate);
            read[c] += normalized[at] * gate / (double)branches;
        }
    }
    free(normalized);
    free(bottleneck);
    return rc;
}

/* src/operators.cpp:86-96 */
int orc_residual_write_reference(const double* streams, const double* output, const double* scales, uint64_t branches,
                                 uint64_t channels, double* result) {
    REQUIRE(branches && channels);
    for (uint64_t b = 0; b < branches; ++b)
        for (uint64_t c = 0; c < channels; ++c) {
            const double v = streams[b * channels + c] + scales[b] * output[c];
            REQUIRE(isfinite(v));
            result[b * channels + c] = v;
        }
    return ORC_OK;
}

/* ------------------------------------------------------------------------- */
/* src/routing.cpp:11-40 — top-k by (logit desc, id asc); softmax / sigmoid weights. */
static double route_activate(const double* logits, uint32_t index, double maximum, uint32_t mode, int normalize) {
    double a, b;
    if (mode == 0) return exp(logits[index] - maximum);
    if (normalize) { orc_stable_softplus(-logits[index], &a); orc_stable_softplus(-maximum, &b); return exp(-a + b); }
    orc_stable_sigmoid(logits[index], &a);
    return a;
}

int orc_route_reference(const double* logits, uint64_t count, uint64_t selected, uint32_t mode,
                        int normalize_selected, uint32_t* ids, double* weights) {
    REQUIRE(count && count <= 4096 && selected && selected <= 64 && selected <= count && mode <= 1);
    for (uint64_t i = 0; i < count; ++i) REQUIRE(isfinite(logits[i]));
    uint8_t taken[4096];
    memset(taken, 0, count);
    /* The comparator is a strict total order, so partial_sort's result is the k smallest keys in
     * order: k rounds of selection produce the same sequence. */
    for (uint64_t j = 0; j < selected; ++j) {
        uint32_t best = UINT32_MAX;
        for (uint32_t i = 0; i < count; ++i) {
            if (taken[i]) continue;
            if (best == UINT32_MAX || logits[i] > logits[best]) best = i; /* ascending scan keeps the lower id on ties */
        }
        taken[best] = 1;
        ids[j] = best;
    }
    const double maximum = logits[ids[0]];
    double denominator = mode == 1 ? 1 : 0;
    if (normalize_selected) {
        denominator = 0;
        for (uint64_t j = 0; j < selected; ++j) denominator += route_activate(logits, ids[j], maximum, mode, normalize_selected);
    } else if (mode == 0) {
        for (uint32_t i = 0; i < count; ++i) denominator += route_activate(logits, i, maximum, mode, normalize_selected);
    }
    REQUIRE(isfinite(denominator) && denominator > 0);
    for (uint64_t j = 0; j < selected; ++j)
        weights[j] = route_activate(logits, ids[j], maximum, mode, normalize_selected) / denominator;
    return ORC_OK;
}

/* src/routing.cpp:42-60 — y[c] = sigmoid(shared_logit)*shared[c] + sum_j w[j]*experts[j][c], j in route order. */
int orc_mixture_reference(const double* experts, const double* weights, uint64_t nweights,
                          const double* shared, uint64_t channels, double shared_logit, double* out) {
    REQUIRE(channels && channels <= 65536 && nweights && nweights <= 64);
    for (uint64_t j = 0; j < nweights; ++j) REQUIRE(isfinite(weights[j]) && weights[j] >= 0);
    double gate;
    REQUIRE(orc_stable_sigmoid(shared_logit, &gate) == ORC_OK);
    for (uint64_t c = 0; c < channels; ++c) {
        REQUIRE(isfinite(shared[c]));
        double value = gate * shared[c];
        for (uint64_t j = 0; j < nweights; ++j) {
            const double contribution = experts[j * channels + c];
            REQUIRE(isfinite(contribution));
            value += weights[j] * contribution;
        }
        REQUIRE(isfinite(value));
        out[c] = value;
    }
    return ORC_OK;
}

/* ------------------------------------------------------------------------- */
/* src/planar_pack_v3.cpp:601-650                                            */
int orc_make_expert_spec(uint32_t source_type, uint32_t columns, uint32_t rows, orc_planar_spec* s) {
    REQUIRE(rows >= 4 && rows % 4 == 0);
    memset(s, 0, sizeof *s);
    s->source_type = source_type; s->columns = columns; s->rows = rows;
    if (source_type == 12 || source_type == 13) {
        REQUIRE(columns >= 256 && columns % 256 == 0);
        s->blocks_per_row = columns / 256;
        const uint64_t total = (uint64_t)rows * s->blocks_per_row;
        if (source_type == 12) {
            s->source_row_bytes = (uint64_t)s->blocks_per_row * 144;
            s->planar_row_bytes = (uint64_t)s->blocks_per_row * 148;
            s->sm_offset = total * 128; s->dm_offset = total * 144;
        } else {
            s->source_row_bytes = (uint64_t)s->blocks_per_row * 176;
            s->planar_row_bytes = (uint64_t)s->blocks_per_row * 180;
            s->qh_offset = total * 128; s->sm_offset = total * 160; s->dm_offset = total * 176;
        }
    } else if (source_type == 7) {
        REQUIRE(columns >= 32 && columns % 32 == 0);
        s->blocks_per_row = columns / 32;
        const uint64_t total = (uint64_t)rows * s->blocks_per_row;
        s->source_row_bytes = s->planar_row_bytes = (uint64_t)s->blocks_per_row * 24;
        s->qh_offset = total * 16; s->dm_offset = total * 20;
    } else if (source_type == 8) {
        REQUIRE(columns >= 32 && columns % 32 == 0);
        s->blocks_per_row = columns / 32;
        const uint64_t total = (uint64_t)rows * s->blocks_per_row;
        REQUIRE(total % 8 == 0);
        s->source_row_bytes = s->planar_row_bytes = (uint64_t)s->blocks_per_row * 34;
        s->dm_offset = total * 32;
    } else return ORC_FORMAT_ERROR;
    s->source_expert_bytes = (uint64_t)rows * s->source_row_bytes;
    s->planar_expert_bytes = (uint64_t)rows * s->planar_row_bytes;
    REQUIRE(s->planar_expert_bytes % 16 == 0);
    return ORC_OK;
}

/* src/planar_pack_v3.cpp:652-661 — 12 packed bytes -> sc[8], mn[8], one byte each (0..63). */
void orc_pack_sm16(const uint8_t s12[12], uint8_t sm[16]) {
    for (uint32_t slot = 0; slot < 4; ++slot) {
        sm[slot] = (uint8_t)(s12[slot] & 0x3fu);
        sm[4 + slot] = (uint8_t)((s12[8 + slot] & 0x0fu) | ((s12[slot] >> 6) << 4));
        sm[8 + slot] = (uint8_t)(s12[4 + slot] & 0x3fu);
        sm[12 + slot] = (uint8_t)((s12[8 + slot] >> 4) | ((s12[4 + slot] >> 6) << 4));
    }
}

/* src/planar_pack_v3.cpp:663-674 */
int orc_unpack_sm16(const uint8_t sm[16], uint8_t s12[12]) {
    for (uint32_t i = 0; i < 16; ++i) REQUIRE((sm[i] & 0xc0u) == 0);
    for (uint32_t slot = 0; slot < 4; ++slot) {
        s12[slot] = (uint8_t)((sm[slot] & 0x3fu) | ((sm[4 + slot] >> 4) << 6));
        s12[4 + slot] = (uint8_t)((sm[8 + slot] & 0x3fu) | ((sm[12 + slot] >> 4) << 6));
        s12[8 + slot] = (uint8_t)((sm[4 + slot] & 0x0fu) | ((sm[12 + slot] & 0x0fu) << 4));
    }
    return ORC_OK;
}

/* src/planar_pack_v3.cpp:676-716 */
int orc_pack_expert_planar_v3(const orc_planar_spec* s, const uint8_t* src, uint64_t gguf_bytes,
                              uint8_t* dst, uint64_t planar_bytes) {
    REQUIRE(gguf_bytes == s->source_expert_bytes && planar_bytes == s->planar_expert_bytes);
    const uint64_t total = (uint64_t)s->rows * s->blocks_per_row;
    for (uint64_t blk = 0; blk < total; ++blk) {
        if (s->source_type == 12) {
            const uint8_t* sb = src + blk * 144;
            memcpy(dst + s->qs_offset + blk * 128, sb + 16, 128);
            orc_pack_sm16(sb + 4, dst + s->sm_offset + blk * 16);
            memcpy(dst + s->dm_offset + blk * 4, sb, 4);
        } else if (s->source_type == 13) {
            const uint8_t* sb = src + blk * 176;
            memcpy(dst + s->qs_offset + blk * 128, sb + 48, 128);
            memcpy(dst + s->qh_offset + blk * 32, sb + 16, 32);
            orc_pack_sm16(sb + 4, dst + s->sm_offset + blk * 16);
            memcpy(dst + s->dm_offset + blk * 4, sb, 4);
        } else if (s->source_type == 7) {
            const uint8_t* sb = src + blk * 24;
            memcpy(dst + s->qs_offset + blk * 16, sb + 8, 16);
            memcpy(dst + s->qh_offset + blk * 4, sb + 4, 4);
            memcpy(dst + s->dm_offset + blk * 4, sb, 4);
        } else if (s->source_type == 8) {
            const uint8_t* sb = src + blk * 34;
            memcpy(dst + s->qs_offset + blk * 32, sb + 2, 32);
            memcpy(dst + s->dm_offset + blk * 2, sb, 2);
        } else return ORC_FORMAT_ERROR;
    }
    return ORC_OK;
}

/* src/planar_pack_v3.cpp:718-758 */
int orc_unpack_expert_planar_v3(const orc_planar_spec* s, const uint8_t* src, uint64_t planar_bytes,
                                uint8_t* dst, uint64_t gguf_bytes) {
    REQUIRE(planar_bytes == s->planar_expert_bytes && gguf_bytes == s->source_expert_bytes);
    const uint64_t total = (uint64_t)s->rows * s->blocks_per_row;
    for (uint64_t blk = 0; blk < total; ++blk) {
        if (s->source_type == 12) {
            uint8_t* sb = dst + blk * 144;
            memcpy(sb, src + s->dm_offset + blk * 4, 4);
            REQUIRE(orc_unpack_sm16(src + s->sm_offset + blk * 16, sb + 4) == ORC_OK);
            memcpy(sb + 16, src + s->qs_offset + blk * 128, 128);
        } else if (s->source_type == 13) {
            uint8_t* sb = dst + blk * 176;
            memcpy(sb, src + s->dm_offset + blk * 4, 4);
            REQUIRE(orc_unpack_sm16(src + s->sm_offset + blk * 16, sb + 4) == ORC_OK);
            memcpy(sb + 16, src + s->qh_offset + blk * 32, 32);
            memcpy(sb + 48, src + s->qs_offset + blk * 128, 128);
        } else if (s->source_type == 7) {
            uint8_t* sb = dst + blk * 24;
            memcpy(sb, src + s->dm_offset + blk * 4, 4);
            memcpy(sb + 4, src + s->qh_offset + blk * 4, 4);
            memcpy(sb + 8, src + s->qs_offset + blk * 16, 16);
        } else if (s->source_type == 8) {
            uint8_t* sb = dst + blk * 34;
            memcpy(sb, src + s->dm_offset + blk * 2, 2);
            memcpy(sb + 2, src + s->qs_offset + blk * 32, 32);
        } else return ORC_FORMAT_ERROR;
    }
    return ORC_OK;
}

/* src/planar_pack_v3.cpp:760-896 — `wide` selects the double (760-827) or float (829-896) arithmetic. */
static int planar_dequant(const orc_planar_spec* s, const uint8_t* base, uint64_t planar_bytes,
                          float* out, uint64_t nelem, int wide) {
    REQUIRE(planar_bytes == s->planar_expert_bytes && nelem == (uint64_t)s->rows * s->columns);
    const uint64_t total = (uint64_t)s->rows * s->blocks_per_row;
    if (s->source_type == 12 || s->source_type == 13) {
        for (uint64_t blk = 0; blk < total; ++blk) {
            const uint8_t* qs = base + s->qs_offset + blk * 128;
            const uint8_t* qh = s->source_type == 13 ? base + s->qh_offset + blk * 32 : NULL;
            const uint8_t* sm = base + s->sm_offset + blk * 16;
            const uint8_t* dm = base + s->dm_offset + blk * 4;
            const float df = orc_binary16(word_le(dm)), dminf = orc_binary16(word_le(dm + 2));
            REQUIRE(isfinite(df) && isfinite(dminf));
            float* o = out + blk * 256;
            for (uint32_t grp = 0; grp < 8; ++grp) {
                const uint32_t pair = grp >> 1, shift = (grp & 1u) * 4u;
                for (uint32_t l = 0; l < 32; ++l) {
                    uint32_t q = (qs[pair * 32 + l] >> shift) & 15u;
                    if (qh) q |= (((uint32_t)qh[l] >> grp) & 1u) << 4;
                    float val;
                    if (wide) {
                        const double dl = (double)df * sm[grp], ml = (double)dminf * sm[8 + grp];
                        val = (float)(dl * q - ml);
                    } else {
                        const float dl = df * (float)sm[grp], ml = dminf * (float)sm[8 + grp];
                        val = dl * (float)q - ml;
                    }
                    REQUIRE(isfinite(val));
                    o[grp * 32 + l] = val;
                }
            }
        }
    } else if (s->source_type == 7) {
        for (uint64_t blk = 0; blk < total; ++blk) {
            const uint8_t* qs = base + s->qs_offset + blk * 16;
            const uint32_t qh = dword_le(base + s->qh_offset + blk * 4);
            const uint8_t* dm = base + s->dm_offset + blk * 4;
            const float df = orc_binary16(word_le(dm)), mf = orc_binary16(word_le(dm + 2));
            REQUIRE(isfinite(df) && isfinite(mf));
            for (uint32_t i = 0; i < 32; ++i) {
                const uint32_t low = (qs[i % 16] >> (4 * (i / 16))) & 15u, high = (qh >> i) & 1u;
                const float val = wide ? (float)((double)df * (low | (high << 4)) + (double)mf)
                                       : df * (float)(low | (high << 4)) + mf;
                REQUIRE(isfinite(val));
                out[blk * 32 + i] = val;
            }
        }
    } else if (s->source_type == 8) {
        for (uint64_t blk = 0; blk < total; ++blk) {
            const int8_t* qs = (const int8_t*)(base + s->qs_offset + blk * 32);
            const float df = orc_binary16(word_le(base + s->dm_offset + blk * 2));
            REQUIRE(isfinite(df));
            for (uint32_t i = 0; i < 32; ++i) {
                const float val = wide ? (float)((double)df * qs[i]) : df * (float)qs[i];
                REQUIRE(isfinite(val));
                out[blk * 32 + i] = val;
            }
        }
    } else return ORC_FORMAT_ERROR;
    return ORC_OK;
}

int orc_dequantize_expert_planar_v3(const orc_planar_spec* s, const uint8_t* planar,
                                    uint64_t planar_bytes, float* out, uint64_t nelem) {
    return planar_dequant(s, planar, planar_bytes, out, nelem, 1);
}
int orc_dequantize_expert_planar_v3_f32(const orc_planar_spec* s, const uint8_t* planar,
                                        uint64_t planar_bytes, float* out, uint64_t nelem) {
    return planar_dequant(s, planar, planar_bytes, out, nelem, 0);
}

/* src/planar_pack_v3.cpp:1061-1123; tests/test_planar_pack_v3.cpp:401-424 */
int orc_pack_coloc_half(const orc_planar_spec* s, const uint8_t* gate_gguf, const uint8_t* up_gguf,
                        uint32_t experts, uint32_t half, uint8_t* out, uint64_t out_bytes) {
    REQUIRE(experts >= 2 && experts % 2 == 0 && half < 2);
    const uint32_t half_e = experts / 2;
    REQUIRE(out_bytes == (uint64_t)half_e * 2 * s->planar_expert_bytes);
    for (uint32_t k = 0; k < half_e; ++k) {
        const uint32_t e = half * half_e + k;
        uint8_t* pair = out + (uint64_t)k * 2 * s->planar_expert_bytes;
        REQUIRE(orc_pack_expert_planar_v3(s, gate_gguf + (uint64_t)e * s->source_expert_bytes, s->source_expert_bytes,
                                          pair, s->planar_expert_bytes) == ORC_OK);
        REQUIRE(orc_pack_expert_planar_v3(s, up_gguf + (uint64_t)e * s->source_expert_bytes, s->source_expert_bytes,
                                          pair + s->planar_expert_bytes, s->planar_expert_bytes) == ORC_OK);
    }
    return ORC_OK;
}

/* ------------------------------------------------------------------------- */
/* src/expert_lanes.cpp:60-119, type 8: [f16 scales x blocks][runs of 16 blocks x 512 B]. */
int orc_q8_lanes_quant_offset(uint32_t columns, uint32_t block, uint32_t index, uint64_t* offset) {
    REQUIRE(columns && columns % 32 == 0 && columns <= 65536);
    const uint32_t blocks = columns / 32;
    REQUIRE(block < blocks && index < 32);
    const uint32_t run = block / 16;
    const uint32_t remaining = blocks - run * 16;
    const uint32_t width = remaining < 16 ? remaining : 16;
    *offset = (uint64_t)blocks * 2 + (uint64_t)run * 512 + (uint64_t)index * width + block % 16;
    return ORC_OK;
}

static int q8_lanes_rows(uint32_t columns, const uint8_t* in, uint8_t* out, uint64_t bytes, int pack) {
    REQUIRE(columns && columns % 32 == 0 && columns <= 65536);
    const uint32_t blocks = columns / 32;
    const uint64_t row_bytes = (uint64_t)blocks * 34;
    REQUIRE(bytes && bytes % row_bytes == 0);
    for (uint64_t row = 0; row < bytes; row += row_bytes) {
        const uint8_t* src = in + row; uint8_t* dst = out + row;
        for (uint32_t b = 0; b < blocks; ++b) {
            if (pack) memcpy(dst + (uint64_t)b * 2, src + (uint64_t)b * 34, 2);
            else memcpy(dst + (uint64_t)b * 34, src + (uint64_t)b * 2, 2);
            for (uint32_t i = 0; i < 32; ++i) {
                uint64_t at;
                orc_q8_lanes_quant_offset(columns, b, i, &at);
                if (pack) dst[at] = src[(uint64_t)b * 34 + 2 + i];
                else dst[(uint64_t)b * 34 + 2 + i] = src[at];
            }
        }
    }
    return ORC_OK;
}
int orc_q8_lanes_pack_rows(uint32_t columns, const uint8_t* original, uint8_t* packed, uint64_t bytes) {
    return q8_lanes_rows(columns, original, packed, bytes, 1);
}
int orc_q8_lanes_unpack_rows(uint32_t columns, const uint8_t* packed, uint8_t* original, uint64_t bytes) {
    return q8_lanes_rows(columns, packed, original, bytes, 0);
}

/* src/expert_lanes.cpp:60-119, type 7: [8-byte heads (d, m, qh) x blocks][runs of 16 blocks x 256 B]. */
int orc_q51_lanes_quant_offset(uint32_t columns, uint32_t block, uint32_t index, uint64_t* offset) {
    REQUIRE(columns && columns % 32 == 0 && columns <= 65536);
    const uint32_t blocks = columns / 32;
    REQUIRE(block < blocks && index < 16);
    const uint32_t run = block / 16;
    const uint32_t remaining = blocks - run * 16;
    const uint32_t width = remaining < 16 ? remaining : 16;
    *offset = (uint64_t)blocks * 8 + (uint64_t)run * 256 + (uint64_t)index * width + block % 16;
    return ORC_OK;
}

static int q51_lanes_rows(uint32_t columns, const uint8_t* in, uint8_t* out, uint64_t bytes, int pack) {
    REQUIRE(columns && columns % 32 == 0 && columns <= 65536);
    const uint32_t blocks = columns / 32;
    const uint64_t row_bytes = (uint64_t)blocks * 24;
    REQUIRE(bytes && bytes % row_bytes == 0);
    for (uint64_t row = 0; row < bytes; row += row_bytes) {
        const uint8_t* src = in + row; uint8_t* dst = out + row;
        for (uint32_t b = 0; b < blocks; ++b) {
            if (pack) memcpy(dst + (uint64_t)b * 8, src + (uint64_t)b * 24, 8);
            else memcpy(dst + (uint64_t)b * 24, src + (uint64_t)b * 8, 8);
            for (uint32_t i = 0; i < 16; ++i) {
                uint64_t at;
                orc_q51_lanes_quant_offset(columns, b, i, &at);
                if (pack) dst[at] = src[(uint64_t)b * 24 + 8 + i];
                else dst[(uint64_t)b * 24 + 8 + i] = src[at];
            }
        }
    }
    return ORC_OK;
}
int orc_q51_lanes_pack_rows(uint32_t columns, const uint8_t* original, uint8_t* packed, uint64_t bytes) {
    return q51_lanes_rows(columns, original, packed, bytes, 1);
}
int orc_q51_lanes_unpack_rows(uint32_t columns, const uint8_t* packed, uint8_t* original, uint64_t bytes) {
    return q51_lanes_rows(columns, packed, original, bytes, 0);
}

/* ------------------------------------------------------------------------- */
/* kernels/grouped_mpp.metal:12-37 — per expert, stable compaction over token order. */
int orc_grouped_routes(const uint32_t* ids, uint32_t experts, uint32_t selected, uint32_t tokens,
                       uint32_t* token_map, uint32_t* counts, uint32_t* error) {
    REQUIRE(experts && selected && tokens);
    for (uint32_t e = 0; e < experts; ++e) {
        uint32_t k = 0;
        for (uint32_t t = 0; t < tokens; ++t) {
            uint32_t slot = UINT32_MAX, matches = 0;
            for (uint32_t i = 0; i < selected; ++i) {
                const uint32_t id = ids[(uint64_t)t * selected + i];
                if (id >= experts) *error |= 4u;
                if (id == e) { slot = i; ++matches; }
            }
            if (matches > 1) *error |= 4u;
            if (matches == 1) token_map[(uint64_t)e * tokens + k++] = t * selected + slot;
        }
        counts[e] = k;
    }
    return ORC_OK;
}

/* kernels/grouped_mpp.metal:41-64 — exclusive scan of tiles per expert, compact task list. */
int orc_grouped_tasks(const uint32_t* counts, uint32_t experts, uint32_t selected, uint32_t tokens,
                      uint32_t tile, uint32_t* tasks, uint32_t* error) {
    REQUIRE(experts && experts <= 512 && tile);
    const uint32_t bound = tokens * selected / tile + experts;
    uint32_t total = 0, routes = 0;
    for (uint32_t i = 0; i < bound; ++i) { tasks[2 + 2 * i] = UINT32_MAX; tasks[3 + 2 * i] = UINT32_MAX; }
    for (uint32_t e = 0; e < experts; ++e) {
        if (counts[e] > tokens) *error |= 4u;
        const uint32_t capped = counts[e] < tokens ? counts[e] : tokens;
        const uint32_t n = (capped + tile - 1) / tile;
        for (uint32_t i = 0; i < n; ++i) if (total + i < bound) {
            tasks[2 + 2 * (total + i)] = e;
            tasks[3 + 2 * (total + i)] = i * tile;
        }
        total += n; routes += counts[e];
    }
    tasks[0] = total < bound ? total : bound;
    tasks[1] = routes;
    if (total > bound || routes != tokens * selected) *error |= 4u;
    return ORC_OK;
}

/* tests/test_planar_union_metadata.mm:27-55; validity rule kernels/planar_moe_v3.metal:419-436.
 * Gate tile = 8 hidden rows, down tile = 16 channels (ordinary build). */
int orc_union_metadata(uint32_t experts, uint32_t selected, uint32_t tokens, uint32_t hidden,
                       uint32_t channels, const uint32_t* ids, uint32_t* meta, uint32_t* error) {
    int valid = experts && experts <= 512 && experts % 2 == 0 && selected && selected <= 16 &&
                selected <= experts && tokens && tokens <= 8 && hidden && channels;
    if (valid) for (uint32_t i = 0; i < tokens * selected; ++i) if (ids[i] >= experts) valid = 0;
    for (uint32_t i = 0; i < 8; ++i) meta[i] = 0;
    if (!valid) { *error |= 4u; return ORC_OK; }
    uint32_t records = 0;
    const uint32_t capacity = tokens <= 4 ? 4 : 8;
    for (uint32_t flat = 0; flat < tokens * selected; ++flat) {
        uint32_t slot = 0;
        while (slot < records && (meta[8 + slot] != ids[flat] || meta[136 + slot] == capacity)) ++slot;
        if (slot == records) {
            ++records;
            meta[8 + slot] = ids[flat];
            meta[136 + slot] = 0;
            for (uint32_t k = 0; k < 8; ++k) { meta[264 + 8 * slot + k] = flat / selected; meta[1288 + 8 * slot + k] = flat; }
        }
        const uint32_t offset = 8 * slot + meta[136 + slot]++;
        meta[264 + offset] = flat / selected;
        meta[1288 + offset] = flat;
    }
    meta[0] = (hidden + 7) / 8; meta[1] = records; meta[2] = 1;
    meta[3] = (channels + 15) / 16; meta[4] = records; meta[5] = 1; meta[6] = records; meta[7] = 0;
    return ORC_OK;
}

/* ------------------------------------------------------------------------- */
/* src/sampling.cpp:473-513 — exact top-64: value desc, id asc, -0 == +0; non-finite skipped. */
static float canon(float v) { return v == 0.0f ? 0.0f : v; }
static int beats(float va, uint32_t ida, float vb, uint32_t idb) {
    const float ca = canon(va), cb = canon(vb);
    return ca > cb || (ca == cb && ida < idb);
}
int orc_logit_topk_row_cpu(const float* logits, uint64_t n, orc_logit_topk_row* out) {
    REQUIRE(n && n <= (1u << 20));
    memset(out, 0, sizeof *out);
    out->vocabulary = (uint32_t)n;
    out->first_nonfinite_col = out->first_subnormal_col = 0xffffffffu;
    for (uint32_t i = 0; i < 64; ++i) out->logits[i] = -INFINITY;
    uint32_t count = 0;
    for (uint64_t i = 0; i < n; ++i) {
        const float raw = logits[i];
        const uint32_t col = (uint32_t)i, bits = f32_bits(raw);
        const uint32_t exp_bits = bits & 0x7f800000u, mant_bits = bits & 0x007fffffu;
        if (exp_bits == 0x7f800000u) { if (out->first_nonfinite_col == 0xffffffffu) out->first_nonfinite_col = col; continue; }
        if (exp_bits == 0 && mant_bits != 0 && out->first_subnormal_col == 0xffffffffu) out->first_subnormal_col = col;
        if (count == 64 && !beats(raw, col, out->logits[63], out->ids[63])) continue;
        uint32_t pos = count < 64 ? count++ : 63;
        while (pos > 0 && beats(raw, col, out->logits[pos - 1], out->ids[pos - 1])) {
            out->logits[pos] = out->logits[pos - 1];
            out->ids[pos] = out->ids[pos - 1];
            --pos;
        }
        out->logits[pos] = raw;
        out->ids[pos] = col;
    }
    out->count = count;
    return ORC_OK;
}

/* ------------------------------------------------------------------------- */
/* src/grouped_mm.cpp:8-47 */
static int row_extent(uint32_t count, uint32_t width, uint64_t stride, uint64_t* out) {
    REQUIRE(count && stride >= (uint64_t)width * 4 && stride % 16 == 0);
    REQUIRE(!mul_overflows(count - 1, stride));
    *out = (uint64_t)(count - 1) * stride + (uint64_t)width * 4;
    return ORC_OK;
}
int orc_grouped_mm_plan_make(uint32_t type, uint32_t layout, uint32_t columns, uint32_t rows,
                             uint32_t experts, uint32_t selected, uint32_t tokens,
                             uint64_t input_stride, uint64_t output_stride, int broadcast,
                             int allow_nax_2k, orc_grouped_mm_plan* p) {
    REQUIRE(type == 7 || type == 8 || type == 12 || type == 13);
    REQUIRE(layout == 0 || (layout == 1 && type == 8) || (layout == 2 && type == 7));
    uint32_t epb, bpb;
    REQUIRE(orc_encoding(type, &epb, &bpb) == ORC_OK);
    const uint32_t max_tokens = allow_nax_2k ? 2048u : 512u;
    REQUIRE(columns && columns <= 65536 && columns % epb == 0 && rows && rows <= 32768 && experts &&
            experts <= 512 && selected && selected <= 16 && selected <= experts && tokens && tokens <= max_tokens);
    if (layout == 2) REQUIRE(columns == 640 && experts > 1);
    if (layout == 1) {
        if (allow_nax_2k) REQUIRE(columns % 32 == 0);
        else REQUIRE(experts == 1 && (columns % 256 == 0 || columns < 512));
    }
    const uint64_t routes = (uint64_t)tokens * selected, stride = (uint64_t)(columns / epb) * bpb;
    const uint64_t expert_stride = stride * rows, maximum_tasks = routes / 32 + experts;
    memset(p, 0, sizeof *p);
    p->args = (orc_grouped_mm_args){columns, rows, (uint32_t)stride, experts, selected, tokens,
                                    (uint32_t)(broadcast != 0), (uint32_t)maximum_tasks, expert_stride,
                                    input_stride, output_stride};
    p->matrix_bytes = expert_stride * experts; p->indices_bytes = routes * 4;
    REQUIRE(row_extent((uint32_t)(broadcast ? tokens : routes), columns, input_stride, &p->input_bytes) == ORC_OK);
    REQUIRE(row_extent((uint32_t)routes, rows, output_stride, &p->output_bytes) == ORC_OK);
    p->token_map_bytes = (uint64_t)experts * tokens * 4; p->counts_bytes = (uint64_t)experts * 4;
    p->tasks_bytes = (2 + maximum_tasks * 2) * 4;
    REQUIRE(p->matrix_bytes <= (2ull << 30));
    const uint64_t spans[5] = {p->input_bytes, p->output_bytes, p->token_map_bytes, p->counts_bytes, p->tasks_bytes};
    for (int i = 0; i < 5; ++i) REQUIRE(spans[i] <= (256ull << 20));
    p->grid_x = (rows + 63) / 64; p->grid_y = (uint32_t)maximum_tasks;
    return ORC_OK;
}

/* src/moe_mm_many_plan.cpp:28-52 */
int orc_moe_mm_many_bytes(uint32_t channels, uint32_t hidden, uint32_t experts, uint32_t selected,
                          uint32_t capacity, int allow_nax_2k, uint64_t views[13], uint64_t* total) {
    const uint64_t max_routes = allow_nax_2k ? 20480ull : 10240ull;
    const uint64_t max_total = allow_nax_2k ? (360ull << 20) : (300ull << 20);
    REQUIRE(channels && channels <= 2560 && channels % 32 == 0 && hidden && hidden <= 640 && hidden % 32 == 0 &&
            experts && experts <= 512 && selected && selected <= 16 && selected <= experts && capacity &&
            capacity <= 2048 && (uint64_t)selected * capacity <= max_routes);
    const uint64_t widths[10] = {experts, selected, selected, (uint64_t)hidden * selected, (uint64_t)hidden * selected,
                                 (uint64_t)channels * selected, hidden, hidden, channels, 1};
    for (int i = 0; i < 10; ++i) views[i] = widths[i] * capacity * 4;
    if (capacity <= 512) {
        orc_grouped_mm_plan meta;
        REQUIRE(orc_grouped_mm_plan_make(8, 0, channels, hidden, experts, selected, capacity, (uint64_t)channels * 4,
                                         (uint64_t)hidden * 4, 1, 0, &meta) == ORC_OK);
        views[10] = meta.token_map_bytes; views[11] = meta.counts_bytes; views[12] = meta.tasks_bytes;
    } else {
        const uint64_t routes = (uint64_t)capacity * selected, maximum_tasks = routes / 32 + experts;
        views[10] = (uint64_t)experts * capacity * 4; views[11] = (uint64_t)experts * 4;
        views[12] = (2 + maximum_tasks * 2) * 4;
    }
    *total = 0;
    for (int i = 0; i < 13; ++i) { REQUIRE(views[i] <= (256ull << 20)); *total += views[i]; }
    REQUIRE(*total <= max_total && views[3] / 4 <= 16777216 && views[6] / 4 <= 16777216);
    return ORC_OK;
}

/* ------------------------------------------------------------------------- */
/* kernels/planar_moe_v3.metal:82-94 */
uint16_t orc_round_bf16_bits(float v, uint32_t* bad) {
    const uint32_t bits = f32_bits(v);
    if ((bits & 0x7f800000u) == 0x7f800000u) { *bad |= 1u; return 0; }
    const uint16_t rounded = (uint16_t)((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
    if ((rounded & 0x7f80u) == 0x7f80u) { *bad |= 1u; return 0; }
    return rounded;
}
float orc_bf16_to_f32(uint16_t bits) { return bits_f32((uint32_t)bits << 16); }

/* ------------------------------------------------------------------------- */
/* tests/test_planar_pack_v3.cpp:519-547 (float silu, float h), src/ffn_check.cpp:117-141 (double). */
typedef struct {
    uint32_t gu_type, dn_type, channels, hidden, selected, route_begin, route_end;
    uint64_t input_stride; int silu_f32, stage_bf16, status;
    const uint8_t *gate, *up, *down; const uint32_t* ids; const float* input;
    double *hidden_out, *down_out;
} moe_job;

static float silu_f32(float x) { return x / (1.0f + expf(-x)); }
static float stage(float v, int bf16) { uint32_t bad = 0; return bf16 ? orc_bf16_to_f32(orc_round_bf16_bits(v, &bad)) : v; }

/* Matrix-core staging of one dequantised Q6_K row (210-byte blocks, f16 d at byte 208): the kernel multiplies the
 * integer product sc * (q - 32) as a half and applies d in f32, so w becomes d * half(w / d). w / d is that integer
 * exactly (w = d * sc * (q - 32) has at most 24 significant bits); only magnitudes above 2048 can round. */
static void stage_q6k_products(const uint8_t* row, float* w, uint32_t columns) {
    for (uint32_t b = 0; b < columns / 256; ++b) {
        const uint8_t* blk = row + (uint64_t)b * 210;
        const double d = orc_binary16((uint16_t)(blk[208] | (blk[209] << 8)));
        for (uint32_t i = 0; i < 256; ++i) {
            float* v = w + b * 256 + i;
            if (d != 0 && isfinite(d)) *v = (float)(d * (double)orc_round_f16((float)((double)*v / d)));
        }
    }
}

static void* moe_worker(void* arg) {
    moe_job* j = (moe_job*)arg;
    uint32_t gu_epb, gu_bpb, dn_epb, dn_bpb;
    j->status = ORC_FORMAT_ERROR;
    if (orc_encoding(j->gu_type, &gu_epb, &gu_bpb) || orc_encoding(j->dn_type, &dn_epb, &dn_bpb)) return NULL;
    const uint64_t gu_row = (uint64_t)(j->channels / gu_epb) * gu_bpb, dn_row = (uint64_t)(j->hidden / dn_epb) * dn_bpb;
    float* wrow = (float*)malloc(sizeof(float) * (j->channels > j->hidden ? j->channels : j->hidden));
    double* h = (double*)malloc(sizeof(double) * j->hidden);
    float* xs = (float*)malloc(sizeof(float) * j->channels);
    if (!wrow || !h || !xs) { free(wrow); free(h); free(xs); return NULL; }
    for (uint32_t rid = j->route_begin; rid < j->route_end; ++rid) {
        const uint32_t e = j->ids[rid];
        const float* x = j->input + (uint64_t)(rid / j->selected) * j->input_stride;
        for (uint32_t c = 0; c < j->channels; ++c) xs[c] = stage(x[c], j->stage_bf16 & 5);
        for (uint32_t r = 0; r < j->hidden; ++r) {
            double dg = 0, du = 0;
            if (orc_dequantize(j->gu_type, j->gate + ((uint64_t)e * j->hidden + r) * gu_row, gu_row, wrow, j->channels)) goto done;
            if (j->stage_bf16 & (2 | 16)) for (uint32_t c = 0; c < j->channels; ++c) wrow[c] = orc_round_f16(wrow[c]);
            for (uint32_t c = 0; c < j->channels; ++c) dg += (double)wrow[c] * xs[c];
            if (orc_dequantize(j->gu_type, j->up + ((uint64_t)e * j->hidden + r) * gu_row, gu_row, wrow, j->channels)) goto done;
            if (j->stage_bf16 & (2 | 16)) for (uint32_t c = 0; c < j->channels; ++c) wrow[c] = orc_round_f16(wrow[c]);
            for (uint32_t c = 0; c < j->channels; ++c) du += (double)wrow[c] * xs[c];
            if (j->silu_f32) h[r] = silu_f32((float)dg) * (float)du;
            else { double s; orc_stable_silu(dg, &s); h[r] = s * du; }
            if (j->stage_bf16 & 1) h[r] = stage((float)h[r], 1);
            if (j->stage_bf16 & 4) h[r] = 256.0 * (double)orc_round_f16((float)h[r] * 0.00390625f);
            if (j->hidden_out) j->hidden_out[(uint64_t)rid * j->hidden + r] = h[r];
        }
        if (j->down && j->down_out) for (uint32_t r = 0; r < j->channels; ++r) {
            double dd = 0;
            if (orc_dequantize(j->dn_type, j->down + ((uint64_t)e * j->channels + r) * dn_row, dn_row, wrow, j->hidden)) goto done;
            if (j->stage_bf16 & (2 | 32)) for (uint32_t c = 0; c < j->hidden; ++c) wrow[c] = orc_round_f16(wrow[c]);
            if ((j->stage_bf16 & 8) && j->dn_type == 14) stage_q6k_products(j->down + ((uint64_t)e * j->channels + r) * dn_row, wrow, j->hidden);
            for (uint32_t c = 0; c < j->hidden; ++c) dd += (double)wrow[c] * h[c];
            j->down_out[(uint64_t)rid * j->channels + r] = dd;
        }
    }
    j->status = ORC_OK;
done:
    free(wrow); free(h); free(xs);
    return NULL;
}

int orc_moe_routed_reference(uint32_t gate_up_type, uint32_t down_type, const uint8_t* gate,
                             const uint8_t* up, const uint8_t* down, uint32_t channels,
                             uint32_t hidden, uint32_t experts, const uint32_t* ids,
                             uint32_t tokens, uint32_t selected, const float* input,
                             uint64_t input_stride_floats, int silu_f32_flag, int stage_bf16,
                             double* hidden_out, double* down_out, uint32_t threads) {
    const uint32_t routes = tokens * selected;
    REQUIRE(routes && channels && hidden && experts);
    for (uint32_t r = 0; r < routes; ++r) REQUIRE(ids[r] < experts);
    if (threads < 1) threads = 1;
    if (threads > 256) threads = 256;
    if (threads > routes) threads = routes;
    pthread_t tids[256]; moe_job jobs[256];
    for (uint32_t t = 0; t < threads; ++t) {
        jobs[t] = (moe_job){gate_up_type, down_type, channels, hidden, selected,
                            (uint32_t)((uint64_t)routes * t / threads), (uint32_t)((uint64_t)routes * (t + 1) / threads),
                            input_stride_floats, silu_f32_flag, stage_bf16, 0, gate, up, down, ids, input, hidden_out, down_out};
        if (threads == 1 || pthread_create(&tids[t], NULL, moe_worker, &jobs[t])) { moe_worker(&jobs[t]); tids[t] = 0; }
    }
    int status = ORC_OK;
    for (uint32_t t = 0; t < threads; ++t) { if (tids[t]) pthread_join(tids[t], NULL); if (jobs[t].status) status = ORC_FORMAT_ERROR; }
    return status;
}

/* ------------------------------------------------------------------------- */
/* tests/grouped_mm_fixture.hpp:10-19 — the reference tests' LCG weight fixture: every byte is the
 * top byte of rng = rng*1664525 + 1013904223 (rng starts at 44), then each block's f16 scale is
 * one of eight cycling patterns and, except for Q8_0, bytes 2..3 are 0x03, 0x1c. */
int orc_fixture_weights(uint32_t type, uint32_t k, uint32_t r, uint32_t e, uint8_t* out, uint64_t nbytes) {
    static const uint16_t ds[8] = {0x0401, 0x0568, 0x068e, 0x0ac2, 0x2401, 0x2803, 0xa401, 0x1801};
    uint32_t epb, bpb;
    REQUIRE(orc_encoding(type, &epb, &bpb) == ORC_OK && k % epb == 0);
    REQUIRE(nbytes == (uint64_t)(k / epb) * bpb * r * e && nbytes <= (32ull << 20));
    uint32_t rng = 44;
    for (uint64_t at = 0; at < nbytes; at += bpb) {
        for (uint32_t i = 0; i < bpb; ++i) { rng = rng * 1664525u + 1013904223u; out[at + i] = (uint8_t)(rng >> 24); }
        const uint16_t d = ds[(at / bpb) % 8];
        out[at] = (uint8_t)(d & 255); out[at + 1] = (uint8_t)(d >> 8);
        if (type != 8) { out[at + 2] = 0x03; out[at + 3] = 0x1c; }
    }
    return ORC_OK;
}

/* ------------------------------------------------------------------------- */
/* IEEE binary32 -> binary16 with round-to-nearest-even, returned as the float the half represents.
 * This is the `half(value)` staging of kernels/grouped_mm.metal:214-216 and
 * kernels/planar_moe_v3.metal:160-166. Overflow gives +-inf like the hardware conversion. */
float orc_round_f16(float v) {
    const uint32_t b = f32_bits(v), sign = b & 0x80000000u, mag = b & 0x7fffffffu;
    if (mag >= 0x7f800000u) return v;                         /* inf / nan */
    if (mag >= 0x477ff000u) return bits_f32(sign | 0x7f800000u); /* rounds to >= 65520 -> inf */
    if (mag < 0x33000001u) return bits_f32(sign);             /* below half of the smallest subnormal (ties to even -> 0) */
    if (mag < 0x38800000u) {                                  /* subnormal half: quantum 2^-24 */
        const float q = bits_f32(mag) * 16777216.0f;          /* exact scaling */
        const float r = nearbyintf(q);                        /* default rounding mode: nearest even */
        return bits_f32(sign | f32_bits(r * 5.9604644775390625e-8f));
    }
    const uint32_t rounded = (mag + 0xfffu + ((mag >> 13) & 1u)) & 0xffffe000u;
    return bits_f32(sign | rounded);
}

/* Declared-precision dense reference (tests/test_moe_mm_many_gpu.cpp:54-63 `dot(..., half)`):
 * out[m][n] = sum_k double(half(dec(W[n,k]))) * double(x[m,k]), sequential double accumulation.
 * `rows_sel` (may be NULL) lists which weight rows to evaluate. */
typedef struct {
    uint32_t type, columns, tokens, begin, end, stage_f16; uint64_t x_stride;
    const uint8_t* matrix; const uint32_t* rows_sel; const float* x; double* out; uint32_t nsel; int status;
} sg_job;

static void* sg_worker(void* arg) {
    sg_job* j = (sg_job*)arg;
    uint32_t epb, bpb;
    j->status = ORC_FORMAT_ERROR;
    if (orc_encoding(j->type, &epb, &bpb)) return NULL;
    const uint64_t row_bytes = (uint64_t)(j->columns / epb) * bpb;
    float* w = (float*)malloc(sizeof(float) * j->columns);
    if (!w) return NULL;
    for (uint32_t i = j->begin; i < j->end; ++i) {
        const uint32_t n = j->rows_sel ? j->rows_sel[i] : i;
        if (orc_dequantize(j->type, j->matrix + (uint64_t)n * row_bytes, row_bytes, w, j->columns)) { free(w); return NULL; }
        if (j->stage_f16 == 1) for (uint32_t c = 0; c < j->columns; ++c) w[c] = orc_round_f16(w[c]);
        if (j->stage_f16 == 2 && j->type == 14) stage_q6k_products(j->matrix + (uint64_t)n * row_bytes, w, j->columns);
        for (uint32_t m = 0; m < j->tokens; ++m) {
            const float* x = j->x + (uint64_t)m * j->x_stride;
            double sum = 0;
            for (uint32_t c = 0; c < j->columns; ++c) sum += (double)w[c] * (double)x[c];
            j->out[(uint64_t)m * j->nsel + i] = sum;
        }
    }
    free(w);
    j->status = ORC_OK;
    return NULL;
}

int orc_staged_gemm(uint32_t type, const uint8_t* matrix, uint32_t columns, const uint32_t* rows_sel, uint32_t nsel,
                    const float* x, uint64_t x_stride_floats, uint32_t tokens, int stage_f16, double* out, uint32_t threads) {
    REQUIRE(nsel && tokens && columns);
    if (threads < 1) threads = 1;
    if (threads > 256) threads = 256;
    if (threads > nsel) threads = nsel;
    pthread_t tids[256]; sg_job jobs[256];
    for (uint32_t t = 0; t < threads; ++t) {
        jobs[t] = (sg_job){type, columns, tokens, (uint32_t)((uint64_t)nsel * t / threads), (uint32_t)((uint64_t)nsel * (t + 1) / threads),
                           (uint32_t)stage_f16, x_stride_floats, matrix, rows_sel, x, out, nsel, 0};
        if (threads == 1 || pthread_create(&tids[t], NULL, sg_worker, &jobs[t])) { sg_worker(&jobs[t]); tids[t] = 0; }
    }
    int status = ORC_OK;
    for (uint32_t t = 0; t < threads; ++t) { if (tids[t]) pthread_join(tids[t], NULL); if (jobs[t].status) status = ORC_FORMAT_ERROR; }
    return status;
}
