// Host-side formats, Pack v3 planar layout, q8_lanes_v1 layout and the pure planners.
// Integer shuffles only; nothing here touches the device.
#include "tsp_common.hpp"

#include <algorithm>
#include <cstring>

namespace tsp {

namespace {
thread_local char g_error[512] = "";
}

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
}

int launch_status(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("%s launch: %s", what, hipGetErrorString(e)); return TSP_ERR_HIP; }
    return TSP_OK;
}

// src/gguf.cpp:21-32: encoded block sizes (elements per block, bytes per block).
const Encoding* find_encoding(uint32_t type) {
    static const Encoding table[] = {
        {0, 1, 4},      {1, 1, 2},      {2, 32, 18},    {3, 32, 20},   {6, 32, 22},   {7, 32, 24},   {8, 32, 34},
        {10, 256, 84},  {11, 256, 110}, {12, 256, 144}, {13, 256, 176}, {14, 256, 210}, {20, 32, 18}, {23, 256, 136},
        {24, 1, 1},     {25, 1, 2},     {26, 1, 4},     {27, 1, 8},    {28, 1, 8},    {30, 1, 2},
    };
    for (const auto& e : table) if (e.id == type) return &e;
    return nullptr;
}

}  // namespace tsp

using namespace tsp;

extern "C" {

const char* tsp_last_error(void) { return g_error; }
uint32_t tsp_abi_version(void) { return 1; }

int tsp_encoding(uint32_t type, uint32_t* elements, uint32_t* bytes) {
    const auto* e = find_encoding(type);
    TSP_REQUIRE(e, "unsupported GGUF tensor encoding %u", type);
    *elements = e->elements; *bytes = e->bytes;
    return TSP_OK;
}

int tsp_can_decode(uint32_t t) {
    return t == 0 || t == 1 || t == 7 || t == 8 || t == 12 || t == 13 || t == 14 || t == 20 || t == 30;
}

int tsp_make_expert_spec(uint32_t source_type, uint32_t columns, uint32_t rows, tsp_planar_spec* s) {
    TSP_REQUIRE(rows >= 4 && rows % 4 == 0, "planar v3 requires rows >= 4 and divisible by 4");
    std::memset(s, 0, sizeof *s);
    s->source_type = source_type; s->columns = columns; s->rows = rows;
    uint32_t per_block = 0, source_block = 0, planar_block = 0;
    if (source_type == 12 || source_type == 13 || source_type == 14) {
        TSP_REQUIRE(columns >= 256 && columns % 256 == 0, "K-quant planar v3 requires columns divisible by 256");
        per_block = 256;
        source_block = source_type == 12 ? 144 : source_type == 13 ? 176 : 210;
        planar_block = source_type == 12 ? 148 : source_type == 13 ? 180 : 210;
    } else if (source_type == 7 || source_type == 8) {
        TSP_REQUIRE(columns >= 32 && columns % 32 == 0, "Q5_1/Q8_0 planar v3 requires columns divisible by 32");
        per_block = 32;
        source_block = planar_block = source_type == 7 ? 24 : 34;
    } else {
        set_error("unsupported encoding for planar v3 expert layout");
        return TSP_ERR_FORMAT;
    }
    s->blocks_per_row = columns / per_block;
    const uint64_t total = uint64_t(rows) * s->blocks_per_row;
    switch (source_type) {
    case 12: s->sm_offset = total * 128; s->dm_offset = total * 144; break;
    case 13: s->qh_offset = total * 128; s->sm_offset = total * 160; s->dm_offset = total * 176; break;
    case 14: s->qh_offset = total * 128; s->sm_offset = total * 192; s->dm_offset = total * 208; break;
    case 7: s->qh_offset = total * 16; s->dm_offset = total * 20; break;
    default:
        TSP_REQUIRE(total % 8 == 0, "Q8_0 planar v3 requires total_blocks divisible by 8 for 16-byte expert alignment");
        s->dm_offset = total * 32;
    }
    if (source_type == 14) TSP_REQUIRE(total % 8 == 0, "Q6_K planar requires total_blocks divisible by 8 for 16-byte plane alignment");
    s->source_row_bytes = uint64_t(s->blocks_per_row) * source_block;
    s->planar_row_bytes = uint64_t(s->blocks_per_row) * planar_block;
    s->source_expert_bytes = uint64_t(rows) * s->source_row_bytes;
    s->planar_expert_bytes = uint64_t(rows) * s->planar_row_bytes;
    TSP_REQUIRE(s->planar_expert_bytes % 16 == 0, "planar v3 expert byte stride must be 16-byte aligned");
    return TSP_OK;
}

void tsp_pack_sm16(const uint8_t s12[12], uint8_t sm[16]) {
    // Sub-blocks 0..3 keep six low bits in bytes 0..7; sub-blocks 4..7 take four bits from bytes 8..11
    // and two from the top of bytes 0..7. Output: sm[0..7] scales, sm[8..15] minima.
    for (int j = 0; j < 4; ++j) {
        sm[j] = s12[j] & 63;
        sm[8 + j] = s12[4 + j] & 63;
        sm[4 + j] = uint8_t((s12[8 + j] & 15) | ((s12[j] >> 6) << 4));
        sm[12 + j] = uint8_t((s12[8 + j] >> 4) | ((s12[4 + j] >> 6) << 4));
    }
}

int tsp_unpack_sm16(const uint8_t sm[16], uint8_t s12[12]) {
    for (int i = 0; i < 16; ++i) TSP_REQUIRE(sm[i] < 64, "corrupt planar v3 scale/min factor exceeds 6-bit [0, 63] range");
    for (int j = 0; j < 4; ++j) {
        s12[j] = uint8_t(sm[j] | ((sm[4 + j] >> 4) << 6));
        s12[4 + j] = uint8_t(sm[8 + j] | ((sm[12 + j] >> 4) << 6));
        s12[8 + j] = uint8_t((sm[4 + j] & 15) | ((sm[12 + j] & 15) << 4));
    }
    return TSP_OK;
}

namespace {
// One plane of a block format: `width` bytes per block, taken from byte `from` of the GGUF block.
struct Plane { uint64_t offset; uint32_t width, from; };
int planes_of(const tsp_planar_spec& s, Plane out[4], uint32_t* source_block) {
    switch (s.source_type) {
    case 12: *source_block = 144; out[0] = {s.qs_offset, 128, 16}; out[1] = {s.dm_offset, 4, 0}; return 2;
    case 13: *source_block = 176; out[0] = {s.qs_offset, 128, 48}; out[1] = {s.qh_offset, 32, 16}; out[2] = {s.dm_offset, 4, 0}; return 3;
    case 14: *source_block = 210; out[0] = {s.qs_offset, 128, 0}; out[1] = {s.qh_offset, 64, 128};
             out[2] = {s.sm_offset, 16, 192}; out[3] = {s.dm_offset, 2, 208}; return 4;
    case 7: *source_block = 24; out[0] = {s.qs_offset, 16, 8}; out[1] = {s.qh_offset, 4, 4}; out[2] = {s.dm_offset, 4, 0}; return 3;
    case 8: *source_block = 34; out[0] = {s.qs_offset, 32, 2}; out[1] = {s.dm_offset, 2, 0}; return 2;
    default: return 0;
    }
}
}  // namespace

int tsp_pack_expert_planar_v3(const tsp_planar_spec* s, const uint8_t* src, uint64_t gguf_bytes, uint8_t* dst, uint64_t planar_bytes) {
    TSP_REQUIRE(gguf_bytes == s->source_expert_bytes && planar_bytes == s->planar_expert_bytes, "pack_expert_planar_v3 span size mismatch");
    Plane planes[4]; uint32_t block = 0;
    const int n = planes_of(*s, planes, &block);
    TSP_REQUIRE(n, "unsupported encoding in pack_expert_planar_v3");
    const uint64_t total = uint64_t(s->rows) * s->blocks_per_row;
    const bool scales = s->source_type == 12 || s->source_type == 13;
    for (uint64_t b = 0; b < total; ++b) {
        const uint8_t* sb = src + b * block;
        for (int p = 0; p < n; ++p) std::memcpy(dst + planes[p].offset + b * planes[p].width, sb + planes[p].from, planes[p].width);
        if (scales) tsp_pack_sm16(sb + 4, dst + s->sm_offset + b * 16);
    }
    return TSP_OK;
}

int tsp_unpack_expert_planar_v3(const tsp_planar_spec* s, const uint8_t* src, uint64_t planar_bytes, uint8_t* dst, uint64_t gguf_bytes) {
    TSP_REQUIRE(planar_bytes == s->planar_expert_bytes && gguf_bytes == s->source_expert_bytes, "unpack_expert_planar_v3 span size mismatch");
    Plane planes[4]; uint32_t block = 0;
    const int n = planes_of(*s, planes, &block);
    TSP_REQUIRE(n, "unsupported encoding in unpack_expert_planar_v3");
    const uint64_t total = uint64_t(s->rows) * s->blocks_per_row;
    const bool scales = s->source_type == 12 || s->source_type == 13;
    for (uint64_t b = 0; b < total; ++b) {
        uint8_t* sb = dst + b * block;
        for (int p = 0; p < n; ++p) std::memcpy(sb + planes[p].from, src + planes[p].offset + b * planes[p].width, planes[p].width);
        if (scales && tsp_unpack_sm16(src + s->sm_offset + b * 16, sb + 4) != TSP_OK) return TSP_ERR_FORMAT;
    }
    return TSP_OK;
}

int tsp_pack_coloc_half(const tsp_planar_spec* s, const uint8_t* gate, const uint8_t* up, uint32_t experts, uint32_t half,
                        uint8_t* out, uint64_t out_bytes) {
    TSP_REQUIRE(experts >= 2 && experts % 2 == 0 && half < 2, "co-located planar v3 requires even experts >= 2");
    const uint32_t per_half = experts / 2;
    TSP_REQUIRE(out_bytes == uint64_t(per_half) * 2 * s->planar_expert_bytes, "co-located planar v3 output span mismatch");
    for (uint32_t k = 0; k < per_half; ++k) {
        const uint64_t e = uint64_t(half) * per_half + k;
        uint8_t* pair = out + uint64_t(k) * 2 * s->planar_expert_bytes;
        int rc = tsp_pack_expert_planar_v3(s, gate + e * s->source_expert_bytes, s->source_expert_bytes, pair, s->planar_expert_bytes);
        if (rc == TSP_OK)
            rc = tsp_pack_expert_planar_v3(s, up + e * s->source_expert_bytes, s->source_expert_bytes,
                                           pair + s->planar_expert_bytes, s->planar_expert_bytes);
        if (rc != TSP_OK) return rc;
    }
    return TSP_OK;
}

int tsp_q8_lanes_quant_offset(uint32_t columns, uint32_t block, uint32_t index, uint64_t* offset) {
    TSP_REQUIRE(columns && columns % 32 == 0 && columns <= 65536, "Q8_0 lane layout needs whole 32-element blocks");
    const uint32_t blocks = columns / 32;
    TSP_REQUIRE(block < blocks && index < 32, "lane layout block/quant bound");
    const uint32_t run = block / 16, width = std::min(16u, blocks - run * 16);
    *offset = uint64_t(blocks) * 2 + uint64_t(run) * 512 + uint64_t(index) * width + block % 16;
    return TSP_OK;
}

namespace {
int q8_lanes_move(uint32_t columns, const uint8_t* in, uint8_t* out, uint64_t bytes, bool pack) {
    TSP_REQUIRE(columns && columns % 32 == 0 && columns <= 65536, "Q8_0 lane layout needs whole 32-element blocks");
    const uint32_t blocks = columns / 32;
    const uint64_t row_bytes = uint64_t(blocks) * 34;
    TSP_REQUIRE(bytes && bytes % row_bytes == 0, "lane layout needs whole rows");
    TSP_REQUIRE(!ranges_overlap(in, bytes, out, bytes), "lane layout input and output overlap");
    for (uint64_t row = 0; row < bytes; row += row_bytes) {
        const uint8_t* src = in + row; uint8_t* dst = out + row;
        for (uint32_t b = 0; b < blocks; ++b) {
            const uint32_t run = b / 16, width = std::min(16u, blocks - run * 16);
            const uint64_t base = uint64_t(blocks) * 2 + uint64_t(run) * 512 + b % 16;
            if (pack) {
                std::memcpy(dst + 2 * b, src + 34 * b, 2);
                for (uint32_t i = 0; i < 32; ++i) dst[base + uint64_t(i) * width] = src[34 * b + 2 + i];
            } else {
                std::memcpy(dst + 34 * b, src + 2 * b, 2);
                for (uint32_t i = 0; i < 32; ++i) dst[34 * b + 2 + i] = src[base + uint64_t(i) * width];
            }
        }
    }
    return TSP_OK;
}
}  // namespace

int tsp_q8_lanes_pack_rows(uint32_t columns, const uint8_t* original, uint8_t* packed, uint64_t bytes) {
    return q8_lanes_move(columns, original, packed, bytes, true);
}
int tsp_q8_lanes_unpack_rows(uint32_t columns, const uint8_t* packed, uint8_t* original, uint64_t bytes) {
    return q8_lanes_move(columns, packed, original, bytes, false);
}

int tsp_q51_lanes_quant_offset(uint32_t columns, uint32_t block, uint32_t index, uint64_t* offset) {
    TSP_REQUIRE(columns && columns % 32 == 0 && columns <= 65536, "Q5_1 lane layout needs whole 32-element blocks");
    const uint32_t blocks = columns / 32;
    TSP_REQUIRE(block < blocks && index < 16, "lane layout block/quant bound");
    const uint32_t run = block / 16, width = std::min(16u, blocks - run * 16);
    *offset = uint64_t(blocks) * 8 + uint64_t(run) * 256 + uint64_t(index) * width + block % 16;
    return TSP_OK;
}

namespace {
int q51_lanes_move(uint32_t columns, const uint8_t* in, uint8_t* out, uint64_t bytes, bool pack) {
    TSP_REQUIRE(columns && columns % 32 == 0 && columns <= 65536, "Q5_1 lane layout needs whole 32-element blocks");
    const uint32_t blocks = columns / 32;
    const uint64_t row_bytes = uint64_t(blocks) * 24;
    TSP_REQUIRE(bytes && bytes % row_bytes == 0, "lane layout needs whole rows");
    TSP_REQUIRE(!ranges_overlap(in, bytes, out, bytes), "lane layout input and output overlap");
    for (uint64_t row = 0; row < bytes; row += row_bytes) {
        const uint8_t* src = in + row; uint8_t* dst = out + row;
        for (uint32_t b = 0; b < blocks; ++b) {
            const uint32_t run = b / 16, width = std::min(16u, blocks - run * 16);
            const uint64_t base = uint64_t(blocks) * 8 + uint64_t(run) * 256 + b % 16;
            if (pack) {
                std::memcpy(dst + 8 * b, src + 24 * b, 8);
                for (uint32_t i = 0; i < 16; ++i) dst[base + uint64_t(i) * width] = src[24 * b + 8 + i];
            } else {
                std::memcpy(dst + 24 * b, src + 8 * b, 8);
                for (uint32_t i = 0; i < 16; ++i) dst[24 * b + 8 + i] = src[base + uint64_t(i) * width];
            }
        }
    }
    return TSP_OK;
}
}  // namespace

int tsp_q51_lanes_pack_rows(uint32_t columns, const uint8_t* original, uint8_t* packed, uint64_t bytes) {
    return q51_lanes_move(columns, original, packed, bytes, true);
}
int tsp_q51_lanes_unpack_rows(uint32_t columns, const uint8_t* packed, uint8_t* original, uint64_t bytes) {
    return q51_lanes_move(columns, packed, original, bytes, false);
}

// ---------------------------------------------------------------- planners

namespace {
int row_extent(uint32_t count, uint32_t width, uint64_t stride, uint64_t* out) {
    TSP_REQUIRE(count && stride >= uint64_t(width) * 4 && stride % 16 == 0 && !mul_overflows(count - 1, stride),
                "tiled prefill FP32 row stride");
    *out = uint64_t(count - 1) * stride + uint64_t(width) * 4;
    return TSP_OK;
}
}  // namespace

int tsp_grouped_mm_plan(uint32_t type, uint32_t layout, uint32_t columns, uint32_t rows, uint32_t experts, uint32_t selected,
                        uint32_t tokens, uint64_t input_stride, uint64_t output_stride, int broadcast, int allow_nax_2k,
                        tsp_grouped_mm_plan_t* p) {
    TSP_REQUIRE(type == 7 || type == 8 || type == 12 || type == 13, "grouped mm encoding");
    TSP_REQUIRE(layout == 0 || (layout == 1 && type == 8) || (layout == 2 && type == 7), "grouped mm layout/encoding mismatch");
    const auto* format = find_encoding(type);
    const uint32_t max_tokens = allow_nax_2k ? 2048u : 512u;
    TSP_REQUIRE(columns && columns <= 65536 && columns % format->elements == 0 && rows && rows <= 32768 && experts &&
                    experts <= 512 && selected && selected <= 16 && selected <= experts && tokens && tokens <= max_tokens,
                "grouped mm geometry");
    if (layout == 2) TSP_REQUIRE(columns == 640 && experts > 1, "registered Q5_1 lane geometry");
    if (layout == 1) {
        if (allow_nax_2k) TSP_REQUIRE(columns % 32 == 0, "registered Q8 lane geometry");
        else TSP_REQUIRE(experts == 1 && (columns % 256 == 0 || columns < 512), "registered Q8 lane geometry");
    }
    const uint64_t routes = uint64_t(tokens) * selected;
    const uint64_t stride = uint64_t(columns / format->elements) * format->bytes;
    const uint64_t expert_stride = stride * rows, maximum_tasks = routes / 32 + experts;
    std::memset(p, 0, sizeof *p);
    p->args = {columns, rows, uint32_t(stride), experts, selected, tokens, uint32_t(broadcast != 0), uint32_t(maximum_tasks),
               expert_stride, input_stride, output_stride};
    p->matrix_bytes = expert_stride * experts;
    p->indices_bytes = routes * 4;
    int rc = row_extent(uint32_t(broadcast ? tokens : routes), columns, input_stride, &p->input_bytes);
    if (rc == TSP_OK) rc = row_extent(uint32_t(routes), rows, output_stride, &p->output_bytes);
    if (rc != TSP_OK) return rc;
    p->token_map_bytes = uint64_t(experts) * tokens * 4;
    p->counts_bytes = uint64_t(experts) * 4;
    p->tasks_bytes = (2 + maximum_tasks * 2) * 4;
    TSP_REQUIRE(p->matrix_bytes <= (2ull << 30), "grouped mm matrix budget");
    for (uint64_t bytes : {p->input_bytes, p->output_bytes, p->token_map_bytes, p->counts_bytes, p->tasks_bytes})
        TSP_REQUIRE(bytes <= (256ull << 20), "grouped mm workspace budget");
    p->grid_x = (rows + 63) / 64;
    p->grid_y = uint32_t(maximum_tasks);
    return TSP_OK;
}

int tsp_dense_mm_q8_plan(uint32_t layout, uint32_t columns, uint32_t rows, uint32_t tokens, uint64_t input_stride,
                         uint64_t output_stride, int allow_nax_2k, tsp_grouped_mm_plan_t* p) {
    const int rc = tsp_grouped_mm_plan(8, layout, columns, rows, 1, 1, tokens, input_stride, output_stride, 1, allow_nax_2k, p);
    if (rc != TSP_OK) return rc;
    p->indices_bytes = p->token_map_bytes = p->counts_bytes = p->tasks_bytes = 0;
    p->args.maximum_tasks = (tokens + 31) / 32;
    p->grid_y = p->args.maximum_tasks;
    return TSP_OK;
}

int tsp_moe_mm_many_bytes(uint32_t channels, uint32_t hidden, uint32_t experts, uint32_t selected, uint32_t capacity,
                          int allow_nax_2k, uint64_t views[13], uint64_t* total) {
    const uint64_t max_routes = allow_nax_2k ? 20480ull : 10240ull;
    const uint64_t max_total = allow_nax_2k ? (360ull << 20) : (300ull << 20);
    TSP_REQUIRE(channels && channels <= 2560 && channels % 32 == 0 && hidden && hidden <= 640 && hidden % 32 == 0 && experts &&
                    experts <= 512 && selected && selected <= 16 && selected <= experts && capacity && capacity <= 2048 &&
                    uint64_t(selected) * capacity <= max_routes,
                "bounded tiled MoE row geometry");
    // logits, indices, weights, gate, up, down, shared_gate, shared_up, shared_down, shared_logit
    const uint64_t widths[10] = {experts, selected, selected, uint64_t(hidden) * selected, uint64_t(hidden) * selected,
                                 uint64_t(channels) * selected, hidden, hidden, channels, 1};
    for (int i = 0; i < 10; ++i) views[i] = widths[i] * capacity * 4;
    if (capacity <= 512) {
        tsp_grouped_mm_plan_t meta;
        const int rc = tsp_grouped_mm_plan(8, 0, channels, hidden, experts, selected, capacity, uint64_t(channels) * 4,
                                           uint64_t(hidden) * 4, 1, 0, &meta);
        if (rc != TSP_OK) return rc;
        views[10] = meta.token_map_bytes; views[11] = meta.counts_bytes; views[12] = meta.tasks_bytes;
    } else {
        const uint64_t maximum_tasks = uint64_t(capacity) * selected / 32 + experts;
        views[10] = uint64_t(experts) * capacity * 4;
        views[11] = uint64_t(experts) * 4;
        views[12] = (2 + maximum_tasks * 2) * 4;
    }
    *total = 0;
    for (int i = 0; i < 13; ++i) {
        TSP_REQUIRE(views[i] <= (256ull << 20), "tiled MoE workspace bound");
        *total += views[i];
    }
    TSP_REQUIRE(*total <= max_total && views[3] / 4 <= 16777216 && views[6] / 4 <= 16777216, "tiled MoE total/activation bound");
    return TSP_OK;
}

int tsp_q8_many_width(uint32_t remaining, uint32_t* width) {
    TSP_REQUIRE(remaining, "empty Q8-many width plan");
    *width = remaining >= 8 ? 8 : remaining >= 4 ? 4 : remaining >= 2 ? 2 : 1;
    return TSP_OK;
}

int tsp_q8_many_chunks(uint32_t rows, uint32_t* chunks) {
    TSP_REQUIRE(rows && rows <= 65536, "Q8-many chunk row bound");
    uint32_t n = 0, w = 0;
    while (rows) { tsp_q8_many_width(rows, &w); rows -= w; ++n; }
    *chunks = n;
    return TSP_OK;
}

}  // extern "C"
