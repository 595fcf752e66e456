// Tests of tokspur::HipGraph on a GPU, written the way the engine's own graph tests are (tests/test_moe.cpp,
// tests/test_planar_pack_v3.cpp): build weights with the tests' LCG fixture, run the operators through the graph
// class, compare with the CPU reference, and check the lifecycle and error contract (idle / encoding phases,
// ledger, budget, sticky error word, no allocation while encoding, canaries).
#include <array>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <cstdlib>
#include <functional>
#include <limits>
#include <string>
#include <vector>

#include "gguf_writer.hpp"
#include "hip_graph.hpp"
#include "pack_v3.hpp"
#include "tokspur_hip.h"
#include "tokspur_oracle.h"

using namespace tokspur;

namespace {
int checks = 0, failures = 0;
void expect(bool ok, const char* what, int line) {
    ++checks;
    if (!ok) { ++failures; std::printf("FAILED line %d: %s\n", line, what); std::fflush(stdout); }
}
#define EXPECT(cond) expect((cond), #cond, __LINE__)
bool throws_format(const std::function<void()>& f) {
    try { f(); } catch (const FormatError&) { return true; } catch (...) { return false; }
    return false;
}
template <class T> std::span<const std::byte> bytes_of(const std::vector<T>& v) { return std::as_bytes(std::span<const T>(v)); }
template <class T> std::vector<T> read_as(HipGraph& g, GpuView v) {
    std::vector<T> out(v.bytes / sizeof(T));
    g.read(v, std::as_writable_bytes(std::span<T>(out)));
    return out;
}
std::vector<float> lcg_floats(uint32_t seed, size_t n) {  // tests/test_planar_pack_v3.cpp input generator
    std::vector<float> out(n);
    uint32_t rng = seed;
    for (auto& v : out) { rng = rng * 1664525u + 1013904223u; v = float(int(rng % 1993u) - 996) / 997.0f; }
    return out;
}
std::vector<uint8_t> fixture(uint32_t type, uint32_t k, uint32_t r, uint32_t e) {
    uint32_t epb = 0, bpb = 0;
    orc_encoding(type, &epb, &bpb);
    std::vector<uint8_t> w(size_t(k / epb) * bpb * r * e);
    if (type == 14) {  // the LCG fixture leaves Q6_K's scale (bytes 208..209) random: give it a small finite half
        uint32_t rng = 77;
        for (auto& b : w) { rng = rng * 1664525u + 1013904223u; b = uint8_t(rng >> 24); }
        for (size_t at = 0; at < w.size(); at += 210) { w[at + 208] = uint8_t(at / 210 % 7); w[at + 209] = 0x1c; }
    } else {
        orc_fixture_weights(type, k, r, e, w.data(), w.size());
    }
    return w;
}
// error in units of the row's largest magnitude: the LCG fixture's scales give outputs of ~1e5 with heavy cancellation, where
// |a - e| / max(1, |e|) per element would measure the cancellation and not the kernel
double row_error(const std::vector<float>& got, const std::vector<double>& want) {
    double worst = 0, scale = 1;
    for (double v : want) scale = std::max(scale, std::fabs(v));
    for (size_t i = 0; i < got.size(); ++i) worst = std::max(worst, std::fabs(double(got[i]) - want[i]) / scale);
    return worst;
}
double scaled_error(const std::vector<float>& got, const std::vector<double>& want) {  // src/ffn_check.cpp:48-56
    double worst = 0;
    for (size_t i = 0; i < got.size(); ++i) worst = std::max(worst, std::fabs(double(got[i]) - want[i]) / std::max(1.0, std::fabs(want[i])));
    return worst;
}
std::vector<uint8_t> coloc_half(const tsp_planar_spec& spec, const std::vector<uint8_t>& gate, const std::vector<uint8_t>& up, uint32_t experts, uint32_t half) {
    std::vector<uint8_t> out(size_t(experts / 2) * 2 * spec.planar_expert_bytes);
    if (tsp_pack_coloc_half(&spec, gate.data(), up.data(), experts, half, out.data(), out.size()) != TSP_OK) std::printf("pack failed: %s\n", tsp_last_error());
    return out;
}
std::vector<uint8_t> planar_stack(const tsp_planar_spec& spec, const std::vector<uint8_t>& gguf, uint32_t experts) {
    std::vector<uint8_t> out(size_t(experts) * spec.planar_expert_bytes);
    for (uint32_t e = 0; e < experts; ++e)
        tsp_pack_expert_planar_v3(&spec, gguf.data() + size_t(e) * spec.source_expert_bytes, spec.source_expert_bytes,
                                  out.data() + size_t(e) * spec.planar_expert_bytes, spec.planar_expert_bytes);
    return out;
}

void test_ledger_and_phases() {
    HipGraph g(1 << 20);
    const GpuView a = g.zeros(4096, "a");
    EXPECT(g.memory().live_bytes == 4096 && g.memory().allocations == 1 && g.memory().budget == (1u << 20));
    EXPECT(throws_format([&] { (void)g.zeros(2u << 20, "too big"); }));  // budget
    std::vector<float> host(1024, 1.5f);
    g.write(a, bytes_of(host));
    EXPECT(read_as<float>(g, g.slice(a, 16, 8))[1] == 1.5f);
    EXPECT(throws_format([&] { (void)g.slice(a, 4090, 16); }));
    const GpuView w = g.upload(bytes_of(host), "weights");
    EXPECT(throws_format([&] { g.write(w, bytes_of(host)); }));  // immutable
    EXPECT(throws_format([&] { g.swiglu(a, a, a); }));           // operator while idle
    HipGraph other(1 << 20);
    EXPECT(throws_format([&] { (void)other.read(a); }));          // foreign view
    g.begin();
    EXPECT(throws_format([&] { (void)g.zeros(16, "while encoding"); }));
    EXPECT(throws_format([&] { (void)g.read(a); }));
    g.abort();
    g.release(a);
    EXPECT(throws_format([&] { (void)g.read(a); }));              // released view is never rebound
    EXPECT(g.memory().live_bytes == 4096 && g.memory().peak_bytes == 8192);
    EXPECT(!g.device_name().empty());
}

void test_gemv_route_mixture_topk() {
    const uint32_t K = 512, R = 96, E = 64, S = 6;
    HipGraph g(64u << 20);
    const auto w = fixture(12, K, R, 1);
    const auto x = lcg_floats(5, K);
    const GpuView dw = g.upload(bytes_of(w), "w"), dx = g.upload(bytes_of(x), "x", false), dy = g.zeros(R * 4, "y");
    const auto logits = lcg_floats(9, E);
    const GpuView dl = g.upload(bytes_of(logits), "logits", false), di = g.zeros(S * 4, "ids"), dwt = g.zeros(S * 4, "weights");
    const GpuView topk_scratch = g.zeros(HipGraph::logit_topk_scratch_bytes(1, E), "scratch"), topk_out = g.zeros(HipGraph::logit_topk_output_bytes(1), "rows");
    g.prepare_logit_topk();
    const uint64_t allocations = g.memory().allocations;
    g.begin();
    g.gemv(12, dw, dx, dy, K, R);
    g.route(dl, di, dwt, S, RouterMode::softmax, true);
    g.logit_topk({dl, 1, E, uint64_t(E) * 4}, topk_scratch, topk_out);
    const BatchResult r = g.submit();
    EXPECT(r.dispatches == 3 && r.gpu_ms > 0 && g.memory().allocations == allocations);  // nothing allocated while encoding
    std::vector<double> want(R);
    orc_reference_gemv(12, w.data(), w.size(), K, R, x.data(), K, want.data());
    EXPECT(scaled_error(read_as<float>(g, dy), want) <= 5e-5);
    std::vector<double> dlogits(logits.begin(), logits.end()), wweights(S);
    std::vector<uint32_t> wids(S);
    orc_route_reference(dlogits.data(), E, S, 0, 1, wids.data(), wweights.data());
    EXPECT(read_as<uint32_t>(g, di) == wids);
    EXPECT(scaled_error(read_as<float>(g, dwt), wweights) <= 1e-6);
    orc_logit_topk_row row{};
    orc_logit_topk_row_cpu(logits.data(), E, &row);
    const auto got = read_as<GpuLogitTopKRow>(g, topk_out);
    EXPECT(got[0].count == row.count && std::memcmp(got[0].ids.data(), row.ids, 256) == 0 && std::memcmp(got[0].logits.data(), row.logits, 256) == 0);
    EXPECT(got[0].ids[0] == wids[0]);  // arg-max agrees with the router's first choice
    // aliasing is refused before anything is encoded
    g.begin();
    EXPECT(throws_format([&] { g.gemv(12, dw, dx, dx, K, K); }));
    g.abort();
}

struct MoeFixture {
    MoeShape shape;
    std::vector<uint8_t> gate, up, down, sgate, sup, sdown;
    std::vector<float> router, shared_router;
};

MoeFixture make_moe(uint32_t channels, uint32_t hidden, uint32_t experts, uint32_t selected) {
    MoeFixture f{{channels, hidden, experts, selected}};
    f.gate = fixture(12, channels, hidden, experts);
    f.up = fixture(12, channels, hidden, experts);
    for (auto& b : f.up) b = uint8_t(b * 3 + 1);
    for (size_t at = 0; at < f.up.size(); at += 144) { std::memcpy(&f.up[at], &f.gate[at], 4); }
    f.down = fixture(14, hidden, channels, experts);
    f.sgate = fixture(12, channels, hidden, 2);
    f.sup = f.sgate;
    f.sdown = fixture(14, hidden, channels, 2);
    f.router = lcg_floats(31, size_t(experts) * channels);
    f.shared_router = lcg_floats(37, channels);
    for (auto& v : f.shared_router) v *= 0.05f;
    return f;
}

struct MoeOnGraph { MoeWeights w; };

MoeOnGraph upload_moe(HipGraph& g, const MoeFixture& f) {
    tsp_planar_spec gu{}, dn{};
    tsp_make_expert_spec(12, f.shape.channels, f.shape.hidden, &gu);
    tsp_make_expert_spec(14, f.shape.hidden, f.shape.channels, &dn);
    const uint32_t E = f.shape.experts;
    MoeOnGraph m{};
    m.w.router = {g.upload(bytes_of(f.router), "router"), 0};
    m.w.gate = {g.upload(bytes_of(coloc_half(gu, f.gate, f.up, E, 0)), "pair_lo"), 12};
    m.w.up = {g.upload(bytes_of(coloc_half(gu, f.gate, f.up, E, 1)), "pair_hi"), 12};
    m.w.down = {g.upload(bytes_of(planar_stack(dn, f.down, E)), "down"), 14};
    g.register_planar_matrix(m.w.gate.view, {12, 2, f.shape.channels, f.shape.hidden, E});
    g.register_planar_matrix(m.w.up.view, {12, 3, f.shape.channels, f.shape.hidden, E});
    g.register_planar_matrix(m.w.down.view, {14, 10, f.shape.hidden, f.shape.channels, E});
    m.w.shared_router = {g.upload(bytes_of(f.shared_router), "shared router"), 0};
    return m;
}

// CPU composition: src/moe.cpp:37-83 order, double accumulation (tests/test_moe.cpp:131-163)
std::vector<double> cpu_moe_token(const MoeFixture& f, const float* x, bool shared_planar_pair) {
    const MoeShape s = f.shape;
    std::vector<double> logits(s.experts), weights(s.selected), out(s.channels);
    orc_reference_gemv(0, reinterpret_cast<const uint8_t*>(f.router.data()), f.router.size() * 4, s.channels, s.experts, x, s.channels, logits.data());
    std::vector<double> flogits(s.experts);
    for (uint32_t e = 0; e < s.experts; ++e) flogits[e] = double(float(logits[e]));
    std::vector<uint32_t> ids(s.selected);
    orc_route_reference(flogits.data(), s.experts, s.selected, 0, 1, ids.data(), weights.data());
    std::vector<double> h(size_t(s.selected) * s.hidden), y(size_t(s.selected) * s.channels);
    std::vector<float> xs(size_t(s.selected) * s.channels);
    orc_moe_routed_reference(12, 14, f.gate.data(), f.up.data(), f.down.data(), s.channels, s.hidden, s.experts, ids.data(), 1, s.selected, x, s.channels, 1, 0,
                             h.data(), y.data(), 1);
    std::vector<double> sh(s.hidden), sy(s.channels);
    const uint32_t zero = 0;
    orc_moe_routed_reference(12, 14, f.sgate.data(), f.sup.data(), f.sdown.data(), s.channels, s.hidden, 2, &zero, 1, 1, x, s.channels, 1, 0, sh.data(), sy.data(), 1);
    double shared_logit = 0;
    orc_reference_gemv(0, reinterpret_cast<const uint8_t*>(f.shared_router.data()), f.shared_router.size() * 4, s.channels, 1, x, s.channels, &shared_logit);
    if (shared_planar_pair == false && std::getenv("TSP_TEST_VERBOSE"))
        std::printf("  cpu ids %u %u %u logits %g %g %g shared_logit %g shared_down[0..1] %g %g down[0] %g\n", ids[0], ids[1], ids[2], logits[0], logits[1],
                    logits[2], shared_logit, sy[0], sy[1], y[0]);
    orc_mixture_reference(y.data(), weights.data(), s.selected, sy.data(), s.channels, double(float(shared_logit)), out.data());
    return out;
}

void test_dense_mm_q8_layouts() {
    // graph.hpp:859-860: a dense Q8_0 matrix in GGUF rows and in q8_lanes_v1 rows, strided f32 rows in and out
    const uint32_t K = 512, R = 160, M = 19;
    HipGraph g(64u << 20);
    const auto w = fixture(8, K, R, 1);
    std::vector<uint8_t> lanes(w.size());
    EXPECT(tsp_q8_lanes_pack_rows(K, w.data(), lanes.data(), w.size()) == TSP_OK);
    const auto x = lcg_floats(21, size_t(M) * (K + 8));
    const GpuView dw = g.upload(bytes_of(w), "w"), dl = g.upload(bytes_of(lanes), "lanes"), dx = g.upload(bytes_of(x), "x", false);
    const std::vector<float> canary(size_t(M) * (R + 4), -7.0f);
    const GpuView y0 = g.upload(bytes_of(canary), "y0", false), y1 = g.upload(bytes_of(canary), "y1", false);
    EXPECT(throws_format([&] { g.configure_block_gemv(4); }));
    g.configure_block_gemv(3);
    g.configure_small_gemv(8);
    g.prepare_dense_mm_q8(PrefillWeightLayout::q8_lanes_v1);
    EXPECT(throws_format([&] { g.prepare_dense_mm_q8(PrefillWeightLayout::planar_v3); }));
    const GpuRowsF32 in{dx, M, K, uint64_t(K + 8) * 4};
    g.begin();
    g.dense_mm_q8(PrefillWeightLayout::gguf, dw, in, {y0, M, R, uint64_t(R + 4) * 4});
    g.dense_mm_q8(PrefillWeightLayout::q8_lanes_v1, dl, in, {y1, M, R, uint64_t(R + 4) * 4});
    (void)g.submit();
    const auto got0 = read_as<float>(g, y0), got1 = read_as<float>(g, y1);
    for (uint32_t m = 0; m < M; ++m) {
        std::vector<double> want(R);
        orc_reference_gemv(8, w.data(), w.size(), K, R, x.data() + size_t(m) * (K + 8), K, want.data());
        const std::vector<float> row0(got0.begin() + size_t(m) * (R + 4), got0.begin() + size_t(m) * (R + 4) + R);
        const std::vector<float> row1(got1.begin() + size_t(m) * (R + 4), got1.begin() + size_t(m) * (R + 4) + R);
        EXPECT(scaled_error(row0, want) <= 5e-5 && scaled_error(row1, want) <= 5e-5);
        for (uint32_t pad = R; pad < R + 4; ++pad) EXPECT(got0[size_t(m) * (R + 4) + pad] == -7.0f && got1[size_t(m) * (R + 4) + pad] == -7.0f);
    }
    // prepared with bounds, 32 rows or more go through the staged form (halves on the matrix cores): same values to the GEMM
    // tolerance, same canaries, and the scratch is charged to the graph's budget (it grows when prepared again with wider bounds)
    const uint32_t M2 = 45;
    const auto x2 = lcg_floats(22, size_t(M2) * (K + 8));
    const GpuView dx2 = g.upload(bytes_of(x2), "x2", false);
    const std::vector<float> canary2(size_t(M2) * (R + 4), -7.0f);
    const GpuView y2 = g.upload(bytes_of(canary2), "y2", false), y3 = g.upload(bytes_of(canary2), "y3", false);
    const uint64_t before = g.memory().live_bytes;
    g.prepare_dense_mm_q8(PrefillWeightLayout::gguf, 32, K, R);
    const uint64_t small = g.memory().live_bytes - before;
    EXPECT(small == tsp_dense_mm_q8_workspace_bytes(32, K, R));
    g.prepare_dense_mm_q8(PrefillWeightLayout::gguf, M2, K, R);
    EXPECT(g.memory().live_bytes - before == tsp_dense_mm_q8_workspace_bytes(M2, K, R));
    EXPECT(throws_format([&] { g.prepare_dense_mm_q8(PrefillWeightLayout::gguf, 0, K, R); }));
    const GpuRowsF32 in2{dx2, M2, K, uint64_t(K + 8) * 4};
    g.begin();
    g.dense_mm_q8(PrefillWeightLayout::gguf, dw, in2, {y2, M2, R, uint64_t(R + 4) * 4});
    g.dense_mm_q8(PrefillWeightLayout::q8_lanes_v1, dl, in2, {y3, M2, R, uint64_t(R + 4) * 4});
    (void)g.submit();
    const auto got2 = read_as<float>(g, y2), got3 = read_as<float>(g, y3);
    for (uint32_t m = 0; m < M2; ++m) {
        std::vector<double> want(R);
        orc_reference_gemv(8, w.data(), w.size(), K, R, x2.data() + size_t(m) * (K + 8), K, want.data());
        double scale = 1, worst = 0;  // the GEMM tolerance: 2e-3 of the row's largest magnitude
        for (double v : want) scale = std::max(scale, std::fabs(v));
        for (uint32_t r = 0; r < R; ++r) {
            worst = std::max(worst, std::fabs(double(got2[size_t(m) * (R + 4) + r]) - want[r]) / scale);
            worst = std::max(worst, std::fabs(double(got3[size_t(m) * (R + 4) + r]) - want[r]) / scale);
        }
        if (m == 0) std::printf("dense_mm_q8 staged: row 0 max error / row max %.3e\n", worst);
        EXPECT(worst <= 2e-3);
        for (uint32_t pad = R; pad < R + 4; ++pad) EXPECT(got2[size_t(m) * (R + 4) + pad] == -7.0f && got3[size_t(m) * (R + 4) + pad] == -7.0f);
    }
}

void test_encode_moe_single_token() {
    const MoeFixture f = make_moe(256, 256, 8, 3);
    HipGraph g(256u << 20);
    MoeOnGraph m = upload_moe(g, f);
    // the single-token composition runs the shared expert as three raw-GGUF GEMVs (src/moe.cpp:71-78)
    const size_t gu_bytes = size_t(f.shape.channels / 256) * 144 * f.shape.hidden, dn_bytes = size_t(f.shape.hidden / 256) * 210 * f.shape.channels;
    m.w.shared_gate = {g.upload(std::as_bytes(std::span(f.sgate.data(), gu_bytes)), "shared gate"), 12};
    m.w.shared_up = {g.upload(std::as_bytes(std::span(f.sup.data(), gu_bytes)), "shared up"), 12};
    m.w.shared_down = {g.upload(std::as_bytes(std::span(f.sdown.data(), dn_bytes)), "shared down"), 14};
    g.prepare_planar_moe_v3(12, 14, false);
    const MoeScratch scratch = allocate_moe_scratch(g, f.shape);
    const auto x = lcg_floats(101, f.shape.channels);
    const GpuView dx = g.upload(bytes_of(x), "x", false), dy = g.zeros(uint64_t(f.shape.channels) * 4, "y");
    EXPECT(is_planar_moe(g, m.w, f.shape) && g.planar_matrix_count() == 3);
    const uint64_t allocations = g.memory().allocations;
    g.begin();
    encode_moe(g, m.w, scratch, dx, dy, f.shape, RouterMode::softmax, true);
    const BatchResult r = g.submit();
    EXPECT(r.dispatches == 9 && g.memory().allocations == allocations);
    // Q6_K integer products above 2048 lose their lowest bit on the matrix cores: a few 1e-5 of the row scale
    const double err = row_error(read_as<float>(g, dy), cpu_moe_token(f, x.data(), false));
    std::printf("encode_moe single token: error / row max %.3e\n", err);
    if (err > 2e-4) {  // say which stage differs
        const auto ids = read_as<uint32_t>(g, scratch.indices);
        const auto lg = read_as<float>(g, scratch.logits);
        const auto sl = read_as<float>(g, scratch.shared_logit);
        const auto sd = read_as<float>(g, scratch.shared_down);
        const auto dn = read_as<float>(g, scratch.down);
        std::printf("  ids %u %u %u logits %g %g %g shared_logit %g shared_down[0..1] %g %g down[0] %g\n", ids[0], ids[1], ids[2], lg[0], lg[1], lg[2], sl[0], sd[0], sd[1], dn[0]);
    }
    EXPECT(err <= 2e-4);
    // a non-finite input poisons only its own batch (tests/test_moe.cpp:175-185)
    std::vector<float> bad = x;
    bad[7] = NAN;
    g.write(dx, bytes_of(bad));
    g.begin();
    encode_moe(g, m.w, scratch, dx, dy, f.shape, RouterMode::softmax, true);
    EXPECT(throws_format([&] { (void)g.submit(); }));
    g.write(dx, bytes_of(x));
    g.begin();
    encode_moe(g, m.w, scratch, dx, dy, f.shape, RouterMode::softmax, true);
    (void)g.submit();
    EXPECT(row_error(read_as<float>(g, dy), cpu_moe_token(f, x.data(), false)) <= 2e-4);
    // registration is closed once a batch has begun; registered matrices stay resident
    EXPECT(throws_format([&] { g.register_planar_matrix(m.w.down.view, {14, 10, f.shape.hidden, f.shape.channels, f.shape.experts}); }));
    EXPECT(throws_format([&] { g.release(m.w.down.view); }));
    release_moe_scratch(g, scratch);
}

void test_encode_moe_batch() {
    const uint32_t T = 70;
    const MoeFixture f = make_moe(256, 256, 8, 3);
    HipGraph g(512u << 20);
    MoeOnGraph m = upload_moe(g, f);
    tsp_planar_spec gu{}, dn{};
    tsp_make_expert_spec(12, f.shape.channels, f.shape.hidden, &gu);
    tsp_make_expert_spec(14, f.shape.hidden, f.shape.channels, &dn);
    m.w.shared_gate = {g.upload(bytes_of(coloc_half(gu, f.sgate, f.sup, 2, 0)), "shared pair_lo"), 12};
    m.w.shared_up = {g.upload(bytes_of(coloc_half(gu, f.sgate, f.sup, 2, 1)), "shared pair_hi"), 12};
    m.w.shared_down = {g.upload(bytes_of(planar_stack(dn, f.sdown, 2)), "shared down"), 14};
    g.register_planar_matrix(m.w.shared_gate.view, {12, 2, f.shape.channels, f.shape.hidden, 2});
    g.register_planar_matrix(m.w.shared_up.view, {12, 3, f.shape.channels, f.shape.hidden, 2});
    g.register_planar_matrix(m.w.shared_down.view, {14, 10, f.shape.hidden, f.shape.channels, 2});
    g.prepare_planar_moe_v3(12, 14, true, T, f.shape.experts, f.shape.selected, f.shape.channels, f.shape.hidden);
    const MoeBatchScratch scratch = allocate_moe_batch_scratch(g, f.shape, T);
    // inputs are bf16-valued (the prefill path carries activations as bf16) with a two-float pad per row that must stay untouched
    const uint32_t stride = f.shape.channels + 2;
    std::vector<float> x = lcg_floats(303, size_t(T) * stride), logits(size_t(T) * f.shape.experts);
    for (auto& v : x) { uint32_t bad = 0; v = orc_bf16_to_f32(orc_round_bf16_bits(v, &bad)); }
    for (uint32_t t = 0; t < T; ++t) {
        std::vector<double> l(f.shape.experts);
        orc_reference_gemv(0, reinterpret_cast<const uint8_t*>(f.router.data()), f.router.size() * 4, f.shape.channels, f.shape.experts, &x[size_t(t) * stride],
                           f.shape.channels, l.data());
        for (uint32_t e = 0; e < f.shape.experts; ++e) logits[size_t(t) * f.shape.experts + e] = float(l[e]);
    }
    const GpuView dx = g.upload(bytes_of(x), "x", false), dl = g.upload(bytes_of(logits), "logits", false);
    std::vector<float> canary(size_t(T) * stride, -9.0f);
    const GpuView dy = g.upload(bytes_of(canary), "y", false);
    const uint64_t allocations = g.memory().allocations;
    g.begin();
    encode_moe_batch(g, m.w, scratch, dl, {dx, T, f.shape.channels, uint64_t(stride) * 4}, {dy, T, f.shape.channels, uint64_t(stride) * 4}, f.shape,
                     RouterMode::softmax, true);
    const BatchResult r = g.submit();
    EXPECT(r.dispatches == 4 && g.memory().allocations == allocations);  // route, grouped MoE with the shared expert riding, shared router, mixture
    const auto y = read_as<float>(g, dy);
    double worst = 0;
    bool pads = true;
    for (uint32_t t = 0; t < T; ++t) {
        const auto want = cpu_moe_token(f, &x[size_t(t) * stride], true);
        double scale = 1;
        for (double v : want) scale = std::max(scale, std::fabs(v));
        for (uint32_t c = 0; c < f.shape.channels; ++c) worst = std::max(worst, std::fabs(double(y[size_t(t) * stride + c]) - want[c]) / scale);
        pads = pads && y[size_t(t) * stride + f.shape.channels] == -9.0f && y[size_t(t) * stride + f.shape.channels + 1] == -9.0f;
    }
    std::printf("encode_moe_batch T=%u: max error / row max %.3e\n", T, worst);
    EXPECT(worst <= 2e-3 && pads);
    // a token that selects one expert twice is a device-side refusal
    std::vector<uint32_t> ids = read_as<uint32_t>(g, scratch.indices);
    g.begin();
    g.prefill_route_batch(dl, scratch.indices, scratch.weights, f.shape.experts, f.shape.selected, T, RouterMode::softmax, true);
    (void)g.submit();
    ids[1] = ids[0];
    g.write(scratch.indices, bytes_of(ids));
    g.begin();
    g.planar_nax_grouped_moe(m.w.gate.view, m.w.up.view, m.w.down.view, scratch.indices, {dx, T, f.shape.channels, uint64_t(stride) * 4},
                             {scratch.expert_down, T * f.shape.selected, f.shape.channels, uint64_t(f.shape.channels) * 4}, scratch.token_map, scratch.counts,
                             scratch.tasks, f.shape.experts, f.shape.selected);
    EXPECT(throws_format([&] { (void)g.submit(); }));
    release_moe_batch_scratch(g, scratch);
}
// CPU composition of the whole sublayer for one token with a dense Q8_0 shared expert (src/moe_mm_many.cpp:126-283 order)
std::vector<double> cpu_moe_token_q8_shared(const MoeFixture& f, const std::vector<uint8_t>& sg, const std::vector<uint8_t>& su, const std::vector<uint8_t>& sd,
                                            const float* x, uint32_t gate_up_type = 12, uint32_t down_type = 14) {
    const MoeShape s = f.shape;
    std::vector<double> logits(s.experts), weights(s.selected), out(s.channels);
    orc_reference_gemv(0, reinterpret_cast<const uint8_t*>(f.router.data()), f.router.size() * 4, s.channels, s.experts, x, s.channels, logits.data());
    for (auto& v : logits) v = double(float(v));
    std::vector<uint32_t> ids(s.selected);
    orc_route_reference(logits.data(), s.experts, s.selected, 0, 1, ids.data(), weights.data());
    std::vector<double> h(size_t(s.selected) * s.hidden), y(size_t(s.selected) * s.channels);
    orc_moe_routed_reference(gate_up_type, down_type, f.gate.data(), f.up.data(), f.down.data(), s.channels, s.hidden, s.experts, ids.data(), 1, s.selected, x,
                             s.channels, 1, 0, h.data(), y.data(), 1);
    std::vector<double> g(s.hidden), u(s.hidden), sy(s.channels);
    orc_reference_gemv(8, sg.data(), sg.size(), s.channels, s.hidden, x, s.channels, g.data());
    orc_reference_gemv(8, su.data(), su.size(), s.channels, s.hidden, x, s.channels, u.data());
    std::vector<float> act(s.hidden);
    for (uint32_t i = 0; i < s.hidden; ++i) { const double v = g[i]; act[i] = float(v / (1.0 + std::exp(-v)) * u[i]); }
    orc_reference_gemv(8, sd.data(), sd.size(), s.hidden, s.channels, act.data(), s.hidden, sy.data());
    double shared_logit = 0;
    orc_reference_gemv(0, reinterpret_cast<const uint8_t*>(f.shared_router.data()), f.shared_router.size() * 4, s.channels, 1, x, s.channels, &shared_logit);
    orc_mixture_reference(y.data(), weights.data(), s.selected, sy.data(), s.channels, double(float(shared_logit)), out.data());
    return out;
}

void encode_moe_mm_many_case(bool router_batch) {
    // planar Q4_K / Q6_K routed experts, dense Q8_0 shared expert (gate in q8_lanes_v1 rows, up and down in GGUF rows), F32 routers;
    // 70 rows take the grouped GEMM, 5 rows the routed kernels for at most eight
    const MoeFixture f = make_moe(256, 256, 8, 3);
    const uint32_t capacity = 70;
    HipGraph g(512u << 20);
    g.configure_moe_router_f32_batch(router_batch);  // src/moe_mm_many.cpp:170-177: the chunk's router logits from one f32 GEMM
    MoeOnGraph m = upload_moe(g, f);
    const auto sg = fixture(8, f.shape.channels, f.shape.hidden, 1), sd = fixture(8, f.shape.hidden, f.shape.channels, 1);
    auto su = sg;
    for (size_t at = 0; at < su.size(); at += 34) for (size_t i = 2; i < 34; ++i) su[at + i] = uint8_t(su[at + i] * 5 + 3);
    std::vector<uint8_t> sg_lanes(sg.size());
    EXPECT(tsp_q8_lanes_pack_rows(f.shape.channels, sg.data(), sg_lanes.data(), sg.size()) == TSP_OK);
    m.w.shared_gate = {g.upload(bytes_of(sg_lanes), "shared gate"), 8};
    m.w.shared_up = {g.upload(bytes_of(su), "shared up"), 8};
    m.w.shared_down = {g.upload(bytes_of(sd), "shared down"), 8};
    MoeMmLayouts layouts;
    layouts.shared_gate = PrefillWeightLayout::q8_lanes_v1;
    prepare_moe_mm_many(g, m.w, f.shape, capacity, layouts);
    const MoeMmManyScratch scratch = allocate_moe_mm_many_scratch(g, f.shape, capacity);
    EXPECT(scratch.capacity == capacity && moe_mm_many_bytes(f.shape, capacity).views[0] == uint64_t(capacity) * f.shape.experts * 4);
    const uint32_t stride = f.shape.channels + 4;  // 16-byte multiple, as the composition demands
    for (const uint32_t T : {70u, 5u}) {
        std::vector<float> x = lcg_floats(400 + T, size_t(T) * stride);
        for (auto& v : x) { uint32_t bad = 0; v = orc_bf16_to_f32(orc_round_bf16_bits(v, &bad)); }
        const GpuView dx = g.upload(bytes_of(x), "x", false);
        const std::vector<float> canary(size_t(T) * stride, -3.0f);
        const GpuView dy = g.upload(bytes_of(canary), "y", false);
        const uint64_t allocations = g.memory().allocations;
        g.begin();
        encode_moe_mm_many(g, m.w, scratch, {dx, T, f.shape.channels, uint64_t(stride) * 4}, {dy, T, f.shape.channels, uint64_t(stride) * 4}, f.shape,
                           RouterMode::softmax, true, layouts);
        (void)g.submit();
        EXPECT(g.memory().allocations == allocations);
        const auto y = read_as<float>(g, dy);
        double worst = 0;
        bool pads = true;
        for (uint32_t t = 0; t < T; ++t) {
            const auto want = cpu_moe_token_q8_shared(f, sg, su, sd, &x[size_t(t) * stride]);
            double scale = 1;
            for (double v : want) scale = std::max(scale, std::fabs(v));
            for (uint32_t c = 0; c < f.shape.channels; ++c) worst = std::max(worst, std::fabs(double(y[size_t(t) * stride + c]) - want[c]) / scale);
            for (uint32_t c = f.shape.channels; c < stride; ++c) pads = pads && y[size_t(t) * stride + c] == -3.0f;
        }
        std::printf("encode_moe_mm_many T=%u%s: max error / row max %.3e\n", T, router_batch ? ", router as one GEMM" : "", worst);
        EXPECT(worst <= 2e-3 && pads);
        g.release(dx);
        g.release(dy);
    }
    // rows beyond the scratch capacity are worked off in chunks; a scratch of another capacity is refused
    {
        const uint32_t T = 150;
        std::vector<float> x = lcg_floats(777, size_t(T) * stride);
        for (auto& v : x) { uint32_t bad = 0; v = orc_bf16_to_f32(orc_round_bf16_bits(v, &bad)); }
        const GpuView dx = g.upload(bytes_of(x), "x", false), dy = g.zeros(uint64_t(T) * stride * 4, "y");
        g.begin();
        encode_moe_mm_many(g, m.w, scratch, {dx, T, f.shape.channels, uint64_t(stride) * 4}, {dy, T, f.shape.channels, uint64_t(stride) * 4}, f.shape,
                           RouterMode::softmax, true, layouts);
        (void)g.submit();
        const auto y = read_as<float>(g, dy);
        const auto want = cpu_moe_token_q8_shared(f, sg, su, sd, &x[size_t(149) * stride]);
        double scale = 1, worst = 0;
        for (double v : want) scale = std::max(scale, std::fabs(v));
        for (uint32_t c = 0; c < f.shape.channels; ++c) worst = std::max(worst, std::fabs(double(y[size_t(149) * stride + c]) - want[c]) / scale);
        EXPECT(worst <= 2e-3);
        MoeMmManyScratch wrong = scratch;
        wrong.capacity = capacity + 1;
        g.begin();
        EXPECT(throws_format([&] {
            encode_moe_mm_many(g, m.w, wrong, {dx, 4, f.shape.channels, uint64_t(stride) * 4}, {dy, 4, f.shape.channels, uint64_t(stride) * 4}, f.shape,
                               RouterMode::softmax, true, layouts);
        }));
        g.abort();
    }
    release_moe_mm_many_scratch(g, scratch);
}
void test_encode_moe_mm_many() { encode_moe_mm_many_case(false); }
void test_encode_moe_mm_many_router_batch() { encode_moe_mm_many_case(true); }

// native/tests/test_moe_mm_many.cpp:35-47 (the plan) and native/tests/test_moe_mm_many_gpu.cpp:194-262 (selection, preparation,
// the 5e-5 logit bound against double sums and against the per-row GEMV, untouched padding, refusals that write nothing)
void test_router_projection_controls() {
    for (const uint32_t n : {1u, 2u, 3u, 8u, 31u, 32u, 33u, 511u, 512u}) {
        const auto p = moe_router_f32_plan(2560, 512, n, 10272, 2080);
        EXPECT(p.matrix_bytes == 5242880 && p.input_bytes == uint64_t(n - 1) * 10272 + 10240 && p.output_bytes == uint64_t(n - 1) * 2080 + 2048);
        EXPECT(p.grid_x == 16 && p.grid_y == (n + 31) / 32 && p.args.tokens == n && p.args.reserved == 0);
    }
    for (const uint32_t n : {0u, 513u, std::numeric_limits<uint32_t>::max()}) EXPECT(throws_format([&] { (void)moe_router_f32_plan(2560, 512, n, 10240, 2048); }));
    EXPECT(throws_format([] { (void)moe_router_f32_plan(2559, 512, 3, 10240, 2048); }));
    EXPECT(throws_format([] { (void)moe_router_f32_plan(2560, 511, 3, 10240, 2048); }));
    EXPECT(throws_format([] { (void)moe_router_f32_plan(2560, 512, 3, 10236, 2048); }));
    EXPECT(throws_format([] { (void)moe_router_f32_plan(2560, 512, 3, 10240, 2044); }));
    EXPECT(throws_format([] { (void)moe_router_f32_plan(2560, 512, 512, std::numeric_limits<uint64_t>::max() - 15, 2048); }));
    EXPECT(throws_format([] { (void)moe_router_f32_plan(2560, 512, 512, 10240, std::numeric_limits<uint64_t>::max() - 15); }));
    EXPECT(throws_format([] { (void)moe_router_f32_plan(2560, 512, 2, 256ull << 20, 2048); }));
    // the device kernel's own limits: any multiple of 32 columns, any expert count
    EXPECT(moe_router_f32_plan(2048, 70, 2048, 8192, 288, false).grid_x == 3);
    EXPECT(throws_format([] { (void)moe_router_f32_plan(2040, 70, 3, 8160, 288, false); }));

    HipGraph g(256u << 20);
    EXPECT(!g.moe_router_f32_batch_enabled() && std::string(g.moe_router_f32_projection_kernel()) == "graph_quantized_gemv");
    g.configure_moe_router_f32_batch(true);
    EXPECT(g.moe_router_f32_batch_enabled() && std::string(g.moe_router_f32_projection_kernel()) == "graph_moe_router_f32_batch");
    constexpr uint32_t c = 2560, e = 512, capacity = 512;
    constexpr uint64_t xs = c * 4 + 32, ys = e * 4 + 32;
    std::vector<float> weights(uint64_t(c) * e), input(capacity * xs / 4, -9876.25f), poison(capacity * ys / 4 + 16, -7654.25f);
    uint32_t rng = 44;
    for (auto& v : weights) { rng = rng * 1664525u + 1013904223u; v = float(int(rng % 1993) - 996) / 997 / 256; }
    for (uint32_t t = 0; t < capacity; ++t)
        for (uint32_t k = 0; k < c; ++k) { rng = rng * 1664525u + 1013904223u; input[t * xs / 4 + k] = float(int(rng % 1993) - 996) / 997; }
    const GpuView w = g.upload(bytes_of(weights), "router"), x = g.upload(bytes_of(input), "x");
    const GpuView y = g.upload(bytes_of(poison), "y", false), scalar = g.upload(bytes_of(poison), "scalar", false);
    g.begin();
    EXPECT(throws_format([&] { g.moe_router_f32_batch(w, {x, 3, c, xs}, {y, 3, e, ys}); }));  // selected but not prepared
    g.abort();
    EXPECT(read_as<float>(g, y) == poison);
    g.prepare_moe_router_f32_batch();
    EXPECT(throws_format([&] { g.configure_moe_router_f32_batch(false); }));
    for (const uint32_t n : {3u, 33u, 512u}) {
        const uint64_t allocations = g.memory().allocations;
        g.begin();
        g.gemv_rows(0, w, {x, n, c, xs}, {scalar, n, e, ys});
        g.moe_router_f32_batch(w, {x, n, c, xs}, {y, n, e, ys});
        const BatchResult r = g.submit();
        EXPECT(r.dispatches == 2 && g.memory().allocations == allocations);
        const auto got = read_as<float>(g, y), legacy = read_as<float>(g, scalar);
        bool bound = true, pads = true;
        for (uint32_t t = 0; t < n; ++t) {
            for (uint32_t expert = 0; expert < e; ++expert) {
                double sum = 0;
                for (uint32_t k = 0; k < c; ++k) sum += double(weights[uint64_t(expert) * c + k]) * input[t * xs / 4 + k];
                const double a = got[t * ys / 4 + expert], b = legacy[t * ys / 4 + expert], tol = 0.00005 * std::max(1.0, std::fabs(sum));
                bound = bound && std::isfinite(a) && std::fabs(a - sum) <= tol && std::fabs(b - sum) <= tol && std::fabs(a - b) <= 0.00005 * std::max(1.0, std::fabs(b));
            }
            for (uint32_t k = e; k < ys / 4; ++k) pads = pads && got[t * ys / 4 + k] == -7654.25f;
        }
        for (size_t k = n * ys / 4; k < got.size(); ++k) pads = pads && got[k] == -7654.25f;
        EXPECT(bound && pads);
    }
    const auto saved = read_as<float>(g, y);
    const auto refused = [&](GpuRowsF32 in, GpuRowsF32 out) {
        g.begin();
        const bool threw = throws_format([&] { g.moe_router_f32_batch(w, in, out); });
        g.abort();
        return threw && read_as<float>(g, y) == saved;
    };
    const GpuRowsF32 in{x, 3, c, xs}, out{y, 3, e, ys};
    GpuRowsF32 bad = out;
    bad.rows = 2;
    EXPECT(refused(in, bad));
    bad = out; bad.stride_bytes = e * 4 - 4;
    EXPECT(refused(in, bad));
    bad = out; bad.view = x;  // immutable, and the input itself
    EXPECT(refused(in, bad));
}

// A block of an adopted Pack v3 file on the graph: synthetic shards on disk -> build_block_pack_v3 -> adopt_block_pack_v3 (full
// authentication) -> upload_moe_block_v3 registers the co-located Q4_K halves and the Q5_1 down planes as they lie in the file ->
// encode_moe_mm_many runs on them, the shared expert's Q8_0 matrices coming from the pack in q8_lanes_v1 rows.
void test_pack_v3_block_on_graph() {
    using gguf_writer::TensorSpec;
    MoeFixture f{{256, 256, 4, 2}};
    f.gate = fixture(12, 256, 256, 4);
    f.up = f.gate;
    for (size_t at = 0; at < f.up.size(); at += 144) for (size_t i = 16; i < 144; ++i) f.up[at + i] ^= 0x5a;
    f.down = fixture(7, 256, 256, 4);
    f.router = lcg_floats(31, size_t(4) * 256);
    f.shared_router = lcg_floats(37, 256);
    for (auto& v : f.shared_router) v *= 0.05f;
    const auto sg = fixture(8, 256, 256, 1), sd = fixture(8, 256, 256, 1);
    auto su = sg;
    for (size_t at = 0; at < su.size(); at += 34) for (size_t i = 2; i < 34; ++i) su[at + i] = uint8_t(su[at + i] * 5 + 3);
    const auto raw = [](const std::vector<float>& v) { std::vector<uint8_t> b(v.size() * 4); std::memcpy(b.data(), v.data(), b.size()); return b; };
    const std::vector<TensorSpec> specs{{"blk.0.ffn_down_exps.weight", 7, {256, 256, 4}, f.down},      {"blk.0.ffn_down_shexp.weight", 8, {256, 256}, sd},
                                        {"blk.0.ffn_gate_exps.weight", 12, {256, 256, 4}, f.gate},     {"blk.0.ffn_gate_inp.weight", 0, {256, 4}, raw(f.router)},
                                        {"blk.0.ffn_gate_inp_shexp.weight", 0, {256}, raw(f.shared_router)}, {"blk.0.ffn_gate_shexp.weight", 8, {256, 256}, sg},
                                        {"blk.0.ffn_up_exps.weight", 12, {256, 256, 4}, f.up},         {"blk.0.ffn_up_shexp.weight", 8, {256, 256}, su}};
    gguf_writer::TempDir dir("tokspur_pack_v3_gpu");
    gguf_writer::write_file(dir.path / "source.gguf", gguf_writer::shard_bytes("qwen35moe", specs));
    const auto source = std::make_shared<const ModelFiles>(std::vector<std::filesystem::path>{dir.path / "source.gguf"});
    const auto pack_path = dir.path / "tokspur-pack-v3-blk0.asa.gguf";
    const auto built = planar_v3::build_block_pack_v3(source, nullptr, 0, pack_path, 2, 1 << 20);
    EXPECT(built.tensors.size() == 8);
    const planar_v3::AdoptedPackV3 pack = planar_v3::adopt_block_pack_v3(source, nullptr, 0, pack_path, 2, derived_pack::default_chunk_bytes, 3);
    EXPECT(pack.plan.tensors.size() == 8 && pack.authentication_workers == 3);

    HipGraph g(512u << 20);
    const planar_v3::PackMoeBlockV3 block = planar_v3::upload_moe_block_v3(g, pack, 0);
    EXPECT(block.channels == 256 && block.hidden == 256 && block.experts == 4 && g.planar_matrix_count() == 3);
    EXPECT(block.gate.encoding == 12 && block.up.encoding == 12 && block.down.encoding == 7);
    EXPECT(throws_format([&] { (void)planar_v3::upload_moe_block_v3(g, pack, 5); }));
    MoeWeights w{};
    const auto from_pack = [&](const char* name) { return g.upload(pack.model->tensor_bytes(name), name); };
    w.router = {from_pack("blk.0.ffn_gate_inp.weight"), 0};
    w.shared_router = {from_pack("blk.0.ffn_gate_inp_shexp.weight"), 0};
    w.gate = block.gate; w.up = block.up; w.down = block.down;
    w.shared_gate = {from_pack("blk.0.ffn_gate_shexp.weight"), 8};
    w.shared_up = {from_pack("blk.0.ffn_up_shexp.weight"), 8};
    w.shared_down = {from_pack("blk.0.ffn_down_shexp.weight"), 8};
    MoeMmLayouts layouts;  // dense Q8_0 matrices lie in the pack in q8_lanes_v1 rows
    layouts.shared_gate = layouts.shared_up = layouts.shared_down = PrefillWeightLayout::q8_lanes_v1;
    for (const auto& t : pack.plan.tensors)
        if (t.name.find("shexp.weight") != std::string::npos && t.type == 8) EXPECT(t.kind == planar_v3::PlanarKind::q8_lanes_v1);
    EXPECT(is_planar_moe(g, w, f.shape));
    const uint32_t capacity = 70;
    g.configure_moe_router_f32_batch(true);
    prepare_moe_mm_many(g, w, f.shape, capacity, layouts);
    const MoeMmManyScratch scratch = allocate_moe_mm_many_scratch(g, f.shape, capacity);
    for (const uint32_t T : {70u, 5u}) {
        std::vector<float> x = lcg_floats(900 + T, size_t(T) * 256);
        for (auto& v : x) { uint32_t bad = 0; v = orc_bf16_to_f32(orc_round_bf16_bits(v, &bad)); }
        const GpuView dx = g.upload(bytes_of(x), "x", false), dy = g.zeros(uint64_t(T) * 256 * 4, "y");
        g.begin();
        encode_moe_mm_many(g, w, scratch, {dx, T, 256, 1024}, {dy, T, 256, 1024}, f.shape, RouterMode::softmax, true, layouts);
        (void)g.submit();
        const auto y = read_as<float>(g, dy);
        double worst = 0;
        for (uint32_t t = 0; t < T; ++t) {
            const auto want = cpu_moe_token_q8_shared(f, sg, su, sd, &x[size_t(t) * 256], 12, 7);
            double scale = 1;
            for (double v : want) scale = std::max(scale, std::fabs(v));
            for (uint32_t c = 0; c < 256; ++c) worst = std::max(worst, std::fabs(double(y[size_t(t) * 256 + c]) - want[c]) / scale);
        }
        std::printf("encode_moe_mm_many on an adopted pack v3 block, T=%u: max error / row max %.3e\n", T, worst);
        EXPECT(worst <= 2e-3);
        g.release(dx);
        g.release(dy);
    }
    release_moe_mm_many_scratch(g, scratch);
}

// native/tests/test_graph.cpp:113-141 `residual_cases` through the graph class: rms -> F32 GEMV -> SiLU in place -> two F32 GEMVs ->
// residual_read -> residual_write, seven operators in one batch with a partial commit in the middle, 5e-5 scaled error
void test_residual_streams_and_partial_commit() {
    HipGraph g(64u << 20);
    for (const auto& shape : {std::array<uint32_t, 3>{1, 7, 3}, std::array<uint32_t, 3>{4, 9, 5}, std::array<uint32_t, 3>{3, 257, 16}, std::array<uint32_t, 3>{4, 2560, 320}}) {
        const uint32_t branches = shape[0], channels = shape[1], rank = shape[2], width = branches * channels;
        auto streams = lcg_floats(11 + channels, width), gains = lcg_floats(12 + channels, width);
        for (auto& v : gains) v = 1 + 0.1f * v;
        auto down = lcg_floats(13 + channels, size_t(width) * rank), up = lcg_floats(14 + channels, size_t(rank) * width), inject = lcg_floats(15 + channels, size_t(width) * branches);
        for (auto* m : {&down, &up, &inject}) for (auto& v : *m) v *= 0.01f;
        const float epsilon = 1e-6f;
        const auto real = [](const std::vector<float>& v) { return std::vector<double>(v.begin(), v.end()); };
        std::vector<double> want_read(channels), want_scales(branches), want_written(width);
        EXPECT(orc_gated_residual_reference(real(streams).data(), real(gains).data(), real(down).data(), real(up).data(), real(inject).data(), branches, channels, rank,
                                            epsilon, want_read.data(), want_scales.data()) == 0);
        EXPECT(orc_residual_write_reference(real(streams).data(), want_read.data(), want_scales.data(), branches, channels, want_written.data()) == 0);
        const GpuView stream = g.upload(bytes_of(streams), "streams"), gain = g.upload(bytes_of(gains), "gains"), w_down = g.upload(bytes_of(down), "down");
        const GpuView w_up = g.upload(bytes_of(up), "up"), w_inject = g.upload(bytes_of(inject), "inject");
        const GpuView normalized = g.zeros(width * 4, "normalized"), bottleneck = g.zeros(rank * 4, "bottleneck"), scores = g.zeros(width * 4, "scores");
        const GpuView logits = g.zeros(branches * 4, "inject logits"), scales = g.zeros(branches * 4, "scales"), output = g.zeros(channels * 4, "output");
        const GpuView written = g.zeros(width * 4, "written");
        const uint64_t allocations = g.memory().allocations;
        g.begin();
        EXPECT(!g.commit_partial());  // nothing encoded yet
        g.rms(stream, gain, normalized, channels, epsilon);
        g.gemv(0, w_down, normalized, bottleneck, width, rank);
        g.activate(bottleneck, bottleneck, Activation::silu, 1.0f / float(branches));
        EXPECT(g.commit_partial());
        g.gemv(0, w_up, bottleneck, scores, rank, width);
        g.gemv(0, w_inject, normalized, logits, width, branches);
        g.residual_read(normalized, scores, logits, output, scales, branches, channels);
        g.residual_write(stream, output, scales, written);
        const BatchResult r = g.submit();
        EXPECT(r.dispatches == 7 && g.memory().allocations == allocations);
        EXPECT(scaled_error(read_as<float>(g, output), want_read) <= 5e-5 && scaled_error(read_as<float>(g, scales), want_scales) <= 5e-5);
        EXPECT(scaled_error(read_as<float>(g, written), want_written) <= 5e-5 && read_as<float>(g, stream) == streams);
        // refusals: a group width that does not divide, a zero epsilon, an output over its input, a gate of another size
        g.begin();
        EXPECT(throws_format([&] { g.rms(stream, gain, normalized, channels + 1, epsilon); }));
        EXPECT(throws_format([&] { g.rms(stream, gain, normalized, channels, 0.0f); }));
        EXPECT(throws_format([&] { g.rms(stream, gain, stream, channels, epsilon); }));  // immutable, and its own input
        EXPECT(throws_format([&] { g.rms_sigmoid_gate(stream, gain, output, normalized, channels, epsilon); }) || width == channels);
        EXPECT(throws_format([&] { g.multiply(normalized, output, scores); }) || width == channels);
        EXPECT(throws_format([&] { g.residual_read(normalized, scores, logits, output, scales, branches + 1, channels); }));
        g.abort();
        for (const GpuView v : {stream, gain, w_down, w_up, w_inject, normalized, bottleneck, scores, logits, scales, output, written}) g.release(v);
    }
}

// the raw-GGUF arm of the same composition (src/moe_mm_many.cpp:214-240): three grouped products over Q4_K expert stacks in
// GGUF rows, nothing registered; `grouped_mm` and `dense_mm` on their own; encodings the grouped product does not take are
// refused while idle, and a refusal part-way through a batch leaves no half-encoded batch behind
void test_encode_moe_mm_many_raw_arm() {
    const MoeShape shape{256, 256, 6, 2};
    const auto gate = fixture(12, shape.channels, shape.hidden, shape.experts);
    auto up = gate;
    for (size_t at = 0; at < up.size(); at += 144) for (size_t i = 16; i < 144; ++i) up[at + i] = uint8_t(up[at + i] * 3 + 1);
    const auto down = fixture(12, shape.hidden, shape.channels, shape.experts);
    const auto sg = fixture(8, shape.channels, shape.hidden, 1), sd = fixture(8, shape.hidden, shape.channels, 1);
    const std::vector<float> router = lcg_floats(41, size_t(shape.experts) * shape.channels);
    std::vector<float> shared_router = lcg_floats(43, shape.channels);
    for (auto& v : shared_router) v *= 0.05f;
    HipGraph g("unused.metallib", 256u << 20);
    MoeWeights w{};
    w.router = {g.upload(bytes_of(router), "router"), 0};
    w.gate = {g.upload(bytes_of(gate), "gate"), 12};
    w.up = {g.upload(bytes_of(up), "up"), 12};
    w.down = {g.upload(bytes_of(down), "down"), 12};
    w.shared_gate = {g.upload(bytes_of(sg), "shared gate"), 8};
    w.shared_up = {g.upload(bytes_of(sg), "shared up"), 8};
    w.shared_down = {g.upload(bytes_of(sd), "shared down"), 8};
    w.shared_router = {g.upload(bytes_of(shared_router), "shared router"), 0};
    g.register_q8_matrix(w.shared_gate.view, shape.channels, shape.hidden);
    EXPECT(g.q8_matrix_count() == 1);
    EXPECT(throws_format([&] { g.register_q8_matrix(w.shared_gate.view, shape.channels, shape.hidden); }));      // overlaps a registered matrix
    EXPECT(throws_format([&] { g.register_q8_matrix(w.shared_down.view, shape.channels + 32, shape.hidden); }));  // byte span
    EXPECT(!is_planar_moe(g, w, shape));
    const uint32_t capacity = 40;
    MoeWeights q5 = w;
    q5.down.encoding = 14;  // Q6_K rows are not among the grouped product's encodings (src/grouped_mm.cpp:8-12)
    EXPECT(throws_format([&] { prepare_moe_mm_many(g, q5, shape, capacity); }));  // refused while idle, not in the middle of a batch
    prepare_moe_mm_many(g, w, shape, capacity);
    const uint64_t after_first = g.memory().allocations;
    prepare_moe_mm_many(g, w, shape, capacity);  // a second layer of the same shape: nothing to do
    EXPECT(g.memory().allocations == after_first);
    prepare_moe_mm_many(g, w, MoeShape{512, 256, 6, 2}, capacity);  // a wider layer: the scratch grows
    g.prepare_dense_mm(32, 256);
    g.prepare_dense_mm(64, 512);
    const MoeMmManyScratch scratch = allocate_moe_mm_many_scratch(g, shape, capacity);
    const uint32_t T = 33, stride = shape.channels + 4;
    // The grouped product carries its input rows as halves: the SwiGLU rows that feed the down product have to stay below
    // 65504 in magnitude, which the fixture's weight scales (outputs of ~1e5 for inputs of ~1) only do for small inputs.
    std::vector<float> x = lcg_floats(900, size_t(T) * stride);
    for (auto& v : x) { uint32_t bad = 0; v = orc_bf16_to_f32(orc_round_bf16_bits(v * 0.0009765625f, &bad)); }
    const GpuView dx = g.upload(bytes_of(x), "x", false), dy = g.zeros(uint64_t(T) * stride * 4, "y");
    g.begin();
    encode_moe_mm_many(g, w, scratch, {dx, T, shape.channels, uint64_t(stride) * 4}, {dy, T, shape.channels, uint64_t(stride) * 4}, shape, RouterMode::softmax, true);
    (void)g.submit();
    const auto y = read_as<float>(g, dy);
    double worst = 0;
    for (uint32_t t = 0; t < T; ++t) {
        const float* xt = &x[size_t(t) * stride];
        std::vector<double> logits(shape.experts), weights(shape.selected), out(shape.channels);
        orc_reference_gemv(0, reinterpret_cast<const uint8_t*>(router.data()), router.size() * 4, shape.channels, shape.experts, xt, shape.channels, logits.data());
        for (auto& v : logits) v = double(float(v));
        std::vector<uint32_t> ids(shape.selected);
        orc_route_reference(logits.data(), shape.experts, shape.selected, 0, 1, ids.data(), weights.data());
        std::vector<double> h(size_t(shape.selected) * shape.hidden), yy(size_t(shape.selected) * shape.channels);
        orc_moe_routed_reference(12, 12, gate.data(), up.data(), down.data(), shape.channels, shape.hidden, shape.experts, ids.data(), 1, shape.selected, xt,
                                 shape.channels, 1, 0, h.data(), yy.data(), 1);
        std::vector<double> sgv(shape.hidden), sy(shape.channels);
        orc_reference_gemv(8, sg.data(), sg.size(), shape.channels, shape.hidden, xt, shape.channels, sgv.data());
        std::vector<float> act(shape.hidden);
        for (uint32_t i = 0; i < shape.hidden; ++i) { const double v = sgv[i]; act[i] = float(v / (1.0 + std::exp(-v)) * sgv[i]); }
        orc_reference_gemv(8, sd.data(), sd.size(), shape.hidden, shape.channels, act.data(), shape.hidden, sy.data());
        double shared_logit = 0;
        orc_reference_gemv(0, reinterpret_cast<const uint8_t*>(shared_router.data()), shared_router.size() * 4, shape.channels, 1, xt, shape.channels, &shared_logit);
        orc_mixture_reference(yy.data(), weights.data(), shape.selected, sy.data(), shape.channels, double(float(shared_logit)), out.data());
        double scale = 1;
        for (double v : out) scale = std::max(scale, std::fabs(v));
        for (uint32_t c = 0; c < shape.channels; ++c) worst = std::max(worst, std::fabs(double(y[size_t(t) * stride + c]) - out[c]) / scale);
    }
    std::printf("encode_moe_mm_many raw arm T=%u: max error / row max %.3e\n", T, worst);
    EXPECT(worst <= 2e-3);
    // the grouped and the dense product on their own (graph.hpp:750-753), against the staged reference of one route
    {
        const std::vector<uint32_t> ids{3, 1, 0, 5, 2, 4};  // 3 tokens x 2
        const GpuView dids = g.upload(bytes_of(ids), "ids"), out = g.zeros(6ull * shape.hidden * 4, "out");
        const GpuView map = g.zeros(uint64_t(shape.experts) * 3 * 4, "map"), counts = g.zeros(shape.experts * 4, "counts"), tasks = g.zeros((2 + 2 * (6 / 32 + shape.experts)) * 4, "tasks");
        const GpuView in3 = g.slice(dx, 0, 2ull * stride * 4 + shape.channels * 4);
        g.begin();
        g.grouped_mm(12, PrefillWeightLayout::gguf, w.gate.view, dids, {in3, 3, shape.channels, uint64_t(stride) * 4}, {out, 6, shape.hidden, uint64_t(shape.hidden) * 4},
                     map, counts, tasks, shape.experts, 2, true);
        (void)g.submit();
        const auto got = read_as<float>(g, out);
        std::vector<double> want(shape.hidden);
        const size_t expert_bytes = gate.size() / shape.experts;
        orc_reference_gemv(12, gate.data() + 5 * expert_bytes, expert_bytes, shape.channels, shape.hidden, &x[size_t(1) * stride], shape.channels, want.data());  // route 3 = token 1, expert 5
        EXPECT(row_error(std::vector<float>(got.begin() + 3 * shape.hidden, got.begin() + 4 * shape.hidden), want) <= 2e-3);
        const GpuView dense_out = g.zeros(3ull * shape.hidden * 4, "dense out"), one = g.slice(w.gate.view, 2 * expert_bytes, expert_bytes);
        g.begin();
        g.dense_mm(12, PrefillWeightLayout::gguf, one, {in3, 3, shape.channels, uint64_t(stride) * 4}, {dense_out, 3, shape.hidden, uint64_t(shape.hidden) * 4});
        (void)g.submit();
        const auto dense = read_as<float>(g, dense_out);
        orc_reference_gemv(12, gate.data() + 2 * expert_bytes, expert_bytes, shape.channels, shape.hidden, &x[size_t(2) * stride], shape.channels, want.data());
        EXPECT(row_error(std::vector<float>(dense.begin() + 2 * shape.hidden, dense.end()), want) <= 2e-3);
    }
    // a refusal inside the composition aborts the batch (src/moe_mm_many.cpp:282): the graph is idle again afterwards
    {
        MoeWeights broken = w;
        broken.router.encoding = 99;  // no such encoding: the router projection refuses
        g.begin();
        EXPECT(throws_format([&] {
            encode_moe_mm_many(g, broken, scratch, {dx, 4, shape.channels, uint64_t(stride) * 4}, {dy, 4, shape.channels, uint64_t(stride) * 4}, shape, RouterMode::softmax, true);
        }));
        EXPECT(throws_format([&] { g.abort(); }));  // nothing left to abort
        g.begin();                                  // and a new batch can start
        g.abort();
    }
    release_moe_mm_many_scratch(g, scratch);
}
// native/tests/test_profile.cpp: the opt-in per-operator profile. Same fixture (an F32 GEMV, SiLU, a product and an RMS
// norm), same checks: rows only when asked for, one per operator with the engine's labels and shape metadata, nothing
// allocated while encoding and no output changed, calibration never fails a batch, a batch longer than one sample chunk,
// the capacity refusal while encoding, no stale profile after a device error, the payload on the ledger and its release.
double checked_timings(const GraphProfile& profile) {
    const double mismatch = profile.cpu_clock_mismatch_fraction;
    const bool calibrated = std::isfinite(mismatch) && mismatch >= 0 && mismatch <= 0.03;
    EXPECT(profile.timings_valid == calibrated);
    double maximum = 0, sum = 0;
    bool ticks = true, millis = true;
    uint64_t previous = 0;
    for (const auto& t : profile.kernels) {
        ticks = ticks && t.start && t.end >= t.start && t.start >= previous;
        previous = t.end;
        if (profile.timings_valid) {
            millis = millis && std::isfinite(t.milliseconds) && t.milliseconds >= 0;
            maximum = std::max(maximum, t.milliseconds);
            sum += t.milliseconds;
        } else millis = millis && std::isnan(t.milliseconds);
    }
    EXPECT(ticks && millis);
    if (profile.timings_valid) EXPECT(profile.gpu_tick_nanoseconds > 0 && std::isfinite(profile.sampled_milliseconds) && profile.sampled_milliseconds == sum);
    else EXPECT(std::isnan(profile.gpu_tick_nanoseconds) && std::isnan(profile.sampled_milliseconds));
    return maximum;
}
void test_profile() {
    EXPECT(profile_calibration_valid(1.0, 0.03) && !profile_calibration_valid(1.0, 0.0301) && !profile_calibration_valid(0.0, 0.0) &&
           !profile_calibration_valid(std::numeric_limits<double>::quiet_NaN(), 0.0) && !profile_calibration_valid(1.0, -0.1));
    HipGraph graph("unused", 128u << 20);
    constexpr uint32_t columns = 4096, rows = 2048;
    std::vector<float> matrix(size_t(columns) * rows), x(columns), ones(rows, 1);
    for (size_t i = 0; i < matrix.size(); ++i) matrix[i] = float(int((i * 13 + 5) % 251) - 125) / 32768;
    for (size_t i = 0; i < x.size(); ++i) x[i] = float(int((i * 17 + 3) % 257) - 128) / 128;
    const GpuView weights = graph.upload(bytes_of(matrix), "profile fixture weights"), input = graph.upload(bytes_of(x), "profile fixture input");
    const GpuView gain = graph.upload(bytes_of(ones), "profile fixture gain");
    const GpuView output = graph.zeros(rows * 4, "profile fixture output"), norm = graph.zeros(rows * 4, "profile fixture norm");
    const uint64_t base = graph.memory().live_bytes;
    const auto encode = [&] {
        graph.gemv(0, weights, input, output, columns, rows);
        graph.activate(output, output, Activation::silu);
        graph.multiply(output, gain, output);
        graph.rms(output, gain, norm, 64, 1e-6f);
    };
    graph.begin(); encode(); (void)graph.submit();
    const auto expected = graph.read(norm);
    EXPECT(graph.last_profile().kernels.empty() && graph.last_profile().mode == ProfileMode::disabled);
    const ProfileMode mode = graph.configure_profiling(4096);
    EXPECT(mode == ProfileMode::dispatch_boundary && graph.memory().profile_counter_payload_bytes == 2 * 32768 &&
           graph.memory().live_bytes == base + 65536);
    double maximum = 0, gemv_ms = 0;
    for (uint32_t repeat = 0; repeat < 8; ++repeat) {
        const uint64_t allocations = graph.memory().allocations;
        graph.begin();
        EXPECT(throws_format([&] { (void)graph.last_profile(); }));
        EXPECT(throws_format([&] { (void)graph.configure_profiling(0); }));
        encode();
        const BatchResult batch = graph.submit();
        const GraphProfile& profile = graph.last_profile();
        EXPECT(batch.dispatches == 4 && profile.kernels.size() == 4 && profile.mode == mode);
        EXPECT(graph.memory().allocations == allocations && graph.read(norm) == expected);
        if (profile.kernels.size() == 4) {
            EXPECT(profile.kernels[0].kernel == "graph_quantized_gemv" && profile.kernels[0].encoding == 0 && profile.kernels[0].shape[0] == columns &&
                   profile.kernels[0].shape[1] == rows);
            EXPECT(profile.kernels[1].kernel == "graph_activate" && profile.kernels[2].kernel == "graph_multiply" && profile.kernels[3].kernel == "graph_rms");
            // the raw samples order the operators whether or not the batch calibrated; the 32 MB GEMV is the long one
            EXPECT(profile.kernels[0].end - profile.kernels[0].start > profile.kernels[1].end - profile.kernels[1].start);
            EXPECT(profile.kernels[3].end <= uint64_t(batch.gpu_ms * 1e6) + 1000);
            if (profile.timings_valid) gemv_ms = std::max(gemv_ms, profile.kernels[0].milliseconds);
        }
        maximum = std::max(maximum, checked_timings(profile));
    }
    // a batch long enough to calibrate, and longer than one chunk of 2048 samples
    graph.begin(); encode();
    for (uint32_t i = 0; i < 2050; ++i) graph.activate(norm, norm, Activation::identity);
    const BatchResult crossing = graph.submit();
    EXPECT(crossing.dispatches == 2054 && graph.last_profile().kernels.size() == 2054 && graph.read(norm) == expected);
    EXPECT(graph.last_profile().kernels.size() == 2054 && graph.last_profile().kernels[2048].kernel == "graph_activate");
    maximum = std::max(maximum, checked_timings(graph.last_profile()));
    {
        const GraphProfile& profile = graph.last_profile();
        std::printf("   profile of %zu operators: valid %d, clock mismatch %.4f, sampled %.3f ms of %.3f ms on the GPU; GEMV row %.1f us\n", profile.kernels.size(),
                    int(profile.timings_valid), profile.cpu_clock_mismatch_fraction, profile.sampled_milliseconds, crossing.gpu_ms,
                    double(profile.kernels[0].end - profile.kernels[0].start) / 1e3);
        // the rows tile the batch: their raw spans add up to the GPU's span of it, first boundary to end
        uint64_t span = 0;
        for (const auto& t : profile.kernels) span += t.end - t.start;
        EXPECT(std::fabs(double(span) / 1e6 - crossing.gpu_ms) <= 0.05 * crossing.gpu_ms + 0.05);
    }
    EXPECT(throws_format([&] { (void)graph.configure_profiling(16385); }));
    const auto before = graph.read(output);
    (void)graph.configure_profiling(1);
    graph.begin();
    graph.gemv(0, weights, input, output, columns, rows);
    EXPECT(throws_format([&] { graph.activate(output, output, Activation::silu); }));  // past the capacity: refused, nothing launched
    graph.abort();
    EXPECT(graph.last_profile().kernels.empty());
    (void)before;  // the GEMV of the aborted batch was launched as it was encoded (operators are not deferred here): its output is the same product
    (void)graph.configure_profiling(8);
    const std::vector<float> infinity(rows, std::numeric_limits<float>::infinity());
    const GpuView invalid = graph.upload(bytes_of(infinity), "profile invalid input");
    graph.begin();
    graph.activate(invalid, output, Activation::sigmoid);
    EXPECT(throws_format([&] { (void)graph.submit(); }));
    EXPECT(graph.last_profile().kernels.empty());  // no stale successful profile after a device error
    graph.begin(); encode(); (void)graph.submit();
    EXPECT(graph.read(norm) == expected && graph.last_profile().kernels.size() == 4);
    graph.release(invalid);
    (void)graph.configure_profiling(0);
    EXPECT(graph.memory().live_bytes == base && graph.memory().profile_counter_payload_bytes == 0);
    graph.begin(); encode(); (void)graph.submit();
    EXPECT(graph.last_profile().kernels.empty() && graph.read(norm) == expected);
    HipGraph limited(16384);
    const uint64_t low = limited.memory().live_bytes;
    EXPECT(throws_format([&] { (void)limited.configure_profiling(16384); }));  // 262144 bytes of samples against a 16 KB budget
    EXPECT(limited.memory().live_bytes == low && limited.last_profile().kernels.empty() && limited.memory().profile_counter_payload_bytes == 0);
    std::printf("   maximum sampled operator %.4f ms, F32 GEMV %.4f ms\n", maximum, gemv_ms);
}
}  // namespace

int main() {
    const std::pair<const char*, void (*)()> tests[] = {{"ledger and phases", test_ledger_and_phases},
                                                         {"gemv, route, mixture, top-k", test_gemv_route_mixture_topk},
                                                         {"dense_mm_q8 in both row layouts", test_dense_mm_q8_layouts},
                                                         {"encode_moe single token", test_encode_moe_single_token},
                                                         {"encode_moe_batch", test_encode_moe_batch},
                                                         {"encode_moe_mm_many", test_encode_moe_mm_many},
                                                         {"encode_moe_mm_many, router projection as one f32 GEMM", test_encode_moe_mm_many_router_batch},
                                                         {"router projection: plan, selection, bounds, refusals", test_router_projection_controls},
                                                         {"pack v3: build, adopt, upload a block, encode_moe_mm_many on it", test_pack_v3_block_on_graph},
                                                         {"RMS, activation, residual streams; partial commit", test_residual_streams_and_partial_commit},
                                                         {"encode_moe_mm_many, raw-GGUF arm; prepare twice; Q8_0 registration", test_encode_moe_mm_many_raw_arm},
                                                         {"per-operator profile", test_profile}};
    for (const auto& [name, fn] : tests) {
        std::printf("== %s\n", name);
        std::fflush(stdout);
        try { fn(); } catch (const std::exception& e) { ++failures; std::printf("FAILED: unexpected exception in %s: %s\n", name, e.what()); }
    }
    std::printf("%d checks, %d failures\n", checks, failures);
    return failures ? 1 : 0;
}
