// Host-only tests of the GGUF reader and the tokspur-pack-v3 builder / adopter, on synthetic shards written to a temporary
// directory as the engine's own test does (tests/test_planar_pack_v3.cpp:283-362): plan, build, zero-footer check, adoption with
// several workers, single-block pack, refusal of a tampered pack. No GPU is touched.
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <fcntl.h>
#include <fstream>
#include <functional>
#include <sys/stat.h>
#include <unistd.h>

#include "gguf_writer.hpp"
#include "hip_graph.hpp"
#include "pack_v3.hpp"
#include "tokspur_hip.h"
#include "tokspur_oracle.h"

using namespace tokspur;
using namespace tokspur::planar_v3;
using gguf_writer::TensorSpec;

namespace {
int checks = 0, failures = 0;
void expect(bool ok, const char* what, int line) {
    ++checks;
    if (!ok) { ++failures; std::printf("FAILED line %d: %s\n", line, what); std::fflush(stdout); }
}
#define EXPECT(cond) expect((cond), #cond, __LINE__)
bool refuses(const std::function<void()>& f) {
    try { f(); } catch (const FormatError&) { return true; } catch (...) { return false; }
    return false;
}
std::vector<uint8_t> weights(uint32_t type, uint32_t columns, uint32_t rows, uint32_t experts, uint8_t twist = 0) {
    uint32_t epb = 0, bpb = 0;
    orc_encoding(type, &epb, &bpb);
    std::vector<uint8_t> w(size_t(columns / epb) * bpb * rows * experts);
    orc_fixture_weights(type, columns, rows, experts, w.data(), w.size());
    // distinct quants per tensor, scale fields untouched (they lead each block: 2 bytes for Q8_0, 4 for Q5_1, 16 for the K kinds)
    const uint32_t lead = type == 8 ? 2 : type == 7 ? 4 : 16;
    if (twist) for (size_t at = 0; at < w.size(); at += bpb) for (uint32_t i = lead; i < bpb; ++i) w[at + i] ^= twist;
    return w;
}
std::string sha_of(const uint8_t* p, size_t n) {
    Sha256 h;
    h.add(std::as_bytes(std::span(p, n)));
    return h.finish();
}
std::span<const std::byte> as_bytes(const std::vector<uint8_t>& v) { return std::as_bytes(std::span(v)); }

void test_sha256_known_answers() {  // FIPS 180-4 examples and the million-a vector
    EXPECT(derived_pack::hash("") == "e3b0c44298fc1c149afbf4c8996fb92427ae41e4649b934ca495991b7852b855");
    EXPECT(derived_pack::hash("abc") == "ba7816bf8f01cfea414140de5dae2223b00361a396177a9cb410ff61f20015ad");
    EXPECT(derived_pack::hash("abcdbcdecdefdefgefghfghighijhijkijkljklmklmnlmnomnopnopq") == "248d6a61d20638b8e5c026930c3e6039a33ce45964ff2167f6ecedd419db06c1");
    Sha256 h;
    const std::vector<uint8_t> chunk(977, 'a');  // an odd chunk size exercises the carried partial block
    size_t fed = 0;
    while (fed < 1'000'000) { const size_t n = std::min(chunk.size(), 1'000'000 - fed); h.add(std::as_bytes(std::span(chunk.data(), n))); fed += n; }
    EXPECT(h.finish() == "cdc76e5c9914fb9281a1c7e284d73e67f1809a48a497200e046d39ccc7112cd0");
}

void test_gguf_reader() {
    const std::vector<TensorSpec> specs{{"a.weight", 0, {8}, std::vector<uint8_t>(32, 1)},
                                        {"b.weight", 8, {64, 3}, weights(8, 64, 3, 1)},
                                        {"c.weight", 12, {256, 2, 2}, weights(12, 256, 2, 2)}};
    const auto file = gguf_writer::shard_bytes("qwen35moe", specs);
    const Gguf g(as_bytes(file));
    EXPECT(g.tensors().size() == 3 && g.string_value("general.architecture") == "qwen35moe" && g.unsigned_value("general.alignment") == 32);
    EXPECT(g.data_offset() % 32 == 0 && g.file_size() == file.size());
    for (size_t i = 0; i < specs.size(); ++i) {
        const Tensor& t = g.tensors()[i];
        EXPECT(t.name == specs[i].name && t.type == specs[i].type && t.dimensions == specs[i].dimensions && t.bytes == specs[i].payload.size());
        const auto b = g.tensor_bytes(t);
        EXPECT(b.size() == t.bytes && std::memcmp(b.data(), specs[i].payload.data(), b.size()) == 0 && t.offset % 32 == 0);
    }
    EXPECT(g.tensors()[2].elements == 1024 && g.tensors()[1].bytes == 2 * 34 * 3);
    const Tensor foreign = g.tensors()[0];
    EXPECT(refuses([&] { (void)g.tensor_bytes(foreign); }));  // membership, not just offsets
    EXPECT(refuses([&] { (void)g.unsigned_value("general.architecture"); }) && refuses([&] { (void)g.string_value("general.alignment"); }));
    // refusals of the bounded parser
    auto broken = file;
    broken[0] ^= 1;
    EXPECT(refuses([&] { Gguf bad(as_bytes(broken)); }));  // magic
    broken = file; broken[4] = 2;
    EXPECT(refuses([&] { Gguf bad(as_bytes(broken)); }));  // version
    broken = file; broken.resize(file.size() - 1);
    EXPECT(refuses([&] { Gguf bad(as_bytes(broken)); }));  // truncated tensor data
    broken = file; broken.resize(40);
    EXPECT(refuses([&] { Gguf bad(as_bytes(broken)); }));  // truncated header
    broken = file; broken[8] = 0xff; broken[9] = 0xff; broken[10] = 0xff;
    EXPECT(refuses([&] { Gguf bad(as_bytes(broken)); }));  // record limit
    EXPECT(refuses([&] { Gguf bad(as_bytes(gguf_writer::shard_bytes("x", {{"a", 0, {8}, std::vector<uint8_t>(32)}, {"a", 0, {8}, std::vector<uint8_t>(32)}}))); }));
    EXPECT(refuses([&] { Gguf bad(as_bytes(gguf_writer::shard_bytes("x", {{"a b", 0, {8}, std::vector<uint8_t>(32)}}))); }));       // space in a name
    EXPECT(refuses([&] { Gguf bad(as_bytes(gguf_writer::shard_bytes("x", {{"a", 12, {200}, std::vector<uint8_t>(144)}}))); }));      // row not block-aligned
    EXPECT(refuses([&] { Gguf bad(as_bytes(gguf_writer::shard_bytes("x", {{"a", 99, {8}, std::vector<uint8_t>(32)}}))); }));         // unknown encoding
    EXPECT(refuses([&] { Gguf bad(as_bytes(gguf_writer::shard_bytes("x", {{"a", 0, {8, 1, 1, 1, 1}, std::vector<uint8_t>(32)}}))); }));  // rank 5
    EXPECT(refuses([&] { Gguf bad(as_bytes(gguf_writer::shard_bytes("x", {{"a", 0, {8}, std::vector<uint8_t>(32)}}, 48))); }));      // alignment not a power of two
    {   // two directory entries over the same bytes; an offset off the alignment
        const std::vector<TensorSpec> two{{"a", 0, {16}, std::vector<uint8_t>(64)}, {"b", 0, {16}, std::vector<uint8_t>(64)}};
        const std::vector<uint64_t> overlapping{0, 32}, unaligned{0, 72};
        EXPECT(refuses([&] { Gguf bad(as_bytes(gguf_writer::shard_bytes("x", two, 32, &overlapping))); }));
        EXPECT(refuses([&] { Gguf bad(as_bytes(gguf_writer::shard_bytes("x", two, 32, &unaligned))); }));
    }
}

struct Shards {
    gguf_writer::TempDir dir{"tokspur_pack_v3"};
    std::vector<TensorSpec> source_specs, sidecar_specs;
    std::shared_ptr<const ModelFiles> source, sidecar;
    Shards() {
        std::vector<float> ones(256, 1.0f);
        std::vector<uint8_t> norm(1024);
        std::memcpy(norm.data(), ones.data(), 1024);
        source_specs = {{"blk.0.attn_norm.weight", 0, {256}, norm},
                        {"blk.0.attn_qkv.weight", 8, {512, 64}, weights(8, 512, 64, 1)},
                        {"blk.0.ffn_down_exps.weight", 7, {32, 256, 4}, weights(7, 32, 256, 4)},
                        {"blk.0.ffn_gate_exps.weight", 12, {256, 32, 4}, weights(12, 256, 32, 4)},
                        {"blk.0.ffn_up_exps.weight", 12, {256, 32, 4}, weights(12, 256, 32, 4, 0x5a)},
                        {"blk.2.ffn_down_exps.weight", 8, {32, 256, 4}, weights(8, 32, 256, 4)},
                        {"blk.2.ffn_gate_exps.weight", 13, {256, 32, 4}, weights(13, 256, 32, 4)},
                        {"blk.2.ffn_up_exps.weight", 13, {256, 32, 4}, weights(13, 256, 32, 4, 0x33)}};
        sidecar_specs = {{"blk.48.ffn_down_exps.weight", 8, {32, 256, 4}, weights(8, 32, 256, 4, 0x11)},
                         {"blk.48.ffn_gate_exps.weight", 8, {256, 32, 4}, weights(8, 256, 32, 4, 0x22)},
                         {"blk.48.ffn_up_exps.weight", 8, {256, 32, 4}, weights(8, 256, 32, 4, 0x44)}};
        gguf_writer::write_file(dir.path / "source.gguf", gguf_writer::shard_bytes("qwen35moe", source_specs));
        gguf_writer::write_file(dir.path / "mtp.gguf", gguf_writer::shard_bytes("qwen35moe", sidecar_specs));
        source = std::make_shared<const ModelFiles>(std::vector<std::filesystem::path>{dir.path / "source.gguf"});
        sidecar = std::make_shared<const ModelFiles>(std::vector<std::filesystem::path>{dir.path / "mtp.gguf"});
    }
    const TensorSpec& spec(const std::string& name) const {
        for (const auto& s : source_specs) if (s.name == name) return s;
        for (const auto& s : sidecar_specs) if (s.name == name) return s;
        throw std::runtime_error("no such spec");
    }
};

std::vector<uint8_t> file_bytes(const std::filesystem::path& p) {
    std::ifstream in(p, std::ios::binary);
    return std::vector<uint8_t>(std::istreambuf_iterator<char>(in), {});
}

void test_plan_and_header(const Shards& s) {
    const PackPlanV3 plan = plan_derived_pack_v3(*s.source, s.sidecar.get());
    EXPECT(plan.tensors.size() == 11 && plan.recipe == "tokspur-pack-v3" && plan.version == 3 && plan.alignment == 16384);
    const auto kind_of = [&](const char* name) { for (const auto& t : plan.tensors) if (t.name == name) return t.kind; return PlanarKind(99); };
    EXPECT(kind_of("blk.0.attn_norm.weight") == PlanarKind::plain && kind_of("blk.0.attn_qkv.weight") == PlanarKind::q8_lanes_v1);
    EXPECT(kind_of("blk.0.ffn_down_exps.weight") == PlanarKind::q51_planar_v3 && kind_of("blk.2.ffn_down_exps.weight") == PlanarKind::q8_planar_v3);
    EXPECT(kind_of("blk.0.ffn_gate_exps.weight") == PlanarKind::q4k_coloc_gate_v3 && kind_of("blk.0.ffn_up_exps.weight") == PlanarKind::q4k_coloc_up_v3);
    EXPECT(kind_of("blk.2.ffn_gate_exps.weight") == PlanarKind::q5k_coloc_gate_v3 && kind_of("blk.48.ffn_up_exps.weight") == PlanarKind::q8_coloc_up_v3);
    uint64_t source_total = 0, packed_total = 0;
    for (size_t i = 0; i < plan.tensors.size(); ++i) {
        const auto& t = plan.tensors[i];
        EXPECT(t.offset % 16384 == 0 && t.layout == planar_kind_name(t.kind) && parse_planar_kind(t.layout) == t.kind);
        if (i) EXPECT(t.offset >= plan.tensors[i - 1].offset + plan.tensors[i - 1].bytes && t.offset - (plan.tensors[i - 1].offset + plan.tensors[i - 1].bytes) < 16384);
        if (is_coloc_gate_kind(t.kind)) EXPECT(i + 1 < plan.tensors.size() && plan.tensors[i + 1].name == t.partner_name && plan.tensors[i + 1].partner_name == t.name);
        source_total += t.source_bytes;
        packed_total += t.bytes;
        EXPECT(t.source_bytes == s.spec(t.name).payload.size() && t.source_dimensions == s.spec(t.name).dimensions && t.source_type == s.spec(t.name).type);
    }
    EXPECT(source_total == plan.source_payload_bytes && packed_total == plan.payload_bytes);
    // the K kinds grow by 4 bytes per super-block (12-byte scale fields become 16) and are then listed as plain bytes
    const auto& gate0 = plan.tensors[3];
    EXPECT(gate0.name == "blk.0.ffn_gate_exps.weight" && gate0.type == 24 && gate0.bytes == gate0.source_bytes + 4ull * 32 * 4 &&
           gate0.dimensions == (std::vector<uint64_t>{148, 32, 4}));
    EXPECT(plan.q4k_superblocks == 2ull * 32 * 4 && plan.q5k_superblocks == 2ull * 32 * 4 &&
           plan.original_12b_scale_header_bytes * 4 == plan.expanded_16b_scale_header_bytes * 3);
    const auto& gate48 = plan.tensors[9];
    EXPECT(gate48.name == "blk.48.ffn_gate_exps.weight" && gate48.type == 8 && gate48.bytes == gate48.source_bytes);
    // the header is a GGUF of its own: five metadata keys, the directory, zero padding to the alignment
    const auto header = build_header_v3(plan);
    EXPECT(header.size() == plan.data_offset && header.size() % 16384 == 0 && plan.file_bytes == plan.data_offset + plan.tensors.back().offset + plan.tensors.back().bytes);
    std::vector<std::byte> whole(header);
    whole.resize(size_t(plan.file_bytes));
    const Gguf parsed{std::span<const std::byte>(whole)};
    EXPECT(parsed.metadata().size() == 5 && parsed.string_value("general.architecture") == "tokspur_pack" && parsed.unsigned_value("tokspur_pack.version") == 3 &&
           parsed.data_offset() == header.size() && parsed.tensors().size() == 11);
    const std::string_view manifest = parsed.string_value("tokspur_pack.manifest");
    const std::string_view opening = "{\"schema\":3,\"recipe\":\"tokspur-pack-v3\",\"source_architecture\":\"qwen4exp\",\"target_revision\":\"";
    EXPECT(manifest.substr(0, opening.size()) == opening && manifest.find(' ') == std::string_view::npos);
    EXPECT(manifest.find("\"source_sha256\":\"" + std::string(64, '0') + "\"") != std::string_view::npos);  // no digests before the build
    const PackPlanV3 block = plan_block_pack_v3(*s.source, s.sidecar.get(), 0);
    EXPECT(block.tensors.size() == 5 && block.recipe == "tokspur-pack-v3-block-0");
    EXPECT(refuses([&] { (void)plan_block_pack_v3(*s.source, s.sidecar.get(), 7); }));            // nothing selected
    EXPECT(refuses([&] { (void)plan_derived_pack_v3(*s.source, s.sidecar.get(), 1000); }));       // byte budget
}

void test_build_adopt_tamper(const Shards& s) {
    const auto pack_path = s.dir.path / "tokspur-pack-v3-synth.asa.gguf", block_path = s.dir.path / "tokspur-pack-v3-blk0.asa.gguf";
    const PackPlanV3 built = build_derived_pack_v3(s.source, s.sidecar, pack_path, 2, 1 << 20);
    EXPECT(built.tensors.size() == 11);
    const auto& last = built.tensors.back();
    EXPECT(built.file_bytes == built.data_offset + last.offset + last.bytes && std::filesystem::file_size(pack_path) == built.file_bytes);  // no footer
    struct stat info{};
    EXPECT(::stat(pack_path.c_str(), &info) == 0 && (info.st_mode & 0222) == 0);
    const auto on_disk = file_bytes(pack_path);
    const auto header = build_header_v3(built);
    EXPECT(on_disk.size() == built.file_bytes && std::memcmp(on_disk.data(), header.data(), header.size()) == 0);
    // digests and planes against independent computations
    for (size_t i = 0; i < built.tensors.size(); ++i) {
        const auto& t = built.tensors[i];
        const auto& src = s.spec(t.name).payload;
        const uint8_t* packed = on_disk.data() + built.data_offset + t.offset;
        EXPECT(t.source_sha256 == sha_of(src.data(), src.size()) && t.packed_sha256 == sha_of(packed, t.bytes));
        if (t.kind == PlanarKind::plain) EXPECT(std::memcmp(packed, src.data(), src.size()) == 0);
        if (t.kind == PlanarKind::q8_lanes_v1) {
            std::vector<uint8_t> want(src.size());
            EXPECT(tsp_q8_lanes_pack_rows(uint32_t(t.source_dimensions[0]), src.data(), want.data(), src.size()) == TSP_OK && std::memcmp(packed, want.data(), want.size()) == 0);
        }
        if (is_coloc_gate_kind(t.kind) || is_coloc_up_kind(t.kind)) {
            const bool hi = is_coloc_up_kind(t.kind);
            const auto& gate = s.spec(hi ? t.partner_name : t.name).payload;
            const auto& up = s.spec(hi ? t.name : t.partner_name).payload;
            tsp_planar_spec spec{};
            EXPECT(tsp_make_expert_spec(t.source_type, uint32_t(t.source_dimensions[0]), uint32_t(t.source_dimensions[1]), &spec) == TSP_OK);
            std::vector<uint8_t> want(t.bytes);
            EXPECT(tsp_pack_coloc_half(&spec, gate.data(), up.data(), uint32_t(t.source_dimensions[2]), hi, want.data(), want.size()) == TSP_OK &&
                   std::memcmp(packed, want.data(), want.size()) == 0);
        }
        if (i + 1 < built.tensors.size())
            for (uint64_t at = t.offset + t.bytes; at < built.tensors[i + 1].offset; ++at) EXPECT(on_disk[built.data_offset + at] == 0);
    }
    const AdoptedPackV3 adopted = adopt_derived_pack_v3(s.source, s.sidecar, pack_path, 2, derived_pack::default_chunk_bytes, 4);
    EXPECT(adopted.authentication_workers == 4 && adopted.plan.tensors.size() == 11 && adopted.model->architecture() == "tokspur_pack");
    EXPECT(adopted.manifest_sha256 == derived_pack::hash(adopted.model->shards()[0].string_value("tokspur_pack.manifest")));
    EXPECT(adopted.plan.tensors[3].packed_sha256 == built.tensors[3].packed_sha256);
    EXPECT(refuses([&] { (void)build_derived_pack_v3(s.source, s.sidecar, pack_path, 2, 1 << 20); }));  // never replaces a file
    EXPECT(refuses([&] { (void)build_derived_pack_v3(s.source, s.sidecar, s.dir.path / "other.gguf", 0, 1 << 20); }));
    EXPECT(refuses([&] { (void)build_derived_pack_v3(s.source, s.sidecar, s.dir.path / "other.gguf", 2, ~0ull >> 1); }));  // reserve cannot be met
    EXPECT(!std::filesystem::exists(s.dir.path / "other.gguf"));
    size_t leftovers = 0;
    for (const auto& e : std::filesystem::directory_iterator(s.dir.path)) leftovers += e.path().filename().string().rfind(".tokspur-pack-v3.", 0) == 0;
    EXPECT(leftovers == 0);  // refused builds leave no temporary behind
    // without the sidecar the plan has three tensors fewer: this pack is not its pack
    EXPECT(refuses([&] { (void)adopt_derived_pack_v3(s.source, nullptr, pack_path, 2); }));

    const PackPlanV3 block = build_block_pack_v3(s.source, s.sidecar, 0, block_path, 2, 1 << 20);
    EXPECT(block.tensors.size() == 5);
    EXPECT(adopt_block_pack_v3(s.source, s.sidecar, 0, block_path, 2, derived_pack::default_chunk_bytes, 2).plan.tensors.size() == 5);
    EXPECT(refuses([&] { (void)adopt_block_pack_v3(s.source, s.sidecar, 2, block_path, 2); }));  // another block's plan
    // a writable pack is refused; so is one payload bit flipped, and one padding byte set
    ::chmod(block_path.c_str(), 0600);
    EXPECT(refuses([&] { (void)adopt_block_pack_v3(s.source, s.sidecar, 0, block_path, 2); }));
    const auto flip = [&](uint64_t at) {
        ::chmod(block_path.c_str(), 0600);
        const int fd = ::open(block_path.c_str(), O_RDWR | O_CLOEXEC);
        uint8_t b = 0;
        EXPECT(fd >= 0 && ::pread(fd, &b, 1, off_t(at)) == 1);
        b ^= 1;
        EXPECT(::pwrite(fd, &b, 1, off_t(at)) == 1);
        ::close(fd);
        ::chmod(block_path.c_str(), 0400);
    };
    ::chmod(block_path.c_str(), 0400);
    EXPECT(adopt_block_pack_v3(s.source, s.sidecar, 0, block_path, 2).plan.tensors.size() == 5);
    flip(block.data_offset);
    EXPECT(refuses([&] { (void)adopt_block_pack_v3(s.source, s.sidecar, 0, block_path, 2, derived_pack::default_chunk_bytes, 2); }));
    flip(block.data_offset);
    EXPECT(adopt_block_pack_v3(s.source, s.sidecar, 0, block_path, 2).plan.tensors.size() == 5);
    const uint64_t pad = block.data_offset + block.tensors[0].offset + block.tensors[0].bytes;  // 1 KiB tensor, 15 KiB of zeros after it
    flip(pad);
    EXPECT(refuses([&] { (void)adopt_block_pack_v3(s.source, s.sidecar, 0, block_path, 2); }));
    flip(pad);
    flip(100);  // inside the manifest text
    EXPECT(refuses([&] { (void)adopt_block_pack_v3(s.source, s.sidecar, 0, block_path, 2); }));
    flip(100);
    // a source that differs in one weight byte: the pack is stale
    auto changed = s.source_specs;
    changed[3].payload[200] ^= 4;
    gguf_writer::write_file(s.dir.path / "changed.gguf", gguf_writer::shard_bytes("qwen35moe", changed));
    const auto other = std::make_shared<const ModelFiles>(std::vector<std::filesystem::path>{s.dir.path / "changed.gguf"});
    EXPECT(refuses([&] { (void)adopt_block_pack_v3(other, s.sidecar, 0, block_path, 2); }));
    EXPECT(adopt_block_pack_v3(s.source, s.sidecar, 0, block_path, 2).plan.tensors.size() == 5);
    // a pack cannot be packed again
    EXPECT(refuses([&] { (void)plan_derived_pack_v3(*adopted.model); }));
}
// include/tokspur/grouped_mm.hpp:22-26: the C++ planners, against the restated ones (themselves bit-equal to the compiled
// reference) on the engine's shapes and on every encoding / layout pair, and the engine's refusals
// native/tests/test_planar_pack_v3.cpp:324-327 and native/tests/test_derived_pack.cpp:390-401: the budget report of a plan, and a
// build interrupted through its cancellation hook, which must leave the directory as it found it.
int g_chunks_before_cancel = 0;
void cancel_after_some_chunks() {
    if (g_chunks_before_cancel-- == 0) throw FormatError("interrupted test build");
}
void test_budget_and_cancellation(const Shards& s) {
    const BudgetReportV3 budget = measure_pack_v3_budget(*s.source, s.sidecar.get(), s.dir.path, {}, 2, 1 << 20);
    const PackPlanV3 plan = plan_derived_pack_v3(*s.source, s.sidecar.get());
    EXPECT(budget.ram_ceiling_satisfied && budget.reserve_satisfied);
    EXPECT(budget.original_12b_scale_header_bytes * 4 == budget.expanded_16b_scale_header_bytes * 3 && budget.expanded_16b_scale_header_bytes > 0);
    EXPECT(budget.planned_pack_v3_file_bytes == plan.file_bytes && budget.planned_pack_v3_payload_bytes == plan.payload_bytes);
    EXPECT(budget.required_reserve_bytes == (1 << 20) && budget.existing_pack_v2_file_bytes == 0);
    EXPECT(budget.free_after_pack_v3_bytes + plan.file_bytes == budget.filesystem_available_bytes);
    // the families add up to the planar tensors of the plan, each counted once
    uint64_t planar = 0, biggest_chunk = 0;
    for (const auto& t : plan.tensors) {
        if (!is_planar_v3_kind(t.kind)) continue;
        planar += t.bytes;
        tsp_planar_spec spec{};
        EXPECT(tsp_make_expert_spec(t.source_type, uint32_t(t.source_dimensions[0]), uint32_t(t.source_dimensions[1]), &spec) == TSP_OK);
        biggest_chunk = std::max<uint64_t>(biggest_chunk, (spec.planar_expert_bytes + 2 * spec.source_expert_bytes) * 2 * (is_coloc_gate_kind(t.kind) ? 2 : 1));
    }
    EXPECT(planar > 0 && budget.q4k_planar_bytes + budget.q5k_planar_bytes + budget.q51_planar_bytes + budget.q8_planar_moe_bytes == planar);
    EXPECT(budget.streaming_ring_buffer_bytes == std::max<uint64_t>(biggest_chunk, 2 * derived_pack::default_chunk_bytes));
    // a block plan with the smallest chunk: the buffers of the plain and lane tensors still count (two chunks)
    const PackPlanV3 block = plan_block_pack_v3(*s.source, s.sidecar.get(), 0);
    const auto existing = s.dir.path / "older-pack.bin";
    { std::ofstream(existing, std::ios::binary) << std::string(777, 'x'); }
    const BudgetReportV3 small = measure_pack_v3_budget(block, s.dir.path, existing, 2, 0, 32768);
    EXPECT(small.planned_pack_v3_file_bytes == block.file_bytes && small.streaming_ring_buffer_bytes >= 65536 && small.existing_pack_v2_file_bytes == 777);
    EXPECT(measure_pack_v3_budget(block, s.dir.path, s.dir.path, 2, 0, 32768).existing_pack_v2_file_bytes == 0);  // a directory is no pack
    EXPECT(!measure_pack_v3_budget(block, s.dir.path, {}, 2, ~0ull >> 1, 32768).reserve_satisfied);
    EXPECT(refuses([&] { (void)measure_pack_v3_budget(block, s.dir.path, {}, 0, 0, 32768); }));
    EXPECT(refuses([&] { (void)measure_pack_v3_budget(block, s.dir.path, {}, 65, 0, 32768); }));
    EXPECT(refuses([&] { (void)measure_pack_v3_budget(block, s.dir.path, {}, 2, 0, 32767); }));
    EXPECT(refuses([&] { (void)measure_pack_v3_budget(block, s.dir.path / "no-such-directory", {}, 2, 0, 32768); }));
    std::filesystem::remove(existing);

    // cancellation at the first chunk, in the middle and just before publication: refused, nothing left behind, and the
    // same build goes through afterwards
    const auto entries = [&] { size_t n = 0; for (const auto& e : std::filesystem::directory_iterator(s.dir.path)) { (void)e; ++n; } return n; };
    const size_t before = entries();
    const auto output = s.dir.path / "cancelled.asa.gguf";
    int chunks = 0;
    g_chunks_before_cancel = 1 << 30;
    {   // count the hook's calls on a build that completes
        (void)build_block_pack_v3(s.source, s.sidecar, 0, output, 2, 0, 32768, cancel_after_some_chunks);
        chunks = (1 << 30) - g_chunks_before_cancel;
        EXPECT(chunks >= 3 && std::filesystem::exists(output));
        EXPECT(::chmod(output.c_str(), 0600) == 0 && std::filesystem::remove(output));
    }
    for (const int at : {0, chunks / 2, chunks - 1}) {
        g_chunks_before_cancel = at;
        bool interrupted = false;
        try { (void)build_block_pack_v3(s.source, s.sidecar, 0, output, 2, 0, 32768, cancel_after_some_chunks); }
        catch (const FormatError& e) { interrupted = std::string(e.what()).find("interrupted test build") != std::string::npos; }
        EXPECT(interrupted && !std::filesystem::exists(output) && entries() == before);
    }
    g_chunks_before_cancel = 1 << 30;
    const PackPlanV3 rebuilt = build_block_pack_v3(s.source, s.sidecar, 0, output, 2, 0, 32768, cancel_after_some_chunks);
    EXPECT(rebuilt.file_bytes == block.file_bytes && std::filesystem::file_size(output) == block.file_bytes);
    EXPECT(::chmod(output.c_str(), 0600) == 0 && std::filesystem::remove(output) && entries() == before);
}

void test_grouped_mm_planners() {
    static_assert(sizeof(GroupedMmArgs) == 56);
    const auto same = [](const GroupedMmPlan& a, const orc_grouped_mm_plan& b) {
        return std::memcmp(&a.args, &b.args, 56) == 0 && a.matrix_bytes == b.matrix_bytes && a.indices_bytes == b.indices_bytes &&
               a.input_bytes == b.input_bytes && a.output_bytes == b.output_bytes && a.token_map_bytes == b.token_map_bytes &&
               a.counts_bytes == b.counts_bytes && a.tasks_bytes == b.tasks_bytes && a.grid_x == b.grid_x && a.grid_y == b.grid_y;
    };
    const std::pair<uint32_t, PrefillWeightLayout> pairs[] = {{7, PrefillWeightLayout::gguf}, {8, PrefillWeightLayout::gguf}, {12, PrefillWeightLayout::gguf},
                                                              {13, PrefillWeightLayout::gguf}, {8, PrefillWeightLayout::q8_lanes_v1}};
    for (const auto& [type, layout] : pairs)
        for (const uint32_t tokens : {1u, 31u, 32u, 33u, 512u, 2048u})
            for (const bool broadcast : {false, true}) {
                const bool big = tokens > 512;
                const uint32_t experts = layout == PrefillWeightLayout::q8_lanes_v1 && !big ? 1 : 64, selected = experts == 1 ? 1 : 10;
                orc_grouped_mm_plan want{};
                EXPECT(orc_grouped_mm_plan_make(type, uint32_t(layout), 2560, 640, experts, selected, tokens, 10240, 2560, broadcast, big, &want) == 0);
                const auto got = grouped_mm_plan(type, layout, 2560, 640, experts, selected, tokens, 10240, 2560, broadcast, big);
                EXPECT(same(got, want) && std::string(got.kernel) == "graph_grouped_mm" && got.threads == 128 && got.threadgroup_bytes == 8192);
            }
    {   // the engine's Q5_1 lane geometry: 640 columns, more than one expert
        orc_grouped_mm_plan want{};
        EXPECT(orc_grouped_mm_plan_make(7, 2, 640, 2560, 512, 10, 512, 2560, 10240, 0, 0, &want) == 0);
        EXPECT(same(grouped_mm_plan(7, PrefillWeightLayout::q51_lanes_v1, 640, 2560, 512, 10, 512, 2560, 10240, false), want));
        EXPECT(refuses([] { (void)grouped_mm_plan(7, PrefillWeightLayout::q51_lanes_v1, 672, 2560, 512, 10, 512, 2688, 10240, false); }));
    }
    // config 1's dense product as the engine would plan it (experts = 1, selected = 1, broadcast)
    const auto c1 = grouped_mm_plan(12, PrefillWeightLayout::gguf, 2048, 8192, 1, 1, 512, 8192, 32768, true);
    EXPECT(c1.args.row_bytes == 1152 && c1.matrix_bytes == 9437184 && c1.grid_x == 128 && c1.grid_y == 17 && c1.args.maximum_tasks == 17);
    const auto d = dense_mm_q8_plan(PrefillWeightLayout::gguf, 2048, 4096, 100, 8192, 16384);
    EXPECT(d.indices_bytes == 0 && d.token_map_bytes == 0 && d.counts_bytes == 0 && d.tasks_bytes == 0 && d.args.maximum_tasks == 4 && d.grid_y == 4 &&
           d.args.row_bytes == 2176 && std::string(d.kernel) == "graph_dense_mm_q8");
    EXPECT(std::string(grouped_mm_kernel(13, PrefillWeightLayout::gguf)) == "graph_grouped_mm");
    EXPECT(std::string(dense_mm_q8_kernel(PrefillWeightLayout::q8_lanes_v1)) == "graph_dense_mm_q8");
    EXPECT(refuses([] { (void)grouped_mm_kernel(14, PrefillWeightLayout::gguf); }));                 // encoding
    EXPECT(refuses([] { (void)grouped_mm_kernel(12, PrefillWeightLayout::q8_lanes_v1); }));          // layout / encoding
    EXPECT(refuses([] { (void)dense_mm_q8_kernel(PrefillWeightLayout::q51_lanes_v1); }));
    EXPECT(refuses([] { (void)grouped_mm_plan(12, PrefillWeightLayout::gguf, 2048, 512, 512, 10, 513, 8192, 2048, true); }));        // rows beyond 512 need allow_nax_2k
    EXPECT(refuses([] { (void)grouped_mm_plan(12, PrefillWeightLayout::gguf, 2048, 512, 512, 10, 2049, 8192, 2048, true, true); }));
    EXPECT(refuses([] { (void)grouped_mm_plan(12, PrefillWeightLayout::gguf, 2000, 512, 512, 10, 8, 8192, 2048, true); }));          // whole blocks
    EXPECT(refuses([] { (void)grouped_mm_plan(12, PrefillWeightLayout::gguf, 2048, 512, 513, 10, 8, 8192, 2048, true); }));
    EXPECT(refuses([] { (void)grouped_mm_plan(12, PrefillWeightLayout::gguf, 2048, 512, 8, 10, 8, 8192, 2048, true); }));            // selected beyond experts
    EXPECT(refuses([] { (void)grouped_mm_plan(12, PrefillWeightLayout::gguf, 2048, 512, 512, 10, 8, 8188, 2048, true); }));          // stride below a row / not in 16s
    EXPECT(refuses([] { (void)grouped_mm_plan(12, PrefillWeightLayout::gguf, 2048, 512, 512, 10, 8, 8192, 2040, true); }));
    EXPECT(refuses([] { (void)dense_mm_q8_plan(PrefillWeightLayout::q8_lanes_v1, 544, 64, 8, 2176, 256); }));                        // lanes: 256s or under 512
}
}  // namespace

int main() {
    std::srand(unsigned(::getpid()));
    const std::pair<const char*, std::function<void()>> tests[] = {
        {"SHA-256 known answers", test_sha256_known_answers},
        {"GGUF reader", test_gguf_reader},
        {"grouped_mm_plan / dense_mm_q8_plan", test_grouped_mm_planners},
        {"pack v3: plan, header, build, adoption, tamper", [] { const Shards s; test_plan_and_header(s); test_build_adopt_tamper(s); }},
        {"pack v3: budget report, cancelled build", [] { const Shards s; test_budget_and_cancellation(s); }}};
    for (const auto& [name, fn] : tests) {
        std::printf("== %s\n", name);
        std::fflush(stdout);
        try { fn(); } catch (const std::exception& e) { ++failures; std::printf("FAILED: unexpected exception in %s: %s\n", name, e.what()); }
    }
    std::printf("%d checks, %d failures\n", checks, failures);
    return failures ? 1 : 0;
}
