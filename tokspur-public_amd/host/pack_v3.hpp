// Weight files for the MoE path: a bounded GGUF v3 reader, and the builder / adopter of the lossless planar
// weight pack "tokspur-pack-v3" (a GGUF container whose tensors are the Pack v3 planes the kernels read).
//
// Interfaces follow the engine's (include/tokspur/gguf.hpp:21-167, include/tokspur/derived_pack.hpp:18-30,
// include/tokspur/planar_pack_v3.hpp:27-248): same type and function names, argument meaning and refusals, so that a pack
// written by either side is adopted by the other: the header (metadata keys, compact manifest JSON in insertion order,
// tensor directory, zero padding to 16 KiB) is rebuilt from the plan and compared byte for byte on adoption.
//
// Left out on purpose: the engine's disk-budget report, the local-seal fast start (every adoption here authenticates in
// full), cancellation hooks, and the census of its one 1254-tensor model with the trailing blk.48 tensors that may
// exist only in the pack.
#pragma once

#include "hip_graph.hpp"

#include <filesystem>
#include <map>
#include <string_view>

namespace tokspur {

uint64_t checked_add(uint64_t a, uint64_t b);
uint64_t checked_mul(uint64_t a, uint64_t b);

// include/tokspur/gguf.hpp:22-28; block sizes as encoded in the file (src/gguf.cpp:21-32)
struct Encoding {
    uint32_t id;
    const char* name;
    uint32_t elements_per_block;
    uint32_t bytes_per_block;
};
const Encoding& encoding(uint32_t id);

// A read-only private mapping of one regular file; nothing is prefetched. include/tokspur/gguf.hpp:36-69
class MappedFile {
public:
    explicit MappedFile(const std::filesystem::path& path);
    ~MappedFile();
    MappedFile(const MappedFile&) = delete;
    MappedFile& operator=(const MappedFile&) = delete;
    MappedFile(MappedFile&& other) noexcept;
    [[nodiscard]] std::span<const std::byte> bytes() const noexcept { return {data_, size_t(size_)}; }
    [[nodiscard]] uint64_t size() const noexcept { return size_; }
    [[nodiscard]] const std::filesystem::path& path() const noexcept { return path_; }
    void assert_unchanged() const;  // size, device, inode, mtime and ctime as they were when mapped

private:
    std::filesystem::path path_;
    int fd_ = -1;
    const std::byte* data_ = nullptr;
    uint64_t size_ = 0, device_ = 0, inode_ = 0;
    int64_t mtime_[2] = {0, 0}, ctime_[2] = {0, 0};
};

// include/tokspur/gguf.hpp:71-86
struct Metadata {
    uint32_t type = 0;
    uint64_t offset = 0, end = 0;
    uint32_t element_type = 0;
    uint64_t elements = 0;
};
struct Tensor {
    std::string name;
    std::vector<uint64_t> dimensions;  // on-disk order: the first dimension is contiguous
    uint32_t type = 0;
    uint64_t offset = 0;  // absolute file offset
    uint64_t bytes = 0, elements = 0;
};

// include/tokspur/gguf.hpp:88-137, parser src/gguf.cpp:356-420: little-endian GGUF v3, at most 100 000 records, header
// within 256 MiB, keys [a-z0-9_.], ASCII tensor names of at most 64 bytes, rank 1..4, block-aligned rows, offsets aligned
// to general.alignment (power of two up to 65536, 32 when absent), no truncated or overlapping tensor data.
class Gguf {
public:
    explicit Gguf(const std::filesystem::path& path);
    explicit Gguf(std::span<const std::byte> bytes);  // borrowed: the caller keeps them alive
    Gguf(const Gguf&) = delete;
    Gguf& operator=(const Gguf&) = delete;
    Gguf(Gguf&&) = default;
    [[nodiscard]] const std::vector<Tensor>& tensors() const { return tensors_; }
    [[nodiscard]] const std::map<std::string, Metadata, std::less<>>& metadata() const { return metadata_; }
    [[nodiscard]] const Metadata* find(std::string_view key) const;
    [[nodiscard]] uint64_t unsigned_value(std::string_view key) const;
    [[nodiscard]] std::string_view string_value(std::string_view key) const;
    [[nodiscard]] std::span<const std::byte> tensor_bytes(const Tensor& tensor) const;
    [[nodiscard]] uint64_t data_offset() const noexcept { return data_offset_; }
    [[nodiscard]] uint64_t file_size() const noexcept { return data_.size(); }
    void assert_unchanged() const;

private:
    void parse();
    std::vector<MappedFile> mapping_;  // zero or one
    std::span<const std::byte> data_;
    std::map<std::string, Metadata, std::less<>> metadata_;
    std::vector<Tensor> tensors_;
    uint64_t data_offset_ = 0;
};

// include/tokspur/gguf.hpp:139-167: one model as 1..1024 shards, tensor names unique across them
class ModelFiles {
public:
    explicit ModelFiles(const std::vector<std::filesystem::path>& paths);
    [[nodiscard]] const std::vector<Gguf>& shards() const { return shards_; }
    [[nodiscard]] const std::map<std::string, std::pair<size_t, size_t>, std::less<>>& tensors() const { return tensors_; }
    [[nodiscard]] bool contains(std::string_view name) const { return tensors_.find(name) != tensors_.end(); }
    [[nodiscard]] const Tensor& tensor(std::string_view name) const;
    [[nodiscard]] std::span<const std::byte> tensor_bytes(std::string_view name) const;
    [[nodiscard]] std::string_view architecture() const { return architecture_; }
    void assert_unchanged() const;

private:
    std::vector<Gguf> shards_;
    std::map<std::string, std::pair<size_t, size_t>, std::less<>> tensors_;  // name -> (shard, index)
    std::string architecture_;
};

// FIPS 180-4 SHA-256, streaming; finish() gives 64 lower-case hex digits
class Sha256 {
public:
    Sha256();
    void add(std::span<const std::byte> data);
    [[nodiscard]] std::string finish();

private:
    void block(const uint8_t* p);
    uint32_t h_[8];
    uint8_t tail_[64];
    uint64_t bytes_ = 0;
};

namespace derived_pack {  // include/tokspur/derived_pack.hpp:18-30
inline constexpr uint64_t pack_alignment = 16384;
inline constexpr const char* pack_architecture = "tokspur_pack";
inline constexpr const char* source_architecture = "qwen4exp";
inline constexpr const char* target_revision = "766911a6b7369840a91dbcd95f9f997acaab6cd6";
inline constexpr const char* mtp_sidecar_sha256 = "5ff54097406a905cf3a724c709124ceb0e3e10235ee862298969e91c96fa96e6";
inline constexpr uint64_t default_reserve_bytes = 50ull << 30;
inline constexpr uint64_t default_chunk_bytes = 4'194'304;
inline constexpr uint32_t max_authentication_workers = 16;
inline constexpr uint64_t max_pack_bytes = 128'000'000'000ull;
[[nodiscard]] std::string hash(std::string_view text);  // SHA-256 hex of the text
[[nodiscard]] inline constexpr bool is_cpu_pinned_embedding(std::string_view name) noexcept {
    return name == "token_embd.weight" || name == "per_layer_token_embd.weight" || name == "per_layer_token_embd";
}
[[nodiscard]] inline bool is_gpu_pack_tensor(std::string_view name) { return !is_cpu_pinned_embedding(name); }
[[nodiscard]] bool check_disk_reserve(uint64_t available_bytes, uint64_t peak_additional_bytes, uint64_t reserve_bytes = default_reserve_bytes);
enum class TrustMode { full, local_seal };  // local_seal is accepted and authenticates in full
}  // namespace derived_pack

namespace planar_v3 {

inline constexpr uint32_t pack_version_v3 = 3;
inline constexpr const char* pack_recipe_v3 = "tokspur-pack-v3";
inline constexpr const char* block_recipe_prefix_v3 = "tokspur-pack-v3-block-";

// include/tokspur/planar_pack_v3.hpp:29-40
enum class PlanarKind : uint32_t {
    plain = 0, q8_lanes_v1 = 1, q4k_coloc_gate_v3 = 2, q4k_coloc_up_v3 = 3, q5k_coloc_gate_v3 = 4, q5k_coloc_up_v3 = 5,
    q8_coloc_gate_v3 = 6, q8_coloc_up_v3 = 7, q51_planar_v3 = 8, q8_planar_v3 = 9,
};
[[nodiscard]] const char* planar_kind_name(PlanarKind kind);
[[nodiscard]] PlanarKind parse_planar_kind(std::string_view name);
[[nodiscard]] bool is_planar_v3_kind(PlanarKind kind) noexcept;
[[nodiscard]] bool is_coloc_gate_kind(PlanarKind kind) noexcept;
[[nodiscard]] bool is_coloc_up_kind(PlanarKind kind) noexcept;

// include/tokspur/planar_pack_v3.hpp:86-115
struct PackTensorV3 {
    std::string name;
    uint32_t type = 0;         // directory type: 24 (I8) when the packed bytes differ in count from the source, else source_type
    uint32_t source_type = 0;
    PlanarKind kind = PlanarKind::plain;
    std::string layout = "plain";
    std::vector<uint64_t> dimensions;         // directory dimensions
    std::vector<uint64_t> source_dimensions;  // the source tensor's
    uint64_t source_bytes = 0, bytes = 0;
    uint64_t offset = 0;  // relative to data_offset, 16 KiB aligned
    std::string partner_name;  // the other tensor of a co-located gate / up pair
    std::string source_sha256, packed_sha256;
};
struct PackPlanV3 {
    std::vector<PackTensorV3> tensors;
    uint64_t source_payload_bytes = 0, payload_bytes = 0, file_bytes = 0, data_offset = 0;
    uint64_t q4k_superblocks = 0, q5k_superblocks = 0;
    uint64_t original_12b_scale_header_bytes = 0, expanded_16b_scale_header_bytes = 0;
    std::string recipe = pack_recipe_v3;
    uint32_t version = pack_version_v3;
    uint32_t alignment = uint32_t(derived_pack::pack_alignment);
};
struct AdoptedPackV3 {
    std::shared_ptr<const ModelFiles> model;  // the pack itself, mapped
    PackPlanV3 plan;
    std::string manifest_sha256;
    uint32_t authentication_workers = 1;
};

[[nodiscard]] std::vector<std::byte> build_header_v3(const PackPlanV3& plan);  // src/planar_pack_v3.cpp:898-920

// include/tokspur/planar_pack_v3.hpp:108-125: what building a plan would cost, before a byte is written
struct BudgetReportV3 {
    uint64_t filesystem_available_bytes = 0;
    uint64_t existing_pack_v2_file_bytes = 0;  // size of a regular file at the given path, 0 if there is none
    uint64_t planned_pack_v3_payload_bytes = 0;
    uint64_t planned_pack_v3_file_bytes = 0;
    uint64_t free_after_pack_v3_bytes = 0;
    uint64_t required_reserve_bytes = derived_pack::default_reserve_bytes;
    uint64_t streaming_ring_buffer_bytes = 0;  // the largest packed + read-back + restored buffers a chunk needs
    uint64_t streaming_ram_ceiling_bytes = 4'000'000'000ull;
    uint64_t q4k_planar_bytes = 0, q5k_planar_bytes = 0, q51_planar_bytes = 0, q8_planar_moe_bytes = 0;
    uint64_t original_12b_scale_header_bytes = 0, expanded_16b_scale_header_bytes = 0;
    bool reserve_satisfied = false;
    bool ram_ceiling_satisfied = false;
};

// src/planar_pack_v3.cpp:394-499: every GPU tensor of the source (and of the optional sidecar), in name order; a
// *.ffn_gate_exps.weight is emitted together with its *.ffn_up_exps.weight as a co-located pair when both are eligible,
// *.ffn_down_exps.weight in Q5_1 / Q8_0 as planes, dense Q8_0 matrices in q8_lanes_v1 rows, everything else as it is.
[[nodiscard]] PackPlanV3 plan_derived_pack_v3(const ModelFiles& source, const ModelFiles* mtp_sidecar = nullptr,
                                              uint64_t byte_budget = derived_pack::max_pack_bytes);
[[nodiscard]] PackPlanV3 plan_block_pack_v3(const ModelFiles& source, const ModelFiles* mtp_sidecar, uint32_t block_id,
                                            uint64_t byte_budget = 4'000'000'000ull);

// src/planar_pack_v3.cpp:931-1000: free space of the output directory against the plan's file size plus the reserve,
// planar bytes per family, and the host buffers one streaming chunk needs against the RAM ceiling. Writes nothing.
[[nodiscard]] BudgetReportV3 measure_pack_v3_budget(const PackPlanV3& plan, const std::filesystem::path& output_directory,
                                                    const std::filesystem::path& existing_pack_v2_path, uint32_t experts_per_chunk,
                                                    uint64_t reserve_bytes, uint64_t chunk_bytes);
[[nodiscard]] BudgetReportV3 measure_pack_v3_budget(const ModelFiles& source, const ModelFiles* mtp_sidecar,
                                                    const std::filesystem::path& output_directory,
                                                    const std::filesystem::path& existing_pack_v2_path = {}, uint32_t experts_per_chunk = 8,
                                                    uint64_t reserve_bytes = derived_pack::default_reserve_bytes);

// src/planar_pack_v3.cpp:1002-1237: streams the plan into a temporary beside `output`, reads every chunk back and proves the
// byte-exact inverse against the source before hashing it, writes the final header (now with digests), makes the file
// read-only and publishes it under `output` without replacing anything. Returns the plan with digests.
// `check_cancelled` (src/planar_pack_v3.cpp:1010,1080-1229), when given, is called before every chunk is written and once
// more before publication; it cancels by throwing, and whatever it throws leaves the directory as it was found.
[[nodiscard]] PackPlanV3 build_pack_v3_from_plan(PackPlanV3 plan, std::shared_ptr<const ModelFiles> source,
                                                 std::shared_ptr<const ModelFiles> mtp_sidecar, const std::filesystem::path& output,
                                                 uint32_t experts_per_chunk = 8, uint64_t reserve_bytes = derived_pack::default_reserve_bytes,
                                                 uint64_t chunk_bytes = derived_pack::default_chunk_bytes, void (*check_cancelled)() = nullptr);
[[nodiscard]] PackPlanV3 build_derived_pack_v3(std::shared_ptr<const ModelFiles> source, std::shared_ptr<const ModelFiles> mtp_sidecar,
                                               const std::filesystem::path& output, uint32_t experts_per_chunk = 8,
                                               uint64_t reserve_bytes = derived_pack::default_reserve_bytes,
                                               uint64_t chunk_bytes = derived_pack::default_chunk_bytes, void (*check_cancelled)() = nullptr);
[[nodiscard]] PackPlanV3 build_block_pack_v3(std::shared_ptr<const ModelFiles> source, std::shared_ptr<const ModelFiles> mtp_sidecar,
                                             uint32_t block_id, const std::filesystem::path& output, uint32_t experts_per_chunk = 8,
                                             uint64_t reserve_bytes = derived_pack::default_reserve_bytes,
                                             uint64_t chunk_bytes = derived_pack::default_chunk_bytes, void (*check_cancelled)() = nullptr);

// src/planar_pack_v3.cpp:1268-1643: the file must be a read-only regular file with one link and exactly the planned size;
// its header must equal the canonical header of the plan (with the manifest's digests); every tensor is unpacked and
// compared with the source byte for byte, both digests are recomputed, padding between tensors must be zero. Tensors
// are verified by up to `authentication_workers` threads (a co-located pair is one unit).
[[nodiscard]] AdoptedPackV3 adopt_pack_v3_with_plan(PackPlanV3 expected_plan, std::shared_ptr<const ModelFiles> source,
                                                    std::shared_ptr<const ModelFiles> mtp_sidecar, const std::filesystem::path& path,
                                                    uint32_t experts_per_chunk = 8, uint64_t chunk_bytes = derived_pack::default_chunk_bytes,
                                                    uint32_t authentication_workers = 1,
                                                    derived_pack::TrustMode trust_mode = derived_pack::TrustMode::full);
[[nodiscard]] AdoptedPackV3 adopt_derived_pack_v3(std::shared_ptr<const ModelFiles> source, std::shared_ptr<const ModelFiles> mtp_sidecar,
                                                  const std::filesystem::path& path, uint32_t experts_per_chunk = 8,
                                                  uint64_t chunk_bytes = derived_pack::default_chunk_bytes, uint32_t authentication_workers = 1,
                                                  derived_pack::TrustMode trust_mode = derived_pack::TrustMode::full);
[[nodiscard]] AdoptedPackV3 adopt_block_pack_v3(std::shared_ptr<const ModelFiles> source, std::shared_ptr<const ModelFiles> mtp_sidecar,
                                                uint32_t block_id, const std::filesystem::path& path, uint32_t experts_per_chunk = 8,
                                                uint64_t chunk_bytes = derived_pack::default_chunk_bytes, uint32_t authentication_workers = 1);

// The routed experts of one block of an adopted pack on the GPU: the co-located halves and the down planes are uploaded
// as they lie in the file and registered with the graph (src/model.cpp registers them the same way through
// graph.hpp:465 `register_planar_matrix`), ready for encode_moe / encode_moe_mm_many.
struct PackMoeBlockV3 {
    GpuMatrix gate, up, down;  // gate.view = pair_lo (experts 0..E/2-1 as [gate, up]), up.view = pair_hi
    uint32_t channels = 0, hidden = 0, experts = 0;
};
[[nodiscard]] PackMoeBlockV3 upload_moe_block_v3(HipGraph& graph, const AdoptedPackV3& pack, uint32_t block_id);

}  // namespace planar_v3
}  // namespace tokspur
