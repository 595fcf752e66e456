// GGUF v3 reader and the tokspur-pack-v3 builder / adopter (host only: files, hashing, the byte-exact inverse proof).
// The plane transforms themselves are the C ABI's host functions (tsp_pack_expert_planar_v3 and friends).
#include "pack_v3.hpp"

#include "../../include/tokspur_hip.h"

#include <algorithm>
#include <array>
#include <atomic>
#include <cerrno>
#include <cstring>
#include <exception>
#include <fcntl.h>
#include <limits>
#include <set>
#include <sys/mman.h>
#include <sys/stat.h>
#include <sys/statvfs.h>
#include <sys/syscall.h>
#include <thread>
#include <unistd.h>
#include <utility>

namespace tokspur {

namespace {

using Bytes = std::vector<std::byte>;

void require(bool condition, const char* message) {
    if (!condition) throw FormatError(message);
}
void abi(int status) {  // host-side refusals of the C ABI keep the engine's exception type
    if (status != TSP_OK) throw FormatError(tsp_last_error());
}
const uint8_t* u8(std::span<const std::byte> s) { return reinterpret_cast<const uint8_t*>(s.data()); }
uint8_t* u8(std::span<std::byte> s) { return reinterpret_cast<uint8_t*>(s.data()); }
bool same(std::span<const std::byte> a, std::span<const std::byte> b) {
    return a.size() == b.size() && (a.empty() || std::memcmp(a.data(), b.data(), a.size()) == 0);
}
bool ends_with(std::string_view s, std::string_view tail) { return s.size() >= tail.size() && s.substr(s.size() - tail.size()) == tail; }
bool starts_with(std::string_view s, std::string_view head) { return s.size() >= head.size() && s.substr(0, head.size()) == head; }

constexpr Encoding kEncodings[] = {
    {0, "F32", 1, 4},      {1, "F16", 1, 2},      {2, "Q4_0", 32, 18},    {3, "Q4_1", 32, 20},    {6, "Q5_0", 32, 22},
    {7, "Q5_1", 32, 24},   {8, "Q8_0", 32, 34},   {10, "Q2_K", 256, 84},  {11, "Q3_K", 256, 110}, {12, "Q4_K", 256, 144},
    {13, "Q5_K", 256, 176}, {14, "Q6_K", 256, 210}, {20, "IQ4_NL", 32, 18}, {23, "IQ4_XS", 256, 136}, {24, "I8", 1, 1},
    {25, "I16", 1, 2},     {26, "I32", 1, 4},     {27, "I64", 1, 8},      {28, "F64", 1, 8},      {30, "BF16", 1, 2},
};
constexpr uint64_t kHeaderLimit = 256ull << 20, kRecordLimit = 100'000, kArrayLimit = 16ull << 20;

bool utf8_ok(std::span<const std::byte> s) {
    for (size_t i = 0; i < s.size();) {
        const uint32_t lead = std::to_integer<uint32_t>(s[i++]);
        if (lead < 0x80) continue;
        const uint32_t more = lead >= 0xf0 ? 3 : lead >= 0xe0 ? 2 : 1;
        if (lead < 0xc2 || lead > 0xf4 || more > s.size() - i) return false;
        uint32_t point = lead & ((1u << (6 - more)) - 1);
        for (uint32_t k = 0; k < more; ++k) {
            const uint32_t next = std::to_integer<uint32_t>(s[i++]);
            if ((next & 0xc0) != 0x80) return false;
            point = (point << 6) | (next & 0x3f);
        }
        const uint32_t least = more == 1 ? 0x80u : more == 2 ? 0x800u : 0x10000u;
        if (point < least || point > 0x10ffff || (point >= 0xd800 && point <= 0xdfff)) return false;
    }
    return true;
}

// bounded little-endian reader over the header bytes
struct Reader {
    std::span<const std::byte> data;
    uint64_t at = 0;
    std::span<const std::byte> take(uint64_t n) {
        const uint64_t end = checked_add(at, n);
        require(end <= data.size() && end <= kHeaderLimit, "truncated or oversized GGUF header");
        const auto out = data.subspan(size_t(at), size_t(n));
        at = end;
        return out;
    }
    uint64_t number(unsigned width) {
        const auto b = take(width);
        uint64_t v = 0;
        for (unsigned i = 0; i < width; ++i) v |= uint64_t(std::to_integer<uint8_t>(b[i])) << (8 * i);
        return v;
    }
    std::string_view text(uint64_t limit = kHeaderLimit) {
        const uint64_t n = number(8);
        require(n <= limit, "GGUF string exceeds limit");
        const auto b = take(n);
        require(utf8_ok(b), "invalid UTF-8 in GGUF string");
        return {reinterpret_cast<const char*>(b.data()), b.size()};
    }
    Metadata value(uint32_t type, unsigned depth = 0) {
        require(depth <= 8, "GGUF array nesting exceeds limit");
        Metadata m{type, at, 0, 0, 0};
        static constexpr uint8_t widths[13] = {1, 1, 2, 2, 4, 4, 4, 0, 0, 0, 8, 8, 8};
        if (type == 7) require(number(1) <= 1, "invalid GGUF boolean");
        else if (type == 8) (void)text();
        else if (type == 9) {
            m.element_type = uint32_t(number(4));
            m.elements = number(8);
            require(m.element_type <= 12 && m.elements <= kArrayLimit, "invalid GGUF array");
            if (widths[m.element_type]) (void)take(checked_mul(m.elements, widths[m.element_type]));
            else for (uint64_t i = 0; i < m.elements; ++i) (void)value(m.element_type, depth + 1);
        } else {
            require(type <= 12 && widths[type], "unknown GGUF metadata type");
            (void)take(widths[type]);
        }
        m.end = at;
        return m;
    }
};

bool key_ok(std::string_view key) {
    if (key.empty() || key.front() == '.' || key.back() == '.') return false;
    char before = '.';
    for (const char c : key) {
        if (!((c >= 'a' && c <= 'z') || (c >= '0' && c <= '9') || c == '_' || c == '.')) return false;
        if (c == '.' && before == '.') return false;
        before = c;
    }
    return true;
}

}  // namespace

uint64_t checked_add(uint64_t a, uint64_t b) {
    if (a > std::numeric_limits<uint64_t>::max() - b) throw FormatError("GGUF offset overflow");
    return a + b;
}
uint64_t checked_mul(uint64_t a, uint64_t b) {
    if (a && b > std::numeric_limits<uint64_t>::max() / a) throw FormatError("GGUF shape overflow");
    return a * b;
}
const Encoding& encoding(uint32_t id) {
    for (const auto& e : kEncodings) if (e.id == id) return e;
    throw FormatError("unsupported GGUF tensor encoding " + std::to_string(id));
}

// ---------------------------------------------------------------------------------------------- files

MappedFile::MappedFile(const std::filesystem::path& path) : path_(path) {
    fd_ = ::open(path.c_str(), O_RDONLY | O_CLOEXEC | O_NONBLOCK);
    if (fd_ < 0) throw FormatError("cannot open weight file");
    struct stat info{};
    if (::fstat(fd_, &info) != 0 || !S_ISREG(info.st_mode) || info.st_size <= 0) {
        ::close(fd_);
        throw FormatError("weight file must be a nonempty regular file");
    }
    size_ = uint64_t(info.st_size);
    device_ = uint64_t(info.st_dev);
    inode_ = uint64_t(info.st_ino);
    mtime_[0] = info.st_mtim.tv_sec; mtime_[1] = info.st_mtim.tv_nsec;
    ctime_[0] = info.st_ctim.tv_sec; ctime_[1] = info.st_ctim.tv_nsec;
    void* mapped = ::mmap(nullptr, size_t(size_), PROT_READ, MAP_PRIVATE, fd_, 0);
    if (mapped == MAP_FAILED) {
        ::close(fd_);
        throw FormatError("cannot map weight file");
    }
    data_ = static_cast<const std::byte*>(mapped);
}
MappedFile::~MappedFile() {
    if (data_) ::munmap(const_cast<std::byte*>(data_), size_t(size_));
    if (fd_ >= 0) ::close(fd_);
}
MappedFile::MappedFile(MappedFile&& o) noexcept
    : path_(std::move(o.path_)), fd_(std::exchange(o.fd_, -1)), data_(std::exchange(o.data_, nullptr)), size_(std::exchange(o.size_, 0)),
      device_(o.device_), inode_(o.inode_), mtime_{o.mtime_[0], o.mtime_[1]}, ctime_{o.ctime_[0], o.ctime_[1]} {}
void MappedFile::assert_unchanged() const {
    struct stat info{};
    if (::fstat(fd_, &info) != 0 || uint64_t(info.st_size) != size_ || uint64_t(info.st_dev) != device_ || uint64_t(info.st_ino) != inode_ ||
        info.st_mtim.tv_sec != mtime_[0] || info.st_mtim.tv_nsec != mtime_[1] || info.st_ctim.tv_sec != ctime_[0] || info.st_ctim.tv_nsec != ctime_[1])
        throw FormatError("weight file changed since mapping");
}

Gguf::Gguf(const std::filesystem::path& path) {
    mapping_.emplace_back(path);
    data_ = mapping_.front().bytes();
    parse();
    assert_unchanged();
}
Gguf::Gguf(std::span<const std::byte> bytes) : data_(bytes) { parse(); }
void Gguf::assert_unchanged() const {
    for (const auto& m : mapping_) m.assert_unchanged();
}
const Metadata* Gguf::find(std::string_view key) const {
    const auto it = metadata_.find(key);
    return it == metadata_.end() ? nullptr : &it->second;
}
uint64_t Gguf::unsigned_value(std::string_view key) const {
    const Metadata* m = find(key);
    if (!m) throw FormatError("missing GGUF metadata " + std::string(key));
    static constexpr uint8_t widths[12] = {1, 1, 2, 2, 4, 4, 0, 0, 0, 0, 8, 8};
    require(m->type < 12 && widths[m->type], "GGUF metadata is not an integer");
    Reader r{data_, m->offset};
    const unsigned width = widths[m->type];
    const uint64_t v = r.number(width);
    require(!((m->type & 1) && (v >> (width * 8 - 1))), "negative GGUF count");  // odd type ids are the signed ones
    return v;
}
std::string_view Gguf::string_value(std::string_view key) const {
    const Metadata* m = find(key);
    if (!m || m->type != 8) throw FormatError("GGUF metadata is not a string: " + std::string(key));
    Reader r{data_, m->offset};
    return r.text();
}
std::span<const std::byte> Gguf::tensor_bytes(const Tensor& tensor) const {
    const bool member = !tensors_.empty() && &tensor >= tensors_.data() && &tensor < tensors_.data() + tensors_.size();
    require(member, "tensor does not belong to this GGUF");
    assert_unchanged();
    return data_.subspan(size_t(tensor.offset), size_t(tensor.bytes));
}

// The header is taken apart in four stages, each over the table the stage before it left, so that reading the bytes and
// judging what they say stay apart: (1) walk the records and note where each one lies (nothing is judged beyond what finding
// the next record needs); (2) admit the metadata keys; (3) admit the tensor records against the alignment the metadata
// declares; (4) lay the data section out behind the header and check every tensor's bytes against the file and each other.
namespace {
struct MetadataRecord { std::string_view key; Metadata value; };
struct TensorRecord {
    std::string_view name;
    uint32_t rank = 0, type = 0;
    std::array<uint64_t, 4> extent{};
    uint64_t offset = 0;  // from the start of the data section
};
struct HeaderWalk {
    std::vector<MetadataRecord> metadata;
    std::vector<TensorRecord> tensors;
    uint64_t end = 0;  // first byte behind the last record
};

// stage 1: where the records lie. A record that cannot be walked over (a string past its limit, a value of no known type, a rank
// with no extents to count) stops the walk; everything else about a record is left to the stages that follow.
HeaderWalk walk_header(std::span<const std::byte> bytes) {
    Reader r{bytes};
    const uint64_t magic = r.number(4), version = r.number(4);
    require(magic == 0x46554747 && version == 3, "expected little-endian GGUF v3");
    const uint64_t tensor_count = r.number(8), metadata_count = r.number(8);
    require(tensor_count <= kRecordLimit && metadata_count <= kRecordLimit, "GGUF record limit exceeded");
    // no record is shorter than its fixed fields: 8 + 4 + 8 + 4 + 8 + one name byte for a tensor, 8 + 4 + one key byte + one
    // value byte for a metadata item; counts that cannot fit in what is left of the file are refused before any table grows
    const uint64_t least = checked_add(checked_mul(tensor_count, 33), checked_mul(metadata_count, 14));
    require(least <= bytes.size() - r.at, "GGUF counts exceed available file bytes");
    HeaderWalk walk;
    walk.metadata.resize(size_t(metadata_count));
    for (MetadataRecord& item : walk.metadata) {
        item.key = r.text(65535);
        require(key_ok(item.key), "invalid GGUF metadata key");  // the key decides whether the value's bytes mean anything at all
        item.value = r.value(uint32_t(r.number(4)));
    }
    walk.tensors.resize(size_t(tensor_count));
    for (TensorRecord& t : walk.tensors) {
        t.name = r.text(64);
        t.rank = uint32_t(r.number(4));
        require(t.rank >= 1 && t.rank <= 4, "unsupported GGUF tensor rank");
        for (uint32_t d = 0; d < t.rank; ++d) t.extent[d] = r.number(8);
        t.type = uint32_t(r.number(4));
        t.offset = r.number(8);
    }
    walk.end = r.at;
    return walk;
}

// stage 3, one record: names are printable ASCII, extents positive, rows whole blocks of the encoding
Tensor admit_tensor(const TensorRecord& record, uint64_t alignment) {
    require(!record.name.empty(), "empty or duplicate tensor name");
    for (const unsigned char c : record.name) require(c >= 0x21 && c <= 0x7e, "non-ASCII tensor name");
    Tensor t;
    t.name = std::string(record.name);
    t.type = record.type;
    t.elements = 1;
    for (uint32_t d = 0; d < record.rank; ++d) {
        require(record.extent[d] != 0, "zero tensor dimension");
        t.dimensions.push_back(record.extent[d]);
        t.elements = checked_mul(t.elements, record.extent[d]);
    }
    const Encoding& e = encoding(t.type);
    require(t.dimensions.front() % e.elements_per_block == 0, "quantized tensor row is not block-aligned");
    t.bytes = checked_mul(t.elements / e.elements_per_block, e.bytes_per_block);
    require(record.offset % alignment == 0, "unaligned GGUF tensor offset");
    t.offset = record.offset;
    return t;
}
}  // namespace

void Gguf::parse() {
    const HeaderWalk walk = walk_header(data_);
    // stage 2: the metadata index
    for (const MetadataRecord& item : walk.metadata) require(metadata_.emplace(std::string(item.key), item.value).second, "duplicate GGUF metadata key");
    uint64_t alignment = 32;
    if (find("general.alignment")) alignment = unsigned_value("general.alignment");
    require(alignment != 0 && alignment <= 65536 && (alignment & (alignment - 1)) == 0, "unsupported GGUF alignment");
    // stage 3: the tensor table, in file order
    tensors_.reserve(walk.tensors.size());
    std::set<std::string_view> seen;
    for (const TensorRecord& record : walk.tensors) {
        Tensor t = admit_tensor(record, alignment);
        require(seen.insert(record.name).second, "empty or duplicate tensor name");
        tensors_.push_back(std::move(t));
    }
    // stage 4: the data section starts at the next multiple of the alignment behind the header (a shard of metadata alone has
    // none and need not be padded); every tensor lies inside the file and no two share a byte
    data_offset_ = checked_add(walk.end, alignment - 1) / alignment * alignment;
    if (tensors_.empty() && data_offset_ > data_.size()) data_offset_ = data_.size();
    require(data_offset_ <= data_.size(), "truncated GGUF header padding");
    std::vector<size_t> by_offset(tensors_.size());
    for (size_t i = 0; i < tensors_.size(); ++i) {
        by_offset[i] = i;
        tensors_[i].offset = checked_add(data_offset_, tensors_[i].offset);
        require(checked_add(tensors_[i].offset, tensors_[i].bytes) <= data_.size(), "truncated GGUF tensor data");
    }
    std::sort(by_offset.begin(), by_offset.end(), [&](size_t a, size_t b) { return tensors_[a].offset < tensors_[b].offset; });
    uint64_t used_to = 0;
    for (const size_t i : by_offset) {
        require(tensors_[i].offset >= used_to, "overlapping GGUF tensors");
        used_to = tensors_[i].offset + tensors_[i].bytes;
    }
}

ModelFiles::ModelFiles(const std::vector<std::filesystem::path>& paths) {
    require(!paths.empty() && paths.size() <= 1024, "expected 1 to 1024 GGUF shards");
    shards_.reserve(paths.size());
    for (const auto& p : paths) shards_.emplace_back(p);
    std::set<uint64_t> numbers;
    uint64_t declared_total = 0;
    bool split = false;
    for (size_t s = 0; s < shards_.size(); ++s) {
        const Gguf& shard = shards_[s];
        const bool has_split = shard.find("split.count") || shard.find("split.no") || shard.find("split.tensors.count");
        if (s == 0) split = has_split;
        require(has_split == split && (split || paths.size() == 1), "inconsistent split-file metadata");
        if (split) {
            const uint64_t count = shard.unsigned_value("split.count"), number = shard.unsigned_value("split.no");
            const uint64_t total = shard.unsigned_value("split.tensors.count");
            require(count == paths.size() && number < count && numbers.insert(number).second && (s == 0 || declared_total == total),
                    "incomplete or mismatched GGUF shard set");
            declared_total = total;
        }
        if (shard.find("general.architecture")) {
            const auto a = shard.string_value("general.architecture");
            require(architecture_.empty() || architecture_ == a, "shard architecture mismatch");
            architecture_ = std::string(a);
        }
        for (size_t t = 0; t < shard.tensors().size(); ++t)
            require(tensors_.emplace(shard.tensors()[t].name, std::pair{s, t}).second, "duplicate tensor across GGUF shards");
    }
    require(!architecture_.empty(), "GGUF model has no architecture");
    require(!split || declared_total == tensors_.size(), "GGUF split tensor count mismatch");
}
const Tensor& ModelFiles::tensor(std::string_view name) const {
    const auto it = tensors_.find(name);
    require(it != tensors_.end(), "unknown tensor");
    return shards_[it->second.first].tensors()[it->second.second];
}
std::span<const std::byte> ModelFiles::tensor_bytes(std::string_view name) const {
    const auto it = tensors_.find(name);
    require(it != tensors_.end(), "unknown tensor");
    const Gguf& shard = shards_[it->second.first];
    return shard.tensor_bytes(shard.tensors()[it->second.second]);
}
void ModelFiles::assert_unchanged() const {
    for (const auto& s : shards_) s.assert_unchanged();
}

// ---------------------------------------------------------------------------------------------- SHA-256

namespace {
constexpr uint32_t kRound[64] = {
    0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5, 0xd807aa98, 0x12835b01, 0x243185be,
    0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174, 0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc, 0x2de92c6f, 0x4a7484aa,
    0x5cb0a9dc, 0x76f988da, 0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147, 0x06ca6351, 0x14292967, 0x27b70a85,
    0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85, 0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3,
    0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070, 0x19a4c116, 0x1e376c08, 0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f,
    0x682e6ff3, 0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208, 0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};
inline uint32_t rotr(uint32_t x, int n) { return (x >> n) | (x << (32 - n)); }
}  // namespace

Sha256::Sha256() : h_{0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a, 0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19}, tail_{} {}
void Sha256::block(const uint8_t* p) {
    uint32_t w[64];
    for (int i = 0; i < 16; ++i) w[i] = uint32_t(p[4 * i]) << 24 | uint32_t(p[4 * i + 1]) << 16 | uint32_t(p[4 * i + 2]) << 8 | p[4 * i + 3];
    for (int i = 16; i < 64; ++i) {
        const uint32_t s0 = rotr(w[i - 15], 7) ^ rotr(w[i - 15], 18) ^ (w[i - 15] >> 3), s1 = rotr(w[i - 2], 17) ^ rotr(w[i - 2], 19) ^ (w[i - 2] >> 10);
        w[i] = w[i - 16] + s0 + w[i - 7] + s1;
    }
    uint32_t a = h_[0], b = h_[1], c = h_[2], d = h_[3], e = h_[4], f = h_[5], g = h_[6], h = h_[7];
    for (int i = 0; i < 64; ++i) {
        const uint32_t t1 = h + (rotr(e, 6) ^ rotr(e, 11) ^ rotr(e, 25)) + ((e & f) ^ (~e & g)) + kRound[i] + w[i];
        const uint32_t t2 = (rotr(a, 2) ^ rotr(a, 13) ^ rotr(a, 22)) + ((a & b) ^ (a & c) ^ (b & c));
        h = g; g = f; f = e; e = d + t1; d = c; c = b; b = a; a = t1 + t2;
    }
    h_[0] += a; h_[1] += b; h_[2] += c; h_[3] += d; h_[4] += e; h_[5] += f; h_[6] += g; h_[7] += h;
}
void Sha256::add(std::span<const std::byte> data) {
    const uint8_t* p = u8(data);
    size_t n = data.size();
    size_t held = size_t(bytes_ % 64);
    bytes_ += n;
    if (held) {
        const size_t fill = std::min(n, 64 - held);
        std::memcpy(tail_ + held, p, fill);
        p += fill; n -= fill; held += fill;
        if (held < 64) return;
        block(tail_);
    }
    for (; n >= 64; p += 64, n -= 64) block(p);
    if (n) std::memcpy(tail_, p, n);
}
std::string Sha256::finish() {
    const uint64_t bits = bytes_ * 8;
    size_t held = size_t(bytes_ % 64);
    tail_[held++] = 0x80;
    if (held > 56) {
        std::memset(tail_ + held, 0, 64 - held);
        block(tail_);
        held = 0;
    }
    std::memset(tail_ + held, 0, 56 - held);
    for (int i = 0; i < 8; ++i) tail_[56 + i] = uint8_t(bits >> (56 - 8 * i));
    block(tail_);
    static constexpr char hex[] = "0123456789abcdef";
    std::string out(64, '0');
    for (int i = 0; i < 32; ++i) {
        const uint8_t byte = uint8_t(h_[i / 4] >> (24 - 8 * (i % 4)));
        out[2 * i] = hex[byte >> 4];
        out[2 * i + 1] = hex[byte & 15];
    }
    return out;
}

namespace derived_pack {
std::string hash(std::string_view text) {
    Sha256 h;
    h.add(std::as_bytes(std::span(text.data(), text.size())));
    return h.finish();
}
bool check_disk_reserve(uint64_t available_bytes, uint64_t peak_additional_bytes, uint64_t reserve_bytes) {
    if (available_bytes == 0 || peak_additional_bytes > std::numeric_limits<uint64_t>::max() - reserve_bytes) return false;
    return available_bytes >= peak_additional_bytes + reserve_bytes;
}
}  // namespace derived_pack

// ---------------------------------------------------------------------------------------------- pack v3

namespace planar_v3 {

namespace {

constexpr uint64_t kMaxHeaderBytes = 256ull << 20;
constexpr const char* kKindNames[] = {"plain", "q8_lanes_v1", "q4k_coloc_gate_v3", "q4k_coloc_up_v3", "q5k_coloc_gate_v3",
                                      "q5k_coloc_up_v3", "q8_coloc_gate_v3", "q8_coloc_up_v3", "q51_planar_v3", "q8_planar_v3"};

uint64_t aligned(uint64_t n, uint64_t boundary = derived_pack::pack_alignment) { return checked_add(n, boundary - 1) / boundary * boundary; }

void put_number(Bytes& b, uint64_t value, unsigned width) {
    for (unsigned i = 0; i < width; ++i) b.push_back(std::byte((value >> (8 * i)) & 255));
}
void put_text(Bytes& b, std::string_view s) {
    put_number(b, s.size(), 8);
    for (const unsigned char c : s) b.push_back(std::byte(c));
}

// ---- the manifest: compact JSON, members in the order written (src/json.cpp:204-244 `Json::dump`)
void json_text(std::string& out, std::string_view s) {
    out += '"';
    for (const unsigned char c : s) {
        if (c == '"' || c == '\\') { out += '\\'; out += char(c); }
        else if (c < 0x20) { static constexpr char hex[] = "0123456789abcdef"; out += "\\u00"; out += hex[c >> 4]; out += hex[c & 15]; }
        else out += char(c);
    }
    out += '"';
}
void json_member(std::string& out, const char* key, bool first = false) {
    if (!first) out += ',';
    json_text(out, key);
    out += ':';
}
void json_numbers(std::string& out, const std::vector<uint64_t>& v) {
    out += '[';
    for (size_t i = 0; i < v.size(); ++i) { if (i) out += ','; out += std::to_string(v[i]); }
    out += ']';
}
std::string manifest_of(const PackPlanV3& plan) {  // src/planar_pack_v3.cpp:120-153
    static const std::string zeros(64, '0');
    std::string m = "{";
    json_member(m, "schema", true); m += std::to_string(plan.version);
    json_member(m, "recipe"); json_text(m, plan.recipe);
    json_member(m, "source_architecture"); json_text(m, derived_pack::source_architecture);
    json_member(m, "target_revision"); json_text(m, derived_pack::target_revision);
    json_member(m, "mtp_sidecar_sha256"); json_text(m, derived_pack::mtp_sidecar_sha256);
    json_member(m, "source_payload_bytes"); m += std::to_string(plan.source_payload_bytes);
    json_member(m, "payload_bytes"); m += std::to_string(plan.payload_bytes);
    json_member(m, "tensors");
    m += '[';
    for (size_t i = 0; i < plan.tensors.size(); ++i) {
        const PackTensorV3& t = plan.tensors[i];
        if (i) m += ',';
        m += '{';
        json_member(m, "name", true); json_text(m, t.name);
        json_member(m, "type"); m += std::to_string(t.type);
        json_member(m, "source_type"); m += std::to_string(t.source_type);
        json_member(m, "layout"); json_text(m, t.layout);
        json_member(m, "dimensions"); json_numbers(m, t.dimensions);
        json_member(m, "source_dimensions"); json_numbers(m, t.source_dimensions);
        json_member(m, "source_bytes"); m += std::to_string(t.source_bytes);
        json_member(m, "bytes"); m += std::to_string(t.bytes);
        json_member(m, "offset"); m += std::to_string(t.offset);
        json_member(m, "partner_name"); json_text(m, t.partner_name);
        json_member(m, "source_sha256"); json_text(m, t.source_sha256.empty() ? zeros : t.source_sha256);
        json_member(m, "packed_sha256"); json_text(m, t.packed_sha256.empty() ? zeros : t.packed_sha256);
        m += '}';
        require(m.size() <= kMaxHeaderBytes, "JSON output byte limit exceeded");
    }
    m += "]}";
    return m;
}

// A reader for the manifest and nothing more general: objects, arrays, strings and unsigned integers; anything else in a
// value position is skipped over as a bare token. Depth and size are bounded by the caller's text.
struct JsonValue {
    enum Kind { text, number, list, object, other } kind = other;
    std::string s;
    uint64_t n = 0;
    std::vector<JsonValue> items;
    std::vector<std::pair<std::string, JsonValue>> members;
    const JsonValue* find(std::string_view key) const {
        for (const auto& m : members) if (m.first == key) return &m.second;
        return nullptr;
    }
};
struct JsonReader {
    std::string_view in;
    size_t at = 0;
    void space() { while (at < in.size() && (in[at] == ' ' || in[at] == '\n' || in[at] == '\r' || in[at] == '\t')) ++at; }
    char peek() { space(); require(at < in.size(), "truncated pack v3 manifest"); return in[at]; }
    void expect(char c) { require(peek() == c, "malformed pack v3 manifest"); ++at; }
    std::string text() {
        expect('"');
        std::string out;
        for (;;) {
            require(at < in.size(), "truncated pack v3 manifest");
            const char c = in[at++];
            if (c == '"') return out;
            if (c != '\\') { out += c; continue; }
            require(at < in.size(), "truncated pack v3 manifest");
            const char e = in[at++];
            if (e == 'u') {
                require(at + 4 <= in.size(), "truncated pack v3 manifest");
                unsigned v = 0;
                for (int i = 0; i < 4; ++i) {
                    const char h = in[at++];
                    v = v * 16 + unsigned(h >= '0' && h <= '9' ? h - '0' : h >= 'a' && h <= 'f' ? h - 'a' + 10 : h >= 'A' && h <= 'F' ? h - 'A' + 10 : 99);
                }
                require(v < 0x80, "pack v3 manifest strings are ASCII");
                out += char(v);
            } else {
                const char* from = "\"\\/bfnrt";
                const char* to = "\"\\/\b\f\n\r\t";
                const char* hit = std::strchr(from, e);
                require(hit && e, "malformed pack v3 manifest escape");
                out += to[hit - from];
            }
        }
    }
    JsonValue value(unsigned depth = 0) {
        require(depth <= 16, "pack v3 manifest nesting exceeds limit");
        JsonValue v;
        const char c = peek();
        if (c == '"') { v.kind = JsonValue::text; v.s = text(); }
        else if (c == '[') {
            v.kind = JsonValue::list;
            ++at;
            if (peek() == ']') { ++at; return v; }
            for (;;) { v.items.push_back(value(depth + 1)); if (peek() == ',') { ++at; continue; } expect(']'); return v; }
        } else if (c == '{') {
            v.kind = JsonValue::object;
            ++at;
            if (peek() == '}') { ++at; return v; }
            for (;;) {
                std::string key = text();
                expect(':');
                require(!v.find(key), "duplicate pack v3 manifest key");
                v.members.emplace_back(std::move(key), value(depth + 1));
                if (peek() == ',') { ++at; continue; }
                expect('}');
                return v;
            }
        } else {
            const size_t start = at;
            while (at < in.size() && std::strchr(",]} \n\r\t", in[at]) == nullptr) ++at;
            const std::string_view token = in.substr(start, at - start);
            require(!token.empty(), "malformed pack v3 manifest");
            if (std::all_of(token.begin(), token.end(), [](char d) { return d >= '0' && d <= '9'; }) && token.size() <= 20) {
                v.kind = JsonValue::number;
                for (const char d : token) {
                    require(v.n <= (std::numeric_limits<uint64_t>::max() - uint64_t(d - '0')) / 10, "pack v3 manifest integer overflow");
                    v.n = v.n * 10 + uint64_t(d - '0');
                }
            }
        }
        return v;
    }
};
JsonValue parse_manifest(std::string_view text) {
    JsonReader r{text};
    JsonValue v = r.value();
    r.space();
    require(r.at == text.size() && v.kind == JsonValue::object, "malformed pack v3 manifest");
    return v;
}

const Tensor* find_tensor(const ModelFiles& source, const ModelFiles* sidecar, std::string_view name) {
    if (source.contains(name)) return &source.tensor(name);
    if (sidecar && sidecar->contains(name)) return &sidecar->tensor(name);
    return nullptr;
}
std::span<const std::byte> find_bytes(const ModelFiles& source, const ModelFiles* sidecar, std::string_view name) {
    if (source.contains(name)) return source.tensor_bytes(name);
    if (sidecar && sidecar->contains(name)) return sidecar->tensor_bytes(name);
    throw FormatError("missing source tensor for pack v3: " + std::string(name));
}

tsp_planar_spec expert_spec(uint32_t type, uint64_t columns, uint64_t rows) {
    require(columns <= UINT32_MAX && rows <= UINT32_MAX, "pack v3 source dimensions mismatch");
    tsp_planar_spec spec{};
    abi(tsp_make_expert_spec(type, uint32_t(columns), uint32_t(rows), &spec));
    return spec;
}

// src/planar_pack_v3.cpp:345-360
bool coloc_eligible(const Tensor& gate, const Tensor& up) {
    if (gate.dimensions.size() != 3 || gate.dimensions != up.dimensions || gate.type != up.type) return false;
    if (gate.type != 12 && gate.type != 13 && gate.type != 8) return false;
    const uint64_t cols = gate.dimensions[0], rows = gate.dimensions[1], experts = gate.dimensions[2];
    if (experts < 2 || experts % 2 || rows < 4 || rows % 4) return false;
    if (gate.type != 8) return cols >= 256 && cols % 256 == 0;
    return cols >= 32 && cols % 32 == 0 && (rows * (cols / 32)) % 8 == 0;
}
bool down_planar_eligible(const Tensor& down) {
    if (down.dimensions.size() != 3 || (down.type != 7 && down.type != 8)) return false;
    const uint64_t cols = down.dimensions[0], rows = down.dimensions[1];
    if (cols < 32 || cols % 32 || rows < 4 || rows % 4) return false;
    return down.type != 8 || (rows * (cols / 32)) % 8 == 0;
}
// src/lane_sidecar.cpp:184-201, the Q8_0 arm: dense two-dimensional matrices outside the embedding and ple_ tables
bool q8_lanes_eligible(const Tensor& t) {
    if (t.type != 8 || t.dimensions.size() != 2 || t.name.empty() || t.name.find("token_embd") != std::string::npos ||
        t.name.find("ple_") != std::string::npos || t.name.find(".ple.") != std::string::npos || starts_with(t.name, "ple."))
        return false;
    const uint64_t columns = t.dimensions[0], rows = t.dimensions[1];
    if (!columns || columns > 65536 || !rows || rows > 1'000'000 || columns % 32 || !(columns % 256 == 0 || columns < 512)) return false;
    return columns / 32 * 34 * rows == t.bytes;
}

PackTensorV3 coloc_entry(const Tensor& t, bool is_gate, std::string partner) {  // src/planar_pack_v3.cpp:362-392
    const tsp_planar_spec spec = expert_spec(t.type, t.dimensions[0], t.dimensions[1]);
    const uint64_t experts = t.dimensions[2], packed = checked_mul(spec.planar_expert_bytes, experts);
    const uint32_t base = t.type == 12 ? 2u : t.type == 13 ? 4u : 6u;
    const PlanarKind kind = PlanarKind(base + (is_gate ? 0u : 1u));
    const bool expanded = packed != t.bytes;  // the 12-byte scale fields grow to 16: the directory then names plain bytes
    PackTensorV3 e;
    e.name = t.name;
    e.type = expanded ? 24u : t.type;
    e.source_type = t.type;
    e.kind = kind;
    e.layout = planar_kind_name(kind);
    e.dimensions = expanded ? std::vector<uint64_t>{spec.planar_row_bytes, t.dimensions[1], experts} : t.dimensions;
    e.source_dimensions = t.dimensions;
    e.source_bytes = t.bytes;
    e.bytes = packed;
    e.partner_name = std::move(partner);
    return e;
}
PackTensorV3 same_size_entry(const Tensor& t, PlanarKind kind) {
    PackTensorV3 e;
    e.name = t.name;
    e.type = e.source_type = t.type;
    e.kind = kind;
    e.layout = planar_kind_name(kind);
    e.dimensions = e.source_dimensions = t.dimensions;
    e.source_bytes = e.bytes = t.bytes;
    return e;
}

void place(PackPlanV3& plan) {  // offsets, header size, file size
    uint64_t at = 0;
    for (auto& t : plan.tensors) {
        at = aligned(at);
        t.offset = at;
        at = checked_add(at, t.bytes);
    }
    plan.data_offset = build_header_v3(plan).size();
    plan.file_bytes = checked_add(plan.data_offset, at);
}

PackPlanV3 plan_filtered(const ModelFiles& source, const ModelFiles* sidecar, std::string_view prefix, std::string recipe, uint64_t byte_budget) {
    source.assert_unchanged();
    require(source.architecture() != derived_pack::pack_architecture, "cannot repack an existing derived pack");
    if (sidecar) sidecar->assert_unchanged();
    std::vector<std::string> names;
    std::set<std::string, std::less<>> seen, done;
    const auto collect = [&](const ModelFiles& files) {
        for (const auto& [name, where] : files.tensors()) {
            (void)where;
            if (!derived_pack::is_gpu_pack_tensor(name) || !starts_with(name, prefix)) continue;
            if (seen.insert(name).second) names.push_back(name);
        }
    };
    collect(source);
    if (sidecar) collect(*sidecar);
    require(!names.empty(), "empty pack v3 tensor selection");

    PackPlanV3 plan;
    plan.recipe = std::move(recipe);
    const auto emit = [&](PackTensorV3 e) {
        plan.source_payload_bytes = checked_add(plan.source_payload_bytes, e.source_bytes);
        plan.payload_bytes = checked_add(plan.payload_bytes, e.bytes);
        done.insert(e.name);
        plan.tensors.push_back(std::move(e));
    };
    constexpr std::string_view gate_tail = ".ffn_gate_exps.weight", down_tail = ".ffn_down_exps.weight";
    for (const auto& name : names) {
        if (done.count(name)) continue;
        const Tensor* t = find_tensor(source, sidecar, name);
        require(t != nullptr, "missing tensor metadata while planning pack v3");
        if (ends_with(name, gate_tail)) {  // the up tensor follows its gate at once: the pair is one unit of the file
            const std::string up_name = name.substr(0, name.size() - gate_tail.size()) + ".ffn_up_exps.weight";
            const Tensor* up = find_tensor(source, sidecar, up_name);
            if (up && seen.count(up_name) && !done.count(up_name) && coloc_eligible(*t, *up)) {
                const uint64_t superblocks = checked_mul(checked_mul(t->dimensions[0] / 256, t->dimensions[1]), t->dimensions[2]) * 2;
                if (t->type == 12) plan.q4k_superblocks = checked_add(plan.q4k_superblocks, superblocks);
                if (t->type == 13) plan.q5k_superblocks = checked_add(plan.q5k_superblocks, superblocks);
                emit(coloc_entry(*t, true, up_name));
                emit(coloc_entry(*up, false, name));
                continue;
            }
        }
        if (ends_with(name, down_tail) && down_planar_eligible(*t)) {
            emit(same_size_entry(*t, t->type == 7 ? PlanarKind::q51_planar_v3 : PlanarKind::q8_planar_v3));
            continue;
        }
        emit(same_size_entry(*t, q8_lanes_eligible(*t) ? PlanarKind::q8_lanes_v1 : PlanarKind::plain));
    }
    const uint64_t superblocks = checked_add(plan.q4k_superblocks, plan.q5k_superblocks);
    plan.original_12b_scale_header_bytes = checked_mul(superblocks, 12);
    plan.expanded_16b_scale_header_bytes = checked_mul(superblocks, 16);
    place(plan);
    require(plan.file_bytes <= byte_budget, "planned pack v3 exceeds byte budget");
    source.assert_unchanged();
    if (sidecar) sidecar->assert_unchanged();
    return plan;
}

// ---- file plumbing
struct Fd {
    int value = -1;
    explicit Fd(int v) : value(v) { require(v >= 0, "cannot open pack v3 file or directory"); }
    ~Fd() { if (value >= 0) ::close(value); }
    Fd(const Fd&) = delete;
    Fd& operator=(const Fd&) = delete;
};
void write_at(int fd, std::span<const std::byte> bytes, uint64_t offset) {
    for (size_t done = 0; done < bytes.size();) {
        const ssize_t n = ::pwrite(fd, bytes.data() + done, bytes.size() - done, off_t(offset + done));
        if (n < 0 && errno == EINTR) continue;
        require(n > 0, "pack v3 write failed");
        done += size_t(n);
    }
}
void read_into(int fd, std::span<std::byte> out, uint64_t offset) {
    for (size_t done = 0; done < out.size();) {
        const ssize_t n = ::pread(fd, out.data() + done, out.size() - done, off_t(offset + done));
        if (n < 0 && errno == EINTR) continue;
        require(n > 0, "pack v3 read failed or file truncated");
        done += size_t(n);
    }
}
Bytes read_at(int fd, size_t bytes, uint64_t offset) {
    Bytes out(bytes);
    read_into(fd, out, offset);
    return out;
}
struct Location {  // the directory (opened) and the leaf name of a pack path
    std::string name;
    std::filesystem::path directory_path;
    int directory = -1;
    explicit Location(const std::filesystem::path& path) {
        require(path.has_filename(), "pack v3 path has no file name");
        name = path.filename().string();
        directory_path = path.has_parent_path() ? path.parent_path() : std::filesystem::path(".");
        directory = ::open(directory_path.c_str(), O_RDONLY | O_DIRECTORY | O_CLOEXEC);
        require(directory >= 0, "cannot open pack v3 directory");
    }
    ~Location() { if (directory >= 0) ::close(directory); }
    Location(const Location&) = delete;
    Location& operator=(const Location&) = delete;
    bool exists() const {
        struct stat info{};
        return ::fstatat(directory, name.c_str(), &info, AT_SYMLINK_NOFOLLOW) == 0;
    }
    uint64_t available_bytes() const {
        struct statvfs v{};
        require(::fstatvfs(directory, &v) == 0, "cannot query free space for pack v3");
        return checked_mul(uint64_t(v.f_bavail), uint64_t(v.f_frsize));
    }
};
struct Temporary {  // an exclusive, owner-only file beside the destination; removed unless published
    int directory;
    std::string name;
    int fd = -1;
    bool published = false;
    explicit Temporary(int dir) : directory(dir) {
        static std::atomic<uint64_t> counter{0};
        for (int attempt = 0; attempt < 64 && fd < 0; ++attempt) {
            name = ".tokspur-pack-v3." + std::to_string(::getpid()) + "." + std::to_string(counter.fetch_add(1)) + ".tmp";
            fd = ::openat(directory, name.c_str(), O_CREAT | O_EXCL | O_RDWR | O_CLOEXEC | O_NOFOLLOW, 0600);
            if (fd < 0 && errno != EEXIST) break;
        }
        require(fd >= 0, "cannot create pack v3 temporary");
    }
    ~Temporary() {
        if (fd >= 0) ::close(fd);
        if (!published) ::unlinkat(directory, name.c_str(), 0);
    }
};

}  // namespace

const char* planar_kind_name(PlanarKind kind) {
    require(uint32_t(kind) < std::size(kKindNames), "unknown PlanarKind");
    return kKindNames[uint32_t(kind)];
}
PlanarKind parse_planar_kind(std::string_view name) {
    for (uint32_t k = 0; k < std::size(kKindNames); ++k) if (name == kKindNames[k]) return PlanarKind(k);
    throw FormatError("unrecognised planar v3 layout string: " + std::string(name));
}
bool is_planar_v3_kind(PlanarKind kind) noexcept { return kind != PlanarKind::plain && kind != PlanarKind::q8_lanes_v1; }
bool is_coloc_gate_kind(PlanarKind k) noexcept { return k == PlanarKind::q4k_coloc_gate_v3 || k == PlanarKind::q5k_coloc_gate_v3 || k == PlanarKind::q8_coloc_gate_v3; }
bool is_coloc_up_kind(PlanarKind k) noexcept { return k == PlanarKind::q4k_coloc_up_v3 || k == PlanarKind::q5k_coloc_up_v3 || k == PlanarKind::q8_coloc_up_v3; }

std::vector<std::byte> build_header_v3(const PackPlanV3& plan) {
    Bytes b;
    put_number(b, 0x46554747, 4);  // "GGUF", version 3
    put_number(b, 3, 4);
    put_number(b, plan.tensors.size(), 8);
    put_number(b, 5, 8);  // metadata entries; type 8 = string, type 4 = u32
    const auto text = [&](const char* key, std::string_view value) { put_text(b, key); put_number(b, 8, 4); put_text(b, value); };
    const auto u32 = [&](const char* key, uint32_t value) { put_text(b, key); put_number(b, 4, 4); put_number(b, value, 4); };
    text("general.architecture", derived_pack::pack_architecture);
    u32("general.alignment", plan.alignment);
    u32("tokspur_pack.version", plan.version);
    text("tokspur_pack.recipe", plan.recipe);
    text("tokspur_pack.manifest", manifest_of(plan));
    for (const auto& t : plan.tensors) {
        put_text(b, t.name);
        put_number(b, t.dimensions.size(), 4);
        for (const uint64_t d : t.dimensions) put_number(b, d, 8);
        put_number(b, t.type, 4);
        put_number(b, t.offset, 8);
    }
    require(b.size() <= kMaxHeaderBytes, "pack v3 header exceeds bound");
    b.resize(size_t(aligned(b.size(), plan.alignment)), std::byte(0));
    return b;
}

PackPlanV3 plan_derived_pack_v3(const ModelFiles& source, const ModelFiles* sidecar, uint64_t byte_budget) {
    return plan_filtered(source, sidecar, {}, pack_recipe_v3, byte_budget);
}
PackPlanV3 plan_block_pack_v3(const ModelFiles& source, const ModelFiles* sidecar, uint32_t block_id, uint64_t byte_budget) {
    return plan_filtered(source, sidecar, "blk." + std::to_string(block_id) + ".", block_recipe_prefix_v3 + std::to_string(block_id), byte_budget);
}

BudgetReportV3 measure_pack_v3_budget(const PackPlanV3& plan, const std::filesystem::path& output_directory,
                                      const std::filesystem::path& existing_pack_v2_path, uint32_t experts_per_chunk, uint64_t reserve_bytes,
                                      uint64_t chunk_bytes) {
    require(experts_per_chunk >= 1 && experts_per_chunk <= 64, "experts_per_chunk must be in 1..64");
    require(chunk_bytes >= 32'768 && chunk_bytes <= 67'108'864, "invalid chunk_bytes bound");
    BudgetReportV3 report;
    {
        const int dir = ::open(output_directory.c_str(), O_RDONLY | O_DIRECTORY | O_CLOEXEC);
        require(dir >= 0, "cannot open pack v3 directory");
        struct statvfs v{};
        const bool ok = ::fstatvfs(dir, &v) == 0;
        ::close(dir);
        require(ok, "cannot query free space for pack v3");
        report.filesystem_available_bytes = checked_mul(uint64_t(v.f_bavail), uint64_t(v.f_frsize));
    }
    if (!existing_pack_v2_path.empty()) {
        struct stat info{};
        if (::stat(existing_pack_v2_path.c_str(), &info) == 0 && S_ISREG(info.st_mode)) report.existing_pack_v2_file_bytes = uint64_t(info.st_size);
    }
    report.planned_pack_v3_payload_bytes = plan.payload_bytes;
    report.planned_pack_v3_file_bytes = plan.file_bytes;
    report.required_reserve_bytes = reserve_bytes;
    report.original_12b_scale_header_bytes = plan.original_12b_scale_header_bytes;
    report.expanded_16b_scale_header_bytes = plan.expanded_16b_scale_header_bytes;
    // which family's counter a planar kind adds to (plain and lane tensors: none)
    uint64_t* const family[10] = {nullptr, nullptr, &report.q4k_planar_bytes, &report.q4k_planar_bytes, &report.q5k_planar_bytes,
                                  &report.q5k_planar_bytes, &report.q8_planar_moe_bytes, &report.q8_planar_moe_bytes,
                                  &report.q51_planar_bytes, &report.q8_planar_moe_bytes};
    // a plain or lane tensor streams through one written and one read-back buffer of chunk_bytes; a planar tensor through
    // the packed chunk, its read-back and the restored source, per expert (a co-located pair counts twice)
    uint64_t buffers = checked_mul(chunk_bytes, 2);
    for (const PackTensorV3& t : plan.tensors) {
        require(uint32_t(t.kind) < std::size(family), "unknown PlanarKind");
        if (uint64_t* const counter = family[uint32_t(t.kind)]) *counter = checked_add(*counter, t.bytes);
        if (!is_planar_v3_kind(t.kind)) continue;
        require(t.source_dimensions.size() >= 2, "planar v3 tensor without expert dimensions");
        const tsp_planar_spec spec = expert_spec(t.source_type, t.source_dimensions[0], t.source_dimensions[1]);
        const uint64_t per_expert = checked_add(spec.planar_expert_bytes, checked_mul(spec.source_expert_bytes, 2));
        buffers = std::max(buffers, checked_mul(per_expert, uint64_t(experts_per_chunk) * (is_coloc_gate_kind(t.kind) ? 2 : 1)));
    }
    report.streaming_ring_buffer_bytes = buffers;
    report.reserve_satisfied = derived_pack::check_disk_reserve(report.filesystem_available_bytes, plan.file_bytes, reserve_bytes);
    report.free_after_pack_v3_bytes = report.filesystem_available_bytes >= plan.file_bytes ? report.filesystem_available_bytes - plan.file_bytes : 0;
    report.ram_ceiling_satisfied = buffers <= report.streaming_ram_ceiling_bytes;
    return report;
}
BudgetReportV3 measure_pack_v3_budget(const ModelFiles& source, const ModelFiles* sidecar, const std::filesystem::path& output_directory,
                                      const std::filesystem::path& existing_pack_v2_path, uint32_t experts_per_chunk, uint64_t reserve_bytes) {
    return measure_pack_v3_budget(plan_derived_pack_v3(source, sidecar), output_directory, existing_pack_v2_path, experts_per_chunk, reserve_bytes,
                                  derived_pack::default_chunk_bytes);
}

PackPlanV3 build_pack_v3_from_plan(PackPlanV3 plan, std::shared_ptr<const ModelFiles> source, std::shared_ptr<const ModelFiles> sidecar,
                                   const std::filesystem::path& output, uint32_t experts_per_chunk, uint64_t reserve_bytes, uint64_t chunk_bytes,
                                   void (*check_cancelled)()) {
    require(bool(source), "missing source model files for pack v3");
    require(experts_per_chunk >= 1 && experts_per_chunk <= 64, "experts_per_chunk must be in 1..64");
    require(chunk_bytes >= 32'768 && chunk_bytes <= 67'108'864, "invalid chunk_bytes bound");
    Location where(output);
    require(!where.exists(), "pack v3 output already exists");
    require(derived_pack::check_disk_reserve(where.available_bytes(), plan.file_bytes, reserve_bytes),
            "insufficient disk space: cannot satisfy pack v3 allocation + reserve");
    Temporary tmp(where.directory);
    const Bytes first_header = build_header_v3(plan);
    write_at(tmp.fd, first_header, 0);
    uint64_t end = first_header.size();
    const auto pad_to = [&](uint64_t target) {
        require(target >= end && target - end < derived_pack::pack_alignment, "nonmonotonic pack v3 write cursor");
        if (target > end) write_at(tmp.fd, Bytes(size_t(target - end), std::byte(0)), end);
        end = target;
    };
    // one chunk: written, read back from the file, and what was read back is what gets unpacked, compared and hashed
    const auto commit = [&](std::span<const std::byte> chunk, std::span<std::byte> readback) {
        if (check_cancelled) check_cancelled();  // throws to cancel: the temporary goes with its owner
        write_at(tmp.fd, chunk, end);
        read_into(tmp.fd, readback, end);
        end = checked_add(end, chunk.size());
    };
    for (size_t i = 0; i < plan.tensors.size(); ++i) {
        source->assert_unchanged();
        if (sidecar) sidecar->assert_unchanged();
        PackTensorV3& t = plan.tensors[i];
        require(derived_pack::check_disk_reserve(where.available_bytes(), plan.file_bytes - end, reserve_bytes),
                "disk space dropped below reserve during pack v3 streaming");
        if (is_coloc_gate_kind(t.kind)) {
            require(i + 1 < plan.tensors.size() && is_coloc_up_kind(plan.tensors[i + 1].kind) && plan.tensors[i + 1].partner_name == t.name &&
                        t.partner_name == plan.tensors[i + 1].name,
                    "co-located gate tensor missing adjacent up partner in plan");
            PackTensorV3& t_up = plan.tensors[i + 1];
            const auto gate = find_bytes(*source, sidecar.get(), t.name), up = find_bytes(*source, sidecar.get(), t_up.name);
            const tsp_planar_spec spec = expert_spec(t.source_type, t.source_dimensions[0], t.source_dimensions[1]);
            const uint32_t experts = uint32_t(t.source_dimensions[2]), half = experts / 2, step = std::min(experts_per_chunk, half);
            require(gate.size() == checked_mul(spec.source_expert_bytes, experts) && up.size() == gate.size(), "pack v3 source dimensions mismatch");
            Sha256 source_digest[2], packed_digest[2];  // [gate, up] and [pair_lo, pair_hi]
            Bytes packed(static_cast<size_t>(checked_mul(spec.planar_expert_bytes * 2, step))), readback(packed.size()), restored(static_cast<size_t>(spec.source_expert_bytes));
            for (uint32_t h = 0; h < 2; ++h) {
                pad_to(checked_add(plan.data_offset, (h ? t_up : t).offset));
                for (uint32_t e = h * half; e < (h + 1) * half;) {
                    const uint32_t count = std::min(step, (h + 1) * half - e);
                    const size_t bytes = size_t(count) * 2 * spec.planar_expert_bytes;
                    for (uint32_t k = 0; k < 2 * count; ++k) {  // [gate e, up e, gate e+1, ...]
                        const auto in = (k & 1 ? up : gate).subspan(size_t((e + k / 2) * spec.source_expert_bytes), size_t(spec.source_expert_bytes));
                        abi(tsp_pack_expert_planar_v3(&spec, u8(in), in.size(), u8(std::span(packed)) + size_t(k) * spec.planar_expert_bytes, spec.planar_expert_bytes));
                        source_digest[k & 1].add(in);
                    }
                    commit(std::span<const std::byte>(packed.data(), bytes), std::span(readback.data(), bytes));
                    for (uint32_t k = 0; k < 2 * count; ++k) {
                        abi(tsp_unpack_expert_planar_v3(&spec, u8(std::span<const std::byte>(readback)) + size_t(k) * spec.planar_expert_bytes,
                                                        spec.planar_expert_bytes, u8(std::span(restored)), restored.size()));
                        const auto in = (k & 1 ? up : gate).subspan(size_t((e + k / 2) * spec.source_expert_bytes), size_t(spec.source_expert_bytes));
                        require(same(in, restored), "co-located gate/up planar v3 inverse byte proof failed");
                    }
                    packed_digest[h].add(std::span<const std::byte>(readback.data(), bytes));
                    e += count;
                }
            }
            t.source_sha256 = source_digest[0].finish();
            t_up.source_sha256 = source_digest[1].finish();
            t.packed_sha256 = packed_digest[0].finish();
            t_up.packed_sha256 = packed_digest[1].finish();
            ++i;
            continue;
        }
        pad_to(checked_add(plan.data_offset, t.offset));
        const auto original = find_bytes(*source, sidecar.get(), t.name);
        require(original.size() == t.source_bytes, "pack v3 source tensor size changed since planning");
        Sha256 source_digest, packed_digest;
        if (t.kind == PlanarKind::q51_planar_v3 || t.kind == PlanarKind::q8_planar_v3) {
            const tsp_planar_spec spec = expert_spec(t.source_type, t.source_dimensions[0], t.source_dimensions[1]);
            const uint32_t experts = uint32_t(t.source_dimensions[2]), step = std::min(experts_per_chunk, experts);
            Bytes packed(static_cast<size_t>(checked_mul(spec.planar_expert_bytes, step))), readback(packed.size()), restored(static_cast<size_t>(spec.source_expert_bytes));
            for (uint32_t e = 0; e < experts;) {
                const uint32_t count = std::min(step, experts - e);
                const size_t bytes = size_t(count) * spec.planar_expert_bytes;
                for (uint32_t k = 0; k < count; ++k) {
                    const auto in = original.subspan(size_t((e + k) * spec.source_expert_bytes), size_t(spec.source_expert_bytes));
                    abi(tsp_pack_expert_planar_v3(&spec, u8(in), in.size(), u8(std::span(packed)) + size_t(k) * spec.planar_expert_bytes, spec.planar_expert_bytes));
                    source_digest.add(in);
                }
                commit(std::span<const std::byte>(packed.data(), bytes), std::span(readback.data(), bytes));
                for (uint32_t k = 0; k < count; ++k) {
                    abi(tsp_unpack_expert_planar_v3(&spec, u8(std::span<const std::byte>(readback)) + size_t(k) * spec.planar_expert_bytes,
                                                    spec.planar_expert_bytes, u8(std::span(restored)), restored.size()));
                    require(same(original.subspan(size_t((e + k) * spec.source_expert_bytes), size_t(spec.source_expert_bytes)), restored),
                            "down planar v3 inverse byte proof failed");
                }
                packed_digest.add(std::span<const std::byte>(readback.data(), bytes));
                e += count;
            }
        } else {
            const bool lanes = t.kind == PlanarKind::q8_lanes_v1;
            const uint32_t columns = uint32_t(t.source_dimensions[0]);
            const uint64_t row_bytes = lanes ? uint64_t(columns / 32) * 34 : 1;
            const uint64_t step = chunk_bytes / row_bytes * row_bytes;  // whole rows for the lane layout
            require(step > 0, "chunk_bytes smaller than single Q8 lane row");
            Bytes packed(lanes ? static_cast<size_t>(step) : 0), readback(static_cast<size_t>(step)), restored(lanes ? static_cast<size_t>(step) : 0);
            for (uint64_t at = 0; at < t.bytes;) {
                const size_t n = size_t(std::min(step, t.bytes - at));
                const auto in = original.subspan(size_t(at), n);
                if (lanes) {
                    abi(tsp_q8_lanes_pack_rows(columns, u8(in), u8(std::span(packed)), n));
                    commit(std::span<const std::byte>(packed.data(), n), std::span(readback.data(), n));
                    abi(tsp_q8_lanes_unpack_rows(columns, u8(std::span<const std::byte>(readback)), u8(std::span(restored)), n));
                    require(same(in, std::span<const std::byte>(restored.data(), n)), "q8_lanes_v1 inverse byte proof failed in pack v3");
                } else {
                    commit(in, std::span(readback.data(), n));
                    require(same(in, std::span<const std::byte>(readback.data(), n)), "plain tensor readback byte proof failed in pack v3");
                }
                source_digest.add(in);
                packed_digest.add(std::span<const std::byte>(readback.data(), n));
                at += n;
            }
        }
        t.source_sha256 = source_digest.finish();
        t.packed_sha256 = packed_digest.finish();
    }
    require(end == plan.file_bytes, "pack v3 final byte size mismatch");
    if (check_cancelled) check_cancelled();
    const Bytes final_header = build_header_v3(plan);
    require(final_header.size() == first_header.size(), "pack v3 manifest changed header size");
    write_at(tmp.fd, final_header, 0);
    require(read_at(tmp.fd, final_header.size(), 0) == final_header, "pack v3 header readback mismatch");
    require(::fchmod(tmp.fd, 0444) == 0 && ::fsync(tmp.fd) == 0, "pack v3 chmod/fsync failed");
    source->assert_unchanged();
    if (sidecar) sidecar->assert_unchanged();
    // published under its name only if nothing is there: never replaces a file
    require(::syscall(SYS_renameat2, where.directory, tmp.name.c_str(), where.directory, where.name.c_str(), 1u /* RENAME_NOREPLACE */) == 0,
            "exclusive pack v3 publication refused");
    tmp.published = true;
    require(::fsync(where.directory) == 0, "directory fsync failed after pack v3 publication");
    return plan;
}

PackPlanV3 build_derived_pack_v3(std::shared_ptr<const ModelFiles> source, std::shared_ptr<const ModelFiles> sidecar, const std::filesystem::path& output,
                                 uint32_t experts_per_chunk, uint64_t reserve_bytes, uint64_t chunk_bytes, void (*check_cancelled)()) {
    require(bool(source), "missing source model files for pack v3");
    auto plan = plan_derived_pack_v3(*source, sidecar.get());
    return build_pack_v3_from_plan(std::move(plan), std::move(source), std::move(sidecar), output, experts_per_chunk, reserve_bytes, chunk_bytes,
                                   check_cancelled);
}
PackPlanV3 build_block_pack_v3(std::shared_ptr<const ModelFiles> source, std::shared_ptr<const ModelFiles> sidecar, uint32_t block_id,
                               const std::filesystem::path& output, uint32_t experts_per_chunk, uint64_t reserve_bytes, uint64_t chunk_bytes,
                               void (*check_cancelled)()) {
    require(bool(source), "missing source model files for pack v3");
    auto plan = plan_block_pack_v3(*source, sidecar.get(), block_id);
    return build_pack_v3_from_plan(std::move(plan), std::move(source), std::move(sidecar), output, experts_per_chunk, reserve_bytes, chunk_bytes,
                                   check_cancelled);
}

namespace {
// src/planar_pack_v3.cpp:501-551: the file's metadata must be exactly the five pack keys, and every manifest entry must
// agree with the expected plan; the digests are taken from the manifest (and proven afterwards).
void manifest_into_plan(PackPlanV3& plan, const Gguf& file) {
    const std::pair<const char*, uint32_t> keys[] = {{"general.architecture", 8}, {"general.alignment", 4}, {"tokspur_pack.version", 4},
                                                     {"tokspur_pack.recipe", 8}, {"tokspur_pack.manifest", 8}};
    require(file.metadata().size() == std::size(keys), "unexpected metadata entries in pack v3 GGUF");
    for (const auto& [key, type] : keys) {
        const Metadata* m = file.find(key);
        require(m && m->type == type, "wrong pack v3 GGUF metadata type");
    }
    require(file.string_value("general.architecture") == derived_pack::pack_architecture &&
                file.unsigned_value("general.alignment") == derived_pack::pack_alignment && file.unsigned_value("tokspur_pack.version") == plan.version &&
                file.string_value("tokspur_pack.recipe") == plan.recipe,
            "stale or incompatible pack v3 metadata");
    const JsonValue manifest = parse_manifest(file.string_value("tokspur_pack.manifest"));
    const JsonValue* entries = manifest.find("tensors");
    require(entries && entries->kind == JsonValue::list, "pack v3 manifest missing tensors array");
    require(entries->items.size() == plan.tensors.size(), "pack v3 manifest tensor count mismatch");
    for (size_t i = 0; i < plan.tensors.size(); ++i) {
        const JsonValue& v = entries->items[i];
        PackTensorV3& t = plan.tensors[i];
        const auto text_is = [&](const char* key, std::string_view want) { const JsonValue* p = v.find(key); return p && p->kind == JsonValue::text && p->s == want; };
        const auto number_is = [&](const char* key, uint64_t want) { const JsonValue* p = v.find(key); return p && p->kind == JsonValue::number && p->n == want; };
        require(text_is("name", t.name), "pack v3 manifest tensor name mismatch");
        require(number_is("type", t.type), "pack v3 manifest tensor type mismatch");
        require(number_is("source_type", t.source_type), "pack v3 manifest source_type mismatch");
        require(text_is("layout", t.layout), "pack v3 manifest layout mismatch");
        require(number_is("source_bytes", t.source_bytes), "pack v3 manifest source_bytes mismatch");
        require(number_is("bytes", t.bytes), "pack v3 manifest bytes mismatch");
        require(number_is("offset", t.offset), "pack v3 manifest offset mismatch");
        const JsonValue *a = v.find("source_sha256"), *b = v.find("packed_sha256");
        require(a && b && a->kind == JsonValue::text && b->kind == JsonValue::text && a->s.size() == 64 && b->s.size() == 64,
                "pack v3 manifest missing SHA-256 digests");
        t.source_sha256 = a->s;
        t.packed_sha256 = b->s;
    }
}
}  // namespace

AdoptedPackV3 adopt_pack_v3_with_plan(PackPlanV3 plan, std::shared_ptr<const ModelFiles> source, std::shared_ptr<const ModelFiles> sidecar,
                                      const std::filesystem::path& path, uint32_t experts_per_chunk, uint64_t chunk_bytes, uint32_t authentication_workers,
                                      derived_pack::TrustMode) {
    require(bool(source), "missing source model files");
    require(authentication_workers >= 1 && authentication_workers <= derived_pack::max_authentication_workers, "authentication_workers must be in 1..16");
    require(experts_per_chunk >= 1 && experts_per_chunk <= 64, "experts_per_chunk must be in 1..64");
    require(chunk_bytes >= 32'768 && chunk_bytes <= 67'108'864, "invalid chunk_bytes bound");
    Location where(path);
    Fd fd(::openat(where.directory, where.name.c_str(), O_RDONLY | O_CLOEXEC | O_NOFOLLOW | O_NONBLOCK));
    struct stat before{};
    require(::fstat(fd.value, &before) == 0 && S_ISREG(before.st_mode) && !(before.st_mode & 0222) && before.st_nlink == 1 && before.st_size > 0,
            "pack v3 must be an immutable regular file");
    // mapped through the descriptor that was just checked, not through the name again
    auto model = std::make_shared<ModelFiles>(std::vector<std::filesystem::path>{"/dev/fd/" + std::to_string(fd.value)});
    require(model->architecture() == derived_pack::pack_architecture && model->shards().size() == 1, "adopted file is not a valid tokspur_pack GGUF");
    const Gguf& file = model->shards()[0];
    require(uint64_t(before.st_size) == plan.file_bytes, "pack v3 must be an immutable regular file of exact planned size");
    manifest_into_plan(plan, file);
    const Bytes canonical = build_header_v3(plan);
    require(file.data_offset() == canonical.size() && read_at(fd.value, canonical.size(), 0) == canonical, "noncanonical or corrupt pack v3 header");

    std::vector<size_t> units;  // a co-located pair is verified as one unit, led by its gate tensor
    for (size_t i = 0; i < plan.tensors.size(); ++i) if (!is_coloc_up_kind(plan.tensors[i].kind)) units.push_back(i);
    const auto directory_agrees = [&](const PackTensorV3& t) {
        const Tensor& m = model->tensor(t.name);
        return m.type == t.type && m.dimensions == t.dimensions && m.bytes == t.bytes && m.offset == checked_add(canonical.size(), t.offset);
    };
    const auto padding_after_is_zero = [&](size_t i) {
        if (i + 1 >= plan.tensors.size()) return;
        const uint64_t end = checked_add(plan.tensors[i].offset, plan.tensors[i].bytes), next = plan.tensors[i + 1].offset;
        if (next <= end) return;
        const Bytes pad = read_at(fd.value, size_t(next - end), checked_add(canonical.size(), end));
        require(std::all_of(pad.begin(), pad.end(), [](std::byte b) { return b == std::byte(0); }), "nonzero padding between pack v3 tensors");
    };
    const auto unchanged = [&] {
        source->assert_unchanged();
        if (sidecar) sidecar->assert_unchanged();
        model->assert_unchanged();
    };
    const auto verify = [&](size_t i) {
        const PackTensorV3& t = plan.tensors[i];
        require(directory_agrees(t), "pack v3 tensor directory metadata mismatch");
        if (is_coloc_gate_kind(t.kind)) {
            require(i + 1 < plan.tensors.size() && is_coloc_up_kind(plan.tensors[i + 1].kind), "missing co-located up tensor during pack v3 adoption");
            const PackTensorV3& t_up = plan.tensors[i + 1];
            require(directory_agrees(t_up), "pack v3 co-located up tensor metadata mismatch");
            const auto gate = find_bytes(*source, sidecar.get(), t.name), up = find_bytes(*source, sidecar.get(), t_up.name);
            const auto lo = model->tensor_bytes(t.name), hi = model->tensor_bytes(t_up.name);
            // the manifest's geometry is not trusted until it accounts for every packed and source byte
            require(t.source_dimensions.size() == 3 && t.source_dimensions[2] != 0 && t.source_dimensions[2] <= UINT32_MAX, "pack v3 source dimensions mismatch");
            const tsp_planar_spec spec = expert_spec(t.source_type, t.source_dimensions[0], t.source_dimensions[1]);
            const uint32_t experts = uint32_t(t.source_dimensions[2]), half = experts / 2;
            require(checked_mul(uint64_t(2) * half, spec.planar_expert_bytes) == lo.size() &&
                        checked_mul(uint64_t(2) * (experts - half), spec.planar_expert_bytes) == hi.size() &&
                        checked_mul(experts, spec.source_expert_bytes) == gate.size() && gate.size() == up.size(),
                    "pack v3 source dimensions mismatch");
            Sha256 source_digest[2], packed_digest[2];
            Bytes restored(static_cast<size_t>(spec.source_expert_bytes));
            for (uint32_t e = 0; e < experts; ++e) {
                unchanged();
                const uint32_t h = e < half ? 0 : 1, local = e - h * half;
                for (uint32_t k = 0; k < 2; ++k) {  // gate, then up
                    const auto packed = (h ? hi : lo).subspan(size_t((2 * local + k) * spec.planar_expert_bytes), size_t(spec.planar_expert_bytes));
                    abi(tsp_unpack_expert_planar_v3(&spec, u8(packed), packed.size(), u8(std::span(restored)), restored.size()));
                    const auto in = (k ? up : gate).subspan(size_t(e * spec.source_expert_bytes), size_t(spec.source_expert_bytes));
                    require(same(in, restored), "pack v3 adoption co-located gate/up inverse byte proof failed");
                    source_digest[k].add(in);
                    packed_digest[h].add(packed);
                }
            }
            require(source_digest[0].finish() == t.source_sha256 && source_digest[1].finish() == t_up.source_sha256 &&
                        packed_digest[0].finish() == t.packed_sha256 && packed_digest[1].finish() == t_up.packed_sha256,
                    "stale source or corrupt co-located tensor digest in pack v3");
            padding_after_is_zero(i);
            padding_after_is_zero(i + 1);
            return;
        }
        const auto original = find_bytes(*source, sidecar.get(), t.name);
        const auto packed = model->tensor_bytes(t.name);
        require(original.size() == t.source_bytes, "pack v3 source dimensions mismatch");
        Sha256 source_digest, packed_digest;
        if (t.kind == PlanarKind::q51_planar_v3 || t.kind == PlanarKind::q8_planar_v3) {
            require(t.source_dimensions.size() == 3 && t.source_dimensions[2] != 0 && t.source_dimensions[2] <= UINT32_MAX, "pack v3 source dimensions mismatch");
            const tsp_planar_spec spec = expert_spec(t.source_type, t.source_dimensions[0], t.source_dimensions[1]);
            const uint32_t experts = uint32_t(t.source_dimensions[2]);
            require(checked_mul(experts, spec.planar_expert_bytes) == packed.size() && checked_mul(experts, spec.source_expert_bytes) == t.source_bytes,
                    "pack v3 source dimensions mismatch");
            Bytes restored(static_cast<size_t>(spec.source_expert_bytes));
            for (uint32_t e = 0; e < experts; ++e) {
                unchanged();
                const auto planes = packed.subspan(size_t(e * spec.planar_expert_bytes), size_t(spec.planar_expert_bytes));
                abi(tsp_unpack_expert_planar_v3(&spec, u8(planes), planes.size(), u8(std::span(restored)), restored.size()));
                const auto in = original.subspan(size_t(e * spec.source_expert_bytes), size_t(spec.source_expert_bytes));
                require(same(in, restored), "pack v3 adoption down inverse byte proof failed");
                source_digest.add(in);
                packed_digest.add(planes);
            }
        } else {
            const bool lanes = t.kind == PlanarKind::q8_lanes_v1;
            require(packed.size() == original.size() && !t.source_dimensions.empty() && t.source_dimensions[0] <= 65536, "pack v3 source dimensions mismatch");
            const uint32_t columns = uint32_t(t.source_dimensions[0]);
            const uint64_t row_bytes = lanes ? uint64_t(columns / 32) * 34 : 1, step = chunk_bytes / std::max<uint64_t>(row_bytes, 1) * row_bytes;
            require(row_bytes && step > 0 && (!lanes || t.bytes % row_bytes == 0), "chunk_bytes smaller than single Q8 lane row");
            Bytes restored(lanes ? static_cast<size_t>(step) : 0);
            for (uint64_t at = 0; at < t.bytes;) {
                unchanged();
                const size_t n = size_t(std::min(step, t.bytes - at));
                const auto in = original.subspan(size_t(at), n), chunk = packed.subspan(size_t(at), n);
                if (lanes) {
                    abi(tsp_q8_lanes_unpack_rows(columns, u8(chunk), u8(std::span(restored)), n));
                    require(same(in, std::span<const std::byte>(restored.data(), n)), "pack v3 adoption q8_lanes_v1 inverse proof failed");
                } else {
                    require(same(in, chunk), "pack v3 adoption plain tensor byte proof failed");
                }
                source_digest.add(in);
                packed_digest.add(chunk);
                at += n;
            }
        }
        require(source_digest.finish() == t.source_sha256 && packed_digest.finish() == t.packed_sha256, "stale source or corrupt tensor digest in pack v3");
        padding_after_is_zero(i);
    };

    const uint32_t workers = std::max<uint32_t>(1, std::min<uint32_t>(authentication_workers, uint32_t(units.size())));
    if (workers == 1) {
        for (const size_t i : units) verify(i);
    } else {
        std::atomic<size_t> next{0};
        std::vector<std::exception_ptr> failures(units.size());
        const auto work = [&] {
            for (size_t u; (u = next.fetch_add(1, std::memory_order_relaxed)) < units.size();) {
                try { verify(units[u]); } catch (...) { failures[u] = std::current_exception(); }
            }
        };
        std::vector<std::thread> pool;
        for (uint32_t w = 1; w < workers; ++w) pool.emplace_back(work);
        work();
        for (auto& t : pool) t.join();
        for (const auto& f : failures) if (f) std::rethrow_exception(f);
    }
    unchanged();
    struct stat after{};
    require(::fstat(fd.value, &after) == 0 && before.st_dev == after.st_dev && before.st_ino == after.st_ino && before.st_size == after.st_size &&
                before.st_mode == after.st_mode && before.st_nlink == after.st_nlink,
            "pack v3 file identity changed during adoption");
    std::string digest = derived_pack::hash(file.string_value("tokspur_pack.manifest"));
    return {std::move(model), std::move(plan), std::move(digest), workers};
}

AdoptedPackV3 adopt_derived_pack_v3(std::shared_ptr<const ModelFiles> source, std::shared_ptr<const ModelFiles> sidecar, const std::filesystem::path& path,
                                    uint32_t experts_per_chunk, uint64_t chunk_bytes, uint32_t authentication_workers, derived_pack::TrustMode trust) {
    require(bool(source), "missing source model files");
    auto plan = plan_derived_pack_v3(*source, sidecar.get());
    return adopt_pack_v3_with_plan(std::move(plan), std::move(source), std::move(sidecar), path, experts_per_chunk, chunk_bytes, authentication_workers, trust);
}
AdoptedPackV3 adopt_block_pack_v3(std::shared_ptr<const ModelFiles> source, std::shared_ptr<const ModelFiles> sidecar, uint32_t block_id,
                                  const std::filesystem::path& path, uint32_t experts_per_chunk, uint64_t chunk_bytes, uint32_t authentication_workers) {
    require(bool(source), "missing source model files");
    auto plan = plan_block_pack_v3(*source, sidecar.get(), block_id);
    return adopt_pack_v3_with_plan(std::move(plan), std::move(source), std::move(sidecar), path, experts_per_chunk, chunk_bytes, authentication_workers,
                                   derived_pack::TrustMode::full);
}

PackMoeBlockV3 upload_moe_block_v3(HipGraph& graph, const AdoptedPackV3& pack, uint32_t block_id) {
    require(bool(pack.model), "pack v3 is not adopted");
    const std::string stem = "blk." + std::to_string(block_id) + ".ffn_";
    const PackTensorV3 *gate = nullptr, *up = nullptr, *down = nullptr;
    for (const auto& t : pack.plan.tensors) {
        if (t.name == stem + "gate_exps.weight") gate = &t;
        if (t.name == stem + "up_exps.weight") up = &t;
        if (t.name == stem + "down_exps.weight") down = &t;
    }
    require(gate && up && down, "pack v3 holds no routed experts for this block");
    require(is_coloc_gate_kind(gate->kind) && is_coloc_up_kind(up->kind) && uint32_t(up->kind) == uint32_t(gate->kind) + 1 &&
                (down->kind == PlanarKind::q51_planar_v3 || down->kind == PlanarKind::q8_planar_v3),
            "pack v3 block is not in planar form");
    require(gate->source_dimensions.size() == 3 && down->source_dimensions.size() == 3 && gate->source_dimensions == up->source_dimensions &&
                down->source_dimensions[0] == gate->source_dimensions[1] && down->source_dimensions[1] == gate->source_dimensions[0] &&
                down->source_dimensions[2] == gate->source_dimensions[2] && gate->source_dimensions[2] <= 4096,
            "pack v3 block geometry mismatch");
    PackMoeBlockV3 out;
    out.channels = uint32_t(gate->source_dimensions[0]);
    out.hidden = uint32_t(gate->source_dimensions[1]);
    out.experts = uint32_t(gate->source_dimensions[2]);
    const auto put = [&](const PackTensorV3& t, uint32_t columns, uint32_t rows) {
        const GpuView view = graph.upload(pack.model->tensor_bytes(t.name), t.name);
        graph.register_planar_matrix(view, {t.source_type, uint32_t(t.kind), columns, rows, out.experts});
        return GpuMatrix{view, t.source_type};
    };
    out.gate = put(*gate, out.channels, out.hidden);
    out.up = put(*up, out.channels, out.hidden);
    out.down = put(*down, out.hidden, out.channels);
    return out;
}

}  // namespace planar_v3
}  // namespace tokspur
