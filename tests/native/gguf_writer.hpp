// A writer of small GGUF v3 shards for tests (the engine's tests build theirs the same way,
// tests/test_planar_pack_v3.cpp:60-141): header, two metadata entries, a tensor directory, payloads at 32-byte alignment.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <filesystem>
#include <unistd.h>
#include <cstdlib>
#include <stdexcept>
#include <algorithm>
#include <fstream>
#include <string>
#include <string_view>
#include <vector>

namespace gguf_writer {

struct TensorSpec {
    std::string name;
    uint32_t type;
    std::vector<uint64_t> dimensions;
    std::vector<uint8_t> payload;
};

inline void put(std::vector<uint8_t>& out, uint64_t value, unsigned width) {
    for (unsigned i = 0; i < width; ++i) out.push_back(uint8_t(value >> (8 * i)));
}
inline void put(std::vector<uint8_t>& out, std::string_view text) {
    put(out, text.size(), 8);
    out.insert(out.end(), text.begin(), text.end());
}

// the whole shard as bytes; `alignment` is written as general.alignment; `directory_offsets` (for tests of refusals)
// replaces the offsets written into the tensor directory while the payloads stay where they belong
inline std::vector<uint8_t> shard_bytes(std::string_view architecture, const std::vector<TensorSpec>& tensors, uint32_t alignment = 32,
                                        const std::vector<uint64_t>* directory_offsets = nullptr) {
    std::vector<uint8_t> file;
    put(file, 0x46554747, 4);
    put(file, 3, 4);
    put(file, tensors.size(), 8);
    put(file, 2, 8);
    put(file, "general.architecture"); put(file, 8, 4); put(file, architecture);
    put(file, "general.alignment"); put(file, 4, 4); put(file, alignment, 4);
    std::vector<uint64_t> offsets;
    uint64_t at = 0;
    for (const auto& t : tensors) {
        at = (at + alignment - 1) / alignment * alignment;
        offsets.push_back(at);
        at += t.payload.size();
    }
    for (size_t i = 0; i < tensors.size(); ++i) {
        put(file, tensors[i].name);
        put(file, tensors[i].dimensions.size(), 4);
        for (const uint64_t d : tensors[i].dimensions) put(file, d, 8);
        put(file, tensors[i].type, 4);
        put(file, directory_offsets ? (*directory_offsets)[i] : offsets[i], 8);
    }
    const uint64_t data = (file.size() + alignment - 1) / alignment * alignment;
    file.resize(size_t(data + at), 0);
    for (size_t i = 0; i < tensors.size(); ++i)
        std::copy(tensors[i].payload.begin(), tensors[i].payload.end(), file.begin() + long(data + offsets[i]));
    return file;
}

inline void write_file(const std::filesystem::path& path, const std::vector<uint8_t>& bytes) {
    std::ofstream out(path, std::ios::binary | std::ios::trunc);
    out.write(reinterpret_cast<const char*>(bytes.data()), long(bytes.size()));
    out.close();
    if (!out) throw std::runtime_error("cannot write " + path.string());
}

struct TempDir {
    std::filesystem::path path;
    explicit TempDir(const std::string& stem) {
        path = std::filesystem::temp_directory_path() / (stem + "_" + std::to_string(::getpid()) + "_" + std::to_string(std::rand()));
        std::filesystem::create_directories(path);
    }
    ~TempDir() {
        std::error_code ec;
        for (const auto& entry : std::filesystem::recursive_directory_iterator(path, ec))
            std::filesystem::permissions(entry.path(), std::filesystem::perms::owner_all, ec);
        std::filesystem::remove_all(path, ec);
    }
};

}  // namespace gguf_writer
