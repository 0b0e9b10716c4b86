// Helpers shared by the C++ tests that need a safetensors file: tensors are written byte by byte
// to the format's definition (u64 header length, JSON header, raw data), independently of the
// reader under test.
#ifndef KX_TESTS_SAFETENSORS_WRITER_H
#define KX_TESTS_SAFETENSORS_WRITER_H

#include <unistd.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "mini_test.h"

namespace stw {

struct Rng {  // SplitMix64
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed) {}
    uint64_t next() {
        uint64_t z = (s += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    double uniform() { return double(next() >> 11) * (1.0 / 9007199254740992.0); }
    double normal() { return std::sqrt(-2.0 * std::log(1.0 - uniform())) * std::cos(6.283185307179586 * uniform()); }
};

struct Blob {
    std::string name, dtype;
    std::vector<int64_t> shape;
    std::vector<uint8_t> bytes;
};

template <typename T>
Blob blob(const std::string& name, const std::string& dtype, std::vector<int64_t> shape, const std::vector<T>& v) {
    Blob b{name, dtype, std::move(shape), {}};
    b.bytes.resize(v.size() * sizeof(T));
    std::memcpy(b.bytes.data(), v.data(), b.bytes.size());
    return b;
}

// A temporary file that disappears with the object.
struct TempFile {
    std::string path;
    TempFile() {
        char name[] = "/tmp/kx_safetensors_XXXXXX";
        const int fd = mkstemp(name);
        if (fd >= 0) close(fd);
        path = name;
    }
    ~TempFile() { std::remove(path.c_str()); }
    void write(const std::string& bytes) const {
        FILE* f = std::fopen(path.c_str(), "wb");
        ASSERT_TRUE(f != nullptr);
        ASSERT_EQ(std::fwrite(bytes.data(), 1, bytes.size(), f), bytes.size());
        std::fclose(f);
    }
};

inline std::string with_length_prefix(const std::string& header, const std::string& data) {
    std::string out(8, '\0');
    uint64_t n = header.size();
    for (int i = 0; i < 8; i++) out[i] = char((n >> (8 * i)) & 0xFF);
    return out + header + data;
}

// header length (u64 LE) | JSON | tensor bytes, entries in the given order, back to back
inline std::string serialise(const std::vector<Blob>& blobs, const std::string& metadata_json = "") {
    std::string header = "{";
    std::string data;
    if (!metadata_json.empty()) header += "\"__metadata__\":" + metadata_json + ",";
    for (size_t i = 0; i < blobs.size(); i++) {
        const Blob& b = blobs[i];
        header += (i ? ",\"" : "\"") + b.name + "\":{\"dtype\":\"" + b.dtype + "\",\"shape\":[";
        for (size_t d = 0; d < b.shape.size(); d++) header += (d ? "," : "") + std::to_string(b.shape[d]);
        header += "],\"data_offsets\":[" + std::to_string(data.size()) + "," +
                  std::to_string(data.size() + b.bytes.size()) + "]}";
        data.append(reinterpret_cast<const char*>(b.bytes.data()), b.bytes.size());
    }
    header += "}";
    while ((header.size() + 8) % 8) header += ' ';  // writers pad the header with spaces
    return with_length_prefix(header, data);
}

}  // namespace stw

#endif  // KX_TESTS_SAFETENSORS_WRITER_H
