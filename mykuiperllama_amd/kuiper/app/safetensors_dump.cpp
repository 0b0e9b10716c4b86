// kx_safetensors_dump <file>: lists the tensors of a safetensors file as the reader sees them,
// one line each:  name dtype dim0xdim1x... bytes fnv1a64-of-the-bytes
// (what a user runs to see whether a checkpoint has the qweight/qzeros/scales tensors the matmul
// layers expect; the checksums let a test compare the reader with another implementation).
#include <cinttypes>
#include <cstdio>

#include "model/safetensors.h"

int main(int argc, char** argv) {
    if (argc != 2) {
        std::fprintf(stderr, "usage: %s file.safetensors\n", argv[0]);
        return 2;
    }
    model::SafetensorsFile file;
    const base::Status status = file.open(argv[1]);
    if (!status) {
        std::fprintf(stderr, "%s\n", status.get_err_msg().c_str());
        return 1;
    }
    for (const auto& kv : file.metadata()) {
        std::printf("# %s = %s\n", kv.first.c_str(), kv.second.c_str());
    }
    for (const model::TensorEntry& e : file.entries()) {
        uint64_t h = 1469598103934665603ull;
        const unsigned char* p = static_cast<const unsigned char*>(file.data(e));
        for (size_t i = 0; i < e.byte_size(); i++) {
            h ^= p[i];
            h *= 1099511628211ull;
        }
        std::string shape;
        for (size_t i = 0; i < e.shape.size(); i++) {
            shape += (i ? "x" : "") + std::to_string(e.shape[i]);
        }
        if (shape.empty()) shape = "scalar";
        std::printf("%s %s %s %zu %016" PRIx64 "\n", e.name.c_str(), e.dtype.c_str(), shape.c_str(), e.byte_size(), h);
    }
    return 0;
}
