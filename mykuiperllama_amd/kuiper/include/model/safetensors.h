// Checkpoint reader for the matmul operator: a safetensors file (8-byte little-endian header
// length, a JSON header {"name": {"dtype", "shape", "data_offsets"}, ...}, then the raw tensor
// bytes) is mapped read-only and its tensors are attached to MatmulLayer objects.
//
// The reference has no loader: its CMake lists kuiper/source/model/ (CMakeLists.txt:79), the
// directory is absent, and the only way weights enter a layer is LayerParam::set_weight /
// set_scales (kuiper/source/op/layer.cpp:245-283).  This fills that hole for the tensors the
// quantised matmul needs, in the checkpoint layout the kernels consume as it lies on disk:
//   <prefix>.qweight  I32 [K, N/8]     <prefix>.qzeros  I32 [K/G, N/8]     <prefix>.scales  F16 [K/G, N]
//   <name>            BF16 [N, K]      for an unquantised layer
#ifndef KUIPER_INCLUDE_MODEL_SAFETENSORS_H
#define KUIPER_INCLUDE_MODEL_SAFETENSORS_H

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "base/base.h"
#include "op/matmul.h"

namespace model {

struct TensorEntry {
    std::string name;
    std::string dtype;           // "I32", "F16", "BF16", "F32", ... as written in the file
    std::vector<int64_t> shape;
    size_t begin = 0;            // byte range inside the data section
    size_t end = 0;

    size_t byte_size() const { return end - begin; }
    int64_t element_count() const;
};

// Bytes per element of a safetensors dtype string; 0 for one this reader does not know.
size_t dtype_size(const std::string& dtype);

class SafetensorsFile {
public:
    SafetensorsFile() = default;
    ~SafetensorsFile();
    SafetensorsFile(const SafetensorsFile&) = delete;
    SafetensorsFile& operator=(const SafetensorsFile&) = delete;

    // Maps the file and parses its header.  Every entry is validated: known dtype, byte range
    // inside the file and equal to shape x element size.  A failure leaves the object closed.
    base::Status open(const std::string& path);
    void close();
    bool is_open() const { return map_ != nullptr; }

    const std::vector<TensorEntry>& entries() const { return entries_; }  // in file order
    const TensorEntry* find(const std::string& name) const;
    const void* data(const TensorEntry& entry) const;  // valid while the file is open
    const std::map<std::string, std::string>& metadata() const { return metadata_; }

private:
    void* map_ = nullptr;
    size_t map_bytes_ = 0;
    size_t data_start_ = 0;
    std::vector<TensorEntry> entries_;
    std::map<std::string, size_t> index_;
    std::map<std::string, std::string> metadata_;
};

// Attaches <prefix>.qweight / .qzeros / .scales to an AWQ MatmulLayer.  Shapes must agree with the
// layer's dim0 (N), dim1 (K) and group size.  The tensors are copied into memory of the layer's
// device (one allocation each through the device's allocator), so the file may be closed afterwards.
base::Status load_awq_linear(const SafetensorsFile& file, const std::string& prefix, op::MatmulLayer& layer);

// The same for several projections that share their input, laid side by side along N (q|k|v,
// gate|up): row k of the fused tensor is row k of the first, then of the second, ...  The layer's
// dim0 must be the sum of the parts' N.  Words are copied whole, so the order of the nibbles inside
// a word is untouched.
base::Status load_awq_linear_fused(const SafetensorsFile& file, const std::vector<std::string>& prefixes,
                                   op::MatmulLayer& layer);

// Attaches a BF16 [N, K] tensor to an unquantised MatmulLayer.
base::Status load_bf16_linear(const SafetensorsFile& file, const std::string& name, op::MatmulLayer& layer);

// A tensor of the given shape as bf16 in memory of `device` (norm gains, embedding table).  BF16 on
// file is copied; F16 and F32 are rounded to bf16 (nearest, ties to even) on the way.
base::Status load_bf16_tensor(const SafetensorsFile& file, const std::string& name, const std::vector<int32_t>& dims,
                              base::DeviceType device, tensor::Tensor& out);

}  // namespace model

#endif  // KUIPER_INCLUDE_MODEL_SAFETENSORS_H
