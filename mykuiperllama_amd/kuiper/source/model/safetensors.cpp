// safetensors reader and the AWQ weight attach (see model/safetensors.h).
#include "model/safetensors.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstring>

#include "base/alloc.h"
#include "kernel/cpu/bf16.h"
#include "tensor/tensor.h"

namespace model {
namespace {

// ---------------------------------------------------------------- a JSON reader for the header
// The header is one object whose values are objects of strings and arrays of non-negative
// integers ("__metadata__": string -> string).  The reader accepts general JSON and keeps what
// the format uses.
struct Json {
    enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
    bool boolean = false;
    double number = 0.0;
    bool integral = false;
    uint64_t integer = 0;
    std::string text;
    std::vector<Json> items;
    std::vector<std::pair<std::string, Json>> members;  // in file order
};

class JsonReader {
public:
    JsonReader(const char* p, size_t n) : p_(p), end_(p + n) {}

    bool parse(Json& out, std::string& why) {
        if (!value(out, 0)) {
            why = why_.empty() ? "malformed JSON" : why_;
            return false;
        }
        skip();
        if (p_ != end_) {
            why = "trailing characters after the header object";
            return false;
        }
        return true;
    }

private:
    static constexpr int kMaxDepth = 16;

    void skip() {
        while (p_ < end_ && (*p_ == ' ' || *p_ == '\t' || *p_ == '\n' || *p_ == '\r')) p_++;
    }
    bool fail(const char* why) {
        if (why_.empty()) why_ = why;
        return false;
    }
    bool literal(const char* word) {
        const size_t n = std::strlen(word);
        if (static_cast<size_t>(end_ - p_) < n || std::memcmp(p_, word, n) != 0) return fail("bad literal");
        p_ += n;
        return true;
    }
    static void append_utf8(std::string& s, uint32_t cp) {
        if (cp < 0x80) {
            s.push_back(static_cast<char>(cp));
        } else if (cp < 0x800) {
            s.push_back(static_cast<char>(0xC0 | (cp >> 6)));
            s.push_back(static_cast<char>(0x80 | (cp & 0x3F)));
        } else if (cp < 0x10000) {
            s.push_back(static_cast<char>(0xE0 | (cp >> 12)));
            s.push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3F)));
            s.push_back(static_cast<char>(0x80 | (cp & 0x3F)));
        } else {
            s.push_back(static_cast<char>(0xF0 | (cp >> 18)));
            s.push_back(static_cast<char>(0x80 | ((cp >> 12) & 0x3F)));
            s.push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3F)));
            s.push_back(static_cast<char>(0x80 | (cp & 0x3F)));
        }
    }
    bool hex4(uint32_t& out) {
        if (end_ - p_ < 4) return fail("short \\u escape");
        out = 0;
        for (int i = 0; i < 4; i++) {
            const char c = *p_++;
            out <<= 4;
            if (c >= '0' && c <= '9') out |= static_cast<uint32_t>(c - '0');
            else if (c >= 'a' && c <= 'f') out |= static_cast<uint32_t>(c - 'a' + 10);
            else if (c >= 'A' && c <= 'F') out |= static_cast<uint32_t>(c - 'A' + 10);
            else return fail("bad \\u escape");
        }
        return true;
    }
    bool string(std::string& out) {
        if (p_ >= end_ || *p_ != '"') return fail("expected a string");
        p_++;
        out.clear();
        while (p_ < end_) {
            const char c = *p_++;
            if (c == '"') return true;
            if (static_cast<unsigned char>(c) < 0x20) return fail("control character in a string");
            if (c != '\\') {
                out.push_back(c);
                continue;
            }
            if (p_ >= end_) break;
            const char e = *p_++;
            switch (e) {
                case '"': out.push_back('"'); break;
                case '\\': out.push_back('\\'); break;
                case '/': out.push_back('/'); break;
                case 'b': out.push_back('\b'); break;
                case 'f': out.push_back('\f'); break;
                case 'n': out.push_back('\n'); break;
                case 'r': out.push_back('\r'); break;
                case 't': out.push_back('\t'); break;
                case 'u': {
                    uint32_t cp = 0;
                    if (!hex4(cp)) return false;
                    if (cp >= 0xD800 && cp <= 0xDBFF) {  // surrogate pair
                        uint32_t lo = 0;
                        if (end_ - p_ < 2 || p_[0] != '\\' || p_[1] != 'u') return fail("lone surrogate");
                        p_ += 2;
                        if (!hex4(lo) || lo < 0xDC00 || lo > 0xDFFF) return fail("bad surrogate pair");
                        cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
                    }
                    append_utf8(out, cp);
                    break;
                }
                default: return fail("bad escape");
            }
        }
        return fail("unterminated string");
    }
    bool number(Json& out) {
        const char* start = p_;
        bool integral = true;
        if (p_ < end_ && *p_ == '-') {
            integral = false;
            p_++;
        }
        if (p_ >= end_ || *p_ < '0' || *p_ > '9') return fail("bad number");
        uint64_t acc = 0;
        bool overflow = false;
        while (p_ < end_ && *p_ >= '0' && *p_ <= '9') {
            const uint64_t d = static_cast<uint64_t>(*p_ - '0');
            if (acc > (UINT64_MAX - d) / 10) overflow = true;
            acc = acc * 10 + d;
            p_++;
        }
        if (p_ < end_ && (*p_ == '.' || *p_ == 'e' || *p_ == 'E')) {
            integral = false;
            while (p_ < end_ && (*p_ == '.' || *p_ == 'e' || *p_ == 'E' || *p_ == '+' || *p_ == '-' ||
                                 (*p_ >= '0' && *p_ <= '9'))) {
                p_++;
            }
        }
        out.kind = Json::Number;
        out.integral = integral && !overflow;
        out.integer = acc;
        out.number = std::strtod(std::string(start, p_).c_str(), nullptr);
        return true;
    }
    bool value(Json& out, int depth) {
        if (depth > kMaxDepth) return fail("nesting too deep");
        skip();
        if (p_ >= end_) return fail("unexpected end of header");
        const char c = *p_;
        if (c == '{') {
            p_++;
            out.kind = Json::Object;
            skip();
            if (p_ < end_ && *p_ == '}') {
                p_++;
                return true;
            }
            while (true) {
                skip();
                std::string key;
                if (!string(key)) return false;
                skip();
                if (p_ >= end_ || *p_ != ':') return fail("expected ':'");
                p_++;
                Json member;
                if (!value(member, depth + 1)) return false;
                out.members.emplace_back(std::move(key), std::move(member));
                skip();
                if (p_ < end_ && *p_ == ',') {
                    p_++;
                    continue;
                }
                if (p_ < end_ && *p_ == '}') {
                    p_++;
                    return true;
                }
                return fail("expected ',' or '}'");
            }
        }
        if (c == '[') {
            p_++;
            out.kind = Json::Array;
            skip();
            if (p_ < end_ && *p_ == ']') {
                p_++;
                return true;
            }
            while (true) {
                Json item;
                if (!value(item, depth + 1)) return false;
                out.items.push_back(std::move(item));
                skip();
                if (p_ < end_ && *p_ == ',') {
                    p_++;
                    continue;
                }
                if (p_ < end_ && *p_ == ']') {
                    p_++;
                    return true;
                }
                return fail("expected ',' or ']'");
            }
        }
        if (c == '"') {
            out.kind = Json::String;
            return string(out.text);
        }
        if (c == 't') {
            out.kind = Json::Bool;
            out.boolean = true;
            return literal("true");
        }
        if (c == 'f') {
            out.kind = Json::Bool;
            out.boolean = false;
            return literal("false");
        }
        if (c == 'n') {
            out.kind = Json::Null;
            return literal("null");
        }
        return number(out);
    }

    const char* p_;
    const char* end_;
    std::string why_;
};

const Json* member(const Json& object, const char* key) {
    for (const auto& kv : object.members) {
        if (kv.first == key) return &kv.second;
    }
    return nullptr;
}

base::Status bad_file(const std::string& why) {
    return base::error::model_parse_error("safetensors: " + why);
}

// ---------------------------------------------------------------- tensors on the layer's device
tensor::Tensor device_tensor(base::DataType type, const std::vector<int32_t>& dims, base::DeviceType device,
                             const void* host_src, size_t bytes) {
    std::shared_ptr<base::DeviceAllocator> alloc;
    if (device == base::DeviceType::DeviceCUDA) {
        alloc = base::CUDADeviceAllocatorFactory::get_instance();
    } else {
        alloc = base::CPUDeviceAllocatorFactory::get_instance();
    }
    tensor::Tensor t(type, dims, true, alloc);
    CHECK_EQ(t.byte_size(), bytes);
    const base::MemcpyKind kind = device == base::DeviceType::DeviceCUDA ? base::MemcpyKind::MemcpyCPU2CUDA
                                                                         : base::MemcpyKind::MemcpyCPU2CPU;
    alloc->memcpy(t.ptr<uint8_t>(), host_src, bytes, kind, nullptr, false);
    return t;
}

struct AwqPart {
    const TensorEntry* qweight = nullptr;
    const TensorEntry* qzeros = nullptr;
    const TensorEntry* scales = nullptr;
    int64_t n = 0;  // output features of this part
};

base::Status find_awq_part(const SafetensorsFile& file, const std::string& prefix, int64_t K, int64_t group,
                           AwqPart& part) {
    part.qweight = file.find(prefix + ".qweight");
    part.qzeros = file.find(prefix + ".qzeros");
    part.scales = file.find(prefix + ".scales");
    if (!part.qweight || !part.qzeros || !part.scales) {
        return base::error::path_not_valid("safetensors: " + prefix + ".qweight/.qzeros/.scales not all present");
    }
    if (part.qweight->dtype != "I32" || part.qzeros->dtype != "I32" || part.scales->dtype != "F16") {
        return bad_file(prefix + ": expected I32 qweight, I32 qzeros, F16 scales");
    }
    if (part.qweight->shape.size() != 2 || part.qzeros->shape.size() != 2 || part.scales->shape.size() != 2) {
        return bad_file(prefix + ": tensors must be two-dimensional");
    }
    const int64_t words = part.qweight->shape[1];
    part.n = words * 8;
    if (part.qweight->shape[0] != K || part.qzeros->shape[0] != K / group || part.qzeros->shape[1] != words ||
        part.scales->shape[0] != K / group || part.scales->shape[1] != part.n) {
        return bad_file(prefix + ": shapes do not describe K = " + std::to_string(K) + ", group " +
                        std::to_string(group));
    }
    return base::error::success();
}

// rows of several [rows, cols_i] tensors laid side by side: out[r] = part0[r] | part1[r] | ...
void concat_rows(const SafetensorsFile& file, const std::vector<const TensorEntry*>& parts, size_t element_size,
                 std::vector<uint8_t>& out) {
    const int64_t rows = parts[0]->shape[0];
    size_t row_bytes = 0;
    for (const TensorEntry* p : parts) row_bytes += static_cast<size_t>(p->shape[1]) * element_size;
    out.resize(static_cast<size_t>(rows) * row_bytes);
    size_t column = 0;
    for (const TensorEntry* p : parts) {
        const size_t part_row = static_cast<size_t>(p->shape[1]) * element_size;
        const uint8_t* src = static_cast<const uint8_t*>(file.data(*p));
        for (int64_t r = 0; r < rows; r++) {
            std::memcpy(out.data() + static_cast<size_t>(r) * row_bytes + column, src + static_cast<size_t>(r) * part_row,
                        part_row);
        }
        column += part_row;
    }
}

}  // namespace

int64_t TensorEntry::element_count() const {
    int64_t n = 1;
    for (int64_t d : shape) n *= d;
    return n;
}

size_t dtype_size(const std::string& dtype) {
    if (dtype == "F64" || dtype == "I64" || dtype == "U64") return 8;
    if (dtype == "F32" || dtype == "I32" || dtype == "U32") return 4;
    if (dtype == "F16" || dtype == "BF16" || dtype == "I16" || dtype == "U16") return 2;
    if (dtype == "I8" || dtype == "U8" || dtype == "BOOL" || dtype == "F8_E4M3" || dtype == "F8_E5M2") return 1;
    return 0;
}

SafetensorsFile::~SafetensorsFile() { close(); }

void SafetensorsFile::close() {
    if (map_ != nullptr) {
        ::munmap(map_, map_bytes_);
    }
    map_ = nullptr;
    map_bytes_ = 0;
    data_start_ = 0;
    entries_.clear();
    index_.clear();
    metadata_.clear();
}

base::Status SafetensorsFile::open(const std::string& path) {
    close();
    const int fd = ::open(path.c_str(), O_RDONLY);
    if (fd < 0) {
        return base::error::path_not_valid("safetensors: cannot open " + path);
    }
    struct stat st;
    if (::fstat(fd, &st) != 0 || st.st_size < 8) {
        ::close(fd);
        return bad_file(path + " is shorter than a header length");
    }
    const size_t bytes = static_cast<size_t>(st.st_size);
    void* map = ::mmap(nullptr, bytes, PROT_READ, MAP_PRIVATE, fd, 0);
    ::close(fd);
    if (map == MAP_FAILED) {
        return base::error::internal_error("safetensors: mmap of " + path + " failed");
    }
    map_ = map;
    map_bytes_ = bytes;

    const uint8_t* raw = static_cast<const uint8_t*>(map_);
    uint64_t header_len = 0;
    for (int i = 7; i >= 0; i--) header_len = (header_len << 8) | raw[i];  // little endian
    if (header_len > bytes - 8) {
        close();
        return bad_file("header length exceeds the file");
    }
    data_start_ = 8 + static_cast<size_t>(header_len);
    const size_t data_bytes = bytes - data_start_;

    Json root;
    std::string why;
    JsonReader reader(reinterpret_cast<const char*>(raw + 8), static_cast<size_t>(header_len));
    if (!reader.parse(root, why) || root.kind != Json::Object) {
        close();
        return bad_file("header: " + (why.empty() ? std::string("not an object") : why));
    }
    for (const auto& kv : root.members) {
        if (kv.first == "__metadata__") {
            if (kv.second.kind == Json::Object) {
                for (const auto& m : kv.second.members) {
                    if (m.second.kind == Json::String) metadata_[m.first] = m.second.text;
                }
            }
            continue;
        }
        const Json& desc = kv.second;
        const Json* dtype = desc.kind == Json::Object ? member(desc, "dtype") : nullptr;
        const Json* shape = desc.kind == Json::Object ? member(desc, "shape") : nullptr;
        const Json* offsets = desc.kind == Json::Object ? member(desc, "data_offsets") : nullptr;
        if (!dtype || dtype->kind != Json::String || !shape || shape->kind != Json::Array || !offsets ||
            offsets->kind != Json::Array || offsets->items.size() != 2) {
            close();
            return bad_file("entry " + kv.first + " lacks dtype, shape or data_offsets");
        }
        TensorEntry entry;
        entry.name = kv.first;
        entry.dtype = dtype->text;
        const size_t esize = dtype_size(entry.dtype);
        if (esize == 0) {
            close();
            return bad_file("entry " + kv.first + " has unknown dtype " + entry.dtype);
        }
        uint64_t count = 1;
        for (const Json& d : shape->items) {
            if (d.kind != Json::Number || !d.integral || d.integer > (1ull << 40)) {
                close();
                return bad_file("entry " + kv.first + " has a bad shape");
            }
            entry.shape.push_back(static_cast<int64_t>(d.integer));
            if (d.integer != 0 && count > (1ull << 50) / d.integer) {
                close();
                return bad_file("entry " + kv.first + " is too large");
            }
            count *= d.integer;
        }
        const Json& b = offsets->items[0];
        const Json& e = offsets->items[1];
        if (b.kind != Json::Number || e.kind != Json::Number || !b.integral || !e.integral || b.integer > e.integer ||
            e.integer > data_bytes) {
            close();
            return bad_file("entry " + kv.first + " points outside the file");
        }
        entry.begin = static_cast<size_t>(b.integer);
        entry.end = static_cast<size_t>(e.integer);
        if (entry.byte_size() != count * esize) {
            close();
            return bad_file("entry " + kv.first + ": byte range does not match shape and dtype");
        }
        if (index_.count(entry.name)) {
            close();
            return bad_file("entry " + kv.first + " appears twice");
        }
        index_[entry.name] = entries_.size();
        entries_.push_back(std::move(entry));
    }
    return base::error::success();
}

const TensorEntry* SafetensorsFile::find(const std::string& name) const {
    auto it = index_.find(name);
    return it == index_.end() ? nullptr : &entries_[it->second];
}

const void* SafetensorsFile::data(const TensorEntry& entry) const {
    CHECK(is_open());
    return static_cast<const uint8_t*>(map_) + data_start_ + entry.begin;
}

base::Status load_awq_linear(const SafetensorsFile& file, const std::string& prefix, op::MatmulLayer& layer) {
    return load_awq_linear_fused(file, {prefix}, layer);
}

base::Status load_awq_linear_fused(const SafetensorsFile& file, const std::vector<std::string>& prefixes,
                                   op::MatmulLayer& layer) {
    if (!file.is_open()) return base::error::invalid_argument("safetensors: the file is not open");
    if (!layer.is_quant_layer()) return base::error::invalid_argument("safetensors: the layer is not quantised");
    if (prefixes.empty()) return base::error::invalid_argument("safetensors: no tensor prefix given");
    const int64_t K = layer.dim1();
    const int64_t N = layer.dim0();
    const int64_t G = layer.group_size();
    std::vector<AwqPart> parts(prefixes.size());
    int64_t total_n = 0;
    for (size_t i = 0; i < prefixes.size(); i++) {
        base::Status st = find_awq_part(file, prefixes[i], K, G, parts[i]);
        if (!st) return st;
        total_n += parts[i].n;
    }
    if (total_n != N) {
        return bad_file("the tensors hold " + std::to_string(total_n) + " output features, the layer " +
                        std::to_string(N));
    }
    const std::vector<int32_t> qw_dims{static_cast<int32_t>(K), static_cast<int32_t>(N / 8)};
    const std::vector<int32_t> qz_dims{static_cast<int32_t>(K / G), static_cast<int32_t>(N / 8)};
    const std::vector<int32_t> sc_dims{static_cast<int32_t>(K / G), static_cast<int32_t>(N)};
    const base::DeviceType device = layer.device_type();
    tensor::Tensor qweight, qzeros, scales;
    if (parts.size() == 1) {
        qweight = device_tensor(base::DataType::DataTypeInt32, qw_dims, device, file.data(*parts[0].qweight),
                                parts[0].qweight->byte_size());
        qzeros = device_tensor(base::DataType::DataTypeInt32, qz_dims, device, file.data(*parts[0].qzeros),
                               parts[0].qzeros->byte_size());
        scales = device_tensor(base::DataType::DataTypeFp16, sc_dims, device, file.data(*parts[0].scales),
                               parts[0].scales->byte_size());
    } else {
        std::vector<const TensorEntry*> list;
        std::vector<uint8_t> staging;
        for (const AwqPart& p : parts) list.push_back(p.qweight);
        concat_rows(file, list, 4, staging);
        qweight = device_tensor(base::DataType::DataTypeInt32, qw_dims, device, staging.data(), staging.size());
        list.clear();
        for (const AwqPart& p : parts) list.push_back(p.qzeros);
        concat_rows(file, list, 4, staging);
        qzeros = device_tensor(base::DataType::DataTypeInt32, qz_dims, device, staging.data(), staging.size());
        list.clear();
        for (const AwqPart& p : parts) list.push_back(p.scales);
        concat_rows(file, list, 2, staging);
        scales = device_tensor(base::DataType::DataTypeFp16, sc_dims, device, staging.data(), staging.size());
    }
    base::Status st = layer.set_weight(0, qweight);
    if (!st) return st;
    st = layer.set_weight(1, qzeros);
    if (!st) return st;
    layer.set_awq_scales(scales);
    return base::error::success();
}

base::Status load_bf16_linear(const SafetensorsFile& file, const std::string& name, op::MatmulLayer& layer) {
    if (!file.is_open()) return base::error::invalid_argument("safetensors: the file is not open");
    if (layer.is_quant_layer()) return base::error::invalid_argument("safetensors: the layer is quantised");
    const TensorEntry* w = file.find(name);
    if (!w) return base::error::path_not_valid("safetensors: " + name + " is not in the file");
    if (w->dtype != "BF16" || w->shape.size() != 2 || w->shape[0] != layer.dim0() || w->shape[1] != layer.dim1()) {
        return bad_file(name + ": expected BF16 [" + std::to_string(layer.dim0()) + ", " +
                        std::to_string(layer.dim1()) + "]");
    }
    tensor::Tensor weight = device_tensor(base::DataType::DataTypeBf16, {layer.dim0(), layer.dim1()},
                                          layer.device_type(), file.data(*w), w->byte_size());
    return layer.set_weight(0, weight);
}

base::Status load_bf16_tensor(const SafetensorsFile& file, const std::string& name, const std::vector<int32_t>& dims,
                              base::DeviceType device, tensor::Tensor& out) {
    if (!file.is_open()) return base::error::invalid_argument("safetensors: the file is not open");
    const TensorEntry* e = file.find(name);
    if (!e) return base::error::path_not_valid("safetensors: " + name + " is not in the file");
    bool same = e->shape.size() == dims.size();
    for (size_t i = 0; same && i < dims.size(); i++) same = e->shape[i] == dims[i];
    if (!same) return bad_file(name + ": shape differs from what the model expects");
    const size_t count = static_cast<size_t>(e->element_count());
    if (e->dtype == "BF16") {
        out = device_tensor(base::DataType::DataTypeBf16, dims, device, file.data(*e), e->byte_size());
        return base::error::success();
    }
    if (e->dtype != "F16" && e->dtype != "F32") return bad_file(name + ": expected BF16, F16 or F32");
    std::vector<uint16_t> rounded(count);
    if (e->dtype == "F32") {
        const float* src = static_cast<const float*>(file.data(*e));
        for (size_t i = 0; i < count; i++) rounded[i] = kernel::float_to_bf16(src[i]);
    } else {
        const uint16_t* src = static_cast<const uint16_t*>(file.data(*e));
        for (size_t i = 0; i < count; i++) rounded[i] = kernel::float_to_bf16(kernel::fp16_to_float(src[i]));
    }
    out = device_tensor(base::DataType::DataTypeBf16, dims, device, rounded.data(), count * sizeof(uint16_t));
    return base::error::success();
}

}  // namespace model
