// Common enums, Status and small helpers of the kuiper host API, MI355X build.
//
// Mirrors kuiper/include/base/base.h of the reference: same names, same numeric values, same
// behaviour.  Additions are strictly additive: DataTypeFp16 (= 4) and DataTypeBf16 (= 5), which
// the quantised matmul path needs for fp16 scales and bf16 activations (the reference stops at
// fp32 / int8 / int32, base.h:41-46).  DeviceType::DeviceCUDA keeps its spelling: it names "the
// GPU", which here is reached through HIP.
#ifndef KUIPER_INCLUDE_BASE_BASE_H
#define KUIPER_INCLUDE_BASE_BASE_H

#include <cstdint>
#include <cstdio>
#include <ostream>
#include <string>

#include "base/log.h"

#define UNUSED(expr) \
    do {             \
        (void)(expr); \
    } while (0)

namespace model {
// Per-step scratch buffers of a decoder model, by role (reference base.h:12-31; value 14 unused).
enum class ModelBufferType {
    InputTokens = 0,
    InputEmbeddings = 1,
    OutputRMSNorm = 2,
    KeyCache = 3,
    ValueCache = 4,
    Query = 5,
    InputPos = 6,
    ScoreStorage = 7,
    OutputMHA = 8,
    AttnOutput = 9,
    W1Output = 10,
    W2Output = 11,
    W3Output = 12,
    FFNRMSNorm = 13,
    ForwardOutput = 15,
    ForwardOutputCPU = 16,
    SinCache = 17,
    CosCache = 18,
};
}  // namespace model

namespace base {

enum class DeviceType : uint8_t {
    DeviceUnknown = 0,
    DeviceCPU = 1,
    DeviceCUDA = 2,  // the GPU (an MI355X behind HIP in this build)
};

enum class DataType : uint8_t {
    DataTypeUnknown = 0,
    DataTypeFp32 = 1,
    DataTypeInt8 = 2,
    DataTypeInt32 = 3,
    DataTypeFp16 = 4,  // added: AWQ scales
    DataTypeBf16 = 5,  // added: activations and unquantised weights of the matmul path
};

enum class ModelType : uint8_t {
    ModelTypeUnown = 0,
    ModelTypeLLama2 = 1,
};

// Size in bytes of one element; unknown types are fatal, as in the reference (base.h:53-64).
inline size_t data_type_size(DataType data_type) {
    switch (data_type) {
        case DataType::DataTypeFp32: return sizeof(float);
        case DataType::DataTypeInt8: return sizeof(int8_t);
        case DataType::DataTypeInt32: return sizeof(int32_t);
        case DataType::DataTypeFp16: return sizeof(uint16_t);
        case DataType::DataTypeBf16: return sizeof(uint16_t);
        default: break;
    }
    LOG(FATAL) << "Unknown data type size for " << int(data_type);
    return 0;
}

class NoCopyable {
protected:
    NoCopyable() = default;
    ~NoCopyable() = default;
    NoCopyable(const NoCopyable&) = delete;
    NoCopyable& operator=(const NoCopyable&) = delete;
};

enum StatusCode : uint8_t {
    Success = 0,
    FunctionUnImplement = 1,
    PathNotValid = 2,
    ModelParseError = 3,
    InternalError = 5,
    KeyValueHasExist = 6,
    InvalidArgument = 7,
};

enum class TokenizerType {
    EncodeUnknown = -1,
    EncodeSpe = 0,
    EncodeBpe = 1,
};

// Error code plus message.  Converts to bool (true on success) and to int (the code).
class Status {
public:
    Status(int code = StatusCode::Success, std::string err_msg = "");
    Status(const Status& other) = default;
    Status& operator=(const Status& other) = default;
    Status& operator=(int code);
    bool operator==(int code) const;
    bool operator!=(int code) const;
    operator int() const;
    operator bool() const;
    int get_err_code() const;
    const std::string& get_err_msg() const;
    void set_err_msg(const std::string& err_msg);

private:
    int code_ = StatusCode::Success;
    std::string err_msg_;
};

namespace error {
// Evaluates `call` once; a failed Status becomes a fatal log entry with file, line, code, message.
#define STATUS_CHECK(call)                                                                 \
    do {                                                                                   \
        const base::Status& status = call;                                                 \
        if (!status) {                                                                     \
            const size_t buf_size = 512;                                                   \
            char buf[buf_size];                                                            \
            snprintf(buf, buf_size - 1,                                                    \
                     "Infer error\n File: %s Line: %d\n Error code: %d\n Error msg: %s\n", \
                     __FILE__, __LINE__, int(status), status.get_err_msg().c_str());       \
            LOG(FATAL) << buf;                                                             \
        }                                                                                  \
    } while (0)

Status success(const std::string& err_msg = "");
Status function_not_implement(const std::string& err_msg = "");
Status path_not_valid(const std::string& err_msg = "");
Status model_parse_error(const std::string& err_msg = "");
Status internal_error(const std::string& err_msg = "");
Status key_has_exits(const std::string& err_msg = "");
Status invalid_argument(const std::string& err_msg = "");
}  // namespace error

std::ostream& operator<<(std::ostream& os, const Status& status);

}  // namespace base

#endif  // KUIPER_INCLUDE_BASE_BASE_H
