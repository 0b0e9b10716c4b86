// kernel::CudaConfig: RAII owner of the stream a layer enqueues its kernels on.  Same class and
// method names as kuiper/include/base/cuda_config.h:17-30; the stream is a hipStream_t (an
// opaque pointer, like cudaStream_t, so callers that pass config->stream() along compile
// unchanged).  The reference's unused <cublas_v2.h> include is gone.
#ifndef KUIPER_INCLUDE_BASE_CUDA_CONFIG_H
#define KUIPER_INCLUDE_BASE_CUDA_CONFIG_H

#include <hip/hip_runtime_api.h>

#include "base/base.h"

namespace kernel {

class CudaConfig : public base::NoCopyable {
public:
    explicit CudaConfig() : stream_(nullptr) {}
    explicit CudaConfig(hipStream_t stream) : stream_(stream) {}
    ~CudaConfig();  // destroys the stream it holds, if any

    void create();  // creates a stream at the default priority; fatal if one is already held
    hipStream_t stream() const;
    void set_stream(hipStream_t stream);

private:
    hipStream_t stream_ = nullptr;
};

}  // namespace kernel

#endif  // KUIPER_INCLUDE_BASE_CUDA_CONFIG_H
