// Stream ownership (reference: kuiper/source/base/cuda_config.cpp:4-23).
#include "base/cuda_config.h"

#include "kernel/hip/matmul_kernel.h"

namespace kernel {

CudaConfig::~CudaConfig() {
    if (stream_ != nullptr) {
        // what the matmul wrapper keeps for this stream goes with it (a later stream may get the same handle);
        // the release waits for the launches still queued on the stream
        matmul_release_workspace(stream_);
        hipError_t err = hipStreamDestroy(stream_);
        if (err != hipSuccess) {
            // a destructor must not throw through a test's fatal handler: report only
            LOG(ERROR) << "Failed to destroy the stream: " << hipGetErrorString(err);
        }
    }
}

void CudaConfig::create() {
    CHECK_EQ(stream_, nullptr);
    hipError_t err = hipStreamCreate(&stream_);
    CHECK_EQ(err, hipSuccess) << "Failed to create a stream: " << hipGetErrorString(err);
}

hipStream_t CudaConfig::stream() const { return stream_; }
void CudaConfig::set_stream(hipStream_t stream) {
    if (stream_ != nullptr && stream_ != stream) matmul_release_workspace(stream_);
    stream_ = stream;
}

}  // namespace kernel
