#include <hip/hip_runtime.h>

#include "base/log.h"
#include "utils.h"

__global__ void fill_value_kernel(float* arr, int32_t size, float value) {
    const int32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < size) arr[i] = value;
}

void set_value_cu(float* arr_cu, int32_t size, float value) {
    (void)hipDeviceSynchronize();
    (void)hipGetLastError();  // start from a clean error state
    hipLaunchKernelGGL(fill_value_kernel, dim3((size + 511) / 512), dim3(512), 0, nullptr, arr_cu, size, value);
    (void)hipDeviceSynchronize();
    const hipError_t err = hipGetLastError();
    CHECK_EQ(err, hipSuccess);
}
