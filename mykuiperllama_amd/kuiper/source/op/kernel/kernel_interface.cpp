// Kernel selection by device; an unknown device is fatal
// (reference: kuiper/source/op/kernel/kernel_interface.cpp:6-14).
#include "kernel_interface.h"

#include "cpu/add_kernel.h"
#include "cpu/decode_kernels.h"
#include "cpu/matmul_kernel.h"
#include "hip/add_kernel.h"
#include "hip/decode_kernels.h"
#include "hip/matmul_kernel.h"

namespace kernel {

AddKernel get_add_kernel(base::DeviceType device_type) {
    switch (device_type) {
        case base::DeviceType::DeviceCPU: return add_kernel_cpu;
        case base::DeviceType::DeviceCUDA: return add_kernel_cu;
        default: break;
    }
    LOG(FATAL) << "Unknown device type for get a add kernel.";
    return nullptr;
}

MatmulKernel get_matmul_kernel(base::DeviceType device_type) {
    switch (device_type) {
        case base::DeviceType::DeviceCPU: return matmul_kernel_cpu;
        case base::DeviceType::DeviceCUDA: return matmul_kernel_cu;
        default: break;
    }
    LOG(FATAL) << "Unknown device type for get a matmul kernel.";
    return nullptr;
}

MatmulKernelAwq get_matmul_kernel_awq(base::DeviceType device_type) {
    switch (device_type) {
        case base::DeviceType::DeviceCPU: return matmul_kernel_awq_cpu;
        case base::DeviceType::DeviceCUDA: return matmul_kernel_awq_cu;
        default: break;
    }
    LOG(FATAL) << "Unknown device type for get a quantised matmul kernel.";
    return nullptr;
}

MatmulChainKernel get_matmul_chain_kernel(base::DeviceType device_type) {
    switch (device_type) {
        case base::DeviceType::DeviceCUDA: return matmul_chain_kernel_cu;
        default: break;  // the fused launches exist on the GPU only; a host layer runs its operators one by one
    }
    LOG(FATAL) << "Unknown device type for get a fused matmul kernel.";
    return nullptr;
}

#define KX_SELECT(Type, getter, cpu_fn, gpu_fn, what)                         \
    Type getter(base::DeviceType device_type) {                               \
        switch (device_type) {                                                \
            case base::DeviceType::DeviceCPU: return cpu_fn;                   \
            case base::DeviceType::DeviceCUDA: return gpu_fn;                  \
            default: break;                                                   \
        }                                                                     \
        LOG(FATAL) << "Unknown device type for get a " what " kernel.";       \
        return nullptr;                                                       \
    }

KX_SELECT(RmsNormKernel, get_rmsnorm_kernel, rmsnorm_kernel_cpu, rmsnorm_kernel_cu, "rmsnorm")
KX_SELECT(SwiGLUKernel, get_swiglu_kernel, swiglu_kernel_cpu, swiglu_kernel_cu, "swiglu")
KX_SELECT(EmbeddingKernel, get_embedding_kernel, embedding_kernel_cpu, embedding_kernel_cu, "embedding")
KX_SELECT(RoPEKernel, get_rope_kernel, rope_kernel_cpu, rope_kernel_cu, "rope")
KX_SELECT(MhaKernel, get_mha_kernel, mha_kernel_cpu, mha_kernel_cu, "mha")
#undef KX_SELECT

}  // namespace kernel
