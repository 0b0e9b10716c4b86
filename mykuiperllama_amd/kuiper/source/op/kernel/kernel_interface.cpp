// Kernel selection by device; an unknown device is fatal
// (reference: kuiper/source/op/kernel/kernel_interface.cpp:6-14).
#include "kernel_interface.h"

#include "cpu/add_kernel.h"
#include "cpu/matmul_kernel.h"
#include "hip/add_kernel.h"
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

}  // namespace kernel
