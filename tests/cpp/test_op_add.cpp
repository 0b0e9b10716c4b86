// The add operator through the kernel-selection interface.  Restates the assertions of the
// reference's test/test_op/test_op_add.cpp (add_cuda_no_stream :7-26, add_cuda_stream :28-51,
// add_cpu :53-70, add_cuda_align :72-91): 32 x 151 fp32, 2 + 3 == 5 exactly; 32 x 151 x 13,
// 2.1 + 3.3 within 1e-4 of 5.4.  Plus the layer wrapper, which the reference leaves untested.
#include <hip/hip_runtime_api.h>

#include <vector>

#include "../../mykuiperllama_amd/kuiper/source/op/kernel/kernel_interface.h"
#include "mini_test.h"
#include "op/add.h"
#include "utils.h"

static void run_gpu_add(std::vector<int32_t> dims, float a, float b, float expect, float tol, bool own_stream) {
    auto allocator_cu = base::CUDADeviceAllocatorFactory::get_instance();
    tensor::Tensor t_in1(base::DataType::DataTypeFp32, dims, true, allocator_cu);
    tensor::Tensor t_in2(base::DataType::DataTypeFp32, dims, true, allocator_cu);
    tensor::Tensor t_out(base::DataType::DataTypeFp32, dims, true, allocator_cu);
    const int32_t size = static_cast<int32_t>(t_out.size());
    set_value_cu(t_in1.ptr<float>(), size, a);
    set_value_cu(t_in2.ptr<float>(), size, b);
    hipStream_t stream = nullptr;
    if (own_stream) ASSERT_EQ(hipStreamCreate(&stream), hipSuccess);
    kernel::get_add_kernel(base::DeviceType::DeviceCUDA)(t_in1, t_in2, t_out, stream);
    ASSERT_EQ(hipDeviceSynchronize(), hipSuccess);
    std::vector<float> back(size, 0.f);
    ASSERT_EQ(hipMemcpy(back.data(), t_out.ptr<float>(), size * sizeof(float), hipMemcpyDeviceToHost), hipSuccess);
    for (int32_t i = 0; i < size; i++) {
        if (tol == 0.f) {
            ASSERT_EQ(back[i], expect);
        } else {
            ASSERT_NEAR(back[i], expect, tol);
        }
    }
    if (own_stream) ASSERT_EQ(hipStreamDestroy(stream), hipSuccess);
}

TEST_GPU(test_op_add, add_cuda_no_stream) { run_gpu_add({32, 151}, 2.f, 3.f, 5.f, 0.f, false); }
TEST_GPU(test_op_add, add_cuda_stream) { run_gpu_add({32, 151}, 2.f, 3.f, 5.f, 0.f, true); }
TEST_GPU(test_op_add, add_cuda_align) { run_gpu_add({32, 151, 13}, 2.1f, 3.3f, 5.4f, 0.0001f, false); }
TEST_GPU(test_op_add, add_cuda_sizes_not_multiple_of_four) { run_gpu_add({7, 3}, 1.5f, 2.25f, 3.75f, 0.f, false); }

TEST_CPU(test_op_add, add_cpu) {
    auto allocator_cpu = base::CPUDeviceAllocatorFactory::get_instance();
    const int32_t size = 32 * 151;
    tensor::Tensor t_in1(base::DataType::DataTypeFp32, 32, 151, true, allocator_cpu);
    tensor::Tensor t_in2(base::DataType::DataTypeFp32, 32, 151, true, allocator_cpu);
    tensor::Tensor t_out(base::DataType::DataTypeFp32, 32, 151, true, allocator_cpu);
    for (int32_t i = 0; i < size; i++) {
        t_in1.index<float>(i) = 2.f;
        t_in2.index<float>(i) = 3.f;
    }
    kernel::get_add_kernel(base::DeviceType::DeviceCPU)(t_in1, t_in2, t_out, nullptr);
    for (int32_t i = 0; i < size; i++) ASSERT_EQ(t_out.ptr<float>()[i], 5.f);
}

TEST_CPU(test_op_add, kernel_selection_and_kernel_checks) {
    ASSERT_FATAL(kernel::get_add_kernel(base::DeviceType::DeviceUnknown));
    auto allocator_cpu = base::CPUDeviceAllocatorFactory::get_instance();
    tensor::Tensor a(base::DataType::DataTypeFp32, 8, true, allocator_cpu);
    tensor::Tensor b(base::DataType::DataTypeFp32, 9, true, allocator_cpu);
    tensor::Tensor out(base::DataType::DataTypeFp32, 8, true, allocator_cpu);
    ASSERT_FATAL(kernel::get_add_kernel(base::DeviceType::DeviceCPU)(a, b, out, nullptr));  // sizes differ
    tensor::Tensor empty;
    ASSERT_FATAL(kernel::get_add_kernel(base::DeviceType::DeviceCPU)(a, empty, out, nullptr));
    // the GPU wrapper refuses host tensors before it touches the device
    ASSERT_FATAL(kernel::get_add_kernel(base::DeviceType::DeviceCUDA)(a, a, out, nullptr));
}

TEST_CPU(test_op_add, layer_cpu) {
    auto allocator_cpu = base::CPUDeviceAllocatorFactory::get_instance();
    op::VecAddLayer layer(base::DeviceType::DeviceCPU);
    ASSERT_TRUE(layer.layer_type() == op::LayerType::LayerAdd);
    ASSERT_EQ(layer.layer_name(), std::string("Add"));
    ASSERT_EQ(layer.input_size(), 2u);
    ASSERT_EQ(layer.output_size(), 1u);
    tensor::Tensor a(base::DataType::DataTypeFp32, 4, 5, true, allocator_cpu);
    tensor::Tensor b(base::DataType::DataTypeFp32, 4, 5, true, allocator_cpu);
    tensor::Tensor out(base::DataType::DataTypeFp32, 4, 5, true, allocator_cpu);
    for (int i = 0; i < 20; i++) {
        a.index<float>(i) = float(i);
        b.index<float>(i) = 0.5f;
    }
    base::Status st = layer.forward(a, b, out);
    ASSERT_TRUE(bool(st));
    for (int i = 0; i < 20; i++) ASSERT_EQ(out.index<float>(i), float(i) + 0.5f);
    // a mismatched output is reported through the Status, not by aborting
    tensor::Tensor bad(base::DataType::DataTypeFp32, 7, true, allocator_cpu);
    st = layer.forward(a, b, bad);
    ASSERT_FALSE(bool(st));
    ASSERT_EQ(st.get_err_code(), int(base::StatusCode::InvalidArgument));
    // wrong element type is a CHECK in set_input
    tensor::Tensor ints(base::DataType::DataTypeInt32, 20, true, allocator_cpu);
    ASSERT_FATAL(layer.set_input(0, ints));
    ASSERT_FATAL(layer.set_input(2, a));
}

TEST_GPU(test_op_add, layer_cuda_needs_a_stream_config) {
    auto allocator_cu = base::CUDADeviceAllocatorFactory::get_instance();
    op::VecAddLayer layer(base::DeviceType::DeviceCUDA);
    tensor::Tensor a(base::DataType::DataTypeFp32, 64, true, allocator_cu);
    tensor::Tensor b(base::DataType::DataTypeFp32, 64, true, allocator_cu);
    tensor::Tensor out(base::DataType::DataTypeFp32, 64, true, allocator_cu);
    set_value_cu(a.ptr<float>(), 64, 2.f);
    set_value_cu(b.ptr<float>(), 64, 3.f);
    ASSERT_FATAL(layer.forward(a, b, out));  // no CudaConfig yet
    auto config = std::make_shared<kernel::CudaConfig>();
    config->create();
    ASSERT_FATAL(config->create());  // already holds a stream
    layer.set_cuda_config(config);
    layer.set_cuda_config(nullptr);  // ignored
    ASSERT_EQ(layer.cuda_config(), config);
    ASSERT_TRUE(bool(layer.forward(a, b, out)));
    ASSERT_EQ(hipStreamSynchronize(config->stream()), hipSuccess);
    out.to_cpu();
    for (int i = 0; i < 64; i++) ASSERT_EQ(out.index<float>(i), 5.f);
}
