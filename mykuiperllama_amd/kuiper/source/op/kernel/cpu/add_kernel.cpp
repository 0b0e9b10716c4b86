// Host add kernel.  The reference wraps the pointers in Armadillo vectors
// (kuiper/source/op/kernel/cpu/add_kernel.cpp:5-26); a plain loop gives the same fp32 sums
// without the dependency.
#include "add_kernel.h"

namespace kernel {

void add_kernel_cpu(const tensor::Tensor& input1, const tensor::Tensor& input2,
                    const tensor::Tensor& output, void* stream) {
    UNUSED(stream);
    CHECK_EQ(input1.is_empty(), false);
    CHECK_EQ(input2.is_empty(), false);
    CHECK_EQ(output.is_empty(), false);
    CHECK_EQ(input1.size(), output.size());
    CHECK_EQ(input2.size(), output.size());

    const float* a = input1.ptr<float>();
    const float* b = input2.ptr<float>();
    float* out = const_cast<float*>(output.ptr<float>());
    const size_t n = output.size();
    for (size_t i = 0; i < n; i++) {
        out[i] = a[i] + b[i];
    }
}

}  // namespace kernel
