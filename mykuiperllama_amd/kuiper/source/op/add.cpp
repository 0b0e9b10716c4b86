// VecAddLayer (reference: kuiper/source/op/add.cpp:5-49): check the three tensors, then hand them
// to the kernel the device selects, on the layer's stream.
#include "op/add.h"

#include "kernel/kernel_interface.h"

namespace op {

VecAddLayer::VecAddLayer(base::DeviceType device_type) : Layer(device_type, LayerType::LayerAdd, "Add") {
    reset_input_size(2);
    reset_output_size(1);
}

base::Status VecAddLayer::check() const {
    // The reference compares against input1.size() passed as one variadic extent (add.cpp:15-16),
    // which is only meaningful for 1-d tensors; the element counts are what matters to the kernel,
    // so they are compared directly here.
    const size_t size = get_input(0).size();
    const char* names[3] = {"input tensor 1", "input tensor 2", "output tensor"};
    const tensor::Tensor* tensors[3] = {&get_input(0), &get_input(1), &get_output(0)};
    for (int i = 0; i < 3; i++) {
        base::Status status = check_tensor(*tensors[i], device_type_, data_type_);
        if (status && tensors[i]->size() != size) {
            status = base::error::invalid_argument("The tensor has a wrong dim in dim0");
        }
        if (!status) {
            LOG(ERROR) << "The " << names[i] << " error in the add layer.";
            return status;
        }
    }
    return base::error::success();
}

base::Status VecAddLayer::forward() {
    base::Status status = check();
    if (!status) {
        return status;
    }
    if (device_type_ == base::DeviceType::DeviceCUDA) {
        CHECK_NE(cuda_config_, nullptr);
    }
    kernel::get_add_kernel(device_type_)(get_input(0), get_input(1), get_output(0),
                                         cuda_config_ ? cuda_config_->stream() : nullptr);
    return base::error::success();
}

}  // namespace op
