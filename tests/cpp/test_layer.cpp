// Status, Layer and LayerParam behaviour that the reference leaves untested but that is part of
// the interface (kuiper/source/base/base.cpp:5-73, kuiper/source/op/layer.cpp:41-304).
#include <sstream>
#include <vector>

#include "mini_test.h"
#include "op/layer.h"

namespace {
// smallest concrete layers: everything else is inherited
struct PlainLayer : op::Layer {
    PlainLayer() : op::Layer(base::DeviceType::DeviceCPU, op::LayerType::LayerSoftmax, "plain") {}
};
struct ParamLayer : op::LayerParam {
    explicit ParamLayer(bool quant) : op::LayerParam(base::DeviceType::DeviceCPU, op::LayerType::LayerLinear, quant, "param") {}
};
}  // namespace

TEST_CPU(test_status, codes_and_conversions) {
    base::Status ok;
    ASSERT_TRUE(bool(ok));
    ASSERT_EQ(int(ok), 0);
    ASSERT_TRUE(ok == base::StatusCode::Success);
    base::Status bad = base::error::invalid_argument("wrong");
    ASSERT_FALSE(bool(bad));
    ASSERT_EQ(bad.get_err_code(), 7);
    ASSERT_TRUE(bad != 0);
    ASSERT_EQ(bad.get_err_msg(), std::string("wrong"));
    std::ostringstream os;
    os << bad;
    ASSERT_EQ(os.str(), std::string("wrong"));
    bad = 0;
    ASSERT_TRUE(bool(bad));
    bad.set_err_msg("kept");
    ASSERT_EQ(bad.get_err_msg(), std::string("kept"));
    ASSERT_EQ(int(base::error::function_not_implement()), 1);
    ASSERT_EQ(int(base::error::path_not_valid()), 2);
    ASSERT_EQ(int(base::error::model_parse_error()), 3);
    ASSERT_EQ(int(base::error::internal_error()), 5);
    ASSERT_EQ(int(base::error::key_has_exits()), 6);
    ASSERT_EQ(int(base::error::success("fine")), 0);
    STATUS_CHECK(base::error::success());
    ASSERT_FATAL(STATUS_CHECK(base::error::internal_error("boom")));
}

TEST_CPU(test_layer, defaults_and_io_slots) {
    PlainLayer layer;
    ASSERT_TRUE(layer.data_type() == base::DataType::DataTypeFp32);
    ASSERT_TRUE(layer.device_type() == base::DeviceType::DeviceCPU);
    ASSERT_TRUE(layer.layer_type() == op::LayerType::LayerSoftmax);
    ASSERT_EQ(layer.layer_name(), std::string("plain"));
    layer.set_layer_name("renamed");
    ASSERT_EQ(layer.layer_name(), std::string("renamed"));
    ASSERT_TRUE(bool(layer.init()));
    ASSERT_EQ(int(layer.check()), int(base::StatusCode::FunctionUnImplement));
    ASSERT_EQ(int(layer.forward()), int(base::StatusCode::FunctionUnImplement));
    ASSERT_EQ(layer.input_size(), 0u);
    ASSERT_FATAL(layer.get_input(0));
    layer.reset_input_size(5);
    layer.reset_output_size(1);
    ASSERT_EQ(layer.input_size(), 5u);
    ASSERT_EQ(layer.output_size(), 1u);
    auto allocator = base::CPUDeviceAllocatorFactory::get_instance();
    std::vector<tensor::Tensor> in;
    for (int i = 0; i < 5; i++) in.emplace_back(base::DataType::DataTypeFp32, 4 + i, true, allocator);
    tensor::Tensor out(base::DataType::DataTypeFp32, 3, true, allocator);
    // the five-input overload fills every slot and then reaches forward()
    ASSERT_EQ(int(layer.forward(in[0], in[1], in[2], in[3], in[4], out)), int(base::StatusCode::FunctionUnImplement));
    for (int i = 0; i < 5; i++) ASSERT_EQ(layer.get_input(i).size(), size_t(4 + i));
    ASSERT_EQ(layer.get_output(0).ptr<void>(), out.ptr<void>());  // slots share the caller's buffer
    ASSERT_EQ(int(layer.set_weight(0, in[0])), int(base::StatusCode::FunctionUnImplement));
    // an empty tensor of the right type may be parked in a slot whatever its device
    tensor::Tensor parked;
    parked.reset(base::DataType::DataTypeFp32, {4});
    layer.set_input(0, parked);
    // a filled tensor on another device may not
    tensor::Tensor foreign(base::DataType::DataTypeFp32, 4, true, allocator);
    foreign.set_device_type(base::DeviceType::DeviceCUDA);
    ASSERT_FATAL(layer.set_output(0, foreign));
}

TEST_CPU(test_layer, check_tensor_helpers) {
    PlainLayer layer;
    auto allocator = base::CPUDeviceAllocatorFactory::get_instance();
    tensor::Tensor t(base::DataType::DataTypeFp32, 3, 7, true, allocator);
    ASSERT_TRUE(bool(layer.check_tensor(t, base::DeviceType::DeviceCPU, base::DataType::DataTypeFp32)));
    ASSERT_FALSE(bool(layer.check_tensor(t, base::DeviceType::DeviceCUDA, base::DataType::DataTypeFp32)));
    ASSERT_FALSE(bool(layer.check_tensor(t, base::DeviceType::DeviceCPU, base::DataType::DataTypeInt8)));
    ASSERT_FALSE(bool(layer.check_tensor(tensor::Tensor(), base::DeviceType::DeviceCPU, base::DataType::DataTypeFp32)));
    ASSERT_TRUE(bool(layer.check_tensor_with_dim(t, base::DeviceType::DeviceCPU, base::DataType::DataTypeFp32, 3, 7)));
    base::Status st = layer.check_tensor_with_dim(t, base::DeviceType::DeviceCPU, base::DataType::DataTypeFp32, 3, 8);
    ASSERT_FALSE(bool(st));
    ASSERT_EQ(st.get_err_msg(), std::string("The tensor has a wrong dim in dim1"));
}

TEST_CPU(test_layer, layer_param_weights_and_quant_members) {
    auto allocator = base::CPUDeviceAllocatorFactory::get_instance();
    ParamLayer layer(false);
    ASSERT_EQ(layer.weights_size(), 0u);
    layer.reset_weights_size(2);
    ASSERT_EQ(layer.weights_size(), 2u);
    tensor::Tensor w(base::DataType::DataTypeFp32, 2, 3, true, allocator);
    ASSERT_TRUE(bool(layer.set_weight(0, w)));
    ASSERT_EQ(layer.get_weight(0).ptr<void>(), w.ptr<void>());
    tensor::Tensor wi(base::DataType::DataTypeInt8, 6, true, allocator);
    ASSERT_FATAL(layer.set_weight(0, wi));  // fp32 only at this level
    ASSERT_FATAL(layer.set_weight(2, w));
    ASSERT_FATAL(layer.get_weight(-1));
    // raw pointer attach borrows the memory as an fp32 tensor of the given dims
    std::vector<float> raw(12, 2.5f);
    ASSERT_TRUE(bool(layer.set_weight(1, {3, 4}, raw.data(), base::DeviceType::DeviceCPU)));
    ASSERT_EQ(layer.get_weight(1).ptr<float>(), raw.data());
    ASSERT_EQ(layer.get_weight(1).dims(), std::vector<int32_t>({3, 4}));
    ASSERT_TRUE(layer.get_weight(1).device_type() == base::DeviceType::DeviceCPU);
    ASSERT_TRUE(layer.get_weight(1).get_buffer()->is_external());
    ASSERT_FATAL(layer.set_weight(1, {3, 4}, nullptr, base::DeviceType::DeviceCPU));
    // a quantised layer stores nothing through the fp32 raw-pointer path
    ParamLayer quant(true);
    quant.reset_weights_size(1);
    ASSERT_TRUE(bool(quant.set_weight(0, {3, 4}, raw.data(), base::DeviceType::DeviceCPU)));
    ASSERT_EQ(quant.get_weight(0).is_empty(), true);
    // scales: same element type and device as the layer, non-empty
    ASSERT_FATAL(quant.get_scale_num());
    tensor::Tensor scales(base::DataType::DataTypeFp32, 10, true, allocator);
    quant.set_scales(scales);
    quant.set_group_size(64);
    ASSERT_EQ(quant.get_scale_num(), 10);
    ASSERT_FATAL(quant.set_scales(tensor::Tensor()));
    tensor::Tensor half(base::DataType::DataTypeFp16, 10, true, allocator);
    ASSERT_FATAL(quant.set_scales(half));
}
