#include "layer.h"

namespace op {

base::Status Layer::check_tensor(const tensor::Tensor& tensor, base::DeviceType device_type,
                                 base::DataType data_type) const {
    if (tensor.is_empty()) return base::error::invalid_argument("The tensor parameter is empty.");
    if (tensor.device_type() != device_type) return base::error::invalid_argument("The tensor has a wrong device type.");
    if (tensor.data_type() != data_type) return base::error::invalid_argument("The tensor has a wrong data type.");
    return base::error::success();
}

base::Status Layer::check_tensor_with_dim(const tensor::Tensor& tensor, base::DeviceType device_type,
                                          base::DataType data_type, std::initializer_list<int32_t> dims) const {
    base::Status status = check_tensor(tensor, device_type, data_type);
    if (!status) return status;
    int32_t i = 0;
    for (int32_t want : dims) {
        if (i >= tensor.dims_size() || tensor.get_dim(i) != want)
            return base::error::invalid_argument("The tensor has a wrong dim in dim" + std::to_string(i));
        ++i;
    }
    if (i != tensor.dims_size()) return base::error::invalid_argument("The tensor has a wrong number of dims");
    return base::error::success();
}

base::Status Layer::forward(const tensor::Tensor& input1, const tensor::Tensor& output1) {
    set_input(0, input1);
    set_output(0, output1);
    return forward();
}
base::Status Layer::forward(const tensor::Tensor& input1, const tensor::Tensor& input2, const tensor::Tensor& output1) {
    set_input(0, input1);
    set_input(1, input2);
    set_output(0, output1);
    return forward();
}
base::Status Layer::forward(const tensor::Tensor& input1, const tensor::Tensor& input2, const tensor::Tensor& input3,
                            const tensor::Tensor& output1) {
    set_input(0, input1);
    set_input(1, input2);
    set_input(2, input3);
    set_output(0, output1);
    return forward();
}
base::Status Layer::forward(const tensor::Tensor& input1, const tensor::Tensor& input2, const tensor::Tensor& input3,
                            const tensor::Tensor& input4, const tensor::Tensor& output1) {
    set_input(0, input1);
    set_input(1, input2);
    set_input(2, input3);
    set_input(3, input4);
    set_output(0, output1);
    return forward();
}
base::Status Layer::forward(const tensor::Tensor& input1, const tensor::Tensor& input2, const tensor::Tensor& input3,
                            const tensor::Tensor& input4, const tensor::Tensor& input5, const tensor::Tensor& output1) {
    set_input(0, input1);
    set_input(1, input2);
    set_input(2, input3);
    set_input(3, input4);
    set_input(4, input5);
    set_output(0, output1);
    return forward();
}

void Layer::set_input(int32_t idx, const tensor::Tensor& input) {
    LLMI_CHECK(idx >= 0 && static_cast<size_t>(idx) < inputs_.size());
    inputs_[idx] = input;
}
void Layer::set_output(int32_t idx, const tensor::Tensor& output) {
    LLMI_CHECK(idx >= 0 && static_cast<size_t>(idx) < outputs_.size());
    outputs_[idx] = output;
}
tensor::Tensor& Layer::get_input(int32_t idx) {
    LLMI_CHECK(idx >= 0 && static_cast<size_t>(idx) < inputs_.size());
    return inputs_[idx];
}
tensor::Tensor& Layer::get_output(int32_t idx) {
    LLMI_CHECK(idx >= 0 && static_cast<size_t>(idx) < outputs_.size());
    return outputs_[idx];
}
const tensor::Tensor& Layer::get_input(int32_t idx) const {
    LLMI_CHECK(idx >= 0 && static_cast<size_t>(idx) < inputs_.size());
    return inputs_[idx];
}
const tensor::Tensor& Layer::get_output(int32_t idx) const {
    LLMI_CHECK(idx >= 0 && static_cast<size_t>(idx) < outputs_.size());
    return outputs_[idx];
}

tensor::Tensor& LayerParam::get_weight(int32_t idx) {
    LLMI_CHECK(idx >= 0 && static_cast<size_t>(idx) < weights_.size());
    return weights_[idx];
}
const tensor::Tensor& LayerParam::get_weight(int32_t idx) const {
    LLMI_CHECK(idx >= 0 && static_cast<size_t>(idx) < weights_.size());
    return weights_[idx];
}
base::Status LayerParam::set_weight(int32_t idx, const tensor::Tensor& weight) {
    LLMI_CHECK(idx >= 0 && static_cast<size_t>(idx) < weights_.size());
    LLMI_CHECK(weight.data_type() == data_type_);
    if (!weight.is_empty()) LLMI_CHECK(weight.device_type() == device_type_);
    weights_[idx] = weight;
    return base::error::success();
}

}  // namespace op
