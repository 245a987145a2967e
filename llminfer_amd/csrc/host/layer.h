// Op layer base classes: hold input/output tensors, check them, pick a kernel
// from the registry. Mirrors code/include/op/layer.h:22-156 and
// code/source/op/layer.cpp:41-212, reduced to what the attention ops use.
#ifndef LLMI_HOST_LAYER_H
#define LLMI_HOST_LAYER_H

#include <initializer_list>
#include <memory>
#include <string>
#include <vector>

#include "hip_config.h"
#include "tensor.h"

namespace op {
enum class LayerType : uint8_t {
    LayerUnknown = 0,
    LayerMatmul = 5,
    LayerRoPE = 6,
    LayerMHA = 7,
};

class Layer {
public:
    // Every layer works on bf16 tensors (layer.cpp:41-42).
    explicit Layer(base::DeviceType device_type, LayerType layer_type, std::string layer_name = "")
        : device_type_(device_type), layer_type_(layer_type), layer_name_(std::move(layer_name)) {}
    virtual ~Layer() = default;

    virtual base::Status init() { return base::error::success(); }
    virtual base::Status check() const { return base::error::function_not_implement("The check function is not implement yet"); }

    base::Status check_tensor(const tensor::Tensor& tensor, base::DeviceType device_type, base::DataType data_type) const;
    // Expected sizes of the leading dimensions, one per dimension of the tensor.
    base::Status check_tensor_with_dim(const tensor::Tensor& tensor, base::DeviceType device_type,
                                       base::DataType data_type, std::initializer_list<int32_t> dims) const;

    virtual base::Status forward() { return base::error::function_not_implement(); }
    base::Status forward(const tensor::Tensor& input1, const tensor::Tensor& output1);
    base::Status forward(const tensor::Tensor& input1, const tensor::Tensor& input2, const tensor::Tensor& output1);
    base::Status forward(const tensor::Tensor& input1, const tensor::Tensor& input2, const tensor::Tensor& input3,
                         const tensor::Tensor& output1);
    base::Status forward(const tensor::Tensor& input1, const tensor::Tensor& input2, const tensor::Tensor& input3,
                         const tensor::Tensor& input4, const tensor::Tensor& output1);
    base::Status forward(const tensor::Tensor& input1, const tensor::Tensor& input2, const tensor::Tensor& input3,
                         const tensor::Tensor& input4, const tensor::Tensor& input5, const tensor::Tensor& output1);

    void set_input(int32_t idx, const tensor::Tensor& input);
    void set_output(int32_t idx, const tensor::Tensor& output);
    size_t inputs_size() const { return inputs_.size(); }
    size_t outputs_size() const { return outputs_.size(); }
    tensor::Tensor& get_input(int32_t idx);
    tensor::Tensor& get_output(int32_t idx);
    const tensor::Tensor& get_input(int32_t idx) const;
    const tensor::Tensor& get_output(int32_t idx) const;
    void reset_inputs_size(size_t size) { inputs_.resize(size); }
    void reset_outputs_size(size_t size) { outputs_.resize(size); }

    void set_hip_config(std::shared_ptr<kernel::HipConfig> hip_config) { hip_config_ = std::move(hip_config); }
    std::shared_ptr<kernel::HipConfig> hip_config() const { return hip_config_; }

    const std::string& layer_name() const { return layer_name_; }
    LayerType layer_type() const { return layer_type_; }
    base::DataType data_type() const { return data_type_; }
    base::DeviceType device_type() const { return device_type_; }
    void set_device_type(base::DeviceType device_type) { device_type_ = device_type; }

protected:
    base::DeviceType device_type_;
    LayerType layer_type_;
    base::DataType data_type_ = base::DataType::DataTypeBf16;
    std::string layer_name_;
    std::vector<tensor::Tensor> inputs_;
    std::vector<tensor::Tensor> outputs_;
    std::shared_ptr<kernel::HipConfig> hip_config_;
};

// Layer with weights (layer.h:122-154), without the quantisation members.
class LayerParam : public Layer {
public:
    using Layer::Layer;
    size_t weights_size() const { return weights_.size(); }
    void reset_weights_size(size_t size) { weights_.resize(size); }
    tensor::Tensor& get_weight(int32_t idx);
    const tensor::Tensor& get_weight(int32_t idx) const;
    base::Status set_weight(int32_t idx, const tensor::Tensor& weight);

protected:
    std::vector<tensor::Tensor> weights_;
};
}  // namespace op
#endif
