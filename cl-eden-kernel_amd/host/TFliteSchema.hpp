// The slice of the model schema the operator constructor reads: tensor types, operator codes, the legacy-model
// attribute and the option tables of the six operators this backend builds, as plain structs with the schema's field
// names (src/model/schema/nnc/v2/schema.fbs:38-58 TensorType, :245-318 BuiltinOperator, :547-567 Conv2DOptions /
// Pool2DOptions, :580-606 DepthwiseConv2DOptions, :659-695 FullyConnectedOptions / AddOptions, :953-962
// TransposeConvOptions, :1456-1465 LegacyModel).  The reference reads flatbuffer tables generated from that schema out
// of a loaded model; the model loader is not part of this backend.
#pragma once

#include <cstdint>
#include <vector>

namespace TFlite {

enum Padding { Padding_SAME = 0, Padding_VALID = 1 };
enum ActivationFunctionType {
    ActivationFunctionType_NONE = 0,
    ActivationFunctionType_RELU = 1,
    ActivationFunctionType_RELU_N1_TO_1 = 2,
    ActivationFunctionType_RELU6 = 3,
};
enum LegacyModel {
    LegacyModel_CAFFE = 0,
    LegacyModel_TENSORFLOW = 1,
    LegacyModel_CAFFE_NCHW = 2,
    LegacyModel_CAFFE_NHWC = 3,
    LegacyModel_TENSORFLOW_NCHW = 4,
    LegacyModel_TENSORFLOW_NHWC = 5,
    LegacyModel_ANDROID_NN = 6,
};
enum TensorType {
    TensorType_FLOAT32 = 0,
    TensorType_FLOAT16 = 1,
    TensorType_INT32 = 2,
    TensorType_UINT8 = 3,
    TensorType_INT64 = 4,
    TensorType_BOOL = 6,
    TensorType_INT16 = 7,
    TensorType_INT8 = 9,
    TensorType_FLOAT64 = 10,
};
enum BuiltinOperator {
    BuiltinOperator_ADD = 0,
    BuiltinOperator_AVERAGE_POOL_2D = 1,
    BuiltinOperator_CONV_2D = 3,
    BuiltinOperator_DEPTHWISE_CONV_2D = 4,
    BuiltinOperator_FULLY_CONNECTED = 9,
    BuiltinOperator_TRANSPOSE_CONV = 67,
};

struct Conv2DOptions {
    Padding padding = Padding_SAME;
    int32_t stride_w = 1, stride_h = 1;
    ActivationFunctionType fused_activation_function = ActivationFunctionType_NONE;
    int32_t dilation_w_factor = 1, dilation_h_factor = 1;
    std::vector<int32_t> padding_value;  // androidNN: explicit {left, right, top, bottom}
    bool use_nchw = false;               // androidNN
};
struct DepthwiseConv2DOptions {
    Padding padding = Padding_SAME;
    int32_t stride_w = 1, stride_h = 1;
    int32_t depth_multiplier = 1;
    ActivationFunctionType fused_activation_function = ActivationFunctionType_NONE;
    int32_t dilation_w_factor = 1, dilation_h_factor = 1;
    std::vector<int32_t> padding_value;
    bool use_nchw = false;
};
struct TransposeConvOptions {
    Padding padding = Padding_SAME;
    int32_t stride_w = 1, stride_h = 1;
    int32_t group = 1;
    ActivationFunctionType fused_activation_function = ActivationFunctionType_NONE;
    std::vector<int32_t> padding_value;
    bool use_nchw = false;
};
struct Pool2DOptions {
    Padding padding = Padding_VALID;
    int32_t stride_w = 1, stride_h = 1;
    int32_t filter_width = 1, filter_height = 1;
    ActivationFunctionType fused_activation_function = ActivationFunctionType_NONE;
    std::vector<int32_t> padding_value;
    bool use_nchw = false;
};
struct FullyConnectedOptions {
    ActivationFunctionType fused_activation_function = ActivationFunctionType_NONE;
};
struct AddOptions {
    ActivationFunctionType fused_activation_function = ActivationFunctionType_NONE;
    bool pot_scale_int16 = true;
    std::vector<float> coeff;
};

}  // namespace TFlite
