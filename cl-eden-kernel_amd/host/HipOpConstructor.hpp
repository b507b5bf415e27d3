// Operator construction from TFLite-style options, and the executor of the resulting list.
//
// Mirrors OperationConstructor / OperationExecutor of the reference
// (src/userdriver/gpu/gpu_op_constructor.cc:63-383 CONV_2D / DEPTHWISE_CONV_2D / TRANSPOSE_CONV /
// FULLY_CONNECTED, :789-860 AVERAGE_POOL_2D, :1166-1205 ADD, :1797-1850 open_oplist, :1884-2009
// layout / precision / padding helpers, :2062-2191 tensor allocation with inter-buffer reuse;
// src/userdriver/gpu/gpu_op_executor.cc:56-103) for the six operators this backend has.
//
// The reference reads flatbuffer tables (TFlite::Conv2DOptions, ...) out of a loaded model.  The
// model loader is not part of this backend, so the option tables are plain structs with the
// schema's field names (src/model/schema/nnc/v2/schema.fbs:547-567,580-606,659-695,953-962), and
// OperatorDesc / TensorDesc stand where model::component::Operator / FeatureMap / Parameter do.
#pragma once

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "HipOperators.hpp"
#include "userdriver_operator.hpp"

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
enum TensorType { TensorType_FLOAT32 = 0, TensorType_FLOAT16 = 1, TensorType_INT32 = 2, TensorType_UINT8 = 3, TensorType_INT8 = 9 };
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

namespace enn {
namespace ud {
namespace hip {

// An edge of the model graph: a feature map (is_const false, buffer_index names its storage) or a
// parameter (is_const true, data points at the host bytes).
struct TensorDesc {
    std::string name;
    NDims shape;
    TFlite::TensorType data_type = TFlite::TensorType_UINT8;
    float scale = 1.0f;
    int32_t zero_point = 0;
    bool is_const = false;
    const void *data = nullptr;
    int32_t buffer_index = UNDEFINED;
    std::vector<float> per_channel_scales;  // symmetric per-channel quantization of a filter; empty otherwise
};

struct OperatorDesc {
    std::string name;
    uint64_t id = 0;
    TFlite::BuiltinOperator code = TFlite::BuiltinOperator_CONV_2D;
    std::vector<std::shared_ptr<TensorDesc>> in_tensors, out_tensors;
    std::shared_ptr<void> option;  // the TFlite::*Options struct that belongs to `code`
};

struct OperatorListDesc {
    uint64_t id = 0;
    TFlite::LegacyModel legacy_model = TFlite::LegacyModel_TENSORFLOW_NHWC;
    std::vector<OperatorDesc> operators;
};

class OperationConstructor {
public:
    explicit OperationConstructor(std::shared_ptr<HipRuntime> runtime) : runtime_(runtime) {}

    // Builds every operator of the list in order (tensors are created as the operators name them; a
    // feature map's storage is handed back to the pool once its last reader has been built) and
    // materialises the pooled buffers.
    EnnReturn open_oplist(const OperatorListDesc &list) {
        operators = std::make_shared<std::vector<std::shared_ptr<UDOperator>>>();
        in_tensors.clear();
        out_tensors.clear();
        alloc_tensors_.clear();
        tensors_used_.clear();
        produced_.clear();
        consumed_.clear();
        legacy_model_ = list.legacy_model;
        for (const auto &op : list.operators) {
            for (const auto &t : op.out_tensors) produced_[t->buffer_index] = true;
            for (const auto &t : op.in_tensors)
                if (!t->is_const) {
                    consumed_[t->buffer_index] = true;
                    tensors_used_[t->buffer_index]++;  // init_inter_buffer
                }
        }
        for (size_t index = 0; index < list.operators.size(); ++index) {
            const auto &op = list.operators[index];
            EnnReturn rc = ENN_RET_FAILED;
            if (fuse_residual_adds && index + 1 < list.operators.size() && fusable_add(op, list.operators[index + 1])) {
                if (create_conv_with_add(op, list.operators[index + 1]) != ENN_RET_SUCCESS) {
                    ERROR_PRINT("OperationConstructor: building %s with its residual add failed\n", op.name.c_str());
                    return ENN_RET_FAILED;
                }
                ++index;  // the Add went into the convolution's launch
                continue;
            }
            switch (op.code) {
                case TFlite::BuiltinOperator_CONV_2D: rc = create_conv(op); break;
                case TFlite::BuiltinOperator_DEPTHWISE_CONV_2D: rc = create_depthwise(op); break;
                case TFlite::BuiltinOperator_TRANSPOSE_CONV: rc = create_deconv(op); break;
                case TFlite::BuiltinOperator_FULLY_CONNECTED: rc = create_fc(op); break;
                case TFlite::BuiltinOperator_AVERAGE_POOL_2D: rc = create_avgpool(op); break;
                case TFlite::BuiltinOperator_ADD: rc = create_add(op); break;
                default: ERROR_PRINT("OperationConstructor: operator code %d is not offered\n", (int)op.code);
            }
            if (rc != ENN_RET_SUCCESS) {
                ERROR_PRINT("OperationConstructor: building %s failed\n", op.name.c_str());
                return ENN_RET_FAILED;
            }
        }
        return runtime_->assignBufferPool() == Status::SUCCESS ? ENN_RET_SUCCESS : ENN_RET_FAILED;
    }

    UDOperators operators;
    UDTensors in_tensors, out_tensors;  // feature maps no operator of the list writes / reads
    // A uint8 ADD right behind the CONV_2D that produces one of its operands, where nothing else reads that
    // operand, runs inside the convolution's launch (HipConvolution::fuseResidualAdd); the list then holds one
    // operator less than the description.  The reference builds one operator per description
    // (gpu_op_constructor.cc:63-383); set to false for that.
    bool fuse_residual_adds = true;

    // ---- helpers, public because tests pin them against hand-computed cases

    static bool is_nchw_layout(const TFlite::LegacyModel &legacy) {
        return !(legacy == TFlite::LegacyModel_TENSORFLOW_NHWC || legacy == TFlite::LegacyModel_CAFFE_NHWC);
    }

    static PrecisionType get_precision(const TFlite::TensorType &type) {
        switch (type) {
            case TFlite::TensorType_INT8: return PrecisionType::INT8;
            case TFlite::TensorType_UINT8: return PrecisionType::UINT8;
            case TFlite::TensorType_FLOAT32: return PrecisionType::FP32;
            default: return PrecisionType::FP16;
        }
    }

    // SAME padding from the input, output and filter extents.  Kept as the reference computes it,
    // including that the dilated filter width takes dilation.h and the height dilation.w
    // (gpu_op_constructor.cc:1966-1967), that Caffe models pad symmetrically with the ceiling, and
    // that an androidNN transposed convolution whose output is smaller than (in - 1) * stride + k gets
    // a negative right / bottom padding.
    static void get_padding(TFlite::LegacyModel legacy_model, TFlite::Padding padding_type, Pad4 &padding, const NDims &input_dim,
                            const NDims &output_dim, const NDims &weight_dim, Dim2 stride, Dim2 dilation, bool deconv, bool nchw) {
        padding.l = padding.r = padding.t = padding.b = 0;
        if (padding_type != TFlite::Padding_SAME) return;
        int32_t input_width, input_height, output_width, output_height, filter_width, filter_height;
        if (!nchw) {
            input_height = (int32_t)input_dim[1];
            input_width = (int32_t)input_dim[2];
            output_height = (int32_t)output_dim[1];
            output_width = (int32_t)output_dim[2];
            filter_height = (int32_t)weight_dim[1];
            filter_width = (int32_t)weight_dim[2];
        } else {
            input_height = (int32_t)input_dim[2];
            input_width = (int32_t)input_dim[3];
            output_height = (int32_t)output_dim[2];
            output_width = (int32_t)output_dim[3];
            filter_height = (int32_t)weight_dim[2];
            filter_width = (int32_t)weight_dim[3];
            if (legacy_model == TFlite::LegacyModel_ANDROID_NN) {  // filters are always [Cout, Kh, Kw, Cin] there
                filter_height = (int32_t)weight_dim[1];
                filter_width = (int32_t)weight_dim[2];
            }
        }
        if (deconv) {
            std::swap(output_width, input_width);
            std::swap(output_height, input_height);
        }
        filter_width = (int32_t)dilation.h * (filter_width - 1) + 1;
        filter_height = (int32_t)dilation.w * (filter_height - 1) + 1;
        const int32_t needed_width = (output_width - 1) * (int32_t)stride.w + filter_width;
        const int32_t needed_height = (output_height - 1) * (int32_t)stride.h + filter_height;
        if (legacy_model == TFlite::LegacyModel_ANDROID_NN && deconv && needed_height < input_height) {
            padding.r = (uint32_t)(needed_width - input_width);
            padding.b = (uint32_t)(needed_height - input_height);
            return;
        }
        const int32_t total_w = std::max(0, needed_width - input_width), total_h = std::max(0, needed_height - input_height);
        if (legacy_model == TFlite::LegacyModel_CAFFE || legacy_model == TFlite::LegacyModel_CAFFE_NHWC ||
            legacy_model == TFlite::LegacyModel_CAFFE_NCHW) {
            padding.l = padding.r = (uint32_t)((total_w + 1) / 2);
            padding.t = padding.b = (uint32_t)((total_h + 1) / 2);
        } else {
            padding.l = (uint32_t)(total_w / 2);
            padding.t = (uint32_t)(total_h / 2);
            padding.r = (uint32_t)((total_w + 1) / 2);
            padding.b = (uint32_t)((total_h + 1) / 2);
        }
    }

private:
    static DataType to_data_type(TFlite::TensorType t) {
        switch (t) {
            case TFlite::TensorType_UINT8: return DataType::UINT8;
            case TFlite::TensorType_INT8: return DataType::INT8;
            case TFlite::TensorType_INT32: return DataType::INT32;
            case TFlite::TensorType_FLOAT16: return DataType::HALF;
            default: return DataType::FLOAT;
        }
    }

    static ActivationInfo to_activation(TFlite::ActivationFunctionType f) {
        return ActivationInfo(static_cast<ActivationInfo::ActivationType>(f), f != TFlite::ActivationFunctionType_NONE);
    }

    bool android_nn() const { return legacy_model_ == TFlite::LegacyModel_ANDROID_NN; }

    template <typename Options>
    void layout_of(const Options &o, bool *androidNN, bool *isNCHW) const {
        *androidNN = android_nn();
        *isNCHW = *androidNN ? o.use_nchw : is_nchw_layout(legacy_model_);
    }

    template <typename Options>
    void padding_of(const Options &o, Pad4 *padding, const UDTensors &in, const UDTensors &out, const NDims &weight_dims, Dim2 stride,
                    Dim2 dilation, bool deconv, bool nchw, bool explicit_for_all_models = false) const {
        if ((android_nn() || explicit_for_all_models) && o.padding_value.size() == 4) {
            padding->l = (uint32_t)o.padding_value[0];
            padding->r = (uint32_t)o.padding_value[1];
            padding->t = (uint32_t)o.padding_value[2];
            padding->b = (uint32_t)o.padding_value[3];
        } else {
            get_padding(legacy_model_, o.padding, *padding, in[0]->getDims(), out[0]->getDims(), weight_dims, stride, dilation, deconv, nchw);
        }
    }

    std::shared_ptr<ITensor> allocate_tensor(const std::shared_ptr<TensorDesc> &edge, const PrecisionType &precision,
                                             const BufferType &buffer_type) {
        if (edge->shape.empty() || edge->shape.size() > 4) {
            ERROR_PRINT("OperationConstructor: tensor %s has %zu dimensions\n", edge->name.c_str(), edge->shape.size());
            return nullptr;
        }
        const Dim4 dims = extendToDim4(edge->shape);
        const DataType type = to_data_type(edge->data_type);
        if (!edge->is_const) {
            auto found = alloc_tensors_.find(edge->buffer_index);
            if (found != alloc_tensors_.end()) return found->second;
            std::shared_ptr<ITensor> tensor = std::make_shared<HipTensor>(runtime_, precision, type, dims, DataOrder::NCHW, edge->scale,
                                                                          edge->zero_point, buffer_type, StorageType::BUFFER, 0,
                                                                          edge->buffer_index);
            alloc_tensors_[edge->buffer_index] = tensor;
            if (!produced_.count(edge->buffer_index))
                in_tensors.push_back(tensor);
            else if (!consumed_.count(edge->buffer_index))
                out_tensors.push_back(tensor);
            return tensor;
        }
        if (edge->data == nullptr) {
            ERROR_PRINT("OperationConstructor: parameter %s has no data\n", edge->name.c_str());
            return nullptr;
        }
        switch (type) {
            case DataType::UINT8:
                return std::make_shared<HipTensor>(runtime_, precision, static_cast<const uint8_t *>(edge->data), dims, DataOrder::NCHW,
                                                   edge->scale, edge->zero_point);
            case DataType::INT8:
                return std::make_shared<HipTensor>(runtime_, precision, static_cast<const int8_t *>(edge->data), dims, DataOrder::NCHW,
                                                   edge->scale, edge->zero_point);
            case DataType::INT32:
                return std::make_shared<HipTensor>(runtime_, precision, static_cast<const int32_t *>(edge->data), dims, DataOrder::NCHW,
                                                   edge->scale, edge->zero_point);
            default: ERROR_PRINT("OperationConstructor: parameter %s has an unsupported type\n", edge->name.c_str());
        }
        return nullptr;
    }

    // outputs first (they may take over storage released by earlier operators), then inputs; an input
    // whose last reader this operator is gives its storage back (gpu_op_constructor.cc:2157-2191)
    bool convert_to_tensors(const OperatorDesc &op, const PrecisionType &precision, UDTensors &in, UDTensors &out) {
        for (const auto &edge : op.out_tensors) {
            auto tensor = allocate_tensor(edge, precision, BufferType::INTER_SHARED_REUSE);
            if (tensor == nullptr) return false;
            out.push_back(tensor);
        }
        for (const auto &edge : op.in_tensors) {
            auto tensor = allocate_tensor(edge, precision, BufferType::INTER_SHARED_NEW);
            if (tensor == nullptr) return false;
            in.push_back(tensor);
            if (!edge->is_const) {
                auto used = tensors_used_.find(edge->buffer_index);
                if (used != tensors_used_.end() && used->second > 0 && --used->second == 0) tensor->resetInterBuffer();
            }
        }
        return true;
    }

    template <typename Op, typename Params>
    EnnReturn finish(const OperatorDesc &op, const PrecisionType &precision, const UDTensors &in, const UDTensors &out,
                     const std::shared_ptr<Params> &parameters) {
        auto impl = std::make_shared<Op>(runtime_, precision);
        if (impl->initialize(in, out, parameters) != Status::SUCCESS) return ENN_RET_FAILED;
        operators->push_back(std::make_shared<EnnUDOperator<Op>>(op.name, op.id, in, out, UDTensors(), impl));
        return ENN_RET_SUCCESS;
    }

    template <typename Options>
    const Options *options_of(const OperatorDesc &op) const {
        return static_cast<const Options *>(op.option.get());
    }

    EnnReturn create_conv(const OperatorDesc &op) {
        if (op.out_tensors.empty() || op.in_tensors.size() < 3 || !op.option) return ENN_RET_FAILED;
        const PrecisionType precision = get_precision(op.out_tensors[0]->data_type);
        UDTensors in, out;
        if (!convert_to_tensors(op, precision, in, out)) return ENN_RET_FAILED;
        const auto *o = options_of<TFlite::Conv2DOptions>(op);
        auto p = std::make_shared<ConvolutionParameters>();
        p->dilation = {(uint32_t)o->dilation_h_factor, (uint32_t)o->dilation_w_factor};
        p->stride = {(uint32_t)o->stride_h, (uint32_t)o->stride_w};
        p->activation_info = std::make_shared<ActivationInfo>(to_activation(o->fused_activation_function));
        p->group_size = 1;
        layout_of(*o, &p->androidNN, &p->isNCHW);
        padding_of(*o, &p->padding, in, out, in[1]->getDims(), p->stride, p->dilation, false, p->isNCHW);
        p->per_channel_quant = !op.in_tensors[1]->per_channel_scales.empty();
        p->scales = op.in_tensors[1]->per_channel_scales;
        return finish<HipConvolution>(op, precision, in, out, p);
    }

    // `add` consumes `conv`'s only output, nothing else does, both are uint8 per-tensor, and the sum is not
    // written over one of the tensors the fused launch still reads
    bool fusable_add(const OperatorDesc &conv, const OperatorDesc &add) const {
        if (conv.code != TFlite::BuiltinOperator_CONV_2D || add.code != TFlite::BuiltinOperator_ADD) return false;
        if (conv.out_tensors.size() != 1 || conv.in_tensors.size() < 3 || add.in_tensors.size() != 2 || add.out_tensors.size() != 1 ||
            !conv.option || !add.option)
            return false;
        const auto &produced = conv.out_tensors[0];
        const bool first = add.in_tensors[0]->buffer_index == produced->buffer_index && !add.in_tensors[0]->is_const;
        const bool second = add.in_tensors[1]->buffer_index == produced->buffer_index && !add.in_tensors[1]->is_const;
        if (first == second) return false;  // neither, or the convolution added to itself
        const auto &other = add.in_tensors[first ? 1 : 0];
        if (other->is_const) return false;
        const auto readers = tensors_used_.find(produced->buffer_index);
        if (readers == tensors_used_.end() || readers->second != 1) return false;
        if (!conv.in_tensors[1]->per_channel_scales.empty()) return false;
        for (const auto &t : {produced, other, add.out_tensors[0], conv.in_tensors[0]})
            if (t->data_type != TFlite::TensorType_UINT8) return false;
        if (produced->shape != other->shape || produced->shape != add.out_tensors[0]->shape) return false;
        const int32_t sum = add.out_tensors[0]->buffer_index;
        return sum != other->buffer_index && sum != produced->buffer_index && sum != conv.in_tensors[0]->buffer_index;
    }

    // The Add's tensors are made first: its output then cannot be given the storage of a feature map the
    // convolution still reads (the convolution's input may see its last reader here and be handed back to the pool
    // once the convolution's own tensors are made).
    EnnReturn create_conv_with_add(const OperatorDesc &conv, const OperatorDesc &add) {
        const PrecisionType precision = get_precision(add.out_tensors[0]->data_type);
        UDTensors add_in, add_out;
        if (!convert_to_tensors(add, precision, add_in, add_out)) return ENN_RET_FAILED;
        if (create_conv(conv) != ENN_RET_SUCCESS) return ENN_RET_FAILED;
        auto wrapper = std::dynamic_pointer_cast<EnnUDOperator<HipConvolution>>(operators->back());
        if (!wrapper) return ENN_RET_FAILED;
        const bool conv_first = add.in_tensors[0]->buffer_index == conv.out_tensors[0]->buffer_index;
        const auto *o = options_of<TFlite::AddOptions>(add);
        return wrapper->getOp()->fuseResidualAdd(add_in[conv_first ? 1 : 0], add_out[0],
                                                          to_activation(o->fused_activation_function)) == Status::SUCCESS
                   ? ENN_RET_SUCCESS
                   : ENN_RET_FAILED;
    }

    EnnReturn create_depthwise(const OperatorDesc &op) {
        if (op.out_tensors.empty() || op.in_tensors.size() < 3 || !op.option) return ENN_RET_FAILED;
        const PrecisionType precision = get_precision(op.out_tensors[0]->data_type);
        UDTensors in, out;
        if (!convert_to_tensors(op, precision, in, out)) return ENN_RET_FAILED;
        const auto *o = options_of<TFlite::DepthwiseConv2DOptions>(op);
        auto p = std::make_shared<DepthwiseConvolutionParameters>();
        p->dilation = {(uint32_t)o->dilation_h_factor, (uint32_t)o->dilation_w_factor};
        p->stride = {(uint32_t)o->stride_h, (uint32_t)o->stride_w};
        p->depth_multiplier = (uint32_t)o->depth_multiplier;
        p->activation_info = std::make_shared<ActivationInfo>(to_activation(o->fused_activation_function));
        layout_of(*o, &p->androidNN, &p->isNCHW);
        padding_of(*o, &p->padding, in, out, in[1]->getDims(), p->stride, p->dilation, false, p->isNCHW);
        p->per_channel_quant = !op.in_tensors[1]->per_channel_scales.empty();
        p->scales = op.in_tensors[1]->per_channel_scales;
        return finish<HipDepthwiseConvolution>(op, precision, in, out, p);
    }

    EnnReturn create_deconv(const OperatorDesc &op) {
        if (op.out_tensors.empty() || op.in_tensors.size() != 3 || !op.option) return ENN_RET_FAILED;
        const PrecisionType precision = get_precision(op.out_tensors[0]->data_type);
        UDTensors in, out;
        if (!convert_to_tensors(op, precision, in, out)) return ENN_RET_FAILED;
        const auto *o = options_of<TFlite::TransposeConvOptions>(op);
        auto p = std::make_shared<DeconvolutionParameters>();
        p->stride = {(uint32_t)o->stride_h, (uint32_t)o->stride_w};
        p->group_size = (uint32_t)o->group;
        p->weights_as_input = !in[1]->is_const();
        p->activation_info = std::make_shared<ActivationInfo>(to_activation(o->fused_activation_function));
        layout_of(*o, &p->androidNN, &p->isNCHW);
        padding_of(*o, &p->padding, in, out, in[1]->getDims(), p->stride, Dim2{1, 1}, true, p->isNCHW);
        p->per_channel_quant = !op.in_tensors[1]->per_channel_scales.empty();
        p->scales = op.in_tensors[1]->per_channel_scales;
        return finish<HipDeconvolution>(op, precision, in, out, p);
    }

    EnnReturn create_fc(const OperatorDesc &op) {
        if (op.out_tensors.empty() || op.in_tensors.size() < 3 || !op.option) return ENN_RET_FAILED;
        const PrecisionType precision = get_precision(op.out_tensors[0]->data_type);
        UDTensors in, out;
        if (!convert_to_tensors(op, precision, in, out)) return ENN_RET_FAILED;
        const auto *o = options_of<TFlite::FullyConnectedOptions>(op);
        auto p = std::make_shared<FullyConnectedParameters>();
        p->androidNN = android_nn();
        p->activation_info = std::make_shared<ActivationInfo>(to_activation(o->fused_activation_function));
        return finish<HipFullyConnected>(op, precision, in, out, p);
    }

    EnnReturn create_avgpool(const OperatorDesc &op) {
        if (op.out_tensors.empty() || op.in_tensors.empty() || !op.option) return ENN_RET_FAILED;
        const PrecisionType precision = get_precision(op.out_tensors[0]->data_type);
        UDTensors in, out;
        if (!convert_to_tensors(op, precision, in, out)) return ENN_RET_FAILED;
        const auto *o = options_of<TFlite::Pool2DOptions>(op);
        auto p = std::make_shared<Pool2DParameters>();
        p->stride = {(uint32_t)o->stride_h, (uint32_t)o->stride_w};
        p->filter = {(uint32_t)o->filter_height, (uint32_t)o->filter_width};
        const bool caffe = legacy_model_ == TFlite::LegacyModel_CAFFE || legacy_model_ == TFlite::LegacyModel_CAFFE_NCHW ||
                           legacy_model_ == TFlite::LegacyModel_CAFFE_NHWC;
        p->compute_type = caffe ? ComputeType::Caffe : ComputeType::TFLite;
        p->activation_info = to_activation(o->fused_activation_function);
        layout_of(*o, &p->androidNN, &p->isNCHW);
        // the pool takes explicit padding values from every model kind (gpu_op_constructor.cc:832-847)
        padding_of(*o, &p->padding, in, out, NDims{1, 1, p->filter.h, p->filter.w}, p->stride, Dim2{1, 1}, false, p->isNCHW, true);
        return finish<HipAveragepool>(op, precision, in, out, p);
    }

    EnnReturn create_add(const OperatorDesc &op) {
        if (op.out_tensors.empty() || op.in_tensors.size() != 2 || !op.option) return ENN_RET_FAILED;
        const PrecisionType precision = get_precision(op.out_tensors[0]->data_type);
        UDTensors in, out;
        if (!convert_to_tensors(op, precision, in, out)) return ENN_RET_FAILED;
        const auto *o = options_of<TFlite::AddOptions>(op);
        auto p = std::make_shared<AddParameters>();
        p->activation_info = to_activation(o->fused_activation_function);
        p->coeff = o->coeff.empty() ? std::vector<float>(in.size(), 1.0f) : o->coeff;
        p->androidNN = android_nn();
        p->isNCHW = false;
        return finish<HipAdd>(op, precision, in, out, p);
    }

    std::shared_ptr<HipRuntime> runtime_;
    TFlite::LegacyModel legacy_model_ = TFlite::LegacyModel_TENSORFLOW_NHWC;
    std::map<int32_t, std::shared_ptr<ITensor>> alloc_tensors_;  // feature maps by buffer index
    std::map<int32_t, int32_t> tensors_used_;                    // readers still to be built, by buffer index
    std::map<int32_t, bool> produced_, consumed_;
};

// Runs a built list: host bytes into the list's input tensors, every operator in order on the
// runtime's stream, the list's output tensors back to the host (gpu_op_executor.cc:56-103).
class OperationExecutor {
public:
    explicit OperationExecutor(std::shared_ptr<HipRuntime> runtime) : runtime_(runtime) {}

    EnnReturn execute(const OperationConstructor &built, const std::vector<const void *> &inputs, const std::vector<void *> &outputs) {
        if (!built.operators || inputs.size() != built.in_tensors.size() || outputs.size() != built.out_tensors.size()) {
            ERROR_PRINT("OperationExecutor: %zu inputs and %zu outputs given, the list has %zu and %zu\n", inputs.size(), outputs.size(),
                        built.in_tensors.size(), built.out_tensors.size());
            return ENN_RET_FAILED;
        }
        for (size_t i = 0; i < inputs.size(); ++i)
            if (built.in_tensors[i]->writeData(const_cast<void *>(inputs[i])) != Status::SUCCESS) return ENN_RET_FAILED;
        auto buffer = std::make_shared<UDBuffer>();
        buffer->set_id(++execution_id_);
        for (auto &op : *built.operators)
            if (op->execute(buffer) != ENN_RET_SUCCESS) {
                ERROR_PRINT("OperationExecutor: %s failed\n", op->getName().c_str());
                return ENN_RET_FAILED;
            }
        for (size_t i = 0; i < outputs.size(); ++i)
            if (built.out_tensors[i]->readData(outputs[i]) != Status::SUCCESS) return ENN_RET_FAILED;
        return ENN_RET_SUCCESS;
    }

private:
    std::shared_ptr<HipRuntime> runtime_;
    uint64_t execution_id_ = 0;
};

}  // namespace hip
}  // namespace ud
}  // namespace enn
