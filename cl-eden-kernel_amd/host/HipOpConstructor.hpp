// Operator construction from TFLite-style options, and the executor of the resulting list.
//
// Mirrors OperationConstructor / OperationExecutor of the reference
// (src/userdriver/gpu/gpu_op_constructor.h:33-56, gpu_op_constructor.cc:63-383 CONV_2D / DEPTHWISE_CONV_2D /
// TRANSPOSE_CONV / FULLY_CONNECTED, :789-860 AVERAGE_POOL_2D, :1166-1205 ADD, :1797-1870 open_oplist / close_oplist,
// :1884-2009 layout / precision / padding helpers, :2062-2191 tensor allocation with inter-buffer reuse;
// src/userdriver/gpu/gpu_op_executor.h:31-44, gpu_op_executor.cc:56-103) for the six operators this backend has.
// Both are built on a HipComputeLibrary, as the reference's are on its CLComputeLibrary: every tensor comes from
// create_tensor / create_and_copy_tensor, every operator from create<Operator>(precision), pooled buffers are
// materialised by assignBuffers().
//
// Where the executor differs: the reference enqueues every operator's kernels on one in-order queue at each execution
// (one clFlush per subgraph).  Here a list whose operators only launch kernels is recorded into a HIP graph the second
// time it runs with the same tensors and quantization parameters, and replayed from then on (one launch per execution
// instead of one per kernel); anything that changes what was recorded (a tensor's scale or zero point, a buffer that
// moved) makes the next execution run operator by operator again and re-record.
#pragma once

#include <algorithm>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "HipComputeLibrary.hpp"
#include "ModelDesc.hpp"
#include "userdriver_operator.hpp"


namespace enn {
namespace ud {
namespace hip {

class OperationConstructor {
public:
    explicit OperationConstructor(std::shared_ptr<HipComputeLibrary> compute_library) : compute_library_(compute_library) {}
    ~OperationConstructor() {
        alloc_tensors_map_.clear();
        tensors_used_.clear();
    }

    // IOperationConstructor (src/userdriver/common/IOperationConstructor.h:28-37)
    EnnReturn initialize_ud_operators() {
        operators = std::make_shared<std::vector<std::shared_ptr<UDOperator>>>();
        in_tensors.clear();
        out_tensors.clear();
        return ENN_RET_SUCCESS;
    }
    const UDOperators &get_ud_operators() { return operators; }
    const UDTensors &get_in_tensors() const { return in_tensors; }
    const UDTensors &get_out_tensors() const { return out_tensors; }

    // Builds every operator of the list in order (tensors are created as the operators name them; a
    // feature map's storage is handed back to the pool once its last reader has been built), materialises
    // the pooled buffers and waits for the device (gpu_op_constructor.cc:1797-1850).
    EnnReturn open_oplist(const OperatorListDesc &list) {
        std::lock_guard<std::mutex> lock_guard(mutex_constructor_);
        if (!operators) initialize_ud_operators();
        operator_list_id_ = list.id;
        legacy_model_ = list.legacy_model;
        produced_.clear();
        consumed_.clear();
        const_tensors_.clear();
        for (const auto &op : list.operators) {
            for (const auto &t : op.out_tensors) produced_[t->buffer_index] = true;
            for (const auto &t : op.in_tensors)
                if (!t->is_const) consumed_[t->buffer_index] = true;
        }
        channels_last_ = store_channels_last && planar_list_can_be_stored_channels_last(list);
        pending_layout_ops_.clear();
        lanes_ = lanes_for(list);
        const auto runtime = compute_library_->runtime();
        for (lane_ = 0; lane_ < lanes_; ++lane_) {
            // every lane builds the whole list on its share of the images, with feature maps in an arena of its own
            runtime->selectArena(lane_);
            tensors_used_.clear();
            for (const auto &op : list.operators)
                for (const auto &t : op.in_tensors)
                    if (!t->is_const) tensors_used_[t->buffer_index]++;  // init_inter_buffer
            const size_t first_operator = operators->size();
            for (size_t index = 0; index < list.operators.size(); ++index) {
                const auto &op = list.operators[index];
                if (fuse_residual_adds && index + 1 < list.operators.size() && fusable_add(op, list.operators[index + 1])) {
                    if (create_conv_with_add(op, list.operators[index + 1]) != ENN_RET_SUCCESS) {
                        ERROR_PRINT("OperationConstructor: building %s with its residual add failed\n", op.name.c_str());
                        return abandon();
                    }
                    ++index;  // the Add went into the convolution's launch
                    append_pending_layout_changes();
                    continue;
                }
                if (fuse_expansions && index + 1 < list.operators.size() && fusable_expansion(op, list.operators[index + 1])) {
                    if (create_conv_with_depthwise(op, list.operators[index + 1]) != ENN_RET_SUCCESS) {
                        ERROR_PRINT("OperationConstructor: building %s with the depthwise convolution behind it failed\n", op.name.c_str());
                        return abandon();
                    }
                    ++index;  // the depthwise convolution went into the pointwise convolution's launch
                    append_pending_layout_changes();
                    continue;
                }
                if (create_ud_operator(op) != ENN_RET_SUCCESS) {
                    ERROR_PRINT("OperationConstructor: building %s failed\n", op.name.c_str());
                    return abandon();
                }
                append_pending_layout_changes();
            }
            for (size_t i = first_operator; i < operators->size(); ++i) (*operators)[i]->setLane(lane_);
        }
        lane_ = 0;
        runtime->selectArena(0);
        compute_library_->assignBuffers();
        compute_library_->synchronize();
        tensors_used_.clear();
        produced_.clear();
        consumed_.clear();
        const_tensors_.clear();
        for (const auto &kv : alloc_tensors_map_[operator_list_id_])  // a pooled buffer that assignBuffers() could not place
            if (kv.second->getNumOfBytes() != 0 && std::static_pointer_cast<HipTensor>(kv.second)->hasStorage() &&
                std::static_pointer_cast<HipTensor>(kv.second)->getDataPtr() == nullptr) {
                ERROR_PRINT("OperationConstructor: feature map %d has no device memory after assignBuffers()\n", kv.first);
                return ENN_RET_FAILED;
            }
        return ENN_RET_SUCCESS;
    }

    // Whether every operator of the list is a planar one this constructor can run on channels-last storage: the six
    // operator kinds, all in planar mode, constant parameters, byte feature maps, and no fully connected layer that
    // flattens more than one pixel per image (its weights are ordered for the planar flattening).
    bool planar_list_can_be_stored_channels_last(const OperatorListDesc &list) const {
        if (list.operators.empty()) return false;
        for (const auto &op : list.operators) {
            bool android = false, nchw = true;
            switch (op.code) {
                case TFlite::BuiltinOperator_CONV_2D:
                    if (!op.option) return false;
                    layout_of(*options_of<TFlite::Conv2DOptions>(op), &android, &nchw);
                    break;
                case TFlite::BuiltinOperator_DEPTHWISE_CONV_2D:
                    if (!op.option) return false;
                    layout_of(*options_of<TFlite::DepthwiseConv2DOptions>(op), &android, &nchw);
                    break;
                case TFlite::BuiltinOperator_TRANSPOSE_CONV:
                    if (!op.option) return false;
                    layout_of(*options_of<TFlite::TransposeConvOptions>(op), &android, &nchw);
                    break;
                case TFlite::BuiltinOperator_AVERAGE_POOL_2D:
                    if (!op.option) return false;
                    layout_of(*options_of<TFlite::Pool2DOptions>(op), &android, &nchw);
                    break;
                case TFlite::BuiltinOperator_FULLY_CONNECTED:
                    if (op.in_tensors.empty()) return false;
                    if (!op.in_tensors[0]->is_const && op.in_tensors[0]->shape.size() == 4 &&
                        (uint64_t)op.in_tensors[0]->shape[2] * op.in_tensors[0]->shape[3] > 1)
                        return false;
                    break;
                case TFlite::BuiltinOperator_ADD: break;
                default: return false;
            }
            if (!nchw) return false;
            // weights and bias that are run-time feature maps have shapes of their own kind: such a list stays as it is
            if (op.code != TFlite::BuiltinOperator_ADD && op.code != TFlite::BuiltinOperator_AVERAGE_POOL_2D)
                for (size_t i = 1; i < op.in_tensors.size(); ++i)
                    if (!op.in_tensors[i]->is_const) return false;
            for (const auto *edges : {&op.in_tensors, &op.out_tensors})
                for (const auto &t : *edges)
                    if (!t->is_const && t->shape.size() == 4 && t->data_type != TFlite::TensorType_UINT8 && t->data_type != TFlite::TensorType_INT8)
                        return false;
        }
        return true;
    }

    // the layout operators that follow the operator built last (those of the list's outputs it writes)
    void append_pending_layout_changes() {
        for (auto &op : pending_layout_ops_) operators->push_back(op);
        pending_layout_ops_.clear();
    }

    // How many lanes the list's images are cut into (1: none).  A list qualifies when every feature map carries the
    // same number of images in its leading dimension, that number divides by image_lanes into shares of at least
    // min_lane_images, and all parameters are constants (a run-time weight tensor has no image dimension to cut).
    // Every operator this constructor builds treats the images of its tensors independently, so the lanes compute
    // exactly what the whole list computes.
    int lanes_for(const OperatorListDesc &list) const {
        if (image_lanes <= 1) return 1;
        uint32_t images = 0;
        for (const auto &op : list.operators) {
            for (const auto *edges : {&op.in_tensors, &op.out_tensors})
                for (const auto &t : *edges) {
                    if (t->is_const) continue;
                    if (t->shape.size() < 2 || t->shape[0] == 0) return 1;
                    if (images == 0) images = t->shape[0];
                    if (t->shape[0] != images) return 1;
                }
            const bool has_parameters = op.code != TFlite::BuiltinOperator_ADD && op.code != TFlite::BuiltinOperator_AVERAGE_POOL_2D;
            if (has_parameters)
                for (size_t i = 1; i < op.in_tensors.size(); ++i)
                    if (!op.in_tensors[i]->is_const) return 1;
        }
        if (images == 0 || images % (uint32_t)image_lanes != 0 || images / (uint32_t)image_lanes < (uint32_t)min_lane_images) return 1;
        return image_lanes;
    }

    // Drops the constructor's own references to the list's feature maps (gpu_op_constructor.cc:1852-1870); the
    // operators keep theirs until the userdriver forgets the list.
    void close_oplist(const uint64_t &oplist_id) {
        std::lock_guard<std::mutex> lock_guard(mutex_constructor_);
        alloc_tensors_map_.erase(oplist_id);
    }

    EnnReturn create_ud_operator(const OperatorDesc &op) {
        switch (op.code) {
            case TFlite::BuiltinOperator_CONV_2D: return create_conv(op);
            case TFlite::BuiltinOperator_DEPTHWISE_CONV_2D: return create_depthwise(op);
            case TFlite::BuiltinOperator_TRANSPOSE_CONV: return create_deconv(op);
            case TFlite::BuiltinOperator_FULLY_CONNECTED: return create_fc(op);
            case TFlite::BuiltinOperator_AVERAGE_POOL_2D: return create_avgpool(op);
            case TFlite::BuiltinOperator_ADD: return create_add(op);
            default: ERROR_PRINT("OperationConstructor: operator code %d is not offered\n", (int)op.code);
        }
        return ENN_RET_FAILED;
    }

    UDOperators operators;
    UDTensors in_tensors, out_tensors;  // feature maps no operator of the list writes / reads
    // A uint8 ADD right behind the CONV_2D that produces one of its operands, where nothing else reads that
    // operand, runs inside the convolution's launch (HipConvolution::fuseResidualAdd); the list then holds one
    // operator less than the description.  The reference builds one operator per description
    // (gpu_op_constructor.cc:63-383); set to false for that.
    bool fuse_residual_adds = true;
    // A feature map no operator of the list writes (a list input) keeps its storage for the life of the list, so that
    // the list can run again on data that is already on the device.  The reference hands such a buffer on to later
    // feature maps once its last reader is built, which is safe there because every ExecuteSubGraph rewrites the
    // inputs first (gpu_userdriver.cc:97-99); set to false for that.
    bool keep_list_inputs = true;
    // A list whose feature maps all carry the same number of images is built image_lanes times over, each time on
    // 1 / image_lanes of the images (a contiguous share of every tensor: the images are the leading dimension), with
    // feature maps of its own; the executor runs the lanes side by side on streams of their own.  The list's inputs
    // and outputs stay whole tensors, of which every lane sees its share.  A launch ends in a tail during which most
    // of the device idles, and the next takes a while to fill it: two lanes fill those gaps for one another
    // (MobileNetV2 at 64 images: 490 -> 444 us per execution; four lanes of 16 images lose more in their smaller
    // launches than they gain).  1 = one operator per description, as the reference builds the list.
    int image_lanes = 2;
    // (from 12 images per lane on two lanes win: MobileNetV2 at batch 24 309 against 327 us, at 32 338 against 352;
    // at batch 16 they tie and below that the lanes' launches no longer overlap and two lanes cost 282 against 248 us at
    // batch 8, 271 against 195 at batch 2)
    int min_lane_images = 12;
    // A uint8 1x1 CONV_2D whose only reader is a 3x3 DEPTHWISE_CONV_2D (an inverted-residual block's expansion) runs
    // with it as one launch where the library's table of measured shapes says that is the faster way
    // (eh_conv_dw_block_listed); the tensor between them then has no storage at all.  false = one operator per
    // description, as the reference builds the list.
    bool fuse_expansions = true;
    bool fuse_unlisted_expansions = false;  // fuse every pair the kernel fits, measured faster or not (tests, experiments)
    // The feature maps inside a PLANAR operator list (a Caffe-style model, or an androidNN one with use_nchw) are stored
    // channels-last: the kernels of this backend work on channels-last data, and a planar tensor costs every operator a
    // transposition on either side (MobileNetV2 at 64 images as a planar list: 1872 us per execution with planar
    // storage).  The list's inputs and outputs stay planar for its owner; one layout operator behind each input and in
    // front of each output is added to the list.  Shapes, parameters and results are those of the planar list.
    // false = every tensor stored as its shape reads, as the reference does.
    bool store_channels_last = true;
    bool stores_channels_last() const { return channels_last_; }  // of the list opened last
    int lanes() const { return lanes_; }  // of the list opened last

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
    // a list that fails half way: its operators and tensors go, and the pooled buffers they asked for are given up
    EnnReturn abandon() {
        if (operators) operators->clear();
        in_tensors.clear();
        out_tensors.clear();
        alloc_tensors_map_.erase(operator_list_id_);
        compute_library_->abandonBuffers();
        return ENN_RET_FAILED;
    }

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

    // The feature map of `edge` as its shape reads: one pooled tensor per buffer index and lane, or, for an input or output
    // of a list that is cut into lanes, one whole tensor and this lane's view of its share.
    std::shared_ptr<ITensor> allocate_feature_map(const std::shared_ptr<TensorDesc> &edge, const PrecisionType &precision, const BufferType &buffer_type,
                                                  const DataOrder &data_order, const NDims &dims, bool list_io) {
        auto &made = alloc_tensors_map_[operator_list_id_];
        if (lanes_ > 1 && list_io) {
            // an input or output of the list: one whole tensor in an arena no lane takes storage from, and this
            // lane's view of its share
            std::shared_ptr<ITensor> &whole = made[edge->buffer_index];
            if (whole == nullptr) {
                compute_library_->runtime()->selectArena(lanes_);
                whole = compute_library_->create_tensor(edge->data_type, precision, dims, edge->buffer_index, BufferType::INTER_SHARED_NEW,
                                                        false, StorageType::BUFFER, data_order, edge->scale, edge->zero_point);
                compute_library_->runtime()->selectArena(lane_);
                if (whole == nullptr) {
                    made.erase(edge->buffer_index);
                    ERROR_PRINT("OperationConstructor: feature map %s could not be made\n", edge->name.c_str());
                    return nullptr;
                }
                (produced_.count(edge->buffer_index) ? out_tensors : in_tensors).push_back(whole);
            }
            std::shared_ptr<ITensor> &view = made[lane_key(edge->buffer_index)];
            if (view == nullptr) {
                const uint32_t share = dims[0] / (uint32_t)lanes_;
                view = std::make_shared<HipTensor>(std::static_pointer_cast<HipTensor>(whole), share * (uint32_t)lane_, share);
            }
            return view;
        }
        auto found = made.find(lane_key(edge->buffer_index));
        if (found != made.end()) return found->second;
        NDims lane_dims = dims;
        lane_dims[0] /= (uint32_t)lanes_;
        std::shared_ptr<ITensor> tensor = compute_library_->create_tensor(edge->data_type, precision, lane_dims, edge->buffer_index, buffer_type,
                                                                          false, StorageType::BUFFER, data_order, edge->scale,
                                                                          edge->zero_point);
        if (tensor == nullptr) {
            ERROR_PRINT("OperationConstructor: feature map %s could not be made\n", edge->name.c_str());
            return nullptr;
        }
        made[lane_key(edge->buffer_index)] = tensor;
        if (lanes_ == 1) {
            if (!produced_.count(edge->buffer_index))
                in_tensors.push_back(tensor);
            else if (!consumed_.count(edge->buffer_index))
                out_tensors.push_back(tensor);
        }
        return tensor;
    }

    // A feature map becomes a pooled run-time tensor, made once per buffer index of the list; a parameter becomes a
    // constant tensor uploaded at once (gpu_op_constructor.cc:2062-2155).
    std::shared_ptr<ITensor> allocate_tensor(const std::shared_ptr<TensorDesc> &edge, const PrecisionType &precision,
                                             const BufferType &buffer_type, const DataOrder &data_order = DataOrder::NCHW) {
        if (edge->shape.empty() || edge->shape.size() > 4) {
            ERROR_PRINT("OperationConstructor: tensor %s has %zu dimensions\n", edge->name.c_str(), edge->shape.size());
            return nullptr;
        }
        // operators read positional (n, c, h, w) extents from a four-entry shape, as the reference's CLTensor gives them
        const Dim4 d4 = extendToDim4(edge->shape);
        const NDims dims = {d4.n, d4.c, d4.h, d4.w};
        if (!edge->is_const) {
            auto &made = alloc_tensors_map_[operator_list_id_];
            const bool list_io = !produced_.count(edge->buffer_index) || !consumed_.count(edge->buffer_index);
            // stored channels-last inside a planar list (a tensor of one pixel per image, or of one channel, is both orders at once)
            const bool channels_last = channels_last_ && edge->shape.size() == 4 && (uint64_t)d4.h * d4.w > 1 && d4.c > 1;
            if (!(channels_last && list_io)) {
                auto tensor = allocate_feature_map(edge, precision, buffer_type, data_order, dims, list_io);
                if (tensor != nullptr && channels_last) std::static_pointer_cast<HipTensor>(tensor)->storeChannelsLast(true);
                return tensor;
            }
            // An input or output of such a list: its owner reads and writes the planar tensor; the operators see a
            // channels-last twin (this lane's share of it), and a layout operator carries the data across.
            const int32_t twin_key = lane_key(edge->buffer_index) + kTwinKeyOffset;
            auto found = made.find(twin_key);
            if (found != made.end()) return found->second;
            auto planar = allocate_feature_map(edge, precision, buffer_type, data_order, dims, list_io);
            if (planar == nullptr) return nullptr;
            NDims lane_dims = dims;
            lane_dims[0] /= (uint32_t)lanes_;
            const bool is_input = !produced_.count(edge->buffer_index);
            std::shared_ptr<ITensor> twin = compute_library_->create_tensor(edge->data_type, precision, lane_dims, edge->buffer_index,
                                                                            is_input ? BufferType::INTER_SHARED_NEW : buffer_type, false,
                                                                            StorageType::BUFFER, data_order, edge->scale, edge->zero_point);
            if (twin == nullptr) {
                ERROR_PRINT("OperationConstructor: the channels-last twin of feature map %s could not be made\n", edge->name.c_str());
                return nullptr;
            }
            std::static_pointer_cast<HipTensor>(twin)->storeChannelsLast(true);
            auto change = std::make_shared<HipLayoutChange>(compute_library_->runtime(), is_input);
            const UDTensors from = {is_input ? planar : twin}, to = {is_input ? twin : planar};
            if (change->initialize(from, to) != Status::SUCCESS) return nullptr;
            auto wrapped = std::make_shared<EnnUDOperator<HipLayoutChange>>((is_input ? "TO_CHANNELS_LAST_" : "TO_PLANAR_") + std::to_string(edge->buffer_index),
                                                                           0, from, to, UDTensors(), change);
            if (is_input)
                operators->push_back(wrapped);  // in front of the operator that is being built, the input's first reader
            else
                pending_layout_ops_.push_back(wrapped);  // behind it, the output's writer
            made[twin_key] = twin;
            return twin;
        }
        // a parameter is uploaded once and read by every lane's operator
        auto shared = const_tensors_.find(edge.get());
        if (shared != const_tensors_.end()) return shared->second;
        if (edge->data == nullptr) {
            ERROR_PRINT("OperationConstructor: parameter %s has no data\n", edge->name.c_str());
            return nullptr;
        }
        DataPtr data = const_cast<DataPtr>(edge->data);
        auto tensor = compute_library_->create_and_copy_tensor(edge->data_type, data, precision, dims, UNDEFINED, buffer_type, false,
                                                               StorageType::BUFFER, data_order, edge->scale, edge->zero_point);
        if (tensor == nullptr) ERROR_PRINT("OperationConstructor: parameter %s could not be made\n", edge->name.c_str());
        if (tensor != nullptr && lanes_ > 1) const_tensors_[edge.get()] = tensor;
        return tensor;
    }

    // feature maps of lane 0 (and whole list inputs / outputs) are filed under their buffer index, those of the other
    // lanes (and all views) above every buffer index
    int32_t lane_key(int32_t buffer_index) const {
        const bool whole_tensor_has_the_index = lanes_ > 1 && (!produced_.count(buffer_index) || !consumed_.count(buffer_index));
        return lane_ == 0 && !whole_tensor_has_the_index ? buffer_index : buffer_index + (lane_ + 1) * kLaneKeyStride;
    }
    static constexpr int32_t kLaneKeyStride = 1 << 24;
    static constexpr int32_t kTwinKeyOffset = 1 << 29;  // the channels-last twins of a planar list's inputs and outputs

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
                if (used != tensors_used_.end() && used->second > 0 && --used->second == 0 &&
                    !(keep_list_inputs && !produced_.count(edge->buffer_index)))
                    tensor->resetInterBuffer();
            }
        }
        return true;
    }

    template <typename Op, typename Params>
    EnnReturn finish(const OperatorDesc &op, const std::shared_ptr<Op> &impl, const UDTensors &in, const UDTensors &out,
                     const std::shared_ptr<Params> &parameters) {
        if (impl == nullptr || impl->initialize(in, out, parameters) != Status::SUCCESS) return ENN_RET_FAILED;
        operators->push_back(std::make_shared<EnnUDOperator<Op>>(op.name, op.id, in, out, UDTensors(), impl));
        return ENN_RET_SUCCESS;
    }

    template <typename Options>
    const Options *options_of(const OperatorDesc &op) const {
        return static_cast<const Options *>(op.option.get());
    }

    // extra_in / extra_out: tensors of an Add taken into this convolution's launch; they ride at the end of the
    // operator's tensor lists so that whoever walks the list (the executor's signature, a dump) sees them
    EnnReturn create_conv(const OperatorDesc &op, const UDTensors &extra_in = UDTensors(), const UDTensors &extra_out = UDTensors()) {
        if (op.out_tensors.empty() || op.in_tensors.size() < 3 || !op.option) return ENN_RET_FAILED;
        const PrecisionType precision = get_precision(op.out_tensors[0]->data_type);
        UDTensors in, out;
        if (!convert_to_tensors(op, precision, in, out)) return ENN_RET_FAILED;
        in.insert(in.end(), extra_in.begin(), extra_in.end());
        out.insert(out.end(), extra_out.begin(), extra_out.end());
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
        return finish(op, compute_library_->createConvolution(precision), in, out, p);
    }

    // `add` consumes `conv`'s only output, nothing else does, all four tensors are uint8, and the sum is not
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
        const bool conv_first = add.in_tensors[0]->buffer_index == conv.out_tensors[0]->buffer_index;
        if (create_conv(conv, {add_in[conv_first ? 1 : 0]}, {add_out[0]}) != ENN_RET_SUCCESS) return ENN_RET_FAILED;
        auto wrapper = std::dynamic_pointer_cast<EnnUDOperator<HipConvolution>>(operators->back());
        if (!wrapper) return ENN_RET_FAILED;
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
        return finish(op, compute_library_->createDepthwiseConvolution(precision), in, out, depthwise_parameters(op, in, out));
    }

    std::shared_ptr<DepthwiseConvolutionParameters> depthwise_parameters(const OperatorDesc &op, const UDTensors &in, const UDTensors &out) const {
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
        return p;
    }

    // `conv` is a channels-last uint8 1x1 convolution (stride 1, constant per-tensor quantized parameters) whose
    // output only `dw` reads, `dw` a 3x3 depthwise convolution of the same kind without dilation or depth multiplier,
    // and the library lists the shape among those where one launch beats two.
    bool fusable_expansion(const OperatorDesc &conv, const OperatorDesc &dw) const {
        if (conv.code != TFlite::BuiltinOperator_CONV_2D || dw.code != TFlite::BuiltinOperator_DEPTHWISE_CONV_2D) return false;
        if (conv.out_tensors.size() != 1 || conv.in_tensors.size() != 3 || dw.in_tensors.size() != 3 || dw.out_tensors.size() != 1 || !conv.option ||
            !dw.option)
            return false;
        const auto &x = conv.in_tensors[0], &e = conv.out_tensors[0], &d = dw.out_tensors[0];
        if (dw.in_tensors[0]->is_const || dw.in_tensors[0]->buffer_index != e->buffer_index) return false;
        const auto readers = tensors_used_.find(e->buffer_index);
        if (readers == tensors_used_.end() || readers->second != 1) return false;
        // weights quantized per tensor in both operators (uint8), or per channel in both (int8)
        const bool per_channel = !conv.in_tensors[1]->per_channel_scales.empty();
        for (const auto *op : {&conv, &dw}) {
            if (!op->in_tensors[1]->is_const || !op->in_tensors[2]->is_const || op->in_tensors[1]->per_channel_scales.empty() == per_channel) return false;
            if (op->in_tensors[1]->data_type != (per_channel ? TFlite::TensorType_INT8 : TFlite::TensorType_UINT8) ||
                op->in_tensors[2]->data_type != TFlite::TensorType_INT32)
                return false;
        }
        for (const auto &t : {x, e, d})
            if (t->is_const || t->data_type != TFlite::TensorType_UINT8 || t->shape.size() != 4) return false;
        const auto *co = options_of<TFlite::Conv2DOptions>(conv);
        const auto *dwo = options_of<TFlite::DepthwiseConv2DOptions>(dw);
        bool android = false, nchw = true, dw_nchw = true;
        layout_of(*co, &android, &nchw);
        layout_of(*dwo, &android, &dw_nchw);
        // channels-last data: the list's own, or a planar list whose feature maps are stored that way
        if (nchw != dw_nchw || (nchw && !channels_last_)) return false;
        // shapes read (n, c, h, w) in a planar list, (n, h, w, c) otherwise; filters (out, kh, kw, in) / (1, kh, kw, c) in
        // androidNN models, (out, in, kh, kw) / (c, 1, kh, kw) otherwise
        const int hi = nchw ? 2 : 1, wi = nchw ? 3 : 2, ci = nchw ? 1 : 3, ki = android ? 1 : 2;
        const auto &cw = conv.in_tensors[1]->shape, &dww = dw.in_tensors[1]->shape;
        if (cw.size() != 4 || cw[ki] != 1 || cw[ki + 1] != 1 || co->stride_h != 1 || co->stride_w != 1 || co->dilation_h_factor != 1 ||
            co->dilation_w_factor != 1)
            return false;
        if (dww.size() != 4 || dww[ki] != 3 || dww[ki + 1] != 3 || dwo->stride_h != dwo->stride_w || dwo->dilation_h_factor != 1 ||
            dwo->dilation_w_factor != 1 || dwo->depth_multiplier != 1)
            return false;
        if (x->shape[hi] != e->shape[hi] || x->shape[wi] != e->shape[wi] || x->shape[0] != e->shape[0]) return false;
        return fuse_unlisted_expansions ||
               eh_conv_dw_block_listed((int32_t)(e->shape[0] / (uint32_t)lanes_), (int32_t)e->shape[hi], (int32_t)e->shape[wi], (int32_t)x->shape[ci],
                                       (int32_t)e->shape[ci], dwo->stride_h) != 0;
    }

    // The depthwise convolution's tensors are made first: its output then cannot be given the storage of the feature
    // map the fused launch still reads (the pointwise convolution's input may see its last reader here).  The
    // expanded tensor between the two operators gets a shape and quantization parameters but no storage.  Should the
    // plans not fit the fused kernel after all, the expanded tensor gets a buffer of its own and the depthwise
    // convolution becomes an operator of the list as usual.
    EnnReturn create_conv_with_depthwise(const OperatorDesc &conv, const OperatorDesc &dw) {
        const PrecisionType precision = get_precision(dw.out_tensors[0]->data_type);
        const auto &edge = conv.out_tensors[0];
        NDims dims = edge->shape;
        dims[0] /= (uint32_t)lanes_;
        auto expanded = std::make_shared<HipTensor>(HipTensor::NoStorage{}, compute_library_->runtime(), precision,
                                                    compute_library_->tensor_type_2_data_type(edge->data_type), dims, DataOrder::NCHW, edge->scale,
                                                    edge->zero_point, static_cast<uint32_t>(edge->data_type), edge->buffer_index);
        expanded->storeChannelsLast(channels_last_);  // (a fused pair's tensors have more than one pixel per image)
        alloc_tensors_map_[operator_list_id_][lane_key(edge->buffer_index)] = expanded;
        UDTensors dw_in, dw_out;
        if (!convert_to_tensors(dw, precision, dw_in, dw_out)) return ENN_RET_FAILED;
        auto depthwise = compute_library_->createDepthwiseConvolution(precision);
        if (depthwise == nullptr || depthwise->initialize(dw_in, dw_out, depthwise_parameters(dw, dw_in, dw_out)) != Status::SUCCESS) return ENN_RET_FAILED;
        if (create_conv(conv, {dw_in[1], dw_in[2]}, {dw_out[0]}) != ENN_RET_SUCCESS) return ENN_RET_FAILED;
        auto wrapper = std::dynamic_pointer_cast<EnnUDOperator<HipConvolution>>(operators->back());
        if (!wrapper) return ENN_RET_FAILED;
        if (wrapper->getOp()->fuseDepthwise(depthwise) == Status::SUCCESS) return ENN_RET_SUCCESS;
        if (expanded->reconfigureDimsAndBuffer(dims) != Status::SUCCESS) return ENN_RET_FAILED;
        operators->push_back(std::make_shared<EnnUDOperator<HipDepthwiseConvolution>>(dw.name, dw.id, dw_in, dw_out, UDTensors(), depthwise));
        return ENN_RET_SUCCESS;
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
        return finish(op, compute_library_->createDeconvolution(precision), in, out, p);
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
        return finish(op, compute_library_->createFullyConnected(precision), in, out, p);
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
        return finish(op, compute_library_->createAveragepool(precision), in, out, p);
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
        return finish(op, compute_library_->createAdd(precision), in, out, p);
    }

    std::shared_ptr<HipComputeLibrary> compute_library_;
    std::mutex mutex_constructor_;
    uint64_t operator_list_id_ = 0;
    TFlite::LegacyModel legacy_model_ = TFlite::LegacyModel_TENSORFLOW_NHWC;
    std::map<uint64_t, std::map<int32_t, std::shared_ptr<ITensor>>> alloc_tensors_map_;  // feature maps by list id and buffer index
    std::map<int32_t, int32_t> tensors_used_;                    // readers still to be built, by buffer index
    std::map<int32_t, bool> produced_, consumed_;
    std::map<const TensorDesc *, std::shared_ptr<ITensor>> const_tensors_;  // parameters of the list being built, shared by its lanes
    int lanes_ = 1, lane_ = 0;
    bool channels_last_ = false;  // the list being opened stores its feature maps channels-last
    std::vector<std::shared_ptr<UDOperator>> pending_layout_ops_;
};

// Runs a built list: every operator in order on the compute library's stream (gpu_op_executor.cc:56-103).  Moving host
// bytes into the list's inputs and out of its outputs is the userdriver's part (gpu_userdriver.cc:97-103).
//
// Record and replay.  A list is recorded when all of its operators are replayable() (they only enqueue kernels whose
// arguments follow from their tensors).  What was recorded stays valid while every tensor of every operator keeps
// its device address, scale and zero point: the executor keeps that signature per list, and an execution whose
// signature differs runs operator by operator (which also lets the operators re-fold biases or send new per-channel
// pairs, things that cannot be recorded), records at the next execution with that same signature, and replays after
// that.  The recorded graph holds kernel launches and device-to-device copies only; buffers are cleared by fill
// kernels, never by memset nodes.
class OperationExecutor {
public:
    explicit OperationExecutor(std::shared_ptr<HipComputeLibrary> compute_library) : compute_library_(compute_library) {}
    ~OperationExecutor() {
        for (auto &kv : recorded_) drop_graphs(kv.second);
    }
    OperationExecutor(const OperationExecutor &) = delete;
    OperationExecutor &operator=(const OperationExecutor &) = delete;

    struct Counters {
        uint64_t direct = 0;     // executions that ran operator by operator
        uint64_t recordings = 0;
        uint64_t replays = 0;
    };

    EnnReturn execute(UDOperators &operators, UDBuffers &buffers, const BufferTable &buffer_table) {
        return execute_times(operators, buffers, buffer_table, 1);
    }

    // `times` executions in a row on the tensors as they stand.  A recorded list asked for kBurst or more executions
    // replays a second graph that holds kBurst of them back to back (made the first time it is needed): one graph
    // launch, whose host-side cost grows with the number of kernel nodes, then covers kBurst executions, which matters
    // once an execution is as short as the launch call (MobileNetV2 at 64 images: 432 -> 417 us per execution).
    EnnReturn execute_times(UDOperators &operators, UDBuffers &buffers, const BufferTable &buffer_table, int times) {
        (void)buffers;
        (void)buffer_table;
        if (!operators || times < 1) return ENN_RET_FAILED;
        for (int done = 0; done < times;) {
            const int ran = execute_some(operators, times - done);
            if (ran < 1) return ENN_RET_FAILED;
            done += ran;
        }
        return ENN_RET_SUCCESS;
    }

    static constexpr int kBurst = 4;

    // Forgets what was recorded for a list (the userdriver calls this when the list is closed, before its operators go).
    void forget(const UDOperators &operators) {
        auto it = recorded_.find(operators.get());
        if (it == recorded_.end()) return;
        if (it->second.graph || it->second.burst) {
            compute_library_->synchronize();
            drop_graphs(it->second);
        }
        recorded_.erase(it);
    }

    const Counters &counters() const { return counters_; }
    bool replay = true;  // false: every execution runs operator by operator, as the reference's does

private:
    enum class State { WARM, RECORDED, DIRECT_ONLY };
    struct Recorded {
        std::vector<uint64_t> signature;
        void *graph = nullptr;
        void *burst = nullptr;  // kBurst executions in one graph
        State state = State::WARM;
    };

    static void drop_graphs(Recorded &r) {
        if (r.graph) eh_graph_destroy(r.graph);
        if (r.burst) eh_graph_destroy(r.burst);
        r.graph = r.burst = nullptr;
    }

    // captures `executions` runs of the list into a graph; null when that fails (the capture is always ended)
    void *record(UDOperators &operators, int executions) {
        void *stream = compute_library_->runtime()->mainStream();
        if (stream == nullptr || eh_graph_begin(stream) != EH_OK) return nullptr;
        EnnReturn ran = ENN_RET_SUCCESS;
        for (int i = 0; i < executions && ran == ENN_RET_SUCCESS; ++i) ran = run_in_order(operators, false);
        void *graph = nullptr;
        const int ended = eh_graph_end(stream, &graph);
        if (ran != ENN_RET_SUCCESS || ended != EH_OK || graph == nullptr) {
            if (graph) eh_graph_destroy(graph);
            return nullptr;
        }
        return graph;
    }

    // one execution, or one burst when `wanted` allows; returns the executions done, 0 on failure
    int execute_some(UDOperators &operators, int wanted) {
        if (!replay) return run_in_order(operators) == ENN_RET_SUCCESS ? 1 : 0;
        Recorded &r = recorded_[operators.get()];
        std::vector<uint64_t> &now = scratch_signature_;
        const bool can_record = signature(operators, &now);
        if (!can_record || now != r.signature || r.state == State::DIRECT_ONLY) {
            const bool changed = now != r.signature;
            if ((r.graph || r.burst) && changed) {
                // what was recorded is stale; the operators are about to rewrite the arrays it reads
                compute_library_->synchronize();
                drop_graphs(r);
            }
            if (changed) r.state = can_record ? State::WARM : State::DIRECT_ONLY;
            r.signature = now;
            return run_in_order(operators) == ENN_RET_SUCCESS ? 1 : 0;
        }
        if (r.state == State::WARM) {  // second execution with this signature: record it
            r.graph = record(operators, 1);
            if (r.graph == nullptr) {
                ERROR_PRINT("OperationExecutor: the list could not be recorded (%s); it runs operator by operator\n", eh_last_error());
                r.state = State::DIRECT_ONLY;
                return run_in_order(operators) == ENN_RET_SUCCESS ? 1 : 0;
            }
            r.state = State::RECORDED;
            ++counters_.recordings;
        }
        void *graph = r.graph;
        int executions = 1;
        if (wanted >= kBurst) {
            if (r.burst == nullptr) r.burst = record(operators, kBurst);  // (if that fails the single graph still serves)
            if (r.burst != nullptr) {
                graph = r.burst;
                executions = kBurst;
            }
        }
        if (eh_graph_launch(graph, compute_library_->runtime()->mainStream()) != EH_OK) {
            ERROR_PRINT("OperationExecutor: replay failed: %s\n", eh_last_error());
            return 0;
        }
        counters_.replays += (uint64_t)executions;
        return executions;
    }

    // Every operator in list order on the compute library's stream; the operators of lanes beyond the first on their
    // lane's stream, forked from the main stream before the first of them and joined to it after the last (under
    // capture the lanes become parallel branches of the graph).  A lane's operators are enqueued in one go.
    EnnReturn run_in_order(UDOperators &operators, bool count = true) {
        if (count) ++counters_.direct;
        int lanes = 1;
        for (auto &op : *operators) lanes = std::max(lanes, op->lane() + 1);
        const auto runtime = compute_library_->runtime();
        void *main_stream = runtime->mainStream();
        if (lanes > 1) {
            void *fork = runtime->event(0);
            if (fork == nullptr || eh_event_record(fork, main_stream) != EH_OK) return ENN_RET_FAILED;
            for (int lane = 1; lane < lanes; ++lane)
                if (runtime->laneStream((size_t)lane - 1) == nullptr || eh_stream_wait_event(runtime->laneStream((size_t)lane - 1), fork) != EH_OK)
                    return ENN_RET_FAILED;
        }
        EnnReturn result = ENN_RET_SUCCESS;
        for (int lane = 0; lane < lanes && result == ENN_RET_SUCCESS; ++lane) {
            runtime->launchOn(lane == 0 ? nullptr : runtime->laneStream((size_t)lane - 1));
            for (auto &op : *operators)
                if (op->lane() == lane && op->execute(nullptr) != ENN_RET_SUCCESS) {
                    ERROR_PRINT("OperationExecutor: %s failed\n", op->getName().c_str());
                    result = ENN_RET_FAILED;
                    break;
                }
        }
        runtime->launchOn(nullptr);
        // the lanes are joined also after a failure: a capture must not end with a lane's stream still forked
        for (int lane = 1; lane < lanes; ++lane) {
            void *join = runtime->event((size_t)lane);
            if (join == nullptr || eh_event_record(join, runtime->laneStream((size_t)lane - 1)) != EH_OK || eh_stream_wait_event(main_stream, join) != EH_OK)
                result = ENN_RET_FAILED;
        }
        return result;
    }

    // device address, scale and zero point of every tensor of every operator; false when an operator cannot be recorded
    static bool signature(const UDOperators &operators, std::vector<uint64_t> *out) {
        bool all = true;
        out->clear();
        out->reserve(operators->size() * 12);
        auto add = [&](const std::shared_ptr<ITensor> &t) {
            if (!t) return;
            const float scale = t->getScale();
            uint32_t bits;
            std::memcpy(&bits, &scale, sizeof bits);
            out->push_back(reinterpret_cast<uint64_t>(static_cast<HipTensor *>(t.get())->getDataPtr()));
            out->push_back(((uint64_t)bits << 32) | (uint32_t)t->getZeroPoint());
        };
        for (auto &op : *operators) {
            all = all && op->replayable();
            for (const auto &t : op->inTensors()) add(t);
            for (const auto &t : op->outTensors()) add(t);
            out->push_back(0xED0ull);  // operator boundary
        }
        return all;
    }

    std::shared_ptr<HipComputeLibrary> compute_library_;
    std::map<const void *, Recorded> recorded_;
    std::vector<uint64_t> scratch_signature_;
    Counters counters_;
};

}  // namespace hip
}  // namespace ud
}  // namespace enn
