// Operator classes of the HIP userdriver backend for the quantized path:
// Convolution, DepthwiseConvolution, FullyConnected, Deconvolution on uint8 tensors.
//
// Each class keeps the reference operator surface: constructed from
// (runtime, precision); initialize({input, weight, bias}, {output}, parameters);
// execute(); release(); every call returns Status and logs instead of throwing.
// Reference counterparts: CLConvolution (src/userdriver/gpu/operators/CLConvolution.hpp:31-66,
// CLConvolution.cpp:34-550), CLDepthwiseConvolution (CLDepthwiseConvolution.hpp:18-38,
// .cpp:88-425), CLFullyConnected (CLFullyConnected.hpp:21-35, .cpp:22-150),
// CLDeconvolution (CLDeconvolution.hpp:20-40, .cpp:36-272); and the two operators a residual
// network needs between them: CLAdd on its quantized path (CLAdd.hpp:21-66,
// cl_optimized_impls/CLAddQuantized.cpp:67-166) and CLAveragepool (CLAveragepool.hpp:15-60,
// CLAveragepool.cpp:175-230, parameters gpu/common/CLParameter.hpp:25-34).
//
// Behaviour kept from the reference: quantization parameters are read from the
// tensors on every execute(); constant weights are packed once in initialize(),
// weights that are run-time inputs (is_const() == false) are re-packed on every
// execute(); a bias scale that does not match input_scale * filter_scale leaves
// the multiplier at zero (every output is the clamped output zero point); an
// empty weight or input tensor makes initialize()/execute() succeed without work;
// in channels-last mode (isNCHW == false) a tensor's Dim4 holds (n, h, w, c)
// positionally; in androidNN mode the weight Dim4 holds (out, kh, kw, in).
// Per-channel quantized weights (per_channel_quant + scales) and INT8 precision are
// offered as the reference offers them; float precisions and texture storage are not
// (initialize() returns FAILURE for them).
#pragma once

#include <memory>
#include <vector>

#include "ActivationInfo.hpp"
#include "HipTensor.hpp"

namespace enn {
namespace ud {
namespace hip {

#define INPUT_INDEX 0
#define WEIGHT_INDEX 1
#define BIAS_INDEX 2
#define OUTPUT_INDEX 0

struct Parameters {
    virtual ~Parameters() {}
};

struct ConvolutionParameters : public Parameters {
    Pad4 padding = {0, 0, 0, 0};
    Dim2 dilation = {1, 1};
    Dim2 stride = {1, 1};
    uint32_t group_size = 1;
    uint32_t axis = 0;
    bool per_channel_quant = false;
    bool androidNN = false;
    bool isNCHW = true;
    StorageType storage_type = StorageType::BUFFER;
    bool openAibWino = false;
    std::shared_ptr<ActivationInfo> activation_info = std::make_shared<ActivationInfo>();
    std::vector<float> scales;
};

struct DepthwiseConvolutionParameters : public Parameters {
    Pad4 padding = {0, 0, 0, 0};
    Dim2 dilation = {1, 1};
    Dim2 stride = {1, 1};
    uint32_t depth_multiplier = 1;
    bool per_channel_quant = false;
    bool androidNN = false;
    bool isNCHW = true;
    StorageType storage_type = StorageType::BUFFER;
    std::shared_ptr<ActivationInfo> activation_info = std::make_shared<ActivationInfo>();
    std::vector<float> scales;
};

struct FullyConnectedParameters : public Parameters {
    bool androidNN = false;
    StorageType storage_type = StorageType::BUFFER;
    std::shared_ptr<ActivationInfo> activation_info = std::make_shared<ActivationInfo>();
};

struct DeconvolutionParameters : public Parameters {
    Pad4 padding = {0, 0, 0, 0};
    Dim2 stride = {1, 1};
    uint32_t group_size = 1;
    bool weights_as_input = false;
    bool per_channel_quant = false;
    bool androidNN = false;
    bool isNCHW = true;
    bool openAibWino = false;
    std::shared_ptr<ActivationInfo> activation_info = std::make_shared<ActivationInfo>();
    std::vector<float> scales;
};

// AddParameters (gpu/operators/CLAdd.hpp:21-28) and Pool2DParameters (gpu/common/CLParameter.hpp:25-34):
// the activation is held by value there
struct AddParameters : public Parameters {
    ActivationInfo activation_info = ActivationInfo();
    bool pot_scale_int16 = false;
    std::vector<float> coeff = {};
    bool androidNN = false;
    bool isNCHW = false;
    StorageType storage_type = StorageType::BUFFER;
};

struct Pool2DParameters : public Parameters {
    Pad4 padding = {0, 0, 0, 0};
    Dim2 stride = {1, 1};
    Dim2 filter = {1, 1};
    ActivationInfo activation_info = ActivationInfo();
    bool androidNN = false;
    bool isNCHW = true;
    StorageType storage_type = StorageType::BUFFER;
    ComputeType compute_type = ComputeType::TFLite;
};

namespace detail {

// How the plan of an operator on planar-shaped (n, c, h, w) tensors addresses them: EH_NCHW when both are stored planar,
// EH_NHWC when they are stored channels-last (HipTensor::storedChannelsLast; a tensor of one pixel per image is both at
// once, and so is one of a single channel), -1 when the two disagree.
inline int planarOperatorLayout(const std::shared_ptr<HipTensor> &a, const std::shared_ptr<HipTensor> &b) {
    const bool al = a->storedChannelsLast(), bl = b->storedChannelsLast();
    if (!al && !bl) return EH_NCHW;
    const Dim4 ad = a->getDim(), bd = b->getDim();
    const bool a_flat = (uint64_t)ad.h * ad.w <= 1 || ad.c <= 1, b_flat = (uint64_t)bd.h * bd.w <= 1 || bd.c <= 1;
    return (al || a_flat) && (bl || b_flat) ? EH_NHWC : -1;
}

inline int toEhActivation(const ActivationInfo &a) {
    switch (a.activation()) {
        case ActivationInfo::ActivationType::RELU: return EH_ACT_RELU;
        case ActivationInfo::ActivationType::RELU1: return EH_ACT_RELU1;
        case ActivationInfo::ActivationType::RELU6: return EH_ACT_RELU6;
        default: return EH_ACT_NONE;
    }
}

// What the reference's quantized operators compute at the top of execute()
// (cl_optimized_impls/CLGEMMConvolutionQuantized.cpp:137-171).
inline eh_requant requantFromTensors(const std::shared_ptr<HipTensor> &in, const std::shared_ptr<HipTensor> &w,
                                     const std::shared_ptr<HipTensor> &bias, const std::shared_ptr<HipTensor> &out,
                                     const ActivationInfo &act) {
    eh_requant q;
    eh_make_requant(in->getScale(), in->getZeroPoint(), w->getScale(), w->getZeroPoint(), bias->getScale(), out->getScale(),
                    out->getZeroPoint(), toEhActivation(act), act.isEnabled() ? 1 : 0, &q);
    return q;
}

// PrecisionType::INT8: every tensor holds int8 bytes and the parameters are int8 values (the SIGNED* kernels,
// cl_optimized_impls/CLGEMMConvolutionQuantized.cpp:47,224-241)
inline eh_requant requantFromTensors(const PrecisionType &precision, const std::shared_ptr<HipTensor> &in,
                                     const std::shared_ptr<HipTensor> &w, const std::shared_ptr<HipTensor> &bias,
                                     const std::shared_ptr<HipTensor> &out, const ActivationInfo &act) {
    if (precision != PrecisionType::INT8) return requantFromTensors(in, w, bias, out, act);
    eh_requant q;
    eh_make_requant_s8(in->getScale(), in->getZeroPoint(), w->getScale(), w->getZeroPoint(), bias->getScale(), out->getScale(),
                       out->getZeroPoint(), toEhActivation(act), act.isEnabled() ? 1 : 0, &q);
    return q;
}

inline bool quantizedPrecision(const PrecisionType &p) { return p == PrecisionType::UINT8 || p == PrecisionType::INT8; }

// data types of {input, weight, bias, output} for a precision: uint8 everywhere (int8 weights in per-channel
// mode), or int8 everywhere
inline bool tensorTypesMatch(const PrecisionType &precision, bool per_channel, const std::shared_ptr<HipTensor> &in,
                             const std::shared_ptr<HipTensor> &w, const std::shared_ptr<HipTensor> &bias,
                             const std::shared_ptr<HipTensor> &out) {
    const DataType io = precision == PrecisionType::INT8 ? DataType::INT8 : DataType::UINT8;
    const DataType wt = (precision == PrecisionType::INT8 || per_channel) ? DataType::INT8 : DataType::UINT8;
    return in->getDataType() == io && w->getDataType() == wt && bias->getDataType() == DataType::INT32 && out->getDataType() == io;
}

// Per-channel mode: int8 weights and one filter scale per output channel
// (cl_optimized_impls/CLConvolutionPerChannelQuantized.cpp:96-120,
// CLDepthwiseConvolutionPerChannelQuantized.cpp:133-160, CLDeconvolutionPerChannelQuantized.cpp:147-179).
// The pairs are derived from the tensors' scales at every execute(), as there; the plan is only told when they change.
struct PerChannelState {
    std::vector<int32_t> multipliers, shifts;  // what the plan holds
    bool sent = false;

    // weight_zp: the convolution ignores the filter's zero point, the depthwise convolution and the
    // deconvolution subtract it.  range_always: the deconvolution derives the activation range even
    // for a disabled activation.
    eh_requant derive(const PrecisionType &precision, const std::shared_ptr<HipTensor> &in, const std::shared_ptr<HipTensor> &out,
                      const ActivationInfo &act, const std::vector<float> &scales, int32_t weight_zp, bool range_always,
                      std::vector<int32_t> *m, std::vector<int32_t> *s) const {
        eh_requant q;
        m->assign(scales.size(), 0);
        s->assign(scales.size(), 0);
        eh_make_requant_perchannel(in->getScale(), in->getZeroPoint(), scales.data(), (int32_t)scales.size(), out->getScale(),
                                   out->getZeroPoint(), toEhActivation(act), (range_always || act.isEnabled()) ? 1 : 0, &q, m->data(),
                                   s->data());
        q.zp_w = weight_zp;
        if (precision == PrecisionType::INT8) {
            q.act_min = -128;
            q.act_max = 127;
            if (range_always || act.isEnabled()) eh_act_range_s8(toEhActivation(act), out->getScale(), out->getZeroPoint(), &q.act_min, &q.act_max);
        }
        return q;
    }
};

}  // namespace detail

class HipDepthwiseConvolution;

class HipConvolution {
public:
    HipConvolution(const std::shared_ptr<HipRuntime> runtime, const PrecisionType &precision)
        : runtime_(runtime), precision_(precision) {}
    ~HipConvolution() { release(); }

    Status initialize(std::vector<std::shared_ptr<ITensor>> inputs, std::vector<std::shared_ptr<ITensor>> outputs,
                      std::shared_ptr<Parameters> parameters) {
        CHECK_EXPR_RETURN_FAILURE(inputs.size() >= 3 && outputs.size() >= 1, "HipConvolution: needs {input, weight, bias} and {output}");
        input_ = std::static_pointer_cast<HipTensor>(inputs.at(INPUT_INDEX));
        weight_ = std::static_pointer_cast<HipTensor>(inputs.at(WEIGHT_INDEX));
        bias_ = std::static_pointer_cast<HipTensor>(inputs.at(BIAS_INDEX));
        output_ = std::static_pointer_cast<HipTensor>(outputs.at(OUTPUT_INDEX));
        parameters_ = std::dynamic_pointer_cast<ConvolutionParameters>(parameters);
        CHECK_EXPR_RETURN_FAILURE(parameters_ != nullptr, "HipConvolution: parameters are not ConvolutionParameters");
        CHECK_EXPR_RETURN_FAILURE(parameters_->activation_info != nullptr, "HipConvolution: null activation info");
        activation_info_ = *parameters_->activation_info;
        weights_as_input_ = !weight_->is_const();
        bias_as_input_ = !bias_->is_const();

        if (weight_->getTotalSizeFromDims() == 0) return Status::SUCCESS;  // zero-sized: nothing to prepare
        CHECK_EXPR_RETURN_FAILURE(detail::quantizedPrecision(precision_), "HipConvolution: only the UINT8 and INT8 paths exist on this backend");
        CHECK_EXPR_RETURN_FAILURE(parameters_->storage_type == StorageType::BUFFER, "HipConvolution: no texture storage");
        per_channel_ = parameters_->per_channel_quant;
        CHECK_EXPR_RETURN_FAILURE(detail::tensorTypesMatch(precision_, per_channel_, input_, weight_, bias_, output_),
                                  "HipConvolution: tensor data types do not fit the precision (uint8 tensors, int8 weights in per-channel mode; int8 tensors for INT8)");

        Dim4 in = input_->getDim(), wd = weight_->getDim();
        if (!parameters_->isNCHW) in = convertDimToNCHW(in);
        const bool ohwi = parameters_->androidNN || !parameters_->isNCHW;  // weight Dim4 = (out, kh, kw, in)
        const uint32_t cout = wd.n, kh = ohwi ? wd.c : wd.h, kw = ohwi ? wd.h : wd.w, cin_g = ohwi ? wd.w : wd.c;
        CHECK_EXPR_RETURN_FAILURE(cin_g != 0 && in.c % cin_g == 0, "HipConvolution: weight channels %u do not divide input channels %u", cin_g, in.c);
        const uint32_t groups = ohwi ? in.c / cin_g : parameters_->group_size;
        CHECK_EXPR_RETURN_FAILURE(groups != 0 && in.c == cin_g * groups, "HipConvolution: group size %u does not match the weight shape", groups);

        eh_conv_desc d;
        d.n = (int32_t)in.n;
        d.c = (int32_t)in.c;
        d.h = (int32_t)in.h;
        d.w = (int32_t)in.w;
        d.cout = (int32_t)cout;
        d.kh = (int32_t)kh;
        d.kw = (int32_t)kw;
        d.stride_h = (int32_t)parameters_->stride.h;
        d.stride_w = (int32_t)parameters_->stride.w;
        d.pad_t = (int32_t)parameters_->padding.t;
        d.pad_b = (int32_t)parameters_->padding.b;
        d.pad_l = (int32_t)parameters_->padding.l;
        d.pad_r = (int32_t)parameters_->padding.r;
        d.dil_h = (int32_t)parameters_->dilation.h;
        d.dil_w = (int32_t)parameters_->dilation.w;
        d.groups = (int32_t)groups;
        d.depth_multiplier = 1;
        d.layout = parameters_->isNCHW ? detail::planarOperatorLayout(input_, output_) : EH_NHWC;
        CHECK_EXPR_RETURN_FAILURE(d.layout >= 0, "HipConvolution: input and output are stored in different element orders");
        d.weight_layout = ohwi ? EH_W_OHWI : EH_W_OIHW;
        desc_ = d;
        const int32_t ho = eh_conv_out_dim(d.h, d.pad_t, d.pad_b, d.kh, d.dil_h, d.stride_h);
        const int32_t wo = eh_conv_out_dim(d.w, d.pad_l, d.pad_r, d.kw, d.dil_w, d.stride_w);
        CHECK_EXPR_RETURN_FAILURE((int64_t)output_->getTotalSizeFromDims() == (int64_t)d.n * d.cout * ho * wo,
                                  "HipConvolution: output tensor has %u elements, the geometry gives %lld", output_->getTotalSizeFromDims(),
                                  (long long)d.n * d.cout * ho * wo);
        if (per_channel_) {
            CHECK_EXPR_RETURN_FAILURE(parameters_->scales.size() == (size_t)desc_.cout, "HipConvolution: %zu filter scales for %d output channels", parameters_->scales.size(), desc_.cout);
            desc_.weight_layout |= EH_W_SIGNED;
        }
        if (precision_ == PrecisionType::INT8) {
            desc_.weight_layout |= EH_W_SIGNED;
            desc_.layout |= EH_IO_SIGNED;
        }
        // Weights or bias that are run-time feature maps of an operator list have no device memory until the list's
        // pooled buffers are assigned: the plan is then made by the first execute(), which is where the reference packs
        // such weights anyway.
        if ((weights_as_input_ || bias_as_input_) && (weight_->getDataPtr() == nullptr || bias_->getDataPtr() == nullptr)) {
            deferred_ = true;
            return Status::SUCCESS;
        }
        return makePlan();
    }

    Status makePlan() {
        deferred_ = false;
        eh_requant q;
        CHECK_EXPR_RETURN_FAILURE(currentRequant(&q) == Status::SUCCESS, "HipConvolution::initialize: requantization parameters");
        const int rc = eh_conv2d_u8_plan(&plan_, &desc_, weight_->getDataPtr(), bias_->getDataPtr(), &q, runtime_->stream());
        CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipConvolution::initialize: %s", eh_last_error());
        if (per_channel_) CHECK_EXPR_RETURN_FAILURE(currentRequant(&q) == Status::SUCCESS, "HipConvolution::initialize: per-channel pairs");
        return Status::SUCCESS;
    }

    Status execute() {
        if (plan_ == nullptr && deferred_) CHECK_EXPR_RETURN_FAILURE(makePlan() == Status::SUCCESS, "HipConvolution::execute: the deferred plan could not be made");
        if (plan_ == nullptr) {  // zero-sized operator
            CHECK_EXPR_RETURN_FAILURE(weight_ && weight_->getTotalSizeFromDims() == 0, "HipConvolution::execute before initialize");
            return Status::SUCCESS;
        }
        if (input_->getTotalSizeFromDims() == 0) return Status::SUCCESS;
        eh_requant q;
        CHECK_EXPR_RETURN_FAILURE(currentRequant(&q) == Status::SUCCESS, "HipConvolution::execute: requantization parameters");
        if (weights_as_input_ || bias_as_input_) {
            const int rc = eh_conv2d_u8_repack(plan_, weight_->getDataPtr(), bias_->getDataPtr(), &q, runtime_->stream());
            CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipConvolution::execute (repack): %s", eh_last_error());
        }
        if (depthwise_) return executeWithDepthwise(q);
        if (residual_) {  // output = add(residual, this convolution), as the CLAdd behind it would compute it
            eh_add_requant aq;
            eh_make_add_requant(residual_->getScale(), residual_->getZeroPoint(), output_->getScale(), output_->getZeroPoint(),
                                sum_->getScale(), sum_->getZeroPoint(), detail::toEhActivation(add_activation_),
                                add_activation_.isEnabled() ? 1 : 0, &aq);
            const int rc = eh_conv2d_u8_run_add(plan_, input_->getDataPtr(), residual_->getDataPtr(), sum_->getDataPtr(), &q, &aq,
                                                runtime_->stream());
            CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipConvolution::execute (with residual add): %s", eh_last_error());
            return Status::SUCCESS;
        }
        const int rc = eh_conv2d_u8_run(plan_, input_->getDataPtr(), output_->getDataPtr(), &q, runtime_->stream());
        CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipConvolution::execute: %s", eh_last_error());
        return Status::SUCCESS;
    }

    // execute() only enqueues kernels unless the weights or bias are run-time inputs (they are then re-packed, which
    // may read device memory back to choose a kernel form)
    bool launchesOnly() const { return !weights_as_input_ && !bias_as_input_; }

    // From now on execute() stores add(residual, convolution) in `sum` and leaves this operator's own output tensor
    // unwritten: the quantized CLAdd that follows this convolution in an operator list, taken into its launch
    // (gpu/operators/CLAdd.cpp:159-163; the sum of the two rescaled operands does not depend on their order).  The
    // output tensor still supplies the scale and zero point the convolution requantizes to.  UINT8 tensors (per-tensor
    // or per-channel weights).
    Status fuseResidualAdd(std::shared_ptr<ITensor> residual, std::shared_ptr<ITensor> sum, const ActivationInfo &add_activation) {
        CHECK_EXPR_RETURN_FAILURE(plan_ != nullptr || deferred_, "HipConvolution::fuseResidualAdd before initialize");
        CHECK_EXPR_RETURN_FAILURE(precision_ == PrecisionType::UINT8, "HipConvolution::fuseResidualAdd: UINT8 tensors only");
        auto r = std::static_pointer_cast<HipTensor>(residual), t = std::static_pointer_cast<HipTensor>(sum);
        CHECK_EXPR_RETURN_FAILURE(r && t && r->getDataType() == DataType::UINT8 && t->getDataType() == DataType::UINT8,
                                  "HipConvolution::fuseResidualAdd: expects uint8 tensors");
        CHECK_EXPR_RETURN_FAILURE(r->getTotalSizeFromDims() == output_->getTotalSizeFromDims() &&
                                      t->getTotalSizeFromDims() == output_->getTotalSizeFromDims() && r != t,
                                  "HipConvolution::fuseResidualAdd: shapes differ");
        residual_ = r;
        sum_ = t;
        add_activation_ = add_activation;
        return Status::SUCCESS;
    }

    // From now on execute() runs this (pointwise) convolution and the depthwise convolution that reads its output as
    // one launch (eh_conv_dw_block_run): the convolution's own output tensor is never written and needs no storage, it
    // still supplies the scale and zero point between the two; the depthwise operator is not executed by anyone else.
    // The reference runs CLConvolution and CLDepthwiseConvolution one after the other (gpu/gpu_op_executor.cc:56-103).
    // FAILURE when the pair does not fit the fused kernel; nothing is changed then.
    Status fuseDepthwise(const std::shared_ptr<HipDepthwiseConvolution> &depthwise);
    bool hasFusedDepthwise() const { return depthwise_ != nullptr; }

    Status release() {
        if (plan_) {
            (void)runtime_->synchronize();
            eh_conv2d_u8_destroy(plan_);
            plan_ = nullptr;
        }
        return Status::SUCCESS;
    }

private:
    Status executeWithDepthwise(const eh_requant &q);

    // The requantization parameters of this execution, read from the tensors now; in per-channel mode
    // also hands the plan the channel pairs when they differ from the ones it holds.
    Status currentRequant(eh_requant *q) {
        if (!per_channel_) {
            *q = detail::requantFromTensors(precision_, input_, weight_, bias_, output_, activation_info_);
            return Status::SUCCESS;
        }
        std::vector<int32_t> m, s;
        *q = pc_.derive(precision_, input_, output_, activation_info_, parameters_->scales, 0, false, &m, &s);
        if (plan_ != nullptr && (!pc_.sent || m != pc_.multipliers || s != pc_.shifts)) {
            const int rc = eh_conv2d_u8_set_perchannel(plan_, m.data(), s.data(), (int32_t)m.size(), runtime_->stream());
            CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipConvolution: %s", eh_last_error());
            pc_.multipliers = m;
            pc_.shifts = s;
            pc_.sent = true;
        }
        return Status::SUCCESS;
    }

    bool per_channel_ = false;
    detail::PerChannelState pc_;
    std::shared_ptr<HipRuntime> runtime_;
    PrecisionType precision_;
    std::shared_ptr<HipTensor> input_, output_, weight_, bias_;
    std::shared_ptr<HipTensor> residual_, sum_;  // set by fuseResidualAdd
    std::shared_ptr<HipDepthwiseConvolution> depthwise_;  // set by fuseDepthwise
    ActivationInfo add_activation_;
    std::shared_ptr<ConvolutionParameters> parameters_;
    ActivationInfo activation_info_;
    bool weights_as_input_ = false, bias_as_input_ = false;
    eh_conv_desc desc_{};
    bool deferred_ = false;
    eh_conv_plan *plan_ = nullptr;
};

class HipDepthwiseConvolution {
public:
    HipDepthwiseConvolution(const std::shared_ptr<HipRuntime> runtime, const PrecisionType &precision)
        : runtime_(runtime), precision_(precision) {}
    ~HipDepthwiseConvolution() { release(); }

    Status initialize(std::vector<std::shared_ptr<ITensor>> inputs, std::vector<std::shared_ptr<ITensor>> outputs,
                      std::shared_ptr<Parameters> parameters) {
        CHECK_EXPR_RETURN_FAILURE(inputs.size() >= 3 && outputs.size() >= 1, "HipDepthwiseConvolution: needs {input, weight, bias} and {output}");
        input_ = std::static_pointer_cast<HipTensor>(inputs.at(INPUT_INDEX));
        weight_ = std::static_pointer_cast<HipTensor>(inputs.at(WEIGHT_INDEX));
        bias_ = std::static_pointer_cast<HipTensor>(inputs.at(BIAS_INDEX));
        output_ = std::static_pointer_cast<HipTensor>(outputs.at(OUTPUT_INDEX));
        parameters_ = std::dynamic_pointer_cast<DepthwiseConvolutionParameters>(parameters);
        CHECK_EXPR_RETURN_FAILURE(parameters_ != nullptr, "HipDepthwiseConvolution: parameters are not DepthwiseConvolutionParameters");
        CHECK_EXPR_RETURN_FAILURE(parameters_->activation_info != nullptr, "HipDepthwiseConvolution: null activation info");
        activation_info_ = *parameters_->activation_info;
        weights_as_input_ = !weight_->is_const() || !bias_->is_const();

        if (weight_->getTotalSizeFromDims() == 0) return Status::SUCCESS;
        CHECK_EXPR_RETURN_FAILURE(detail::quantizedPrecision(precision_), "HipDepthwiseConvolution: only the UINT8 and INT8 paths exist on this backend");
        CHECK_EXPR_RETURN_FAILURE(parameters_->storage_type == StorageType::BUFFER, "HipDepthwiseConvolution: no texture storage");
        per_channel_ = parameters_->per_channel_quant;
        CHECK_EXPR_RETURN_FAILURE(detail::tensorTypesMatch(precision_, per_channel_, input_, weight_, bias_, output_),
                                  "HipDepthwiseConvolution: tensor data types do not fit the precision (uint8 tensors, int8 weights in per-channel mode; int8 tensors for INT8)");

        Dim4 in = input_->getDim();
        if (!parameters_->isNCHW) in = convertDimToNCHW(in);
        // [C * depth_multiplier][1][kh][kw]; androidNN models hold [1][kh][kw][C * depth_multiplier]
        // (gpu/operators/CLDepthwiseConvolution.cpp:128-131,146)
        Dim4 wd = weight_->getDim();
        const bool hwo = parameters_->androidNN;
        if (hwo) wd = Dim4{wd.w, wd.n, wd.c, wd.h};
        eh_conv_desc d;
        d.n = (int32_t)in.n;
        d.c = (int32_t)in.c;
        d.h = (int32_t)in.h;
        d.w = (int32_t)in.w;
        d.cout = (int32_t)(in.c * parameters_->depth_multiplier);
        d.kh = (int32_t)wd.h;
        d.kw = (int32_t)wd.w;
        d.stride_h = (int32_t)parameters_->stride.h;
        d.stride_w = (int32_t)parameters_->stride.w;
        d.pad_t = (int32_t)parameters_->padding.t;
        d.pad_b = (int32_t)parameters_->padding.b;
        d.pad_l = (int32_t)parameters_->padding.l;
        d.pad_r = (int32_t)parameters_->padding.r;
        d.dil_h = (int32_t)parameters_->dilation.h;
        d.dil_w = (int32_t)parameters_->dilation.w;
        d.groups = 1;
        d.depth_multiplier = (int32_t)parameters_->depth_multiplier;
        d.layout = parameters_->isNCHW ? detail::planarOperatorLayout(input_, output_) : EH_NHWC;
        CHECK_EXPR_RETURN_FAILURE(d.layout >= 0, "HipDepthwiseConvolution: input and output are stored in different element orders");
        d.weight_layout = hwo ? EH_W_OHWI : EH_W_OIHW;
        CHECK_EXPR_RETURN_FAILURE(wd.n == (uint32_t)d.cout && wd.c == 1, "HipDepthwiseConvolution: weight shape [%u %u %u %u] is not [C*dm][1][kh][kw]", wd.n, wd.c, wd.h, wd.w);
        desc_ = d;
        if (per_channel_) {
            CHECK_EXPR_RETURN_FAILURE(parameters_->scales.size() == (size_t)desc_.cout, "HipDepthwiseConvolution: %zu filter scales for %d output channels", parameters_->scales.size(), desc_.cout);
            desc_.weight_layout |= EH_W_SIGNED;
        }
        if (precision_ == PrecisionType::INT8) {
            desc_.weight_layout |= EH_W_SIGNED;
            desc_.layout |= EH_IO_SIGNED;
        }
        // Weights or bias that are run-time feature maps of an operator list have no device memory until the list's
        // pooled buffers are assigned: the plan is then made by the first execute(), which is where the reference packs
        // such weights anyway.
        if (weights_as_input_ && (weight_->getDataPtr() == nullptr || bias_->getDataPtr() == nullptr)) {
            deferred_ = true;
            return Status::SUCCESS;
        }
        return makePlan();
    }

    Status makePlan() {
        deferred_ = false;
        eh_requant q;
        CHECK_EXPR_RETURN_FAILURE(currentRequant(&q) == Status::SUCCESS, "HipDepthwiseConvolution::initialize: requantization parameters");
        const int rc = eh_dwconv2d_u8_plan(&plan_, &desc_, weight_->getDataPtr(), bias_->getDataPtr(), &q, runtime_->stream());
        CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipDepthwiseConvolution::initialize: %s", eh_last_error());
        if (per_channel_) CHECK_EXPR_RETURN_FAILURE(currentRequant(&q) == Status::SUCCESS, "HipDepthwiseConvolution::initialize: per-channel pairs");
        return Status::SUCCESS;
    }

    Status execute() {
        if (plan_ == nullptr && deferred_) CHECK_EXPR_RETURN_FAILURE(makePlan() == Status::SUCCESS, "HipDepthwiseConvolution::execute: the deferred plan could not be made");
        if (plan_ == nullptr) {  // zero-sized operator
            CHECK_EXPR_RETURN_FAILURE(weight_ && weight_->getTotalSizeFromDims() == 0, "HipDepthwiseConvolution::execute before initialize");
            return Status::SUCCESS;
        }
        if (input_->getTotalSizeFromDims() == 0) return Status::SUCCESS;
        eh_requant q;
        CHECK_EXPR_RETURN_FAILURE(currentRequant(&q) == Status::SUCCESS, "HipDepthwiseConvolution::execute: requantization parameters");
        if (weights_as_input_) {
            const int rc = eh_dwconv2d_u8_repack(plan_, weight_->getDataPtr(), bias_->getDataPtr(), &q, runtime_->stream());
            CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipDepthwiseConvolution::execute (repack): %s", eh_last_error());
        }
        const int rc = eh_dwconv2d_u8_run(plan_, input_->getDataPtr(), output_->getDataPtr(), &q, runtime_->stream());
        CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipDepthwiseConvolution::execute: %s", eh_last_error());
        return Status::SUCCESS;
    }

    bool launchesOnly() const { return !weights_as_input_; }  // a re-pack reads the weights back to choose the dot-product form
    Status release() {
        if (plan_) {
            (void)runtime_->synchronize();
            eh_dwconv2d_u8_destroy(plan_);
            plan_ = nullptr;
        }
        return Status::SUCCESS;
    }

    // for the pointwise convolution that takes this operator into its launch (HipConvolution::fuseDepthwise)
    eh_dwconv_plan *plan() const { return plan_; }
    bool perTensorUint8() const { return !per_channel_ && precision_ == PrecisionType::UINT8 && !weights_as_input_; }
    bool perChannelUint8() const { return per_channel_ && precision_ == PrecisionType::UINT8 && !weights_as_input_; }
    const std::shared_ptr<HipTensor> &inputTensor() const { return input_; }
    const std::shared_ptr<HipTensor> &outputTensor() const { return output_; }
    Status requantNow(eh_requant *q) { return currentRequant(q); }

private:
    // The requantization parameters of this execution, read from the tensors now; in per-channel mode
    // also hands the plan the channel pairs when they differ from the ones it holds.
    Status currentRequant(eh_requant *q) {
        if (!per_channel_) {
            *q = detail::requantFromTensors(precision_, input_, weight_, bias_, output_, activation_info_);
            return Status::SUCCESS;
        }
        std::vector<int32_t> m, s;
        *q = pc_.derive(precision_, input_, output_, activation_info_, parameters_->scales, weight_->getZeroPoint(), false, &m, &s);
        if (plan_ != nullptr && (!pc_.sent || m != pc_.multipliers || s != pc_.shifts)) {
            const int rc = eh_dwconv2d_u8_set_perchannel(plan_, m.data(), s.data(), (int32_t)m.size(), runtime_->stream());
            CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipDepthwiseConvolution: %s", eh_last_error());
            pc_.multipliers = m;
            pc_.shifts = s;
            pc_.sent = true;
        }
        return Status::SUCCESS;
    }

    bool per_channel_ = false;
    detail::PerChannelState pc_;
    std::shared_ptr<HipRuntime> runtime_;
    PrecisionType precision_;
    std::shared_ptr<HipTensor> input_, output_, weight_, bias_;
    std::shared_ptr<DepthwiseConvolutionParameters> parameters_;
    ActivationInfo activation_info_;
    bool weights_as_input_ = false;
    eh_conv_desc desc_{};
    bool deferred_ = false;
    eh_dwconv_plan *plan_ = nullptr;
};

inline Status HipConvolution::fuseDepthwise(const std::shared_ptr<HipDepthwiseConvolution> &depthwise) {
    CHECK_EXPR_RETURN_FAILURE(plan_ != nullptr && !deferred_ && depthwise && depthwise->plan() != nullptr, "HipConvolution::fuseDepthwise before initialize");
    CHECK_EXPR_RETURN_FAILURE(precision_ == PrecisionType::UINT8 && launchesOnly() && !residual_ &&
                                  (per_channel_ ? depthwise->perChannelUint8() : depthwise->perTensorUint8()),
                              "HipConvolution::fuseDepthwise: uint8 tensors, constant weights quantized per tensor in both operators or per channel in both, no residual add");
    CHECK_EXPR_RETURN_FAILURE(depthwise->inputTensor() == output_, "HipConvolution::fuseDepthwise: the depthwise convolution does not read this convolution's output");
    if (!eh_conv_dw_block_applies(plan_, depthwise->plan())) return Status::FAILURE;  // (not an error: the caller runs the two operators apart)
    depthwise_ = depthwise;
    return Status::SUCCESS;
}

inline Status HipConvolution::executeWithDepthwise(const eh_requant &q) {
    eh_requant q_dw;
    CHECK_EXPR_RETURN_FAILURE(depthwise_->requantNow(&q_dw) == Status::SUCCESS, "HipConvolution::execute: the depthwise stage's requantization parameters");
    const int rc = eh_conv_dw_block_run(plan_, depthwise_->plan(), input_->getDataPtr(), depthwise_->outputTensor()->getDataPtr(), &q, &q_dw, 0, 0,
                                        runtime_->stream());
    CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipConvolution::execute (with the depthwise stage): %s", eh_last_error());
    return Status::SUCCESS;
}

class HipFullyConnected {
public:
    HipFullyConnected(const std::shared_ptr<HipRuntime> runtime, const PrecisionType &precision)
        : runtime_(runtime), precision_(precision) {}
    ~HipFullyConnected() { release(); }

    Status initialize(const std::vector<std::shared_ptr<ITensor>> &input_tensors,
                      const std::vector<std::shared_ptr<ITensor>> &output_tensors, const std::shared_ptr<Parameters> parameters) {
        CHECK_EXPR_RETURN_FAILURE(input_tensors.size() >= 3 && output_tensors.size() >= 1, "HipFullyConnected: needs {input, weight, bias} and {output}");
        input_ = std::static_pointer_cast<HipTensor>(input_tensors.at(INPUT_INDEX));
        weight_ = std::static_pointer_cast<HipTensor>(input_tensors.at(WEIGHT_INDEX));
        bias_ = std::static_pointer_cast<HipTensor>(input_tensors.at(BIAS_INDEX));
        output_ = std::static_pointer_cast<HipTensor>(output_tensors.at(OUTPUT_INDEX));
        parameters_ = std::dynamic_pointer_cast<FullyConnectedParameters>(parameters);
        CHECK_EXPR_RETURN_FAILURE(parameters_ != nullptr, "HipFullyConnected: parameters are not FullyConnectedParameters");
        CHECK_EXPR_RETURN_FAILURE(parameters_->activation_info != nullptr, "HipFullyConnected: null activation info");
        activation_info_ = *parameters_->activation_info;
        weights_as_input_ = !weight_->is_const() || !bias_->is_const();

        if (weight_->getTotalSizeFromDims() == 0) return Status::SUCCESS;
        CHECK_EXPR_RETURN_FAILURE(detail::quantizedPrecision(precision_), "HipFullyConnected: only the UINT8 and INT8 paths exist on this backend");
        CHECK_EXPR_RETURN_FAILURE(parameters_->storage_type == StorageType::BUFFER, "HipFullyConnected: no texture storage");
        CHECK_EXPR_RETURN_FAILURE(detail::tensorTypesMatch(precision_, false, input_, weight_, bias_, output_),
                                  "HipFullyConnected: expects uint8 (INT8 precision: int8) input/weight/output and int32 bias");
        // weight [units][k]; the input is flattened to [size / k][k] (in the order its shape reads: a tensor stored
        // channels-last must be one pixel per image)
        CHECK_EXPR_RETURN_FAILURE(!input_->storedChannelsLast() || (uint64_t)input_->getDim().h * input_->getDim().w <= 1,
                                  "HipFullyConnected: the input is stored channels-last and has more than one pixel per image");
        // (CLFullyConnected.cpp:46-57: in androidNN mode the batch is whatever the element count gives)
        const Dim4 wd = weight_->getDim();
        const uint32_t units = wd.n, k = wd.c * wd.h * wd.w;
        CHECK_EXPR_RETURN_FAILURE(k != 0 && input_->getTotalSizeFromDims() % k == 0, "HipFullyConnected: input of %u elements is not a multiple of k = %u", input_->getTotalSizeFromDims(), k);
        const uint32_t m = input_->getTotalSizeFromDims() / k;
        CHECK_EXPR_RETURN_FAILURE(parameters_->androidNN || m == input_->getDim().n, "HipFullyConnected: input batch %u does not match %u rows of k = %u", input_->getDim().n, m, k);
        CHECK_EXPR_RETURN_FAILURE(output_->getTotalSizeFromDims() == m * units, "HipFullyConnected: output has %u elements, expected %u", output_->getTotalSizeFromDims(), m * units);
        m_ = (int32_t)m;
        k_ = (int32_t)k;
        units_ = (int32_t)units;
        if (weights_as_input_ && (weight_->getDataPtr() == nullptr || bias_->getDataPtr() == nullptr)) {  // see HipConvolution::initialize
            deferred_ = true;
            return Status::SUCCESS;
        }
        return makePlan();
    }

    Status makePlan() {
        deferred_ = false;
        const eh_requant q = detail::requantFromTensors(precision_, input_, weight_, bias_, output_, activation_info_);
        const int32_t flags = precision_ == PrecisionType::INT8 ? (EH_W_SIGNED | EH_IO_SIGNED) : 0;
        const int rc = eh_fc_q8_plan(&plan_, m_, k_, units_, flags, weight_->getDataPtr(), bias_->getDataPtr(), &q, runtime_->stream());
        CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipFullyConnected::initialize: %s", eh_last_error());
        return Status::SUCCESS;
    }

    Status execute() {
        if (plan_ == nullptr && deferred_) CHECK_EXPR_RETURN_FAILURE(makePlan() == Status::SUCCESS, "HipFullyConnected::execute: the deferred plan could not be made");
        if (plan_ == nullptr) {
            CHECK_EXPR_RETURN_FAILURE(weight_ && weight_->getTotalSizeFromDims() == 0, "HipFullyConnected::execute before initialize");
            return Status::SUCCESS;
        }
        if (m_ == 0) return Status::SUCCESS;
        const eh_requant q = detail::requantFromTensors(precision_, input_, weight_, bias_, output_, activation_info_);
        if (weights_as_input_) {
            const int rc = eh_fc_u8_repack(plan_, weight_->getDataPtr(), bias_->getDataPtr(), &q, runtime_->stream());
            CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipFullyConnected::execute (repack): %s", eh_last_error());
        }
        const int rc = eh_fc_u8_run(plan_, input_->getDataPtr(), output_->getDataPtr(), &q, runtime_->stream());
        CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipFullyConnected::execute: %s", eh_last_error());
        return Status::SUCCESS;
    }

    bool launchesOnly() const { return !weights_as_input_; }
    Status release() {
        if (plan_) {
            (void)runtime_->synchronize();
            eh_fc_u8_destroy(plan_);
            plan_ = nullptr;
        }
        return Status::SUCCESS;
    }

private:
    std::shared_ptr<HipRuntime> runtime_;
    PrecisionType precision_;
    std::shared_ptr<HipTensor> input_, output_, weight_, bias_;
    std::shared_ptr<FullyConnectedParameters> parameters_;
    ActivationInfo activation_info_;
    bool weights_as_input_ = false;
    int32_t m_ = 0, k_ = 0, units_ = 0;
    bool deferred_ = false;
    eh_fc_plan *plan_ = nullptr;
};

class HipDeconvolution {
public:
    HipDeconvolution(const std::shared_ptr<HipRuntime> runtime, const PrecisionType &precision)
        : runtime_(runtime), precision_(precision) {}
    ~HipDeconvolution() { release(); }

    Status initialize(std::vector<std::shared_ptr<ITensor>> inputs_tensors, std::vector<std::shared_ptr<ITensor>> outputs_tensors,
                      std::shared_ptr<Parameters> parameters) {
        CHECK_EXPR_RETURN_FAILURE(inputs_tensors.size() >= 3 && outputs_tensors.size() >= 1, "HipDeconvolution: needs {input, weight, bias} and {output}");
        input_ = std::static_pointer_cast<HipTensor>(inputs_tensors.at(INPUT_INDEX));
        weight_ = std::static_pointer_cast<HipTensor>(inputs_tensors.at(WEIGHT_INDEX));
        bias_ = std::static_pointer_cast<HipTensor>(inputs_tensors.at(BIAS_INDEX));
        output_ = std::static_pointer_cast<HipTensor>(outputs_tensors.at(OUTPUT_INDEX));
        parameters_ = std::dynamic_pointer_cast<DeconvolutionParameters>(parameters);
        CHECK_EXPR_RETURN_FAILURE(parameters_ != nullptr, "HipDeconvolution: parameters are not DeconvolutionParameters");
        CHECK_EXPR_RETURN_FAILURE(parameters_->activation_info != nullptr, "HipDeconvolution: null activation info");
        activation_info_ = *parameters_->activation_info;
        weights_as_input_ = parameters_->weights_as_input || !weight_->is_const() || !bias_->is_const();

        if (weight_->getTotalSizeFromDims() == 0) return Status::SUCCESS;
        CHECK_EXPR_RETURN_FAILURE(detail::quantizedPrecision(precision_), "HipDeconvolution: only the UINT8 and INT8 paths exist on this backend");
        per_channel_ = parameters_->per_channel_quant;
        CHECK_EXPR_RETURN_FAILURE(detail::tensorTypesMatch(precision_, per_channel_, input_, weight_, bias_, output_),
                                  "HipDeconvolution: tensor data types do not fit the precision (uint8 tensors, int8 weights in per-channel mode; int8 tensors for INT8)");

        Dim4 in = input_->getDim();
        if (!parameters_->isNCHW) in = convertDimToNCHW(in);
        const Dim4 wd = weight_->getDim();
        const bool nn = parameters_->androidNN;  // weight Dim4 = (out, kh, kw, in); otherwise (in, out / groups, kh, kw)
        const uint32_t groups = nn ? 1 : parameters_->group_size;
        eh_conv_desc d;
        d.n = (int32_t)in.n;
        d.c = (int32_t)in.c;
        d.h = (int32_t)in.h;
        d.w = (int32_t)in.w;
        d.cout = (int32_t)(nn ? wd.n : wd.c * groups);
        d.kh = (int32_t)(nn ? wd.c : wd.h);
        d.kw = (int32_t)(nn ? wd.h : wd.w);
        d.stride_h = (int32_t)parameters_->stride.h;
        d.stride_w = (int32_t)parameters_->stride.w;
        d.pad_t = (int32_t)parameters_->padding.t;
        d.pad_b = (int32_t)parameters_->padding.b;
        d.pad_l = (int32_t)parameters_->padding.l;
        d.pad_r = (int32_t)parameters_->padding.r;
        d.dil_h = 1;
        d.dil_w = 1;
        d.groups = (int32_t)groups;
        d.depth_multiplier = 1;
        d.layout = parameters_->isNCHW ? detail::planarOperatorLayout(input_, output_) : EH_NHWC;
        CHECK_EXPR_RETURN_FAILURE(d.layout >= 0, "HipDeconvolution: input and output are stored in different element orders");
        d.weight_layout = nn ? EH_W_OHWI : EH_W_IOHW;
        CHECK_EXPR_RETURN_FAILURE((nn ? wd.w : wd.n) == in.c, "HipDeconvolution: weight input channels %u do not match the input's %u", nn ? wd.w : wd.n, in.c);
        desc_ = d;
        const int32_t oh = eh_deconv_out_dim(d.h, d.pad_t, d.pad_b, d.kh, d.stride_h);
        const int32_t ow = eh_deconv_out_dim(d.w, d.pad_l, d.pad_r, d.kw, d.stride_w);
        CHECK_EXPR_RETURN_FAILURE((int64_t)output_->getTotalSizeFromDims() == (int64_t)d.n * d.cout * oh * ow,
                                  "HipDeconvolution: output tensor has %u elements, the geometry gives %lld", output_->getTotalSizeFromDims(),
                                  (long long)d.n * d.cout * oh * ow);
        if (per_channel_) {
            CHECK_EXPR_RETURN_FAILURE(parameters_->scales.size() == (size_t)desc_.cout, "HipDeconvolution: %zu filter scales for %d output channels", parameters_->scales.size(), desc_.cout);
            desc_.weight_layout |= EH_W_SIGNED;
        }
        if (precision_ == PrecisionType::INT8) {
            desc_.weight_layout |= EH_W_SIGNED;
            desc_.layout |= EH_IO_SIGNED;
        }
        // Weights or bias that are run-time feature maps of an operator list have no device memory until the list's
        // pooled buffers are assigned: the plan is then made by the first execute(), which is where the reference packs
        // such weights anyway.
        if (weights_as_input_ && (weight_->getDataPtr() == nullptr || bias_->getDataPtr() == nullptr)) {
            deferred_ = true;
            return Status::SUCCESS;
        }
        return makePlan();
    }

    Status makePlan() {
        deferred_ = false;
        eh_requant q;
        CHECK_EXPR_RETURN_FAILURE(currentRequant(&q) == Status::SUCCESS, "HipDeconvolution::initialize: requantization parameters");
        const int rc = eh_deconv2d_u8_plan(&plan_, &desc_, weight_->getDataPtr(), bias_->getDataPtr(), &q, runtime_->stream());
        CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipDeconvolution::initialize: %s", eh_last_error());
        if (per_channel_) CHECK_EXPR_RETURN_FAILURE(currentRequant(&q) == Status::SUCCESS, "HipDeconvolution::initialize: per-channel pairs");
        return Status::SUCCESS;
    }

    Status execute() {
        if (plan_ == nullptr && deferred_) CHECK_EXPR_RETURN_FAILURE(makePlan() == Status::SUCCESS, "HipDeconvolution::execute: the deferred plan could not be made");
        if (plan_ == nullptr) {  // zero-sized operator
            CHECK_EXPR_RETURN_FAILURE(weight_ && weight_->getTotalSizeFromDims() == 0, "HipDeconvolution::execute before initialize");
            return Status::SUCCESS;
        }
        if (input_->getTotalSizeFromDims() == 0) return Status::SUCCESS;
        eh_requant q;
        CHECK_EXPR_RETURN_FAILURE(currentRequant(&q) == Status::SUCCESS, "HipDeconvolution::execute: requantization parameters");
        if (weights_as_input_) {
            const int rc = eh_deconv2d_u8_repack(plan_, weight_->getDataPtr(), bias_->getDataPtr(), &q, runtime_->stream());
            CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipDeconvolution::execute (repack): %s", eh_last_error());
        }
        const int rc = eh_deconv2d_u8_run(plan_, input_->getDataPtr(), output_->getDataPtr(), &q, runtime_->stream());
        CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipDeconvolution::execute: %s", eh_last_error());
        return Status::SUCCESS;
    }

    bool launchesOnly() const { return !weights_as_input_; }
    Status release() {
        if (plan_) {
            (void)runtime_->synchronize();
            eh_deconv2d_u8_destroy(plan_);
            plan_ = nullptr;
        }
        return Status::SUCCESS;
    }

private:
    // The requantization parameters of this execution, read from the tensors now; in per-channel mode
    // also hands the plan the channel pairs when they differ from the ones it holds.
    Status currentRequant(eh_requant *q) {
        if (!per_channel_) {
            *q = detail::requantFromTensors(precision_, input_, weight_, bias_, output_, activation_info_);
            return Status::SUCCESS;
        }
        std::vector<int32_t> m, s;
        *q = pc_.derive(precision_, input_, output_, activation_info_, parameters_->scales, weight_->getZeroPoint(), true, &m, &s);
        if (plan_ != nullptr && (!pc_.sent || m != pc_.multipliers || s != pc_.shifts)) {
            const int rc = eh_deconv2d_u8_set_perchannel(plan_, m.data(), s.data(), (int32_t)m.size(), runtime_->stream());
            CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipDeconvolution: %s", eh_last_error());
            pc_.multipliers = m;
            pc_.shifts = s;
            pc_.sent = true;
        }
        return Status::SUCCESS;
    }

    bool per_channel_ = false;
    detail::PerChannelState pc_;
    std::shared_ptr<HipRuntime> runtime_;
    PrecisionType precision_;
    std::shared_ptr<HipTensor> input_, output_, weight_, bias_;
    std::shared_ptr<DeconvolutionParameters> parameters_;
    ActivationInfo activation_info_;
    bool weights_as_input_ = false;
    eh_conv_desc desc_{};
    bool deferred_ = false;
    eh_deconv_plan *plan_ = nullptr;
};

// Element-wise sum of two equally shaped uint8 tensors, requantized to the output tensor's
// scale (quantization parameters are read from the three tensors at every execute()).
// Broadcasting and the int16 power-of-two variant are not offered here; coefficients are ignored, as the
// reference's quantized path ignores them.
class HipAdd {
public:
    HipAdd(const std::shared_ptr<HipRuntime> runtime, const PrecisionType &precision) : runtime_(runtime), precision_(precision) {}

    Status initialize(const std::vector<std::shared_ptr<ITensor>> &input_tensors,
                      const std::vector<std::shared_ptr<ITensor>> &output_tensors, const std::shared_ptr<Parameters> parameters) {
        CHECK_EXPR_RETURN_FAILURE(input_tensors.size() == 2 && output_tensors.size() >= 1, "HipAdd: needs two inputs and one output");
        a_ = std::static_pointer_cast<HipTensor>(input_tensors.at(0));
        b_ = std::static_pointer_cast<HipTensor>(input_tensors.at(1));
        output_ = std::static_pointer_cast<HipTensor>(output_tensors.at(0));
        parameters_ = std::dynamic_pointer_cast<AddParameters>(parameters);
        CHECK_EXPR_RETURN_FAILURE(parameters_ != nullptr, "HipAdd: parameters are not AddParameters");
        CHECK_EXPR_RETURN_FAILURE(precision_ == PrecisionType::UINT8, "HipAdd: only the UINT8 path exists on this backend");
        CHECK_EXPR_RETURN_FAILURE(parameters_->storage_type == StorageType::BUFFER, "HipAdd: no texture storage");
        // coefficients belong to the float kernels: the quantized path never reads them (gpu/operators/CLAdd.cpp:159-163)
        CHECK_EXPR_RETURN_FAILURE(!parameters_->pot_scale_int16, "HipAdd: int16 scaling is not offered");
        CHECK_EXPR_RETURN_FAILURE(a_->getDataType() == DataType::UINT8 && b_->getDataType() == DataType::UINT8 &&
                                      output_->getDataType() == DataType::UINT8, "HipAdd: expects uint8 tensors");
        CHECK_EXPR_RETURN_FAILURE(a_->getTotalSizeFromDims() == b_->getTotalSizeFromDims() &&
                                      a_->getTotalSizeFromDims() == output_->getTotalSizeFromDims(), "HipAdd: shapes differ (no broadcast)");
        // element by element: any element order, as long as it is the same one
        CHECK_EXPR_RETURN_FAILURE(a_->storedChannelsLast() == b_->storedChannelsLast() && a_->storedChannelsLast() == output_->storedChannelsLast(),
                                  "HipAdd: the tensors are stored in different element orders");
        ready_ = true;
        return Status::SUCCESS;
    }

    Status execute() {
        CHECK_EXPR_RETURN_FAILURE(ready_, "HipAdd::execute before initialize");
        eh_add_requant q;
        eh_make_add_requant(a_->getScale(), a_->getZeroPoint(), b_->getScale(), b_->getZeroPoint(), output_->getScale(),
                            output_->getZeroPoint(), detail::toEhActivation(parameters_->activation_info),
                            parameters_->activation_info.isEnabled() ? 1 : 0, &q);
        const int rc = eh_add_u8(a_->getDataPtr(), b_->getDataPtr(), output_->getDataPtr(), (int64_t)output_->getTotalSizeFromDims(), &q,
                                 runtime_->stream());
        CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipAdd::execute: %s", eh_last_error());
        return Status::SUCCESS;
    }

    bool launchesOnly() const { return true; }
    Status release() { return Status::SUCCESS; }

private:
    std::shared_ptr<HipRuntime> runtime_;
    PrecisionType precision_;
    std::shared_ptr<HipTensor> a_, b_, output_;
    std::shared_ptr<AddParameters> parameters_;
    bool ready_ = false;
};

// Average pool on a uint8 tensor: windows clipped to the image, (sum + count / 2) / count, clamp to
// the activation range of the output tensor.  Input and output share one scale and zero point.
class HipAveragepool {
public:
    HipAveragepool(const std::shared_ptr<HipRuntime> runtime, const PrecisionType &precision)
        : runtime_(runtime), precision_(precision) {}

    Status initialize(const std::vector<std::shared_ptr<ITensor>> &input_tensors,
                      const std::vector<std::shared_ptr<ITensor>> &output_tensors, const std::shared_ptr<Parameters> parameters) {
        CHECK_EXPR_RETURN_FAILURE(input_tensors.size() >= 1 && output_tensors.size() >= 1, "HipAveragepool: needs an input and an output");
        input_ = std::static_pointer_cast<HipTensor>(input_tensors.at(0));
        output_ = std::static_pointer_cast<HipTensor>(output_tensors.at(0));
        parameters_ = std::dynamic_pointer_cast<Pool2DParameters>(parameters);
        CHECK_EXPR_RETURN_FAILURE(parameters_ != nullptr, "HipAveragepool: parameters are not Pool2DParameters");
        CHECK_EXPR_RETURN_FAILURE(detail::quantizedPrecision(precision_), "HipAveragepool: only the UINT8 and INT8 paths exist on this backend");
        CHECK_EXPR_RETURN_FAILURE(parameters_->storage_type == StorageType::BUFFER, "HipAveragepool: no texture storage");
        CHECK_EXPR_RETURN_FAILURE(parameters_->compute_type == ComputeType::TFLite, "HipAveragepool: only the TFLite window rule");
        const DataType io = precision_ == PrecisionType::INT8 ? DataType::INT8 : DataType::UINT8;
        CHECK_EXPR_RETURN_FAILURE(input_->getDataType() == io && output_->getDataType() == io,
                                  "HipAveragepool: expects uint8 tensors (INT8 precision: int8)");
        const Dim4 id = input_->getDim();
        const bool nchw = parameters_->isNCHW;
        d_.n = (int32_t)id.n;
        d_.c = (int32_t)(nchw ? id.c : id.w);  // channels-last tensors hold (n, h, w, c) positionally
        d_.h = (int32_t)(nchw ? id.h : id.c);
        d_.w = (int32_t)(nchw ? id.w : id.h);
        d_.kh = (int32_t)parameters_->filter.h;
        d_.kw = (int32_t)parameters_->filter.w;
        d_.stride_h = (int32_t)parameters_->stride.h;
        d_.stride_w = (int32_t)parameters_->stride.w;
        d_.pad_t = (int32_t)parameters_->padding.t;
        d_.pad_b = (int32_t)parameters_->padding.b;
        d_.pad_l = (int32_t)parameters_->padding.l;
        d_.pad_r = (int32_t)parameters_->padding.r;
        const int order = nchw ? detail::planarOperatorLayout(input_, output_) : EH_NHWC;
        CHECK_EXPR_RETURN_FAILURE(order >= 0, "HipAveragepool: input and output are stored in different element orders");
        d_.layout = order | (precision_ == PrecisionType::INT8 ? EH_IO_SIGNED : 0);
        CHECK_EXPR_RETURN_FAILURE(d_.kh > 0 && d_.kw > 0 && d_.stride_h > 0 && d_.stride_w > 0, "HipAveragepool: bad window or stride");
        const int32_t ho = (d_.h + d_.pad_t + d_.pad_b - d_.kh) / d_.stride_h + 1, wo = (d_.w + d_.pad_l + d_.pad_r - d_.kw) / d_.stride_w + 1;
        CHECK_EXPR_RETURN_FAILURE((uint64_t)output_->getTotalSizeFromDims() == (uint64_t)d_.n * d_.c * ho * wo,
                                  "HipAveragepool: output has %u elements, expected %d x %d x %d x %d", output_->getTotalSizeFromDims(), d_.n, d_.c, ho, wo);
        ready_ = true;
        return Status::SUCCESS;
    }

    Status execute() {
        CHECK_EXPR_RETURN_FAILURE(ready_, "HipAveragepool::execute before initialize");
        eh_pool_desc d = d_;
        // the range comes from the activation type alone, as in CLAveragepool::averagepool_quant (CLAveragepool.cpp:183-198)
        (precision_ == PrecisionType::INT8 ? eh_act_range_s8 : eh_act_range_u8)(detail::toEhActivation(parameters_->activation_info),
                                                                                output_->getScale(), output_->getZeroPoint(),
                                                                                &d.act_min, &d.act_max);
        const int rc = eh_avgpool_u8(input_->getDataPtr(), output_->getDataPtr(), &d, runtime_->stream());
        CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipAveragepool::execute: %s", eh_last_error());
        return Status::SUCCESS;
    }

    bool launchesOnly() const { return true; }
    Status release() { return Status::SUCCESS; }

private:
    std::shared_ptr<HipRuntime> runtime_;
    PrecisionType precision_;
    std::shared_ptr<HipTensor> input_, output_;
    std::shared_ptr<Pool2DParameters> parameters_;
    eh_pool_desc d_{};
    bool ready_ = false;
};

// Planar <-> channels-last storage of one byte tensor whose shape reads (n, c, h, w): the operator constructor puts one
// behind every input and in front of every output of a planar operator list whose feature maps it stores channels-last
// (nchw2nhwc_uint8 / nhwc2nchw_uint8, cl_kernels/NormalizationKernels and CLTensor.cpp:181-225, as operators of the list).
class HipLayoutChange {
public:
    HipLayoutChange(const std::shared_ptr<HipRuntime> runtime, bool to_channels_last) : runtime_(runtime), to_channels_last_(to_channels_last) {}

    Status initialize(const std::vector<std::shared_ptr<ITensor>> &input_tensors, const std::vector<std::shared_ptr<ITensor>> &output_tensors,
                      const std::shared_ptr<Parameters> = nullptr) {
        CHECK_EXPR_RETURN_FAILURE(input_tensors.size() == 1 && output_tensors.size() == 1, "HipLayoutChange: needs one input and one output");
        input_ = std::static_pointer_cast<HipTensor>(input_tensors.at(0));
        output_ = std::static_pointer_cast<HipTensor>(output_tensors.at(0));
        CHECK_EXPR_RETURN_FAILURE(input_->getNumOfBytes() == input_->getTotalSizeFromDims() && output_->getNumOfBytes() == input_->getNumOfBytes(),
                                  "HipLayoutChange: byte tensors of one size");
        CHECK_EXPR_RETURN_FAILURE(input_->storedChannelsLast() != to_channels_last_ && output_->storedChannelsLast() == to_channels_last_,
                                  "HipLayoutChange: the tensors' element orders do not fit the direction");
        ready_ = true;
        return Status::SUCCESS;
    }

    Status execute() {
        CHECK_EXPR_RETURN_FAILURE(ready_, "HipLayoutChange::execute before initialize");
        if (input_->getTotalSizeFromDims() == 0) return Status::SUCCESS;
        const Dim4 d = input_->getDim();
        const int rc = (to_channels_last_ ? eh_transpose_u8_nchw2nhwc : eh_transpose_u8_nhwc2nchw)(input_->getDataPtr(), output_->getDataPtr(), (int32_t)d.n,
                                                                                                  (int32_t)d.c, (int32_t)d.h, (int32_t)d.w,
                                                                                                  runtime_->stream());
        CHECK_EXPR_RETURN_FAILURE(rc == EH_OK, "HipLayoutChange::execute: %s", eh_last_error());
        return Status::SUCCESS;
    }

    bool launchesOnly() const { return true; }
    Status release() { return Status::SUCCESS; }

private:
    std::shared_ptr<HipRuntime> runtime_;
    bool to_channels_last_;
    std::shared_ptr<HipTensor> input_, output_;
    bool ready_ = false;
};

}  // namespace hip
}  // namespace ud
}  // namespace enn
