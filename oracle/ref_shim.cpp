// C-callable view of the reference's own host arithmetic, used to pin the
// oracle.  TEST INFRASTRUCTURE ONLY.  This file holds no reference code: it
// includes the reference's headers where they lie and is linked against the
// reference's QuantizationUtil.cpp and KernelUtil.cpp, compiled in place by
// oracle/Makefile into oracle/_ref/ (never committed, never shipped as product).
#include <cstdint>

#include "userdriver/gpu/operators/cl_quantized_utils/QuantizationUtil.hpp"
#include "userdriver/common/operator_interfaces/common/ActivationInfo.hpp"

namespace enn {
namespace ud {
namespace gpu {
// declared in cl_quantized_utils/KernelUtil.hpp; re-declared here because that
// header also pulls in the OpenCL tensor class, which this shim does not need
Status GetQuantizedConvolutionMultipler(double, double, double, double, double *);
void CalculateActivationRangeUint8(ActivationInfo::ActivationType, float, int32_t, int32_t *, int32_t *);
void CalculateActivationRangeInt8(ActivationInfo::ActivationType, float, int32_t, int32_t *, int32_t *);
}  // namespace gpu
}  // namespace ud
}  // namespace enn

extern "C" {

void ref_quantize_multiplier(double m, int32_t *q, int32_t *shift) {
    int s = 0;
    enn::ud::gpu::QuantizeMultiplier(m, q, &s);
    *shift = s;
}

int ref_conv_multiplier(float s_in, float s_w, float s_bias, float s_out, double *m) {
    return enn::ud::gpu::GetQuantizedConvolutionMultipler(s_in, s_w, s_bias, s_out, m) == Status::SUCCESS ? 0 : 1;
}

void ref_act_range_u8(int act, float scale, int32_t zp, int32_t *amin, int32_t *amax) {
    enn::ud::gpu::CalculateActivationRangeUint8(static_cast<ActivationInfo::ActivationType>(act), scale, zp, amin, amax);
}

void ref_act_range_s8(int act, float scale, int32_t zp, int32_t *amin, int32_t *amax) {
    enn::ud::gpu::CalculateActivationRangeInt8(static_cast<ActivationInfo::ActivationType>(act), scale, zp, amin, amax);
}

int32_t ref_srdhm(int32_t a, int32_t b) { return gemmlowp::SaturatingRoundingDoublingHighMul(a, b); }

int32_t ref_rdivpot(int32_t x, int32_t e) { return gemmlowp::RoundingDivideByPOT(x, e); }

int32_t ref_mbqm(int32_t x, int32_t q, int32_t shift) { return enn::ud::gpu::MultiplyByQuantizedMultiplier(x, q, shift); }

}  // extern "C"
