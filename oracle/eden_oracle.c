/*
 * eden_oracle — CPU restatement of the reference's quantized operator semantics.
 * TEST INFRASTRUCTURE ONLY: see eden_oracle.h for who may call it and for the
 * pinning status of each function.
 *
 * All reference citations are relative to the reference repository root.
 */
#include "eden_oracle.h"

#include <limits.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------ */
/* host arithmetic                                                          */
/* ------------------------------------------------------------------------ */

/* src/userdriver/gpu/operators/cl_quantized_utils/QuantizationUtil.cpp:8-21 */
void eo_quantize_multiplier(double m, int32_t *q, int32_t *shift) {
    if (m == 0.) {
        *q = 0;
        *shift = 0;
        return;
    }
    int e = 0;
    const double frac = frexp(m, &e);
    int64_t q_fixed = (int64_t)round(frac * (double)(1ll << 31));
    if (q_fixed == (1ll << 31)) {
        q_fixed /= 2;
        ++e;
    }
    *q = (int32_t)q_fixed;
    *shift = e;
}

/* src/userdriver/gpu/operators/cl_quantized_utils/KernelUtil.cpp:7-25
 * Returns 0 on success; on failure returns 1 and leaves *m untouched, which is
 * how the callers end up with multiplier 0
 * (cl_optimized_impls/CLGEMMConvolutionQuantized.cpp:163-166). */
int eo_conv_multiplier(float s_in, float s_w, float s_bias, float s_out, double *m) {
    const double in_scale = (double)s_in, w_scale = (double)s_w;
    const double bias_scale = (double)s_bias, out_scale = (double)s_out;
    const double product = in_scale * w_scale;
    const double lim = 1e-6 * (product < bias_scale ? product : bias_scale);
    if (!(fabs(product - bias_scale) <= lim)) return 1;
    if (!(product >= 0)) return 1;
    *m = product / out_scale;
    return 0;
}

/* src/userdriver/gpu/operators/cl_quantized_utils/KernelUtil.cpp:27-60
 * (the lambda divides a float by a float and calls double round()) */
static int32_t quantize_real(float f, float scale, int32_t zp) {
    return zp + (int32_t)round((double)(f / scale));
}

static void act_range(int act, float scale, int32_t zp, int32_t qmin, int32_t qmax, int32_t *amin, int32_t *amax);

void eo_act_range_u8(int act, float scale, int32_t zp, int32_t *amin, int32_t *amax) {
    act_range(act, scale, zp, 0, 255, amin, amax);
}

/* src/userdriver/gpu/operators/cl_quantized_utils/KernelUtil.cpp:62-71: the same clamps over [-128, 127] */
void eo_act_range_s8(int act, float scale, int32_t zp, int32_t *amin, int32_t *amax) {
    act_range(act, scale, zp, -128, 127, amin, amax);
}

static void act_range(int act, float scale, int32_t zp, int32_t qmin, int32_t qmax, int32_t *amin, int32_t *amax) {
    if (act == EO_ACT_RELU) {
        const int32_t lo = quantize_real(0.0f, scale, zp);
        *amin = qmin > lo ? qmin : lo;
        *amax = qmax;
    } else if (act == EO_ACT_RELU6) {
        const int32_t lo = quantize_real(0.0f, scale, zp);
        const int32_t hi = quantize_real(6.0f, scale, zp);
        *amin = qmin > lo ? qmin : lo;
        *amax = qmax < hi ? qmax : hi;
    } else if (act == EO_ACT_RELU1) {
        const int32_t lo = quantize_real(-1.0f, scale, zp);
        const int32_t hi = quantize_real(1.0f, scale, zp);
        *amin = qmin > lo ? qmin : lo;
        *amax = qmax < hi ? qmax : hi;
    } else {
        *amin = qmin;
        *amax = qmax;
    }
}

/* src/userdriver/gpu/common/CLKernels.hpp:120-126,
 * src/userdriver/gpu/operators/cl_quantized_utils/QuantizationUtil.cpp:100-108 */
int32_t eo_srdhm(int32_t a, int32_t b) {
    if (a == b && a == INT32_MIN) return INT32_MAX;
    const int64_t ab = (int64_t)a * (int64_t)b;
    const int64_t nudge = ab >= 0 ? (1ll << 30) : (1 - (1ll << 30));
    return (int32_t)((ab + nudge) / (1ll << 31)); /* C division truncates toward zero */
}

/* src/userdriver/gpu/common/CLKernels.hpp:143-149,
 * src/userdriver/gpu/operators/cl_quantized_utils/QuantizationUtil.cpp:110-117 */
int32_t eo_rdivpot(int32_t x, int32_t exponent) {
    const int32_t mask = (int32_t)((1ll << exponent) - 1);
    const int32_t remainder = x & mask;
    const int32_t threshold = (mask >> 1) + (x < 0 ? 1 : 0);
    return (x >> exponent) + (remainder > threshold ? 1 : 0);
}

/* src/userdriver/gpu/operators/cl_quantized_utils/QuantizationUtil.hpp:102-110;
 * the product x * (1 << ls) wraps like the int32 multiply in the device code
 * (src/userdriver/gpu/operators/cl_kernels/ConvolutionKernels.cpp:1066). */
int32_t eo_mbqm(int32_t x, int32_t q, int32_t shift) {
    const int32_t ls = shift > 0 ? shift : 0;
    const int32_t rs = shift > 0 ? 0 : -shift;
    const int32_t shifted = (int32_t)((uint32_t)x << ls);
    return eo_rdivpot(eo_srdhm(shifted, q), rs);
}

/* src/userdriver/gpu/common/CLKernels.hpp:151-170 */
uint8_t eo_requant(int32_t acc, const eo_quant *q) {
    int32_t x = eo_mbqm(acc, q->multiplier, q->shift) + q->zp_out;
    if (x < q->act_min) x = q->act_min;
    if (x > q->act_max) x = q->act_max;
    return (uint8_t)x;
}

/* What an operator's execute() derives from its tensors:
 * cl_optimized_impls/CLGEMMConvolutionQuantized.cpp:137-171 */
void eo_make_quant(float s_in, int32_t zp_in, float s_w, int32_t zp_w, float s_bias,
                   float s_out, int32_t zp_out, int act, int act_enabled, eo_quant *q) {
    double m = 0.0;
    (void)eo_conv_multiplier(s_in, s_w, s_bias, s_out, &m); /* status ignored, as the callers do */
    eo_quantize_multiplier(m, &q->multiplier, &q->shift);
    q->zp_in = zp_in;
    q->zp_w = zp_w;
    q->zp_out = zp_out;
    if (act_enabled) {
        eo_act_range_u8(act, s_out, zp_out, &q->act_min, &q->act_max);
    } else {
        q->act_min = 0;
        q->act_max = 255;
    }
}

/* INT8 precision: cl_optimized_impls/CLGEMMConvolutionQuantized.cpp:224-241 */
void eo_make_quant_s8(float s_in, int32_t zp_in, float s_w, int32_t zp_w, float s_bias,
                      float s_out, int32_t zp_out, int act, int act_enabled, eo_quant *q) {
    eo_make_quant(s_in, zp_in, s_w, zp_w, s_bias, s_out, zp_out, act, 0, q);
    if (act_enabled) {
        eo_act_range_s8(act, s_out, zp_out, &q->act_min, &q->act_max);
    } else {
        q->act_min = -128;
        q->act_max = 127;
    }
}

/* src/userdriver/gpu/operators/CLConvolution.cpp:99-104 */
int32_t eo_conv_out_dim(int32_t in, int32_t pad_a, int32_t pad_b, int32_t k, int32_t dil, int32_t stride) {
    return (in + pad_a + pad_b - (dil * (k - 1) + 1) + stride) / stride;
}

/* src/userdriver/gpu/operators/CLDeconvolution.cpp:82-87 */
int32_t eo_deconv_out_dim(int32_t in, int32_t pad_a, int32_t pad_b, int32_t k, int32_t stride) {
    return in * stride + k - stride - pad_a - pad_b;
}

/* ------------------------------------------------------------------------ */
/* operators                                                                */
/* ------------------------------------------------------------------------ */

/* Accumulate one (input plane, tap) pair into an int32 output plane.  The
 * index relation iy = oy*stride + ky*dil - pad and the skip of out-of-range
 * taps follow src/userdriver/gpu/op_test/convolution_guard.h:118-144 and
 * cl_kernels/ConvolutionKernels.cpp:1321-1350; a skipped tap is the same as
 * a tap that reads zp_in (cl_optimized_impls/CLPadConvert.cpp:185). */
static void accumulate_tap(int32_t *plane, const uint8_t *src, int in_is_signed, int32_t wv, int32_t zp_in,
                           int32_t H, int32_t W, int32_t Ho, int32_t Wo,
                           int32_t oy_off, int32_t ox_off, int32_t sh, int32_t sw) {
    /* iy = oy*sh + oy_off, ix = ox*sw + ox_off */
    for (int32_t oy = 0; oy < Ho; ++oy) {
        const int32_t iy = oy * sh + oy_off;
        if (iy < 0 || iy >= H) continue;
        int32_t ox0 = 0;
        if (ox_off < 0) ox0 = (-ox_off + sw - 1) / sw;
        int32_t ox1 = Wo;
        if ((Wo - 1) * sw + ox_off >= W) ox1 = (W - 1 - ox_off) / sw + 1;
        if (ox_off > W - 1) ox1 = 0;
        const uint8_t *row = src + (int64_t)iy * W;
        int32_t *dst = plane + (int64_t)oy * Wo;
        if (in_is_signed) {
            const int8_t *srow = (const int8_t *)row;
            for (int32_t ox = ox0; ox < ox1; ++ox) dst[ox] += ((int32_t)srow[ox * sw + ox_off] - zp_in) * wv;
        } else {
            for (int32_t ox = ox0; ox < ox1; ++ox) dst[ox] += ((int32_t)row[ox * sw + ox_off] - zp_in) * wv;
        }
    }
}

static void conv_core(const uint8_t *in, int in_is_signed, const void *w, int w_is_signed, const int32_t *bias, uint8_t *out,
                      const eo_conv_shape *s, const eo_quant *q, const int32_t *multipliers,
                      const int32_t *shifts, int32_t *acc_out) {
    const int32_t Ho = eo_conv_out_dim(s->h, s->pad_t, s->pad_b, s->kh, s->dil_h, s->stride_h);
    const int32_t Wo = eo_conv_out_dim(s->w, s->pad_l, s->pad_r, s->kw, s->dil_w, s->stride_w);
    const int32_t G = s->groups, Cig = s->c / G, Cog = s->cout / G;
    const int64_t plane = (int64_t)Ho * Wo;
    const int64_t jobs = (int64_t)s->n * s->cout;
    if (plane <= 0 || jobs <= 0) return;
#pragma omp parallel
    {
        int32_t *acc = (int32_t *)malloc(sizeof(int32_t) * (size_t)plane);
#pragma omp for schedule(static)
        for (int64_t job = 0; job < jobs; ++job) {
            const int32_t n = (int32_t)(job / s->cout), oc = (int32_t)(job % s->cout);
            const int32_t g = oc / Cog;
            for (int64_t i = 0; i < plane; ++i) acc[i] = bias ? bias[oc] : 0;
            for (int32_t ic = 0; ic < Cig; ++ic) {
                const uint8_t *src = in + ((int64_t)n * s->c + g * Cig + ic) * s->h * s->w;
                for (int32_t ky = 0; ky < s->kh; ++ky)
                    for (int32_t kx = 0; kx < s->kw; ++kx) {
                        const int64_t wi = (((int64_t)oc * Cig + ic) * s->kh + ky) * s->kw + kx;
                        const int32_t wv = w_is_signed ? (int32_t)((const int8_t *)w)[wi] - q->zp_w
                                                       : (int32_t)((const uint8_t *)w)[wi] - q->zp_w;
                        accumulate_tap(acc, src, in_is_signed, wv, q->zp_in, s->h, s->w, Ho, Wo,
                                       ky * s->dil_h - s->pad_t, kx * s->dil_w - s->pad_l,
                                       s->stride_h, s->stride_w);
                    }
            }
            eo_quant ql = *q;
            if (multipliers) {
                ql.multiplier = multipliers[oc];
                ql.shift = shifts[oc];
            }
            uint8_t *dst = out + job * plane;
            for (int64_t i = 0; i < plane; ++i) dst[i] = eo_requant(acc[i], &ql);
            if (acc_out) memcpy(acc_out + job * plane, acc, sizeof(int32_t) * (size_t)plane);
        }
        free(acc);
    }
}

/* Semantics: cl_kernels/ConvolutionKernels.cpp:956-1076 (GEMM form) and
 * :1317-1375 (naive per-channel form); weights [Cout][Cin/g][kh][kw]. */
void eo_conv2d_u8(const uint8_t *in, const uint8_t *w, const int32_t *bias, uint8_t *out,
                  const eo_conv_shape *s, const eo_quant *q, int32_t *acc) {
    conv_core(in, 0, w, 0, bias, out, s, q, NULL, NULL, acc);
}

/* cl_kernels/ConvolutionKernels.cpp:1317-1375: int8 weights, one multiplier
 * and shift per output channel. */
void eo_conv2d_u8_perchannel(const uint8_t *in, const int8_t *w, const int32_t *bias, uint8_t *out,
                             const eo_conv_shape *s, const eo_quant *q,
                             const int32_t *multipliers, const int32_t *shifts, int32_t *acc) {
    conv_core(in, 0, w, 1, bias, out, s, q, multipliers, shifts, acc);
}

/* cl_kernels/DepthwiseconvolutionKernels.cpp:1273-1321; weights [C*dm][1][kh][kw],
 * output channel c*dm+d reads input channel c. */
static void dw_core(const uint8_t *in, int in_is_signed, const void *w, int w_is_signed, const int32_t *bias, uint8_t *out,
                    const eo_conv_shape *s, const eo_quant *q, const int32_t *multipliers,
                    const int32_t *shifts, int32_t *acc_out) {
    const int32_t Ho = eo_conv_out_dim(s->h, s->pad_t, s->pad_b, s->kh, s->dil_h, s->stride_h);
    const int32_t Wo = eo_conv_out_dim(s->w, s->pad_l, s->pad_r, s->kw, s->dil_w, s->stride_w);
    const int32_t dm = s->dm > 0 ? s->dm : 1;
    const int32_t Cout = s->c * dm;
    const int64_t plane = (int64_t)Ho * Wo;
    const int64_t jobs = (int64_t)s->n * Cout;
    if (plane <= 0 || jobs <= 0) return;
#pragma omp parallel
    {
        int32_t *acc = (int32_t *)malloc(sizeof(int32_t) * (size_t)plane);
#pragma omp for schedule(static)
        for (int64_t job = 0; job < jobs; ++job) {
            const int32_t n = (int32_t)(job / Cout), oc = (int32_t)(job % Cout);
            const int32_t ic = oc / dm;
            for (int64_t i = 0; i < plane; ++i) acc[i] = bias ? bias[oc] : 0;
            const uint8_t *src = in + ((int64_t)n * s->c + ic) * s->h * s->w;
            for (int32_t ky = 0; ky < s->kh; ++ky)
                for (int32_t kx = 0; kx < s->kw; ++kx) {
                    const int64_t wi = ((int64_t)oc * s->kh + ky) * s->kw + kx;
                    const int32_t wv = w_is_signed ? (int32_t)((const int8_t *)w)[wi] - q->zp_w
                                                   : (int32_t)((const uint8_t *)w)[wi] - q->zp_w;
                    accumulate_tap(acc, src, in_is_signed, wv, q->zp_in, s->h, s->w, Ho, Wo,
                                   ky * s->dil_h - s->pad_t, kx * s->dil_w - s->pad_l,
                                   s->stride_h, s->stride_w);
                }
            eo_quant ql = *q;
            if (multipliers) {
                ql.multiplier = multipliers[oc];
                ql.shift = shifts[oc];
            }
            uint8_t *dst = out + job * plane;
            for (int64_t i = 0; i < plane; ++i) dst[i] = eo_requant(acc[i], &ql);
            if (acc_out) memcpy(acc_out + job * plane, acc, sizeof(int32_t) * (size_t)plane);
        }
        free(acc);
    }
}

void eo_dwconv2d_u8(const uint8_t *in, const uint8_t *w, const int32_t *bias, uint8_t *out,
                    const eo_conv_shape *s, const eo_quant *q, int32_t *acc_out) {
    dw_core(in, 0, w, 0, bias, out, s, q, NULL, NULL, acc_out);
}

/* cl_kernels/DepthwiseconvolutionKernels.cpp:1323-1371 (int8 weight bytes, the multiplier and
 * shift of output channel c*dm+d), driven by
 * cl_optimized_impls/CLDepthwiseConvolutionPerChannelQuantized.cpp:133-153. */
void eo_dwconv2d_u8_perchannel(const uint8_t *in, const int8_t *w, const int32_t *bias, uint8_t *out,
                               const eo_conv_shape *s, const eo_quant *q,
                               const int32_t *multipliers, const int32_t *shifts, int32_t *acc_out) {
    dw_core(in, 0, w, 1, bias, out, s, q, multipliers, shifts, acc_out);
}

/* Layout a[m][k], w[n][k], out[m][n]: src/userdriver/gpu/op_test/fullyconnected_test.cpp:93-105.
 * Arithmetic: the convolution integer pipeline applied to a 1x1 problem
 * (cl_kernels/ConvolutionKernels.cpp:956-1076), not the reference's float
 * detour for uint8 FullyConnected. */
void eo_fc_u8(const uint8_t *a, const uint8_t *w, const int32_t *bias, uint8_t *out,
              int32_t m, int32_t k, int32_t n, const eo_quant *q, int32_t *acc_out) {
    const int32_t zp_a = q->zp_in, zp_w = q->zp_w;
#pragma omp parallel for schedule(static) collapse(2)
    for (int32_t i = 0; i < m; ++i)
        for (int32_t j = 0; j < n; ++j) {
            const uint8_t *ar = a + (int64_t)i * k, *wr = w + (int64_t)j * k;
            int32_t acc = 0;
            for (int32_t t = 0; t < k; ++t) acc += ((int32_t)ar[t] - zp_a) * ((int32_t)wr[t] - zp_w);
            acc += bias ? bias[j] : 0;
            out[(int64_t)i * n + j] = eo_requant(acc, q);
            if (acc_out) acc_out[(int64_t)i * n + j] = acc;
        }
}

/* Gather form in double precision, shared by the uint8 operator and by the
 * float known-answer vectors of the reference's own tests (double arithmetic on
 * integer-valued data below 2^53 is exact, so the uint8 path loses nothing).
 * Index relation h_im = oy + pad = h_col*stride + ky:
 * cl_kernels/DeconvolutionKernels.cpp:147-198 over the products of :24-60;
 * weights [Cin][Cout/g][kh][kw] (src/userdriver/gpu/op_test/deconv_guard.h:53-69).
 * `in` and `w` already have their zero points removed. */
void eo_deconv2d_f64(const double *in, const double *w, const double *bias, double *out,
                     const eo_conv_shape *s) {
    const int32_t Ho = eo_deconv_out_dim(s->h, s->pad_t, s->pad_b, s->kh, s->stride_h);
    const int32_t Wo = eo_deconv_out_dim(s->w, s->pad_l, s->pad_r, s->kw, s->stride_w);
    const int32_t G = s->groups, Cig = s->c / G, Cog = s->cout / G;
    const int64_t jobs = (int64_t)s->n * s->cout;
    if (Ho <= 0 || Wo <= 0 || jobs <= 0) return;
#pragma omp parallel for schedule(static)
    for (int64_t job = 0; job < jobs; ++job) {
        const int32_t n = (int32_t)(job / s->cout), oc = (int32_t)(job % s->cout);
        const int32_t g = oc / Cog, ocg = oc % Cog;
        for (int32_t oy = 0; oy < Ho; ++oy)
            for (int32_t ox = 0; ox < Wo; ++ox) {
                double acc = 0;
                const int32_t h_im = oy + s->pad_t, w_im = ox + s->pad_l;
                for (int32_t ky = 0; ky < s->kh; ++ky) {
                    const int32_t t = h_im - ky;
                    if (t < 0 || t % s->stride_h) continue;
                    const int32_t iy = t / s->stride_h;
                    if (iy >= s->h) continue;
                    for (int32_t kx = 0; kx < s->kw; ++kx) {
                        const int32_t u = w_im - kx;
                        if (u < 0 || u % s->stride_w) continue;
                        const int32_t ix = u / s->stride_w;
                        if (ix >= s->w) continue;
                        for (int32_t ic = 0; ic < Cig; ++ic) {
                            const int32_t cin = g * Cig + ic;
                            acc += in[(((int64_t)n * s->c + cin) * s->h + iy) * s->w + ix] *
                                   w[(((int64_t)cin * Cog + ocg) * s->kh + ky) * s->kw + kx];
                        }
                    }
                }
                acc += bias ? bias[oc] : 0;
                out[(job * Ho + oy) * Wo + ox] = acc;
            }
    }
}

static void deconv_core(const uint8_t *in, int in_is_signed, const void *w, int w_is_signed, const int32_t *bias, uint8_t *out,
                        const eo_conv_shape *s, const eo_quant *q, const int32_t *multipliers,
                        const int32_t *shifts, int32_t *acc_out) {
    const int32_t Ho = eo_deconv_out_dim(s->h, s->pad_t, s->pad_b, s->kh, s->stride_h);
    const int32_t Wo = eo_deconv_out_dim(s->w, s->pad_l, s->pad_r, s->kw, s->stride_w);
    const int64_t n_in = (int64_t)s->n * s->c * s->h * s->w;
    const int64_t n_w = (int64_t)s->c * (s->cout / s->groups) * s->kh * s->kw;
    const int64_t n_out = (int64_t)s->n * s->cout * Ho * Wo;
    if (n_out <= 0) return;
    double *din = (double *)malloc(sizeof(double) * (size_t)(n_in > 0 ? n_in : 1));
    double *dw = (double *)malloc(sizeof(double) * (size_t)(n_w > 0 ? n_w : 1));
    double *db = (double *)malloc(sizeof(double) * (size_t)s->cout);
    double *dout = (double *)malloc(sizeof(double) * (size_t)n_out);
    for (int64_t i = 0; i < n_in; ++i)
        din[i] = (double)((in_is_signed ? (int32_t)((const int8_t *)in)[i] : (int32_t)in[i]) - q->zp_in);
    for (int64_t i = 0; i < n_w; ++i)
        dw[i] = (double)((w_is_signed ? (int32_t)((const int8_t *)w)[i] : (int32_t)((const uint8_t *)w)[i]) - q->zp_w);
    for (int32_t i = 0; i < s->cout; ++i) db[i] = bias ? (double)bias[i] : 0.0;
    eo_deconv2d_f64(din, dw, db, dout, s);
    for (int64_t i = 0; i < n_out; ++i) {
        const int32_t acc = (int32_t)dout[i];
        eo_quant ql = *q;
        if (multipliers) {
            const int32_t oc = (int32_t)((i / ((int64_t)Ho * Wo)) % s->cout);
            ql.multiplier = multipliers[oc];
            ql.shift = shifts[oc];
        }
        out[i] = eo_requant(acc, &ql);
        if (acc_out) acc_out[i] = acc;
    }
    free(din);
    free(dw);
    free(db);
    free(dout);
}

void eo_deconv2d_u8(const uint8_t *in, const uint8_t *w, const int32_t *bias, uint8_t *out,
                    const eo_conv_shape *s, const eo_quant *q, int32_t *acc_out) {
    deconv_core(in, 0, w, 0, bias, out, s, q, NULL, NULL, acc_out);
}

/* cl_kernels/DeconvolutionKernels.cpp:200-249 (the gather with the pair of channel
 * get_global_id(0) % channels) over int8 weight bytes (:449-454), driven by
 * cl_optimized_impls/CLDeconvolutionPerChannelQuantized.cpp:147-176. */
void eo_deconv2d_u8_perchannel(const uint8_t *in, const int8_t *w, const int32_t *bias, uint8_t *out,
                               const eo_conv_shape *s, const eo_quant *q,
                               const int32_t *multipliers, const int32_t *shifts, int32_t *acc_out) {
    deconv_core(in, 0, w, 1, bias, out, s, q, multipliers, shifts, acc_out);
}

/* PrecisionType::INT8: int8 input, weight and output bytes, zero points and clamp bounds in [-128, 127] (the
 * SIGNED* kernels: cl_kernels/ConvolutionKernels.cpp SIGNEDquantizedGemmBlocked,
 * cl_kernels/DepthwiseconvolutionKernels.cpp:2410-2450, cl_kernels/DeconvolutionKernels.cpp:340-440).  The
 * arithmetic is the uint8 one on the signed values; `multipliers` may be NULL (per-tensor). */
void eo_conv2d_s8(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out, const eo_conv_shape *s,
                  const eo_quant *q, const int32_t *multipliers, const int32_t *shifts) {
    conv_core((const uint8_t *)in, 1, w, 1, bias, (uint8_t *)out, s, q, multipliers, shifts, NULL);
}

void eo_dwconv2d_s8(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out, const eo_conv_shape *s,
                    const eo_quant *q, const int32_t *multipliers, const int32_t *shifts) {
    dw_core((const uint8_t *)in, 1, w, 1, bias, (uint8_t *)out, s, q, multipliers, shifts, NULL);
}

void eo_deconv2d_s8(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out, const eo_conv_shape *s,
                    const eo_quant *q, const int32_t *multipliers, const int32_t *shifts) {
    deconv_core((const uint8_t *)in, 1, w, 1, bias, (uint8_t *)out, s, q, multipliers, shifts, NULL);
}

void eo_fc_s8(const int8_t *a, const int8_t *w, const int32_t *bias, int8_t *out, int32_t m, int32_t k, int32_t n,
              const eo_quant *q) {
#pragma omp parallel for schedule(static) collapse(2)
    for (int32_t i = 0; i < m; ++i)
        for (int32_t j = 0; j < n; ++j) {
            const int8_t *ar = a + (int64_t)i * k, *wr = w + (int64_t)j * k;
            int32_t acc = 0;
            for (int32_t t = 0; t < k; ++t) acc += ((int32_t)ar[t] - q->zp_in) * ((int32_t)wr[t] - q->zp_w);
            acc += bias ? bias[j] : 0;
            out[(int64_t)i * n + j] = (int8_t)eo_requant(acc, q);
        }
}

/* Scatter form: col = W^T x A (cl_kernels/DeconvolutionKernels.cpp:24-60), then
 * every col entry is added to the output pixel it maps to
 * (src/userdriver/gpu/op_test/deconv_guard.h:77-110). */
void eo_deconv2d_u8_scatter(const uint8_t *in, const uint8_t *w, const int32_t *bias, uint8_t *out,
                            const eo_conv_shape *s, const eo_quant *q, int32_t *acc_out) {
    const int32_t Ho = eo_deconv_out_dim(s->h, s->pad_t, s->pad_b, s->kh, s->stride_h);
    const int32_t Wo = eo_deconv_out_dim(s->w, s->pad_l, s->pad_r, s->kw, s->stride_w);
    const int32_t G = s->groups, Cig = s->c / G, Cog = s->cout / G;
    const int64_t total = (int64_t)s->n * s->cout * Ho * Wo;
    if (Ho <= 0 || Wo <= 0 || total <= 0) return;
    int32_t *acc = (int32_t *)malloc(sizeof(int32_t) * (size_t)total);
    for (int32_t n = 0; n < s->n; ++n)
        for (int32_t oc = 0; oc < s->cout; ++oc) {
            int32_t *p = acc + ((int64_t)n * s->cout + oc) * Ho * Wo;
            for (int64_t i = 0; i < (int64_t)Ho * Wo; ++i) p[i] = bias ? bias[oc] : 0;
        }
    for (int32_t n = 0; n < s->n; ++n)
        for (int32_t g = 0; g < G; ++g)
            for (int32_t ocg = 0; ocg < Cog; ++ocg)
                for (int32_t ky = 0; ky < s->kh; ++ky)
                    for (int32_t kx = 0; kx < s->kw; ++kx)
                        for (int32_t iy = 0; iy < s->h; ++iy)
                            for (int32_t ix = 0; ix < s->w; ++ix) {
                                int32_t col = 0;
                                for (int32_t ic = 0; ic < Cig; ++ic) {
                                    const int32_t cin = g * Cig + ic;
                                    const int32_t av = (int32_t)in[(((int64_t)n * s->c + cin) * s->h + iy) * s->w + ix] - q->zp_in;
                                    const int32_t wv = (int32_t)w[(((int64_t)cin * Cog + ocg) * s->kh + ky) * s->kw + kx] - q->zp_w;
                                    col += wv * av;
                                }
                                const int32_t oy = iy * s->stride_h + ky - s->pad_t;
                                const int32_t ox = ix * s->stride_w + kx - s->pad_l;
                                if (oy < 0 || oy >= Ho || ox < 0 || ox >= Wo) continue;
                                acc[(((int64_t)n * s->cout + g * Cog + ocg) * Ho + oy) * Wo + ox] += col;
                            }
    for (int64_t i = 0; i < total; ++i) out[i] = eo_requant(acc[i], q);
    if (acc_out) memcpy(acc_out, acc, sizeof(int32_t) * (size_t)total);
    free(acc);
}

/* out[n,hw,c] = in[n,c,hw]: src/userdriver/gpu/common/CLKernels.hpp:429-459 */
void eo_nchw2nhwc_u8(const uint8_t *in, uint8_t *out, int32_t n, int32_t c, int32_t h, int32_t w) {
    const int64_t hw = (int64_t)h * w;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < n; ++b)
        for (int64_t p = 0; p < hw; ++p)
            for (int32_t ch = 0; ch < c; ++ch) out[(b * hw + p) * c + ch] = in[(b * c + ch) * hw + p];
}

/* src/userdriver/gpu/common/CLKernels.hpp:461-491 */
void eo_nhwc2nchw_u8(const uint8_t *in, uint8_t *out, int32_t n, int32_t c, int32_t h, int32_t w) {
    const int64_t hw = (int64_t)h * w;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < n; ++b)
        for (int32_t ch = 0; ch < c; ++ch)
            for (int64_t p = 0; p < hw; ++p) out[(b * c + ch) * hw + p] = in[(b * hw + p) * c + ch];
}

/* The hand-optimised kernels compute mul_hi(x << (2+ls), M) then rhadd(., 0)
 * (cl_kernels/DirectConvolutionKernel.cpp:4424-4437,
 * cl_kernels/DepthwiseconvolutionKernels.cpp:2068-2069), i.e.
 * floor((x*2^ls*M + 2^30) / 2^31).  eo_srdhm's nudge-and-truncate is the same
 * function (round half up) for every product, so the two forms differ only
 * where x << (2+ls) leaves int32.  This counts those accumulators. */
int64_t eo_count_fastpath_overflow(const int32_t *acc, int64_t count, const eo_quant *q) {
    const int32_t ls = q->shift > 0 ? q->shift : 0;
    int64_t n = 0;
    for (int64_t i = 0; i < count; ++i) {
        const int64_t v = (int64_t)acc[i] * (1ll << (ls + 2));
        if (v > INT32_MAX || v < INT32_MIN) ++n;
    }
    return n;
}

/* The fast-path high-mul itself, for the equivalence test. */
int32_t eo_srdhm_fastpath(int32_t x_shifted_by_ls, int32_t m) {
    const int32_t x4 = (int32_t)((uint32_t)x_shifted_by_ls << 2);
    const int32_t hi = (int32_t)(((int64_t)x4 * (int64_t)m) >> 32); /* mul_hi */
    return (int32_t)(((int64_t)hi + 1) >> 1);                       /* rhadd(hi, 0) */
}

/* ------------------------------------------------------------------------ */
/* network glue: add, average pool                                          */
/* ------------------------------------------------------------------------ */

/* cl_optimized_impls/CLAddQuantized.cpp:70-115 */
void eo_make_add_quant(float s_a, int32_t zp_a, float s_b, int32_t zp_b, float s_out, int32_t zp_out,
                       int act, int act_enabled, eo_add_quant *q) {
    q->zp_a = zp_a;
    q->zp_b = zp_b;
    q->zp_out = zp_out;
    q->left_shift = 20;
    const float mx = s_a > s_b ? s_a : s_b; /* std::max on floats, then promoted */
    const double twice_max = 2 * (double)mx;
    const double ma = (double)s_a / twice_max, mb = (double)s_b / twice_max;
    const double mo = twice_max / ((double)(1 << q->left_shift) * (double)s_out);
    eo_quantize_multiplier(ma, &q->mult_a, &q->shift_a);
    eo_quantize_multiplier(mb, &q->mult_b, &q->shift_b);
    eo_quantize_multiplier(mo, &q->mult_out, &q->shift_out);
    if (act_enabled) {
        eo_act_range_u8(act, s_out, zp_out, &q->act_min, &q->act_max);
    } else {
        q->act_min = 0;
        q->act_max = 255;
    }
}

/* cl_kernels/AddKernelsQauntized.cpp:135-215.  The kernel leaves a scaled
 * value unset when a shift is positive; shifts here are required to be <= 0
 * (true whenever each multiplier is < 1) and a positive one is treated as 0. */
void eo_add_u8(const uint8_t *a, const uint8_t *b, uint8_t *out, int64_t count, const eo_add_quant *q) {
    const int32_t rsa = q->shift_a < 0 ? -q->shift_a : 0;
    const int32_t rsb = q->shift_b < 0 ? -q->shift_b : 0;
    const int32_t rso = q->shift_out < 0 ? -q->shift_out : 0;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < count; ++i) {
        const int32_t va = ((int32_t)a[i] - q->zp_a) * (1 << q->left_shift);
        const int32_t vb = ((int32_t)b[i] - q->zp_b) * (1 << q->left_shift);
        const int32_t sa = eo_rdivpot(eo_srdhm(va, q->mult_a), rsa);
        const int32_t sb = eo_rdivpot(eo_srdhm(vb, q->mult_b), rsb);
        int32_t r = eo_rdivpot(eo_srdhm(sa + sb, q->mult_out), rso) + q->zp_out;
        if (r < q->act_min) r = q->act_min;
        if (r > q->act_max) r = q->act_max;
        out[i] = (uint8_t)r;
    }
}

/* cl_kernels/AveragepoolKernels.cpp:8-44: window clipped to the image,
 * (sum + n/2) / n, clamp; NCHW. */
void eo_avgpool_u8(const uint8_t *in, uint8_t *out, int32_t n, int32_t c, int32_t h, int32_t w,
                   int32_t kh, int32_t kw, int32_t stride_h, int32_t stride_w,
                   int32_t pad_t, int32_t pad_b, int32_t pad_l, int32_t pad_r,
                   int32_t act_min, int32_t act_max) {
    const int32_t Ho = (h + pad_t + pad_b - kh) / stride_h + 1;
    const int32_t Wo = (w + pad_l + pad_r - kw) / stride_w + 1;
    for (int64_t p = 0; p < (int64_t)n * c; ++p)
        for (int32_t oy = 0; oy < Ho; ++oy)
            for (int32_t ox = 0; ox < Wo; ++ox) {
                int32_t y0 = oy * stride_h - pad_t, x0 = ox * stride_w - pad_l;
                int32_t y1 = y0 + kh < h ? y0 + kh : h, x1 = x0 + kw < w ? x0 + kw : w;
                if (y0 < 0) y0 = 0;
                if (x0 < 0) x0 = 0;
                const int32_t cnt = (y1 - y0) * (x1 - x0);
                int32_t sum = 0;
                for (int32_t y = y0; y < y1; ++y)
                    for (int32_t x = x0; x < x1; ++x) sum += in[(p * h + y) * w + x];
                int32_t v = cnt > 0 ? (sum + cnt / 2) / cnt : 0;
                if (v < act_min) v = act_min;
                if (v > act_max) v = act_max;
                out[(p * Ho + oy) * Wo + ox] = (uint8_t)v;
            }
}

/* cl_kernels/AveragepoolKernels.cpp:8-38 with the int8 rounding of :70-74: the signed sum is rounded half away from
 * zero by C's truncating division. */
void eo_avgpool_s8(const int8_t *in, int8_t *out, int32_t n, int32_t c, int32_t h, int32_t w,
                   int32_t kh, int32_t kw, int32_t stride_h, int32_t stride_w,
                   int32_t pad_t, int32_t pad_b, int32_t pad_l, int32_t pad_r,
                   int32_t act_min, int32_t act_max) {
    const int32_t Ho = (h + pad_t + pad_b - kh) / stride_h + 1;
    const int32_t Wo = (w + pad_l + pad_r - kw) / stride_w + 1;
    for (int64_t p = 0; p < (int64_t)n * c; ++p)
        for (int32_t oy = 0; oy < Ho; ++oy)
            for (int32_t ox = 0; ox < Wo; ++ox) {
                int32_t y0 = oy * stride_h - pad_t, x0 = ox * stride_w - pad_l;
                int32_t y1 = y0 + kh < h ? y0 + kh : h, x1 = x0 + kw < w ? x0 + kw : w;
                if (y0 < 0) y0 = 0;
                if (x0 < 0) x0 = 0;
                const int32_t cnt = (y1 - y0) * (x1 - x0);
                int32_t sum = 0;
                for (int32_t y = y0; y < y1; ++y)
                    for (int32_t x = x0; x < x1; ++x) sum += in[(p * h + y) * w + x];
                int32_t v = 0;
                if (cnt > 0) v = sum > 0 ? (sum + cnt / 2) / cnt : (sum - cnt / 2) / cnt;
                if (v < act_min) v = act_min;
                if (v > act_max) v = act_max;
                out[(p * Ho + oy) * Wo + ox] = (int8_t)v;
            }
}

/* ------------------------------------------------------------------------ */
/* seeded data                                                              */
/* ------------------------------------------------------------------------ */

uint64_t eo_splitmix64(uint64_t seed, uint64_t index) {
    uint64_t z = seed + (index + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

void eo_fill_u8(uint8_t *dst, int64_t count, uint64_t seed, int32_t lo, int32_t hi) {
    const uint64_t span = (uint64_t)(hi - lo + 1);
    for (int64_t i = 0; i < count; ++i) dst[i] = (uint8_t)(lo + (int32_t)((eo_splitmix64(seed, (uint64_t)i) >> 11) % span));
}

void eo_fill_i32(int32_t *dst, int64_t count, uint64_t seed, int32_t lo, int32_t hi) {
    const uint64_t span = (uint64_t)((int64_t)hi - lo + 1);
    for (int64_t i = 0; i < count; ++i) dst[i] = (int32_t)(lo + (int64_t)((eo_splitmix64(seed, (uint64_t)i) >> 11) % span));
}

/* Sum of twelve 16-bit uniforms has mean 6*65535 and variance 65536^2 (to 2e-5):
 * value = mean + round_half_away(sd * (sum - 6*65535) / 65536), clipped to [0,255]. */
void eo_fill_u8_normal(uint8_t *dst, int64_t count, uint64_t seed, int32_t mean, int32_t sd) {
    for (int64_t i = 0; i < count; ++i) {
        int64_t sum = 0;
        for (int t = 0; t < 3; ++t) {
            const uint64_t r = eo_splitmix64(seed, (uint64_t)i * 3 + (uint64_t)t);
            sum += (int64_t)(r & 0xFFFF) + (int64_t)((r >> 16) & 0xFFFF) + (int64_t)((r >> 32) & 0xFFFF) +
                   (int64_t)((r >> 48) & 0xFFFF);
        }
        const int64_t num = (int64_t)sd * (sum - 6 * 65535);
        const int64_t dev = num >= 0 ? (num + 32768) / 65536 : -((-num + 32768) / 65536);
        int64_t v = mean + dev;
        if (v < 0) v = 0;
        if (v > 255) v = 255;
        dst[i] = (uint8_t)v;
    }
}

int eo_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
