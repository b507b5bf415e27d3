/*
 * eden_oracle — CPU restatement of the reference's quantized operator semantics.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (the HIP library, the host
 * operator classes) may link, load or call this file; only tests, the smoke
 * check and the bench's cpu_baseline leg use it, and only as the checker.
 *
 * Every function cites the reference file:line (relative to the reference
 * repository root) whose arithmetic it restates.  Pinning status (what fixes
 * each function independently of this file) is listed per function below.
 *
 *   eo_quantize_multiplier   pinned: closed forms + reference build (oracle/_ref) + golden vectors
 *   eo_conv_multiplier       pinned: reference build + golden vectors
 *   eo_act_range_u8          pinned: closed forms + reference build + golden vectors
 *   eo_srdhm / eo_rdivpot / eo_mbqm
 *                            pinned: identities, 128-bit brute force, vendored gemmlowp build, golden vectors
 *   eo_conv2d_u8             pinned: reference float KATs reused as u8 (scale 1, zp 0), per-channel u8 KAT,
 *                                    brute-force vs fold form, invariants
 *   eo_dwconv2d_u8           pinned: reference KATs, equality with grouped conv (groups == C)
 *   eo_fc_u8                 pinned: reference KAT, equality with 1x1 conv
 *   eo_deconv2d_u8           pinned: reference KATs (integer data), scatter form == gather form,
 *                                    stride-1 deconv == conv with flipped kernel
 *   eo_conv2d_u8_perchannel  pinned: the reference's uint8 per-channel KAT
 *   eo_dwconv2d_u8_perchannel / eo_deconv2d_u8_perchannel
 *                            pinned by reduction: channel c of the result equals channel c of the per-tensor
 *                                    function above run on the weight bytes + 128 with weight zero point + 128
 *                                    and channel c's (multiplier, shift); no reference vector exists for them
 *   eo_act_range_s8          pinned: reference build + golden vectors
 *   eo_conv2d_s8 / eo_dwconv2d_s8 / eo_deconv2d_s8 / eo_fc_s8
 *                            pinned by reduction: the result + 128 equals the uint8 function above on every byte,
 *                                    zero point and clamp bound + 128; no reference vector exists for them
 *   eo_nchw2nhwc_u8 / eo_nhwc2nchw_u8  pinned: round trip + index closed form
 *   eo_add_u8 / eo_avgpool_u8
 *                            no reference vector exists (the reference's add and average-pool tests are float only);
 *                                    pinned by mathematics: every output against exact rational arithmetic over all byte
 *                                    pairs (add) or a sweep of windows, strides and paddings (pool), with mutants of
 *                                    the plausible mistakes (swapped multipliers, a shift off by one; a divisor that
 *                                    counts padded taps, truncation, ties to even) failing the same checks
 *   eo_avgpool_s8            parity unpinned by reference vectors (closed forms and exact rational arithmetic only)
 */
#ifndef EDEN_ORACLE_H_
#define EDEN_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Activation kinds, numbered like ActivationInfo::ActivationType
 * (src/userdriver/common/operator_interfaces/common/ActivationInfo.hpp:5-12). */
enum { EO_ACT_NONE = 0, EO_ACT_RELU = 1, EO_ACT_RELU1 = 2, EO_ACT_RELU6 = 3 };

typedef struct eo_quant {
    int32_t zp_in;      /* input zero point  */
    int32_t zp_w;       /* weight zero point */
    int32_t zp_out;     /* output zero point */
    int32_t multiplier; /* Q31 significand   */
    int32_t shift;      /* >0 left, <0 right */
    int32_t act_min;
    int32_t act_max;
} eo_quant;

typedef struct eo_conv_shape {
    int32_t n, c, h, w;         /* input NCHW dims */
    int32_t cout, kh, kw;
    int32_t stride_h, stride_w;
    int32_t pad_t, pad_b, pad_l, pad_r;
    int32_t dil_h, dil_w;
    int32_t groups;             /* conv: groups; dw: depth multiplier lives in `dm` */
    int32_t dm;                 /* depthwise only */
} eo_conv_shape;

/* host arithmetic */
void    eo_quantize_multiplier(double m, int32_t *q, int32_t *shift);
int     eo_conv_multiplier(float s_in, float s_w, float s_bias, float s_out, double *m);
void    eo_act_range_u8(int act, float scale, int32_t zp, int32_t *amin, int32_t *amax);
void    eo_act_range_s8(int act, float scale, int32_t zp, int32_t *amin, int32_t *amax);
int32_t eo_srdhm(int32_t a, int32_t b);
int32_t eo_rdivpot(int32_t x, int32_t exponent);
int32_t eo_mbqm(int32_t x, int32_t q, int32_t shift);
uint8_t eo_requant(int32_t acc, const eo_quant *q);
/* fill an eo_quant from tensor scales exactly as an operator's execute() does */
void    eo_make_quant(float s_in, int32_t zp_in, float s_w, int32_t zp_w, float s_bias,
                      float s_out, int32_t zp_out, int act, int act_enabled, eo_quant *q);

void    eo_make_quant_s8(float s_in, int32_t zp_in, float s_w, int32_t zp_w, float s_bias,
                         float s_out, int32_t zp_out, int act, int act_enabled, eo_quant *q);

/* output-size formulas */
int32_t eo_conv_out_dim(int32_t in, int32_t pad_a, int32_t pad_b, int32_t k, int32_t dil, int32_t stride);
int32_t eo_deconv_out_dim(int32_t in, int32_t pad_a, int32_t pad_b, int32_t k, int32_t stride);

/* operators; all NCHW.  `acc` (optional, may be NULL) receives the int32
 * accumulator (bias included) of every output element. */
void eo_conv2d_u8(const uint8_t *in, const uint8_t *w, const int32_t *bias, uint8_t *out,
                  const eo_conv_shape *s, const eo_quant *q, int32_t *acc);
void eo_conv2d_u8_perchannel(const uint8_t *in, const int8_t *w, const int32_t *bias, uint8_t *out,
                             const eo_conv_shape *s, const eo_quant *q,
                             const int32_t *multipliers, const int32_t *shifts, int32_t *acc);
void eo_dwconv2d_u8(const uint8_t *in, const uint8_t *w, const int32_t *bias, uint8_t *out,
                    const eo_conv_shape *s, const eo_quant *q, int32_t *acc);
void eo_dwconv2d_u8_perchannel(const uint8_t *in, const int8_t *w, const int32_t *bias, uint8_t *out,
                               const eo_conv_shape *s, const eo_quant *q,
                               const int32_t *multipliers, const int32_t *shifts, int32_t *acc);
void eo_deconv2d_u8_perchannel(const uint8_t *in, const int8_t *w, const int32_t *bias, uint8_t *out,
                               const eo_conv_shape *s, const eo_quant *q,
                               const int32_t *multipliers, const int32_t *shifts, int32_t *acc);
/* INT8 precision: int8 bytes everywhere, parameters in [-128, 127]; multipliers/shifts NULL = per-tensor */
void eo_conv2d_s8(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out, const eo_conv_shape *s,
                  const eo_quant *q, const int32_t *multipliers, const int32_t *shifts);
void eo_dwconv2d_s8(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out, const eo_conv_shape *s,
                    const eo_quant *q, const int32_t *multipliers, const int32_t *shifts);
void eo_deconv2d_s8(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out, const eo_conv_shape *s,
                    const eo_quant *q, const int32_t *multipliers, const int32_t *shifts);
void eo_fc_s8(const int8_t *a, const int8_t *w, const int32_t *bias, int8_t *out, int32_t m, int32_t k, int32_t n,
              const eo_quant *q);
void eo_fc_u8(const uint8_t *a, const uint8_t *w, const int32_t *bias, uint8_t *out,
              int32_t m, int32_t k, int32_t n, const eo_quant *q, int32_t *acc);
/* gather form (each output pixel sums its contributing taps) */
void eo_deconv2d_u8(const uint8_t *in, const uint8_t *w, const int32_t *bias, uint8_t *out,
                    const eo_conv_shape *s, const eo_quant *q, int32_t *acc);
/* the gather form's index math in double precision on zero-point-free data;
 * this is the core eo_deconv2d_u8 runs on */
void eo_deconv2d_f64(const double *in, const double *w, const double *bias, double *out,
                     const eo_conv_shape *s);
/* GEMM + col2im scatter form; must agree with the gather form bit for bit */
void eo_deconv2d_u8_scatter(const uint8_t *in, const uint8_t *w, const int32_t *bias, uint8_t *out,
                            const eo_conv_shape *s, const eo_quant *q, int32_t *acc);

void eo_nchw2nhwc_u8(const uint8_t *in, uint8_t *out, int32_t n, int32_t c, int32_t h, int32_t w);
void eo_nhwc2nchw_u8(const uint8_t *in, uint8_t *out, int32_t n, int32_t c, int32_t h, int32_t w);

/* number of accumulators on which the reference's mul_hi/rhadd fast-path
 * rounding would differ from the exact form: those whose x << (2+ls) overflows
 * int32 (everywhere else the two forms are the same function). */
int64_t eo_count_fastpath_overflow(const int32_t *acc, int64_t count, const eo_quant *q);
int32_t eo_srdhm_fastpath(int32_t x_shifted_by_ls, int32_t m);

/* quantized element-wise add and average pool (network glue) */
typedef struct eo_add_quant {
    int32_t zp_a, zp_b, zp_out;
    int32_t left_shift;
    int32_t mult_a, shift_a, mult_b, shift_b, mult_out, shift_out;
    int32_t act_min, act_max;
} eo_add_quant;
void eo_make_add_quant(float s_a, int32_t zp_a, float s_b, int32_t zp_b, float s_out, int32_t zp_out,
                       int act, int act_enabled, eo_add_quant *q);
void eo_add_u8(const uint8_t *a, const uint8_t *b, uint8_t *out, int64_t count, const eo_add_quant *q);
void eo_avgpool_u8(const uint8_t *in, uint8_t *out, int32_t n, int32_t c, int32_t h, int32_t w,
                   int32_t kh, int32_t kw, int32_t stride_h, int32_t stride_w,
                   int32_t pad_t, int32_t pad_b, int32_t pad_l, int32_t pad_r,
                   int32_t act_min, int32_t act_max);
void eo_avgpool_s8(const int8_t *in, int8_t *out, int32_t n, int32_t c, int32_t h, int32_t w,
                   int32_t kh, int32_t kw, int32_t stride_h, int32_t stride_w,
                   int32_t pad_t, int32_t pad_b, int32_t pad_l, int32_t pad_r,
                   int32_t act_min, int32_t act_max);

/* seeded integer generator shared by every harness (SplitMix64, counter based) */
uint64_t eo_splitmix64(uint64_t seed, uint64_t index);
void eo_fill_u8(uint8_t *dst, int64_t count, uint64_t seed, int32_t lo, int32_t hi);
void eo_fill_i32(int32_t *dst, int64_t count, uint64_t seed, int32_t lo, int32_t hi);
/* clip(round(N(mean, sd)), 0, 255) by a 12-term Irwin–Hall sum in integer arithmetic */
void eo_fill_u8_normal(uint8_t *dst, int64_t count, uint64_t seed, int32_t mean, int32_t sd);

int eo_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif /* EDEN_ORACLE_H_ */
