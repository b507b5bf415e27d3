/*
 * eden_hip.h — C ABI of the MI355X (gfx950) backend for the quantized operator
 * path of the EDEN/ENN userdriver: Convolution, DepthwiseConvolution,
 * FullyConnected and Deconvolution on asymmetric uint8 tensors with int32 bias
 * and fixed-point requantization, plus layout conversion and device buffers.
 *
 * The reference has no C ABI: its operator classes call the OpenCL runtime
 * directly.  Each entry point below names the reference interface it stands in
 * for (paths relative to the reference repository root).  The C++ operator
 * classes under cl-eden-kernel_amd/host/ are the only intended callers.
 *
 * Conventions: every function returns EH_OK (0) or a negative eh_status; no
 * exceptions and no C++ types cross this boundary; device pointers are plain
 * `void *` owned by the caller unless a plan allocated them; `stream` is a
 * hipStream_t passed as `void *` (NULL = the default stream); all launches are
 * asynchronous on that stream.  eh_last_error() gives the text of the last
 * failure on the calling thread.
 */
#ifndef EDEN_HIP_H_
#define EDEN_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum eh_status {
    EH_OK = 0,
    EH_FAILURE = -1,        /* Status::FAILURE        (operator_interfaces/common/Common.hpp:113-119) */
    EH_DEVICE_FAILURE = -2, /* Status::CL_FAILURE: the device runtime reported an error               */
    EH_INVALID_PARAMS = -3  /* Status::INVALID_PARAMS                                                  */
} eh_status;

/* ActivationInfo::ActivationType (operator_interfaces/common/ActivationInfo.hpp:5-12) */
typedef enum eh_activation { EH_ACT_NONE = 0, EH_ACT_RELU = 1, EH_ACT_RELU1 = 2, EH_ACT_RELU6 = 3 } eh_activation;

/* DataOrder (operator_interfaces/common/Common.hpp:20-25) */
typedef enum eh_layout { EH_NCHW = 0, EH_NHWC = 1 } eh_layout;

/* Weight element order.  OIHW is the reference's default [Cout][Cin/g][kh][kw];
 * OHWI is its androidNN order [Cout][kh][kw][Cin/g] (deconvolution: groups == 1 only)
 * (gpu/operators/cl_optimized_impls/CLDeconvolutionQuantized.cpp:39-46), for a depthwise
 * convolution [1][kh][kw][C*dm] (gpu/operators/CLDepthwiseConvolution.cpp:128-131,146);
 * IOHW is the deconvolution order [Cin][Cout/g][kh][kw] (gpu/op_test/deconv_guard.h:53-69). */
typedef enum eh_weight_layout { EH_W_OIHW = 0, EH_W_OHWI = 1, EH_W_IOHW = 2 } eh_weight_layout;
/* Or-ed into eh_conv_desc.weight_layout (convolution, depthwise convolution, deconvolution): the weight
 * bytes are int8 values, as the per-channel quantized operators take them
 * (CLConvolutionPerChannelQuantized.cpp:73-159, cl_kernels/DepthwiseconvolutionKernels.cpp:2323-2340,
 * cl_kernels/DeconvolutionKernels.cpp:449-454);
 * eh_requant.zp_w is then an int8 zero point in [-128, 127] (0 in the reference). */
#define EH_W_SIGNED 0x100
/* Or-ed into eh_conv_desc.layout: the input and output tensors hold int8 values (PrecisionType::INT8: the
 * SIGNED* kernels, e.g. gpu/operators/cl_optimized_impls/CLGEMMConvolutionQuantized.cpp:47,110-114,226-241);
 * eh_requant.zp_in, zp_out, act_min and act_max are then int8 values in [-128, 127].  The reference pairs this
 * precision with int8 weights (EH_W_SIGNED); the two flags are independent here. */
#define EH_IO_SIGNED 0x200
/* Or-ed into eh_conv_desc.layout (convolution, deconvolution) or into eh_fc_q8_plan's flags: keep the plan from staging
 * a channel-padded copy of its input.  Without the flag, a plan whose channels per group (a fully connected layer's row
 * length) are no multiple of 16 and fit none of the kernels for few channels copies the input, on every run, into an
 * image of its own with each group padded to the next multiple of 16 (the role of the reference's pad-and-align pass,
 * gpu/operators/cl_kernels/PadConvertKernels.cpp:25-167) and runs the wide-load kernels on that; with it, the
 * byte-gathering kernel reads the caller's tensor directly: several times slower, no staging memory.  The flag also
 * keeps convolution groups of fewer than 16 channels as one problem per group; without it neighbouring groups run in
 * bundles as block-diagonal problems over 16 to 64 adjacent channels, for which the plan keeps a copy of the
 * weights (it packs them again when a run brings another weight zero point).  A depthwise plan with a depth
 * multiplier or output channels off the multiples of 4 (channels-last), or planar tensors (multiplier 1, channels a
 * multiple of 4), likewise owns staging images (the input with every channel repeated and the pixels' tails padded, the
 * result at the padded width; the two transposed tensors) unless the flag is set, which keeps it on the
 * one-output-per-thread kernel.  Results are the same bytes either way. */
#define EH_EXACT_CHANNELS 0x400

/* Integer requantization parameters of one operator execution: what
 * CLGEMMConvolutionQuantized::execute derives from its tensors
 * (gpu/operators/cl_optimized_impls/CLGEMMConvolutionQuantized.cpp:137-171). */
typedef struct eh_requant {
    int32_t zp_in;      /* input tensor zero point, 0..255  */
    int32_t zp_w;       /* weight tensor zero point, 0..255 */
    int32_t zp_out;     /* output tensor zero point         */
    int32_t multiplier; /* Q31 significand, >= 0            */
    int32_t shift;      /* > 0 left shift, < 0 right shift  */
    int32_t act_min;    /* clamp range in the quantized domain */
    int32_t act_max;
} eh_requant;

/* Parameters of a quantized element-wise add: what CLAddQuantized::execute derives
 * from its three tensors (gpu/operators/cl_optimized_impls/CLAddQuantized.cpp:70-115). */
typedef struct eh_add_requant {
    int32_t zp_a, zp_b, zp_out;
    int32_t left_shift;           /* 20 */
    int32_t mult_a, shift_a;      /* scale_a / (2 max(scale_a, scale_b)) */
    int32_t mult_b, shift_b;
    int32_t mult_out, shift_out;  /* 2 max(scale_a, scale_b) / (2^left_shift scale_out) */
    int32_t act_min, act_max;
} eh_add_requant;

/* Geometry of an average pool (Pool2DParameters, gpu/common/CLParameter.hpp:25-34);
 * the clamp range is what CLAveragepool::averagepool_quant derives from the output
 * tensor (gpu/operators/CLAveragepool.cpp:175-198), see eh_act_range_u8. */
typedef struct eh_pool_desc {
    int32_t n, c, h, w;
    int32_t kh, kw, stride_h, stride_w;
    int32_t pad_t, pad_b, pad_l, pad_r;
    int32_t layout;               /* EH_NCHW or EH_NHWC, input and output alike */
    int32_t act_min, act_max;
} eh_pool_desc;

/* Geometry of a convolution-like operator.  Input dims are (n, c, h, w) whatever
 * the memory order; `layout` says how input and output bytes are ordered.
 * Mirrors ConvolutionParameters / DepthwiseConvolutionParameters /
 * DeconvolutionParameters (gpu/operators/CLConvolution.hpp:31-44,
 * CLDepthwiseConvolution.hpp:18-29, CLDeconvolution.hpp:20-31).
 * Limits the plan calls check (EH_ERR_UNSUPPORTED beyond them): every tensor below 2 GiB, kernel extents times
 * dilation below 32000, and reductions (c * kh * kw; k of a fully connected layer) of at most 2^24 terms. */
typedef struct eh_conv_desc {
    int32_t n, c, h, w;
    int32_t cout;
    int32_t kh, kw;
    int32_t stride_h, stride_w;
    int32_t pad_t, pad_b, pad_l, pad_r;
    int32_t dil_h, dil_w;
    int32_t groups;           /* convolution / deconvolution */
    int32_t depth_multiplier; /* depthwise only              */
    int32_t layout;           /* eh_layout of input and output */
    int32_t weight_layout;    /* eh_weight_layout              */
} eh_conv_desc;

/* ---- host arithmetic (pure CPU, usable without a GPU) ------------------- */

/* QuantizeMultiplier (gpu/operators/cl_quantized_utils/QuantizationUtil.cpp:8-21) */
void eh_quantize_multiplier(double real_multiplier, int32_t *quantized_multiplier, int32_t *shift);
/* GetQuantizedConvolutionMultipler (gpu/operators/cl_quantized_utils/KernelUtil.cpp:7-25):
 * EH_FAILURE leaves *multiplier untouched. */
int eh_conv_multiplier(float input_scale, float filter_scale, float bias_scale, float output_scale, double *multiplier);
/* CalculateActivationRangeUint8 (gpu/operators/cl_quantized_utils/KernelUtil.cpp:27-60) */
void eh_act_range_u8(int activation, float scale, int32_t zero_point, int32_t *act_min, int32_t *act_max);
/* CalculateActivationRangeInt8 (gpu/operators/cl_quantized_utils/KernelUtil.cpp:62-71) */
void eh_act_range_s8(int activation, float scale, int32_t zero_point, int32_t *act_min, int32_t *act_max);
/* The whole derivation an operator's execute() performs, including the
 * reference's behaviour of continuing with multiplier 0 when the bias scale
 * does not match (CLGEMMConvolutionQuantized.cpp:163-166). */
void eh_make_requant(float input_scale, int32_t input_zp, float filter_scale, int32_t filter_zp, float bias_scale,
                     float output_scale, int32_t output_zp, int activation, int activation_enabled, eh_requant *out);
/* The same for PrecisionType::INT8 (EH_IO_SIGNED plans): range [-128, 127] or CalculateActivationRangeInt8
 * (gpu/operators/cl_optimized_impls/CLGEMMConvolutionQuantized.cpp:224-241). */
void eh_make_requant_s8(float input_scale, int32_t input_zp, float filter_scale, int32_t filter_zp, float bias_scale,
                        float output_scale, int32_t output_zp, int activation, int activation_enabled, eh_requant *out);
/* The requantization every kernel epilogue applies to an int32 accumulator (bias
 * and zero-point terms already added): MultiplyByQuantizedMultiplier, output
 * zero point, activation clamp (gpu/common/CLKernels.hpp:120-170), evaluated on
 * the host with the same source the kernels compile.  form 0 evaluates it the
 * way the kernels would for these parameters (a single 64-bit multiply-add and
 * shift where that is exact, *single_shift reports which), form 1 always takes
 * the two-step reference order.  Forms 2 and 3 are the single-shift forms the
 * kernels use with one multiplier and shift per channel (conv_per_channel_quantized,
 * gpu/operators/cl_kernels/ConvolutionKernels.cpp:1317-1375), q's pair standing for
 * the channel's: 2 with the rounding term computed from the shift (-20 <= shift <= -1),
 * 3 with it taken from a per-channel table (-20 <= shift <= -2); parameters outside
 * those ranges are an error, as the kernels then take the two-step order.  Form 4 is
 * the per-tensor single-shift form as the kernels' epilogues evaluate it: four accumulators
 * at a time, the clamp applied before the shift, and a row term (here a value that varies
 * with the group of four) kept out of the accumulators and folded into the rounding term. */
int eh_requant_apply(const eh_requant *q, const int32_t *acc, uint8_t *out, int64_t count, int32_t form,
                     int32_t *single_shift);
/* What CLConvolutionPerChannelQuantized::execute derives (CLConvolutionPerChannelQuantized.cpp:88-121):
 * one (multiplier, shift) per output channel from input_scale * filter_scales[i] / output_scale, and
 * the clamp range; out->multiplier / out->shift are unused in per-channel mode. */
void eh_make_requant_perchannel(float input_scale, int32_t input_zp, const float *filter_scales, int32_t channels,
                                float output_scale, int32_t output_zp, int activation, int activation_enabled, eh_requant *out,
                                int32_t *multipliers, int32_t *shifts);
/* output extents: CLConvolution.cpp:99-104 and CLDeconvolution.cpp:82-87 */
int32_t eh_conv_out_dim(int32_t in, int32_t pad_a, int32_t pad_b, int32_t kernel, int32_t dilation, int32_t stride);
int32_t eh_deconv_out_dim(int32_t in, int32_t pad_a, int32_t pad_b, int32_t kernel, int32_t stride);

/* ---- runtime and device buffers ------------------------------------------
 * Stand in for CLRuntime::initialize / allocBuffer / releaseBuffer /
 * writeBuffer / readBuffer / copyBuffer and clFinish
 * (gpu/common/CLRuntime.cpp:1339-1372,1409-1416; CLRuntime.hpp:59-110). */
int eh_init(int device);
int eh_device_name(char *dst, size_t cap);
int eh_malloc(void **ptr, size_t bytes);             /* zero-initialised, 256-byte aligned */
int eh_free(void *ptr);
int eh_memset(void *ptr, int value, size_t bytes, void *stream);
int eh_h2d(void *dst, const void *src, size_t bytes, void *stream);
int eh_d2h(void *dst, const void *src, size_t bytes, void *stream);
int eh_d2d(void *dst, const void *src, size_t bytes, void *stream);
int eh_stream_create(void **stream);                 /* default priority, non-blocking w.r.t. the null stream */
int eh_stream_destroy(void *stream);
int eh_stream_sync(void *stream);
const char *eh_last_error(void);

/* Pooled buffers of an operator list: CLRuntime::getBuffer with BufferType INTER_SHARED_NEW / INTER_SHARED_REUSE /
 * INTRA_SHARED, resetInterBuffer, resetIntraBuffer and assignBufferPool (gpu/common/CLRuntime.cpp:34-157), as the
 * operator constructor drives them (gpu/gpu_op_constructor.cc:2157-2191: an operator's outputs are requested with
 * REUSE before the inputs it reads last are handed back).  A request returns a slot, sized but without memory;
 * eh_pool_assign lays every slot requested since the last assignment out in ONE device allocation (each at a
 * 1024-byte aligned address with the reference's 1024 bytes of slack in front and 32 behind, zero-filled) and, as the
 * reference does, forgets the pools: later requests collect the next list.  eh_pool_layout reports what an
 * assignment would allocate without allocating; eh_pool_slot gives a slot's address (null before its assignment)
 * and final size; eh_pool_release is releaseBuffer for a pooled buffer (the allocation is freed with its last
 * slot); eh_pool_destroy frees whatever is left.  Not thread-safe: one builder at a time, as under the reference's
 * constructor mutex. */
typedef struct eh_pool eh_pool;
typedef enum eh_pool_kind { EH_POOL_INTER_NEW = 0, EH_POOL_INTER_REUSE = 1, EH_POOL_INTRA = 2 } eh_pool_kind;
int eh_pool_create(eh_pool **pool);
int eh_pool_request(eh_pool *pool, int kind, size_t bytes, int32_t *slot);
int eh_pool_reset_inter(eh_pool *pool, int32_t slot);
int eh_pool_reset_intra(eh_pool *pool);
int eh_pool_layout(eh_pool *pool, size_t *arena_bytes, int32_t *slot_count);
int eh_pool_assign(eh_pool *pool, size_t *arena_bytes);
int eh_pool_slot(const eh_pool *pool, int32_t slot, void **ptr, size_t *bytes);
int eh_pool_release(eh_pool *pool, int32_t slot);
int eh_pool_destroy(eh_pool *pool);

/* Replay of a fixed launch sequence.  The reference submits a whole subgraph to
 * one in-order queue and flushes once (gpu/gpu_userdriver.cc:78-112); on HIP the
 * same sequence is captured once and replayed as a graph, which removes the
 * per-kernel launch cost of short layers.  Capture needs a stream made by
 * eh_stream_create; only `*_run` and the transposes may be called between
 * begin and end (no allocation, no plan creation, no eh_memset). */
int eh_graph_begin(void *stream);
int eh_graph_end(void *stream, void **graph);
int eh_graph_launch(void *graph, void *stream);
int eh_graph_destroy(void *graph);

/* ---- machine probe -----------------------------------------------------------
 * Sustained rate (TOP/s, 1 op = 1 multiply or 1 add) of v_mfma_i32_32x32x32_i8 issued
 * from registers on every SIMD of the device, with constant operands or with operands
 * whose bits toggle like data (the clock the device sustains differs).  The measured
 * ceiling the benchmark prints beside the published peak; no counterpart in the
 * reference.  Synchronous; allocates and frees a small device buffer. */
int eh_probe_mfma_i8(int32_t iterations, int32_t toggling_operands, double *tops);
/* What a CU's matrix pipe can be fed with: `workgroups` workgroups of four waves repeat an iteration of so many matrix
 * instructions, 16-byte-per-lane LDS fragment reads, 1 KiB direct-to-LDS loads from an L2-resident region and 1 KiB
 * loads into registers per wave (returned in per_iteration[0..3], may be NULL), in the proportions of a GEMM tile's
 * inner loop.  mix: 0 direct-to-LDS loads alone, 1 fragment reads alone, 2 matrix instructions alone, 3 the 128x128
 * tile, 4 the 64x64 split-reduction tile, 5 256x128, 6 256x256, 7 / 8 the 128x128 / 256x256 tile with the weight
 * operand loaded straight into registers.  Returns the nanoseconds one iteration takes (all workgroups in parallel).
 * A yardstick like eh_probe_mfma_i8; no counterpart in the reference.  Synchronous; allocates and frees 8 MiB. */
int eh_probe_feed(int32_t mix, int32_t workgroups, int32_t iterations, double *ns_per_iteration, int32_t *per_iteration);
/* A kernel that only moves bytes (16 per lane, whole lines per wave), launched on `stream`:
 * the yardstick beside the HBM-bound kernels' figures.  mode 0 copies out_bytes; mode 1
 * writes every 16-byte source chunk six times (reads out_bytes / 6: the ratio of a 24 -> 144
 * pointwise layer); mode 2 folds four source chunks into each written one (reads
 * 4 * out_bytes: the ratio of a stride-2 depthwise layer).  No counterpart in the reference. */
int eh_probe_stream(const void *src, void *dst, int64_t out_bytes, int32_t mode, void *stream);

/* ---- layout conversion -----------------------------------------------------
 * nchw2nhwc_uint8 / nhwc2nchw_uint8 (gpu/common/CLKernels.hpp:429-491) as
 * driven by CLRuntime::NCHW2NHWC / NHWC2NCHW (gpu/common/CLRuntime.cpp:1477-1619). */
int eh_transpose_u8_nchw2nhwc(const void *src, void *dst, int32_t n, int32_t c, int32_t h, int32_t w, void *stream);
int eh_transpose_u8_nhwc2nchw(const void *src, void *dst, int32_t n, int32_t c, int32_t h, int32_t w, void *stream);

/* ---- element-wise add and average pool --------------------------------------
 * The two operators between the convolutions of a quantized residual network.
 * eh_make_add_requant is host arithmetic (CLAddQuantized.cpp:70-115); eh_add_u8 is
 * the quantized add kernel (gpu/operators/cl_kernels/AddKernelsQauntized.cpp:135-215)
 * over `count` bytes of two equally shaped tensors; eh_avgpool_u8 is
 * avepooling_tflite_INT8 (gpu/operators/cl_kernels/AveragepoolKernels.cpp:8-44):
 * windows clipped to the image, (sum + count / 2) / count, clamp; with EH_IO_SIGNED or-ed into
 * eh_pool_desc.layout it is SIGNEDavepooling_tflite_INT8 (:64-85): int8 bytes, a clamp range within
 * [-128, 127], the signed mean rounded half away from zero.  The int8 Add of the reference
 * (SIGNEDeltwiseAddQuantized, AddKernelsQauntized.cpp:97-127) is a float kernel and is not offered.  Both are
 * asynchronous on `stream` and may be captured in a graph. */
void eh_make_add_requant(float scale_a, int32_t zp_a, float scale_b, int32_t zp_b, float scale_out, int32_t zp_out,
                         int activation, int activation_enabled, eh_add_requant *out);
int eh_add_u8(const void *a, const void *b, void *out, int64_t count, const eh_add_requant *q, void *stream);
int eh_avgpool_u8(const void *in, void *out, const eh_pool_desc *desc, void *stream);

/* ---- operators -------------------------------------------------------------
 * A plan owns everything initialize() prepares once: packed int8 weights, the
 * bias with the zero-point terms folded in, and scratch.  `*_plan` reads the
 * weights and bias from device memory on `stream`; `*_run` enqueues one
 * execution.  Passing a requant whose zero points differ from the plan's
 * re-folds the bias first (the reference reads quantization parameters from
 * the tensors on every execute).  `*_repack` is the weights-as-input case:
 * the reference re-packs non-constant weights on every execute.
 *
 * A plan belongs to ONE stream at a time, like the reference's operators on their single in-order queue: the
 * re-fold and re-pack rewrite the plan's own device arrays in stream order, so work queued on another stream, or a
 * captured graph, that still uses the plan must have finished (or must never be replayed again) before a `*_run`
 * with other zero points, a `*_repack` or a `*_set_perchannel` on it.  In particular the zero points (and, in
 * per-channel mode, the pairs) a plan was captured with have to stay the same for as long as the graph is replayed:
 * `*_run` bakes them into the kernel arguments it records, while the folded bias they must match lives in the plan. */
typedef struct eh_conv_plan eh_conv_plan;
typedef struct eh_dwconv_plan eh_dwconv_plan;
typedef struct eh_fc_plan eh_fc_plan;
typedef struct eh_deconv_plan eh_deconv_plan;

/* CLConvolution::initialize / execute / release, uint8 branch
 * (gpu/operators/CLConvolution.cpp:139-218,458-550) with the work of
 * CLGEMMConvolutionQuantized and CLQuantizedDirectConvolution
 * (gpu/operators/cl_optimized_impls/CLGEMMConvolutionQuantized.cpp:33-280,
 * CLQuantizedDirectConvolution.cpp:30-249) and their kernels. */
int eh_conv2d_u8_plan(eh_conv_plan **plan, const eh_conv_desc *desc, const void *weight, const void *bias,
                      const eh_requant *q, void *stream);
/* Which kernel family a plan made from `desc` would run, one eh_kernel_id per part (convolution group;
 * deconvolution output phase and group), without a GPU: the choice CLConvolution::initialize makes among its
 * implementations (gpu/operators/CLConvolution.cpp:139-218).  Writes at most `cap` ids, returns the number of
 * parts or a negative eh_status. */
typedef enum eh_kernel_id {
    EH_KERNEL_STAGED = 0,         /* register-staged implicit GEMM, any channel count               */
    EH_KERNEL_DMA_256x128 = 1,    /* direct-to-LDS implicit GEMM tiles                              */
    EH_KERNEL_DMA_128x128 = 2,
    EH_KERNEL_DMA_128x64 = 3,
    EH_KERNEL_DMA_64x64_SPLITK = 4,
    EH_KERNEL_DMA_256x256 = 5,
    EH_KERNEL_ONE_TAP = 6,        /* 1x1 problems with short reductions or few pixels               */
    EH_KERNEL_C3K3 = 7,           /* 3x3 on three input channels (first layers)                     */
    EH_KERNEL_CONV3X3_PATCH = 8,  /* 3x3, stride 1: input patch staged in LDS once                  */
    EH_KERNEL_FEW_CHANNEL_ROWS = 9, /* 1 - 4 input channels, 3 - 11 kernel rows of at most 32 bytes  */
    EH_KERNEL_SKINNY = 10         /* one tap, at most 64 output pixels, reductions beyond 256 bytes */
} eh_kernel_id;
int eh_conv2d_u8_kernels(const eh_conv_desc *desc, int32_t *kernel_ids, int32_t cap);
int eh_deconv2d_u8_kernels(const eh_conv_desc *desc, int32_t *kernel_ids, int32_t cap);
/* Per-channel mode (conv_per_channel_quantized, gpu/operators/cl_kernels/ConvolutionKernels.cpp:1317-1375):
 * `count` == cout host arrays of multipliers and shifts replace the requant's single pair on every
 * following run; two null pointers return to per-tensor mode.  Copies synchronously. */
int eh_conv2d_u8_set_perchannel(eh_conv_plan *plan, const int32_t *multipliers, const int32_t *shifts, int32_t count,
                                void *stream);
int eh_conv2d_u8_repack(eh_conv_plan *plan, const void *weight, const void *bias, const eh_requant *q, void *stream);
int eh_conv2d_u8_run(eh_conv_plan *plan, const void *input, void *output, const eh_requant *q, void *stream);
/* eh_conv2d_u8_run for callers that must not allocate (code under graph capture, tight serving loops, harnesses
 * that forbid it): no counterpart in the reference.  Calls no hipMalloc / hipFree and allocates no host memory.  A
 * planar (EH_NCHW) plan computes channels-last between two layout conversions; here the two channels-last staging
 * images live in a static device array of EH_STATIC_SCRATCH_BYTES that each GPU holds from the moment the library
 * is loaded on it, instead of in the plan's own buffers; so does the channel-padded copy of the input that a plan
 * with a channel count off the multiples of 16 reads (see EH_EXACT_CHANNELS).  Any other EH_NHWC plan needs no staging
 * and runs as eh_conv2d_u8_run does.  Fails with EH_INVALID_PARAMS, launching nothing, when the staging
 * (planar: n*c*h*w + n*cout*ho*wo bytes; padded: n*h*w*groups*ceil16(c/groups); each rounded up to 256 plus 256)
 * exceeds the array or the plan runs as more than 8 problems (groups, slices of a long reduction).  What a plan
 * allocated when it was made (packed weights, the int32 image of a sliced reduction) stays the plan's.  Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU (two streams, two
 * threads) race; calls ordered on one stream do not.  Results are bit for bit those of eh_conv2d_u8_run.  The first
 * launch of a persistent-grid kernel variant (the one-tap and the few-channel first-layer kernels) at a given LDS size
 * asks the driver once how many of its workgroups a CU holds
 * (an occupancy query: no allocation, no stream operation, legal under capture); every later launch reads the cached
 * answer. */
#define EH_STATIC_SCRATCH_BYTES (32u << 20)
int eh_conv2d_u8_run_static(eh_conv_plan *plan, const void *input, void *output, const eh_requant *q, void *stream);
/* Convolution followed by the quantized residual add, output = add(residual, convolution) with `aq` as eh_add_u8
 * applies it (the residual is the add's first operand; it has the output's shape and layout and must not be the
 * output buffer).  Bit for bit what eh_conv2d_u8_run into a temporary followed by eh_add_u8 gives; the one-tap and
 * split-reduction GEMM kernels add in their epilogue, other kernels run the add as a second launch in place.  No
 * counterpart in the reference, whose operator list runs CLConvolution and CLAdd one after the other
 * (gpu/gpu_op_executor.cc:56-103); offered for uint8 tensors only. */
int eh_conv2d_u8_run_add(eh_conv_plan *plan, const void *input, const void *residual, void *output, const eh_requant *q,
                         const eh_add_requant *aq, void *stream);
/* 1 when eh_conv2d_u8_run_add on this plan is a single launch (the add happens in the kernel's epilogue), else 0 */
int eh_conv2d_u8_fuses_add(const eh_conv_plan *plan);
int eh_conv2d_u8_destroy(eh_conv_plan *plan);

/* CLDepthwiseConvolution::initialize / execute / release, uint8 branch
 * (gpu/operators/CLDepthwiseConvolution.cpp:88-200,388-425;
 * cl_optimized_impls/CLDepthwiseConvolutionQuantized.cpp:82-674). */
int eh_dwconv2d_u8_plan(eh_dwconv_plan **plan, const eh_conv_desc *desc, const void *weight, const void *bias,
                        const eh_requant *q, void *stream);
/* Per-channel mode of the depthwise convolution
 * (cl_optimized_impls/CLDepthwiseConvolutionPerChannelQuantized.cpp:133-153,
 * cl_kernels/DepthwiseconvolutionKernels.cpp:1323-1371); arguments as eh_conv2d_u8_set_perchannel. */
int eh_dwconv2d_u8_set_perchannel(eh_dwconv_plan *plan, const int32_t *multipliers, const int32_t *shifts, int32_t count,
                                  void *stream);
int eh_dwconv2d_u8_repack(eh_dwconv_plan *plan, const void *weight, const void *bias, const eh_requant *q, void *stream);
int eh_dwconv2d_u8_run(eh_dwconv_plan *plan, const void *input, void *output, const eh_requant *q, void *stream);
int eh_dwconv2d_u8_destroy(eh_dwconv_plan *plan);

/* A pointwise (1x1) convolution followed by a 3x3 depthwise convolution on its output, as ONE launch: the expanded
 * tensor between them lives in LDS only (an output tile's rows plus their halo are computed per workgroup, the halo
 * rows twice).  Bit for bit what eh_conv2d_u8_run into a temporary followed by eh_dwconv2d_u8_run gives.  No counterpart
 * in the reference, whose operator list runs CLConvolution and CLDepthwiseConvolution one after the other
 * (gpu/gpu_op_executor.cc:56-103), the expanded tensor written by quantizedGemmBlocked and read back by
 * depthwise_conv_3x3s2_pad_merge (cl_kernels/DepthwiseconvolutionKernels.cpp:1964-2083).  Takes the two operators' own
 * plans; `_applies` says whether the pair fits (1) or has to run as two launches (0): channels-last uint8 tensors, a
 * pointwise layer of at most 256 input channels (a multiple of 8) whose output is the depthwise input, depthwise 3x3 at
 * stride 1 or 2 without dilation or depth multiplier on a multiple of 16 channels, requantization per tensor in both or per channel in both.
 * `_preferred` says whether the one launch is also the faster choice for the pair's shape (1) or the two launches
 * are (0): below 32 images per launch every fitting pair (a launch is mostly latency there, and a whole network
 * measured faster with all of them fused at every batch from 1 to 24); from 32 images on a table of shapes timed
 * inside a network, kept beside the kernel: a caller that fuses wherever `_preferred` says so never loses to the
 * two launches on a measured shape, and unmeasured shapes stay unfused.
 * rows_per_tile, cols_per_tile: the tile of output pixels a workgroup owns, 0 lets the library choose.
 * q_pointwise->zp_out must equal q_depthwise->zp_in (they describe the same tensor). */
int eh_conv_dw_block_applies(const eh_conv_plan *pointwise, const eh_dwconv_plan *depthwise);
int eh_conv_dw_block_preferred(const eh_conv_plan *pointwise, const eh_dwconv_plan *depthwise);
/* The table alone, for a caller that has to decide before the plans exist (an operator constructor that does not
 * give the expanded tensor any storage): images per launch, the square image's extent, pointwise input channels,
 * expanded channels, depthwise stride.  `_preferred` is `_applies` and this (below 32 images it is 1 for every
 * shape: whether the pair fits is `_applies`' business). */
int eh_conv_dw_block_listed(int32_t images, int32_t image_h, int32_t image_w, int32_t in_channels, int32_t expanded_channels, int32_t stride);
int eh_conv_dw_block_run(eh_conv_plan *pointwise, eh_dwconv_plan *depthwise, const void *input, void *output,
                         const eh_requant *q_pointwise, const eh_requant *q_depthwise, int32_t rows_per_tile, int32_t cols_per_tile,
                         void *stream);

/* CLFullyConnected::initialize / execute / release (gpu/operators/CLFullyConnected.cpp:22-150):
 * input [m][k], weight [n][k], bias [n], output [m][n]
 * (gpu/op_test/fullyconnected_test.cpp:93-105), computed in the convolution's
 * integer pipeline rather than the reference's float detour. */
int eh_fc_u8_plan(eh_fc_plan **plan, int32_t m, int32_t k, int32_t n, const void *weight, const void *bias,
                  const eh_requant *q, void *stream);
/* The same with `flags` = any of EH_W_SIGNED | EH_IO_SIGNED: int8 weights and/or int8 input and output
 * (PrecisionType::INT8 takes the quantized path too, cl_optimized_impls/CLBaseFullyConnected.cpp:88,147-148). */
int eh_fc_q8_plan(eh_fc_plan **plan, int32_t m, int32_t k, int32_t n, int32_t flags, const void *weight, const void *bias,
                  const eh_requant *q, void *stream);
int eh_fc_u8_repack(eh_fc_plan *plan, const void *weight, const void *bias, const eh_requant *q, void *stream);
int eh_fc_u8_run(eh_fc_plan *plan, const void *input, void *output, const eh_requant *q, void *stream);
int eh_fc_u8_destroy(eh_fc_plan *plan);

/* CLDeconvolution::initialize / execute / release, uint8 branch
 * (gpu/operators/CLDeconvolution.cpp:36-272;
 * cl_optimized_impls/CLDeconvolutionQuantized.cpp:18-288).  Output extent is
 * in*stride + k - stride - pads. */
int eh_deconv2d_u8_plan(eh_deconv_plan **plan, const eh_conv_desc *desc, const void *weight, const void *bias,
                        const eh_requant *q, void *stream);
/* Per-channel mode of the deconvolution
 * (cl_optimized_impls/CLDeconvolutionPerChannelQuantized.cpp:147-176,
 * cl_kernels/DeconvolutionKernels.cpp:200-249); arguments as eh_conv2d_u8_set_perchannel. */
int eh_deconv2d_u8_set_perchannel(eh_deconv_plan *plan, const int32_t *multipliers, const int32_t *shifts, int32_t count,
                                  void *stream);
int eh_deconv2d_u8_repack(eh_deconv_plan *plan, const void *weight, const void *bias, const eh_requant *q, void *stream);
int eh_deconv2d_u8_run(eh_deconv_plan *plan, const void *input, void *output, const eh_requant *q, void *stream);
int eh_deconv2d_u8_destroy(eh_deconv_plan *plan);

/* Timing aid for harnesses: runs `fn`-independent HIP event pairs on `stream`.
 * eh_event_* wrap hipEventCreate / Record / ElapsedTime so that a harness can
 * time the stream the kernels are launched on without linking HIP itself. */
int eh_event_create(void **event);
int eh_event_record(void *event, void *stream);
int eh_event_elapsed_ms(void *start, void *stop, float *ms); /* synchronises on `stop` */
/* Work enqueued on `stream` after this call waits for what `event` recorded (hipStreamWaitEvent): the way a caller
 * forks independent work onto a second stream and joins it again, under graph capture too. */
int eh_stream_wait_event(void *stream, void *event);
int eh_event_destroy(void *event);

#ifdef __cplusplus
}
#endif
#endif /* EDEN_HIP_H_ */
