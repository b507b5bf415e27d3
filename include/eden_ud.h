/*
 * eden_ud.h — C ABI of the userdriver level of the MI355X (gfx950) backend: open an operator list (build its
 * operators once), execute it on host buffers, close it.  This is the level at which the reference's runtime binds a
 * userdriver (enn::ud::UserDriver, src/userdriver/common/UserDriver.h:52-122, implemented for the OpenCL GPU by
 * GpuUserDriver, src/userdriver/gpu/gpu_userdriver.h:34-94); each entry point names the member it stands in for.
 * Behind it sit the C++ classes of cl-eden-kernel_amd/host/ (HipUserDriver -> OperationConstructor /
 * OperationExecutor -> HipComputeLibrary -> operator classes), which call the kernels through eden_hip.h.
 *
 * The reference hands its userdriver C++ model objects made by its flatbuffer loader.  A C caller describes the same
 * things with eud_oplist_*: feature maps (run-time tensors named by a buffer index), parameters (constant tensors with
 * host data, copied when added) and operators with the TFLite option fields of src/model/schema/nnc/v2/schema.fbs.
 *
 * Conventions: 0 = success (ENN_RET_SUCCESS), non-zero = failure, text in eud_last_error(); no exceptions and no C++
 * types cross the boundary; a driver object serialises its own entry points (the reference's constructor mutex).
 * Loaded by bench.py and the tests through ctypes (cl-eden-kernel_amd/userdriver.py).
 */
#ifndef EDEN_UD_H_
#define EDEN_UD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct eud_driver eud_driver;
typedef struct eud_oplist eud_oplist;

/* TFlite::BuiltinOperator values of the operators this backend builds (schema.fbs:245-318) */
enum { EUD_OP_ADD = 0, EUD_OP_AVERAGE_POOL_2D = 1, EUD_OP_CONV_2D = 3, EUD_OP_DEPTHWISE_CONV_2D = 4, EUD_OP_FULLY_CONNECTED = 9, EUD_OP_TRANSPOSE_CONV = 67 };
/* TFlite::TensorType (schema.fbs:38-58) */
enum { EUD_TENSOR_INT32 = 2, EUD_TENSOR_UINT8 = 3, EUD_TENSOR_INT8 = 9 };
/* TFlite::LegacyModel (schema.fbs:1456-1465) */
enum { EUD_MODEL_CAFFE = 0, EUD_MODEL_TENSORFLOW = 1, EUD_MODEL_CAFFE_NCHW = 2, EUD_MODEL_CAFFE_NHWC = 3, EUD_MODEL_TENSORFLOW_NCHW = 4, EUD_MODEL_TENSORFLOW_NHWC = 5, EUD_MODEL_ANDROID_NN = 6 };

/* The option fields of Conv2DOptions / DepthwiseConv2DOptions / TransposeConvOptions / Pool2DOptions /
 * FullyConnectedOptions / AddOptions (schema.fbs:547-567,580-606,659-695,953-962); an operator reads the fields its
 * table has and ignores the rest. */
typedef struct eud_options {
    int32_t padding;                   /* TFlite::Padding: 0 SAME, 1 VALID */
    int32_t stride_w, stride_h;
    int32_t dilation_w_factor, dilation_h_factor;
    int32_t depth_multiplier;          /* DEPTHWISE_CONV_2D */
    int32_t group;                     /* TRANSPOSE_CONV */
    int32_t filter_width, filter_height; /* AVERAGE_POOL_2D */
    int32_t fused_activation_function; /* TFlite::ActivationFunctionType: 0 NONE, 1 RELU, 2 RELU_N1_TO_1, 3 RELU6 */
    int32_t has_padding_value;         /* 1: padding_value = explicit {left, right, top, bottom} */
    int32_t padding_value[4];
    int32_t use_nchw;                  /* androidNN models */
} eud_options;

const char *eud_last_error(void);

/* UserDriver::Initialize / Deinitialize (gpu_userdriver.cc:36-49,131-143): makes the compute library for `device`, the
 * operator constructor and the executor; fails on anything but a gfx950 device. */
int eud_initialize(eud_driver **driver, int device);
int eud_deinitialize(eud_driver *driver);

/* The description of one operator list: model::component::OperatorList with its Attribute's legacy_model
 * (gpu_op_constructor.cc:1797-1812).  Tensors are numbered in the order they are added; the number is what
 * eud_oplist_operator takes. */
int eud_oplist_create(eud_oplist **list, uint64_t id, int32_t legacy_model);
/* model::component::FeatureMap: shape (1 to 4 extents), TensorType, per-tensor scale and zero point, buffer index */
int32_t eud_oplist_feature_map(eud_oplist *list, int32_t buffer_index, const uint32_t *shape, int32_t rank, int32_t tensor_type,
                               float scale, int32_t zero_point);
/* model::component::Parameter: the same plus `bytes` of host data (copied) and, for a per-channel quantized filter,
 * one scale per output channel (else scales = NULL, scale_count = 0) */
int32_t eud_oplist_parameter(eud_oplist *list, const uint32_t *shape, int32_t rank, int32_t tensor_type, float scale, int32_t zero_point,
                             const void *data, size_t bytes, const float *scales, int32_t scale_count);
/* model::component::Operator: code, tensors by number, options */
int eud_oplist_operator(eud_oplist *list, const char *name, int32_t builtin_code, const int32_t *inputs, int32_t input_count,
                        const int32_t *outputs, int32_t output_count, const eud_options *options);
int eud_oplist_destroy(eud_oplist *list);

/* UserDriver::OpenSubGraph (gpu_userdriver.cc:51-70): builds every operator (weights packed, pooled feature maps laid out
 * in one device allocation).  fuse_residual_adds = 0 builds one operator per description as the reference does;
 * 1 lets a uint8 ADD right behind the CONV_2D that feeds it run inside that convolution's launch. */
int eud_open_subgraph(eud_driver *driver, const eud_oplist *list, int32_t fuse_residual_adds);
/* UserDriver::PrepareSubGraph (gpu_userdriver.cc:72-76): nothing to do */
int eud_prepare_subgraph(eud_driver *driver, uint64_t list_id);
/* UserDriver::ExecuteSubGraph (gpu_userdriver.cc:78-112) with the request's BufferTable
 * (src/model/memory/buffer_table.hpp:19-44) given as parallel arrays: host bytes into the list's inputs, the operators,
 * outputs back (blocking). */
int eud_execute_subgraph(eud_driver *driver, uint64_t list_id, const int32_t *buffer_indices, void *const *addresses,
                         const size_t *sizes, int32_t buffer_count);
/* UserDriver::CloseSubGraph (gpu_userdriver.cc:114-129) */
int eud_close_subgraph(eud_driver *driver, uint64_t list_id);

/* ---- for callers whose tensors already live on the device, and for measurements.  No counterpart in the
 * reference, whose ExecuteSubGraph always copies. */
/* OperationExecutor::execute (gpu_op_executor.cc:56-103) `times` times on the tensors as they stand; asynchronous */
int eud_execute_operators(eud_driver *driver, uint64_t list_id, int32_t times);
/* replay = 0: every execution runs operator by operator, as the reference's executor does */
int eud_set_replay(eud_driver *driver, int32_t replay);
/* Lists opened from now on whose feature maps all carry the same number of images are built `lanes` times over, each
 * on 1 / lanes of the images, and the lanes run side by side on streams of their own (parallel branches of the recorded
 * graph), when a share holds at least min_lane_images images.  Default 2 lanes from 12 images per lane; lanes = 1 builds
 * one operator per description as the reference does.  Results do not depend on it. */
int eud_set_image_lanes(eud_driver *driver, int32_t lanes, int32_t min_lane_images);
/* Lists opened from now on: a uint8 1x1 CONV_2D whose only reader is a 3x3 DEPTHWISE_CONV_2D runs with it as one launch
 * (eh_conv_dw_block_run; the tensor between them gets no storage) for mode 1 where the library lists the shape as
 * faster that way (the default), for mode 2 wherever the kernel fits, for mode 0 never (one operator per description,
 * as the reference builds the list).  Results do not depend on it. */
int eud_set_fuse_expansions(eud_driver *driver, int32_t mode);
/* Lists opened from now on: the feature maps inside a PLANAR list (a Caffe-style model, or an androidNN one whose
 * operators say use_nchw) are stored channels-last, the order the kernels work in, instead of being transposed on either
 * side of every operator; the list's inputs and outputs stay planar, and one layout operator behind each input and in
 * front of each output joins the list (on: the default).  off: every tensor is stored as its shape reads, as the
 * reference does.  Results do not depend on it. */
int eud_set_store_channels_last(eud_driver *driver, int32_t on);
int eud_synchronize(eud_driver *driver);         /* IComputeLibrary::synchronize */
void *eud_stream(eud_driver *driver);            /* the hipStream_t the operators are enqueued on */
/* operators built for the list, and what the executor has done so far (over all lists) */
int eud_stats(eud_driver *driver, uint64_t list_id, int32_t *operator_count, uint64_t *direct, uint64_t *recordings, uint64_t *replays,
              size_t *pool_bytes);
/* host <-> device copy of the list's i-th input / output tensor (ITensor::writeData / readData, blocking) */
int eud_write_input(eud_driver *driver, uint64_t list_id, int32_t i, const void *host, size_t bytes);
int eud_read_output(eud_driver *driver, uint64_t list_id, int32_t i, void *host, size_t bytes);
/* ITensor::setScale / setZeroPoint on the list's i-th input (is_output = 0) or output (1) tensor: the operators read
 * quantization parameters from their tensors at every execution */
int eud_set_quant(eud_driver *driver, uint64_t list_id, int32_t is_output, int32_t i, float scale, int32_t zero_point);

#ifdef __cplusplus
}
#endif
#endif /* EDEN_UD_H_ */
