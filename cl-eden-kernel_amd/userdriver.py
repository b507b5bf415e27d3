"""ctypes binding of libedenud.so (the userdriver-level C ABI in include/eden_ud.h) for the test and benchmark
harnesses: describe an operator list, open it (the C++ OperationConstructor builds HipConvolution ... operators on a
HipComputeLibrary), execute it (OperationExecutor, recorded into a HIP graph and replayed), close it.

No CPU fallback: a missing library raises in load(), a missing or non-gfx950 GPU makes UserDriver() raise."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libedenud.so")

OP_ADD, OP_AVERAGE_POOL_2D, OP_CONV_2D, OP_DEPTHWISE_CONV_2D, OP_FULLY_CONNECTED, OP_TRANSPOSE_CONV = 0, 1, 3, 4, 9, 67
TENSOR_INT32, TENSOR_UINT8, TENSOR_INT8 = 2, 3, 9
(MODEL_CAFFE, MODEL_TENSORFLOW, MODEL_CAFFE_NCHW, MODEL_CAFFE_NHWC, MODEL_TENSORFLOW_NCHW, MODEL_TENSORFLOW_NHWC,
 MODEL_ANDROID_NN) = range(7)
PADDING_SAME, PADDING_VALID = 0, 1
ACT_NONE, ACT_RELU, ACT_RELU_N1_TO_1, ACT_RELU6 = 0, 1, 2, 3


class EdenUdError(RuntimeError):
    pass


class Options(C.Structure):
    _fields_ = [("padding", C.c_int32), ("stride_w", C.c_int32), ("stride_h", C.c_int32), ("dilation_w_factor", C.c_int32),
                ("dilation_h_factor", C.c_int32), ("depth_multiplier", C.c_int32), ("group", C.c_int32), ("filter_width", C.c_int32),
                ("filter_height", C.c_int32), ("fused_activation_function", C.c_int32), ("has_padding_value", C.c_int32),
                ("padding_value", C.c_int32 * 4), ("use_nchw", C.c_int32)]


def options(padding=PADDING_VALID, stride=(1, 1), dilation=(1, 1), depth_multiplier=1, group=1, filter=(1, 1), activation=ACT_NONE,
            padding_value=None, use_nchw=False):
    """stride, dilation and filter are (h, w); padding_value is the explicit (left, right, top, bottom)"""
    o = Options(padding, stride[1], stride[0], dilation[1], dilation[0], depth_multiplier, group, filter[1], filter[0], activation,
                1 if padding_value is not None else 0, (C.c_int32 * 4)(*(padding_value or (0, 0, 0, 0))), int(use_nchw))
    return o


EXPORTS = {
    "eud_last_error": (C.c_char_p, []),
    "eud_initialize": (C.c_int, [C.POINTER(C.c_void_p), C.c_int]),
    "eud_deinitialize": (C.c_int, [C.c_void_p]),
    "eud_oplist_create": (C.c_int, [C.POINTER(C.c_void_p), C.c_uint64, C.c_int32]),
    "eud_oplist_feature_map": (C.c_int32, [C.c_void_p, C.c_int32, C.c_void_p, C.c_int32, C.c_int32, C.c_float, C.c_int32]),
    "eud_oplist_parameter": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_float, C.c_int32, C.c_void_p, C.c_size_t,
                                         C.c_void_p, C.c_int32]),
    "eud_oplist_operator": (C.c_int, [C.c_void_p, C.c_char_p, C.c_int32, C.c_void_p, C.c_int32, C.c_void_p, C.c_int32, C.POINTER(Options)]),
    "eud_oplist_destroy": (C.c_int, [C.c_void_p]),
    "eud_open_subgraph": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32]),
    "eud_prepare_subgraph": (C.c_int, [C.c_void_p, C.c_uint64]),
    "eud_execute_subgraph": (C.c_int, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32]),
    "eud_close_subgraph": (C.c_int, [C.c_void_p, C.c_uint64]),
    "eud_execute_operators": (C.c_int, [C.c_void_p, C.c_uint64, C.c_int32]),
    "eud_set_replay": (C.c_int, [C.c_void_p, C.c_int32]),
    "eud_set_image_lanes": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32]),
    "eud_set_fuse_expansions": (C.c_int, [C.c_void_p, C.c_int32]),
    "eud_set_store_channels_last": (C.c_int, [C.c_void_p, C.c_int32]),
    "eud_synchronize": (C.c_int, [C.c_void_p]),
    "eud_stream": (C.c_void_p, [C.c_void_p]),
    "eud_stats": (C.c_int, [C.c_void_p, C.c_uint64, C.POINTER(C.c_int32), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64),
                            C.POINTER(C.c_uint64), C.POINTER(C.c_size_t)]),
    "eud_write_input": (C.c_int, [C.c_void_p, C.c_uint64, C.c_int32, C.c_void_p, C.c_size_t]),
    "eud_read_output": (C.c_int, [C.c_void_p, C.c_uint64, C.c_int32, C.c_void_p, C.c_size_t]),
    "eud_set_quant": (C.c_int, [C.c_void_p, C.c_uint64, C.c_int32, C.c_int32, C.c_float, C.c_int32]),
}

_lib = None


def load():
    """Loads libedenud.so and checks that every export of include/eden_ud.h is there."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise EdenUdError("%s is missing: run `python cl-eden-kernel_amd/build.py` (there is no CPU fallback)" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in EXPORTS.items():
            fn = getattr(lib, name, None)
            if fn is None:
                raise EdenUdError("libedenud.so does not export %s" % name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def check(rc, what=""):
    if rc != 0:
        raise EdenUdError("%s%s" % (what + ": " if what else "", (load().eud_last_error() or b"").decode()))


class OperatorList:
    """The description of an operator list (what the reference's model loader hands OpenSubGraph)."""

    def __init__(self, list_id, legacy_model=MODEL_TENSORFLOW_NHWC):
        self.id = list_id
        self.h = C.c_void_p()
        check(load().eud_oplist_create(C.byref(self.h), list_id, legacy_model))

    def feature_map(self, buffer_index, shape, scale, zero_point, tensor_type=TENSOR_UINT8):
        s = (C.c_uint32 * len(shape))(*shape)
        t = load().eud_oplist_feature_map(self.h, buffer_index, s, len(shape), tensor_type, scale, zero_point)
        if t < 0:
            check(1, "feature_map")
        return t

    def parameter(self, array, scale=1.0, zero_point=0, shape=None, per_channel_scales=None):
        a = np.ascontiguousarray(array)
        kind = {np.dtype(np.uint8): TENSOR_UINT8, np.dtype(np.int8): TENSOR_INT8, np.dtype(np.int32): TENSOR_INT32}[a.dtype]
        shape = tuple(shape if shape is not None else a.shape)
        s = (C.c_uint32 * len(shape))(*shape)
        pcs = np.ascontiguousarray(per_channel_scales, np.float32) if per_channel_scales is not None else None
        t = load().eud_oplist_parameter(self.h, s, len(shape), kind, scale, zero_point, a.ctypes.data, a.nbytes,
                                        pcs.ctypes.data if pcs is not None else None, len(pcs) if pcs is not None else 0)
        if t < 0:
            check(1, "parameter")
        return t

    def operator(self, name, code, inputs, outputs, opts=None):
        opts = opts if opts is not None else options()
        i, o = (C.c_int32 * len(inputs))(*inputs), (C.c_int32 * len(outputs))(*outputs)
        check(load().eud_oplist_operator(self.h, name.encode(), code, i, len(inputs), o, len(outputs), C.byref(opts)), "operator " + name)

    def __del__(self):
        try:
            if self.h:
                load().eud_oplist_destroy(self.h)
                self.h = C.c_void_p()
        except Exception:
            pass


class UserDriver:
    """HipUserDriver behind the C ABI: Initialize at construction, Deinitialize at close()."""

    def __init__(self, device=0):
        self.h = C.c_void_p()
        check(load().eud_initialize(C.byref(self.h), device), "eud_initialize")

    def open_subgraph(self, oplist, fuse_residual_adds=True):
        check(load().eud_open_subgraph(self.h, oplist.h, int(fuse_residual_adds)), "open_subgraph")

    def execute_subgraph(self, list_id, buffers):
        """buffers: {buffer_index: numpy array}; inputs are read from, outputs written into the arrays"""
        n = len(buffers)
        idx = (C.c_int32 * n)(*buffers.keys())
        for a in buffers.values():
            assert a.flags["C_CONTIGUOUS"]
        addr = (C.c_void_p * n)(*[a.ctypes.data for a in buffers.values()])
        size = (C.c_size_t * n)(*[a.nbytes for a in buffers.values()])
        check(load().eud_execute_subgraph(self.h, list_id, idx, addr, size, n), "execute_subgraph")

    def close_subgraph(self, list_id):
        check(load().eud_close_subgraph(self.h, list_id), "close_subgraph")

    def execute_operators(self, list_id, times=1):
        check(load().eud_execute_operators(self.h, list_id, times), "execute_operators")

    def set_replay(self, on):
        check(load().eud_set_replay(self.h, int(on)))

    def set_image_lanes(self, lanes, min_lane_images=12):
        """Lists opened from now on run as `lanes` chains of images side by side when a chain gets min_lane_images or more."""
        check(load().eud_set_image_lanes(self.h, lanes, min_lane_images), "set_image_lanes")

    def set_fuse_expansions(self, mode):
        """0: never; 1: where the library's measured table prefers the one launch (default); 2: wherever the kernel fits"""
        check(load().eud_set_fuse_expansions(self.h, mode), "set_fuse_expansions")

    def set_store_channels_last(self, on):
        """Lists opened from now on: feature maps inside a planar list are stored channels-last (default) or as their shapes read."""
        check(load().eud_set_store_channels_last(self.h, int(on)), "set_store_channels_last")

    def synchronize(self):
        check(load().eud_synchronize(self.h), "synchronize")

    @property
    def stream(self):
        return load().eud_stream(self.h)

    def stats(self, list_id):
        n, d, r, p, b = C.c_int32(), C.c_uint64(), C.c_uint64(), C.c_uint64(), C.c_size_t()
        check(load().eud_stats(self.h, list_id, C.byref(n), C.byref(d), C.byref(r), C.byref(p), C.byref(b)), "stats")
        return dict(operators=n.value, direct=d.value, recordings=r.value, replays=p.value, pool_bytes=b.value)

    def write_input(self, list_id, i, array):
        a = np.ascontiguousarray(array)
        check(load().eud_write_input(self.h, list_id, i, a.ctypes.data, a.nbytes), "write_input")

    def read_output(self, list_id, i, shape, dtype=np.uint8):
        out = np.empty(shape, dtype)
        check(load().eud_read_output(self.h, list_id, i, out.ctypes.data, out.nbytes), "read_output")
        return out

    def set_quant(self, list_id, is_output, i, scale, zero_point):
        check(load().eud_set_quant(self.h, list_id, int(is_output), i, scale, zero_point))

    def close(self):
        if self.h:
            load().eud_deinitialize(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
