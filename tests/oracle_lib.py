"""ctypes view of oracle/liboracle.so (the CPU checker) and, where it was built,
oracle/_ref/libedenref.so (the reference's own host arithmetic).

Test infrastructure: imported by tests, the smoke check and the bench's
cpu_baseline leg only."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
_LIB = os.path.join(ORACLE_DIR, "liboracle.so")
_REF = os.path.join(ORACLE_DIR, "_ref", "libedenref.so")

ACT_NONE, ACT_RELU, ACT_RELU1, ACT_RELU6 = 0, 1, 2, 3


class Quant(C.Structure):
    _fields_ = [(n, C.c_int32) for n in
                ("zp_in", "zp_w", "zp_out", "multiplier", "shift", "act_min", "act_max")]

    def as_tuple(self):
        return tuple(getattr(self, n) for n, _ in self._fields_)


class ConvShape(C.Structure):
    _fields_ = [(n, C.c_int32) for n in
                ("n", "c", "h", "w", "cout", "kh", "kw", "stride_h", "stride_w",
                 "pad_t", "pad_b", "pad_l", "pad_r", "dil_h", "dil_w", "groups", "dm")]


class AddQuant(C.Structure):
    _fields_ = [(n, C.c_int32) for n in
                ("zp_a", "zp_b", "zp_out", "left_shift", "mult_a", "shift_a", "mult_b", "shift_b",
                 "mult_out", "shift_out", "act_min", "act_max")]


def _load():
    if not os.path.exists(_LIB):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "-s"])
    lib = C.CDLL(_LIB)
    i32, i64, u64, f32, f64, vp = C.c_int32, C.c_int64, C.c_uint64, C.c_float, C.c_double, C.c_void_p
    P = C.POINTER
    sig = {
        "eo_quantize_multiplier": (None, [f64, P(i32), P(i32)]),
        "eo_conv_multiplier": (C.c_int, [f32, f32, f32, f32, P(f64)]),
        "eo_act_range_u8": (None, [C.c_int, f32, i32, P(i32), P(i32)]),
        "eo_act_range_s8": (None, [C.c_int, f32, i32, P(i32), P(i32)]),
        "eo_make_quant_s8": (None, [f32, i32, f32, i32, f32, f32, i32, C.c_int, C.c_int, P(Quant)]),
        "eo_conv2d_s8": (None, [vp, vp, vp, vp, P(ConvShape), P(Quant), vp, vp]),
        "eo_dwconv2d_s8": (None, [vp, vp, vp, vp, P(ConvShape), P(Quant), vp, vp]),
        "eo_deconv2d_s8": (None, [vp, vp, vp, vp, P(ConvShape), P(Quant), vp, vp]),
        "eo_fc_s8": (None, [vp, vp, vp, vp, i32, i32, i32, P(Quant)]),
        "eo_srdhm": (i32, [i32, i32]),
        "eo_rdivpot": (i32, [i32, i32]),
        "eo_mbqm": (i32, [i32, i32, i32]),
        "eo_requant": (C.c_uint8, [i32, P(Quant)]),
        "eo_make_quant": (None, [f32, i32, f32, i32, f32, f32, i32, C.c_int, C.c_int, P(Quant)]),
        "eo_conv_out_dim": (i32, [i32] * 6),
        "eo_deconv_out_dim": (i32, [i32] * 5),
        "eo_conv2d_u8": (None, [vp, vp, vp, vp, P(ConvShape), P(Quant), vp]),
        "eo_conv2d_u8_perchannel": (None, [vp, vp, vp, vp, P(ConvShape), P(Quant), vp, vp, vp]),
        "eo_dwconv2d_u8": (None, [vp, vp, vp, vp, P(ConvShape), P(Quant), vp]),
        "eo_dwconv2d_u8_perchannel": (None, [vp, vp, vp, vp, P(ConvShape), P(Quant), vp, vp, vp]),
        "eo_deconv2d_u8_perchannel": (None, [vp, vp, vp, vp, P(ConvShape), P(Quant), vp, vp, vp]),
        "eo_fc_u8": (None, [vp, vp, vp, vp, i32, i32, i32, P(Quant), vp]),
        "eo_deconv2d_u8": (None, [vp, vp, vp, vp, P(ConvShape), P(Quant), vp]),
        "eo_deconv2d_u8_scatter": (None, [vp, vp, vp, vp, P(ConvShape), P(Quant), vp]),
        "eo_deconv2d_f64": (None, [vp, vp, vp, vp, P(ConvShape)]),
        "eo_nchw2nhwc_u8": (None, [vp, vp, i32, i32, i32, i32]),
        "eo_nhwc2nchw_u8": (None, [vp, vp, i32, i32, i32, i32]),
        "eo_count_fastpath_overflow": (i64, [vp, i64, P(Quant)]),
        "eo_srdhm_fastpath": (i32, [i32, i32]),
        "eo_make_add_quant": (None, [f32, i32, f32, i32, f32, i32, C.c_int, C.c_int, P(AddQuant)]),
        "eo_add_u8": (None, [vp, vp, vp, i64, P(AddQuant)]),
        "eo_avgpool_u8": (None, [vp, vp] + [i32] * 14),
        "eo_avgpool_s8": (None, [vp, vp] + [i32] * 14),
        "eo_splitmix64": (u64, [u64, u64]),
        "eo_fill_u8": (None, [vp, i64, u64, i32, i32]),
        "eo_fill_i32": (None, [vp, i64, u64, i32, i32]),
        "eo_fill_u8_normal": (None, [vp, i64, u64, i32, i32]),
        "eo_num_threads": (C.c_int, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    return lib


lib = _load()


def load_ref():
    """The reference's own QuantizationUtil/KernelUtil/gemmlowp arithmetic, or None
    when oracle/_ref was not built (it needs the reference tree)."""
    if not os.path.exists(_REF):
        return None
    ref = C.CDLL(_REF)
    i32, f32, f64 = C.c_int32, C.c_float, C.c_double
    P = C.POINTER
    ref.ref_quantize_multiplier.argtypes = [f64, P(i32), P(i32)]
    ref.ref_quantize_multiplier.restype = None
    ref.ref_conv_multiplier.argtypes = [f32, f32, f32, f32, P(f64)]
    ref.ref_conv_multiplier.restype = C.c_int
    ref.ref_act_range_u8.argtypes = [C.c_int, f32, i32, P(i32), P(i32)]
    ref.ref_act_range_u8.restype = None
    ref.ref_act_range_s8.argtypes = [C.c_int, f32, i32, P(i32), P(i32)]
    ref.ref_act_range_s8.restype = None
    for n in ("ref_srdhm", "ref_rdivpot"):
        getattr(ref, n).argtypes = [i32, i32]
        getattr(ref, n).restype = i32
    ref.ref_mbqm.argtypes = [i32, i32, i32]
    ref.ref_mbqm.restype = i32
    return ref


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def quantize_multiplier(m):
    q, s = C.c_int32(), C.c_int32()
    lib.eo_quantize_multiplier(m, C.byref(q), C.byref(s))
    return q.value, s.value


def act_range_u8(act, scale, zp):
    lo, hi = C.c_int32(), C.c_int32()
    lib.eo_act_range_u8(act, scale, zp, C.byref(lo), C.byref(hi))
    return lo.value, hi.value


def act_range_s8(act, scale, zp):
    lo, hi = C.c_int32(), C.c_int32()
    lib.eo_act_range_s8(act, scale, zp, C.byref(lo), C.byref(hi))
    return lo.value, hi.value


def make_quant_s8(s_in, zp_in, s_w, zp_w, s_out, zp_out, act=ACT_NONE, act_enabled=False, s_bias=None):
    """INT8 precision: zero points and the activation range are int8 values"""
    q = Quant()
    if s_bias is None:
        s_bias = float(np.float32(s_in) * np.float32(s_w))
    lib.eo_make_quant_s8(s_in, zp_in, s_w, zp_w, s_bias, s_out, zp_out, act, int(act_enabled), C.byref(q))
    return q


def _s8_op(fn, x, w, bias, s, q, out_shape, multipliers, shifts):
    x, w, bias = _c(x, np.int8), _c(w, np.int8), _c(bias, np.int32)
    out = np.zeros(out_shape, np.int8)
    m = _c(multipliers, np.int32) if multipliers is not None else None
    sh = _c(shifts, np.int32) if shifts is not None else None
    fn(_ptr(x), _ptr(w), _ptr(bias), _ptr(out), C.byref(s), C.byref(q), _ptr(m), _ptr(sh))
    return out


def conv2d_s8(x, w, bias, s, q, multipliers=None, shifts=None):
    ho, wo = conv_out_hw(s)
    return _s8_op(lib.eo_conv2d_s8, x, w, bias, s, q, (s.n, s.cout, ho, wo), multipliers, shifts)


def dwconv2d_s8(x, w, bias, s, q, multipliers=None, shifts=None):
    ho, wo = conv_out_hw(s)
    return _s8_op(lib.eo_dwconv2d_s8, x, w, bias, s, q, (s.n, s.c * max(s.dm, 1), ho, wo), multipliers, shifts)


def deconv2d_s8(x, w, bias, s, q, multipliers=None, shifts=None):
    ho, wo = deconv_out_hw(s)
    return _s8_op(lib.eo_deconv2d_s8, x, w, bias, s, q, (s.n, s.cout, ho, wo), multipliers, shifts)


def fc_s8(a, w, bias, q):
    a, w, bias = _c(a, np.int8), _c(w, np.int8), _c(bias, np.int32)
    out = np.zeros((a.shape[0], w.shape[0]), np.int8)
    lib.eo_fc_s8(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), a.shape[0], a.shape[1], w.shape[0], C.byref(q))
    return out


def make_quant(s_in, zp_in, s_w, zp_w, s_out, zp_out, act=ACT_NONE, act_enabled=False, s_bias=None):
    """Quant parameters exactly as an operator's execute() derives them from its
    tensors; the bias scale defaults to the float32 product s_in*s_w."""
    if s_bias is None:
        s_bias = float(np.float32(s_in) * np.float32(s_w))
    q = Quant()
    lib.eo_make_quant(s_in, zp_in, s_w, zp_w, s_bias, s_out, zp_out, act, int(act_enabled), C.byref(q))
    return q


def perchannel_pairs(s_in, filter_scales, s_out):
    """One (multiplier, shift) per output channel as the per-channel operators derive them at execute()
    (cl_optimized_impls/CLConvolutionPerChannelQuantized.cpp:88-97): the per-tensor derivation with the channel's
    filter scale and the bias scale s_in * scale."""
    pairs = [make_quant(s_in, 0, float(s), 0, s_out, 0) for s in np.asarray(filter_scales, np.float32)]
    return np.array([q.multiplier for q in pairs], np.int32), np.array([q.shift for q in pairs], np.int32)


def raw_quant(zp_in=0, zp_w=0, zp_out=0, multiplier=1 << 30, shift=1, act_min=0, act_max=255):
    """Explicit integer parameters; the default multiplier/shift is M == 1."""
    return Quant(zp_in, zp_w, zp_out, multiplier, shift, act_min, act_max)


def conv_shape(n, c, h, w, cout, kh, kw, stride=(1, 1), pad=(0, 0, 0, 0), dil=(1, 1), groups=1, dm=1):
    """pad = (top, bottom, left, right)"""
    return ConvShape(n, c, h, w, cout, kh, kw, stride[0], stride[1], pad[0], pad[1], pad[2], pad[3],
                     dil[0], dil[1], groups, dm)


def conv_out_hw(s):
    return (lib.eo_conv_out_dim(s.h, s.pad_t, s.pad_b, s.kh, s.dil_h, s.stride_h),
            lib.eo_conv_out_dim(s.w, s.pad_l, s.pad_r, s.kw, s.dil_w, s.stride_w))


def deconv_out_hw(s):
    return (lib.eo_deconv_out_dim(s.h, s.pad_t, s.pad_b, s.kh, s.stride_h),
            lib.eo_deconv_out_dim(s.w, s.pad_l, s.pad_r, s.kw, s.stride_w))


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def conv2d(x, w, bias, s, q, want_acc=False):
    x, w, bias = _c(x, np.uint8), _c(w, np.uint8), _c(bias, np.int32)
    ho, wo = conv_out_hw(s)
    out = np.zeros((s.n, s.cout, ho, wo), np.uint8)
    acc = np.zeros(out.shape, np.int32) if want_acc else None
    lib.eo_conv2d_u8(_ptr(x), _ptr(w), _ptr(bias), _ptr(out), C.byref(s), C.byref(q), _ptr(acc))
    return (out, acc) if want_acc else out


def conv2d_perchannel(x, w_i8, bias, s, q, multipliers, shifts):
    x, w, bias = _c(x, np.uint8), _c(w_i8, np.int8), _c(bias, np.int32)
    m, sh = _c(multipliers, np.int32), _c(shifts, np.int32)
    ho, wo = conv_out_hw(s)
    out = np.zeros((s.n, s.cout, ho, wo), np.uint8)
    lib.eo_conv2d_u8_perchannel(_ptr(x), _ptr(w), _ptr(bias), _ptr(out), C.byref(s), C.byref(q),
                                _ptr(m), _ptr(sh), None)
    return out


def dwconv2d(x, w, bias, s, q, want_acc=False):
    x, w, bias = _c(x, np.uint8), _c(w, np.uint8), _c(bias, np.int32)
    ho, wo = conv_out_hw(s)
    out = np.zeros((s.n, s.c * max(s.dm, 1), ho, wo), np.uint8)
    acc = np.zeros(out.shape, np.int32) if want_acc else None
    lib.eo_dwconv2d_u8(_ptr(x), _ptr(w), _ptr(bias), _ptr(out), C.byref(s), C.byref(q), _ptr(acc))
    return (out, acc) if want_acc else out


def dwconv2d_perchannel(x, w_i8, bias, s, q, multipliers, shifts):
    x, w, bias = _c(x, np.uint8), _c(w_i8, np.int8), _c(bias, np.int32)
    m, sh = _c(multipliers, np.int32), _c(shifts, np.int32)
    ho, wo = conv_out_hw(s)
    out = np.zeros((s.n, s.c * max(s.dm, 1), ho, wo), np.uint8)
    lib.eo_dwconv2d_u8_perchannel(_ptr(x), _ptr(w), _ptr(bias), _ptr(out), C.byref(s), C.byref(q), _ptr(m), _ptr(sh), None)
    return out


def deconv2d_perchannel(x, w_i8, bias, s, q, multipliers, shifts):
    x, w, bias = _c(x, np.uint8), _c(w_i8, np.int8), _c(bias, np.int32)
    m, sh = _c(multipliers, np.int32), _c(shifts, np.int32)
    ho, wo = deconv_out_hw(s)
    out = np.zeros((s.n, s.cout, ho, wo), np.uint8)
    lib.eo_deconv2d_u8_perchannel(_ptr(x), _ptr(w), _ptr(bias), _ptr(out), C.byref(s), C.byref(q), _ptr(m), _ptr(sh), None)
    return out


def fc(a, w, bias, q, want_acc=False):
    a, w, bias = _c(a, np.uint8), _c(w, np.uint8), _c(bias, np.int32)
    m, k = a.shape
    n = w.shape[0]
    assert w.shape[1] == k
    out = np.zeros((m, n), np.uint8)
    acc = np.zeros(out.shape, np.int32) if want_acc else None
    lib.eo_fc_u8(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), m, k, n, C.byref(q), _ptr(acc))
    return (out, acc) if want_acc else out


def deconv2d(x, w, bias, s, q, want_acc=False, scatter=False):
    x, w, bias = _c(x, np.uint8), _c(w, np.uint8), _c(bias, np.int32)
    ho, wo = deconv_out_hw(s)
    out = np.zeros((s.n, s.cout, ho, wo), np.uint8)
    acc = np.zeros(out.shape, np.int32) if want_acc else None
    fn = lib.eo_deconv2d_u8_scatter if scatter else lib.eo_deconv2d_u8
    fn(_ptr(x), _ptr(w), _ptr(bias), _ptr(out), C.byref(s), C.byref(q), _ptr(acc))
    return (out, acc) if want_acc else out


def deconv2d_f64(x, w, bias, s):
    x, w, bias = _c(x, np.float64), _c(w, np.float64), _c(bias, np.float64)
    ho, wo = deconv_out_hw(s)
    out = np.zeros((s.n, s.cout, ho, wo), np.float64)
    lib.eo_deconv2d_f64(_ptr(x), _ptr(w), _ptr(bias), _ptr(out), C.byref(s))
    return out


def nchw2nhwc(x):
    x = _c(x, np.uint8)
    n, c, h, w = x.shape
    out = np.zeros((n, h, w, c), np.uint8)
    lib.eo_nchw2nhwc_u8(_ptr(x), _ptr(out), n, c, h, w)
    return out


def nhwc2nchw(x):
    x = _c(x, np.uint8)
    n, h, w, c = x.shape
    out = np.zeros((n, c, h, w), np.uint8)
    lib.eo_nhwc2nchw_u8(_ptr(x), _ptr(out), n, c, h, w)
    return out


def count_fastpath_overflow(acc, q):
    acc = _c(acc, np.int32)
    return lib.eo_count_fastpath_overflow(_ptr(acc), acc.size, C.byref(q))


def make_add_quant(s_a, zp_a, s_b, zp_b, s_out, zp_out, act=ACT_NONE, act_enabled=False):
    q = AddQuant()
    lib.eo_make_add_quant(s_a, zp_a, s_b, zp_b, s_out, zp_out, act, int(act_enabled), C.byref(q))
    return q


def add(a, b, q):
    a, b = _c(a, np.uint8), _c(b, np.uint8)
    out = np.zeros(a.shape, np.uint8)
    lib.eo_add_u8(_ptr(a), _ptr(b), _ptr(out), a.size, C.byref(q))
    return out


def avgpool(x, kh, kw, stride=(1, 1), pad=(0, 0, 0, 0), act_min=0, act_max=255):
    x = _c(x, np.uint8)
    n, c, h, w = x.shape
    ho = (h + pad[0] + pad[1] - kh) // stride[0] + 1
    wo = (w + pad[2] + pad[3] - kw) // stride[1] + 1
    out = np.zeros((n, c, ho, wo), np.uint8)
    lib.eo_avgpool_u8(_ptr(x), _ptr(out), n, c, h, w, kh, kw, stride[0], stride[1],
                      pad[0], pad[1], pad[2], pad[3], act_min, act_max)
    return out


def avgpool_s8(x, kh, kw, stride=(1, 1), pad=(0, 0, 0, 0), act_min=-128, act_max=127):
    x = _c(x, np.int8)
    n, c, h, w = x.shape
    ho = (h + pad[0] + pad[1] - kh) // stride[0] + 1
    wo = (w + pad[2] + pad[3] - kw) // stride[1] + 1
    out = np.zeros((n, c, ho, wo), np.int8)
    lib.eo_avgpool_s8(_ptr(x), _ptr(out), n, c, h, w, kh, kw, stride[0], stride[1],
                      pad[0], pad[1], pad[2], pad[3], act_min, act_max)
    return out


def fill_u8(shape, seed, lo=0, hi=255):
    out = np.zeros(shape, np.uint8)
    lib.eo_fill_u8(_ptr(out), out.size, seed, lo, hi)
    return out


def fill_i32(shape, seed, lo, hi):
    out = np.zeros(shape, np.int32)
    lib.eo_fill_i32(_ptr(out), out.size, seed, lo, hi)
    return out


def fill_u8_normal(shape, seed, mean, sd):
    out = np.zeros(shape, np.uint8)
    lib.eo_fill_u8_normal(_ptr(out), out.size, seed, mean, sd)
    return out
