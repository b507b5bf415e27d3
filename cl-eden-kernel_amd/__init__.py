"""ctypes binding of libedenhip.so (the C ABI in include/eden_hip.h) for the test
and benchmark harnesses.  The product's host layer is the C++ operator classes
under host/; this module only makes the same C ABI callable from Python.

There is no CPU fallback: a missing library raises on import of `lib`, and a
missing or non-gfx950 GPU makes `init()` raise."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libedenhip.so")

EH_OK = 0
ACT_NONE, ACT_RELU, ACT_RELU1, ACT_RELU6 = 0, 1, 2, 3
NCHW, NHWC = 0, 1
W_OIHW, W_OHWI, W_IOHW = 0, 1, 2
W_SIGNED = 0x100  # or-ed into a convolution's weight layout: int8 weight bytes
IO_SIGNED = 0x200  # or-ed into a convolution's tensor layout: int8 input and output (zero points and range in [-128, 127])
EXACT_CHANNELS = 0x400  # or-ed into a convolution's tensor layout or a fully connected plan's flags: no channel-padded staging copy


class EdenHipError(RuntimeError):
    pass


class Requant(C.Structure):
    _fields_ = [(n, C.c_int32) for n in
                ("zp_in", "zp_w", "zp_out", "multiplier", "shift", "act_min", "act_max")]

    def as_tuple(self):
        return tuple(getattr(self, n) for n, _ in self._fields_)


class ConvDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in
                ("n", "c", "h", "w", "cout", "kh", "kw", "stride_h", "stride_w",
                 "pad_t", "pad_b", "pad_l", "pad_r", "dil_h", "dil_w", "groups",
                 "depth_multiplier", "layout", "weight_layout")]


class AddRequant(C.Structure):
    _fields_ = [(n, C.c_int32) for n in
                ("zp_a", "zp_b", "zp_out", "left_shift", "mult_a", "shift_a", "mult_b", "shift_b", "mult_out", "shift_out",
                 "act_min", "act_max")]


class PoolDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in
                ("n", "c", "h", "w", "kh", "kw", "stride_h", "stride_w", "pad_t", "pad_b", "pad_l", "pad_r", "layout",
                 "act_min", "act_max")]


EXPORTS = {
    # name: (restype, argtypes)
    "eh_quantize_multiplier": (None, [C.c_double, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "eh_conv_multiplier": (C.c_int, [C.c_float] * 4 + [C.POINTER(C.c_double)]),
    "eh_act_range_u8": (None, [C.c_int, C.c_float, C.c_int32, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "eh_act_range_s8": (None, [C.c_int, C.c_float, C.c_int32, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "eh_make_requant_s8": (None, [C.c_float, C.c_int32, C.c_float, C.c_int32, C.c_float, C.c_float, C.c_int32,
                                  C.c_int, C.c_int, C.POINTER(Requant)]),
    "eh_requant_apply": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_void_p]),
    "eh_make_requant": (None, [C.c_float, C.c_int32, C.c_float, C.c_int32, C.c_float, C.c_float, C.c_int32,
                               C.c_int, C.c_int, C.POINTER(Requant)]),
    "eh_make_add_requant": (None, [C.c_float, C.c_int32, C.c_float, C.c_int32, C.c_float, C.c_int32, C.c_int, C.c_int,
                                   C.POINTER(AddRequant)]),
    "eh_add_u8": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.POINTER(AddRequant), C.c_void_p]),
    "eh_avgpool_u8": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(PoolDesc), C.c_void_p]),
    "eh_probe_mfma_i8": (C.c_int, [C.c_int32, C.c_int32, C.POINTER(C.c_double)]),
    "eh_probe_feed": (C.c_int, [C.c_int32, C.c_int32, C.c_int32, C.POINTER(C.c_double), C.POINTER(C.c_int32)]),
    "eh_probe_stream": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_void_p]),
    "eh_make_requant_perchannel": (None, [C.c_float, C.c_int32, C.c_void_p, C.c_int32, C.c_float, C.c_int32, C.c_int, C.c_int,
                                          C.POINTER(Requant), C.c_void_p, C.c_void_p]),
    "eh_conv2d_u8_run_add": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(Requant), C.POINTER(AddRequant),
                                       C.c_void_p]),
    "eh_conv2d_u8_fuses_add": (C.c_int, [C.c_void_p]),
    "eh_conv_dw_block_applies": (C.c_int, [C.c_void_p, C.c_void_p]),
    "eh_conv_dw_block_preferred": (C.c_int, [C.c_void_p, C.c_void_p]),
    "eh_conv_dw_block_listed": (C.c_int, [C.c_int32] * 6),
    "eh_conv_dw_block_run": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(Requant), C.POINTER(Requant), C.c_int32,
                                       C.c_int32, C.c_void_p]),
    "eh_conv2d_u8_run_static": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(Requant), C.c_void_p]),
    "eh_conv2d_u8_kernels": (C.c_int, [C.POINTER(ConvDesc), C.c_void_p, C.c_int32]),
    "eh_deconv2d_u8_kernels": (C.c_int, [C.POINTER(ConvDesc), C.c_void_p, C.c_int32]),
    "eh_conv2d_u8_set_perchannel": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p]),
    "eh_dwconv2d_u8_set_perchannel": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p]),
    "eh_deconv2d_u8_set_perchannel": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p]),
    "eh_conv_out_dim": (C.c_int32, [C.c_int32] * 6),
    "eh_deconv_out_dim": (C.c_int32, [C.c_int32] * 5),
    "eh_init": (C.c_int, [C.c_int]),
    "eh_device_name": (C.c_int, [C.c_char_p, C.c_size_t]),
    "eh_malloc": (C.c_int, [C.POINTER(C.c_void_p), C.c_size_t]),
    "eh_free": (C.c_int, [C.c_void_p]),
    "eh_memset": (C.c_int, [C.c_void_p, C.c_int, C.c_size_t, C.c_void_p]),
    "eh_h2d": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "eh_d2h": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "eh_d2d": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "eh_pool_create": (C.c_int, [C.POINTER(C.c_void_p)]),
    "eh_pool_request": (C.c_int, [C.c_void_p, C.c_int, C.c_size_t, C.POINTER(C.c_int32)]),
    "eh_pool_reset_inter": (C.c_int, [C.c_void_p, C.c_int32]),
    "eh_pool_reset_intra": (C.c_int, [C.c_void_p]),
    "eh_pool_layout": (C.c_int, [C.c_void_p, C.POINTER(C.c_size_t), C.POINTER(C.c_int32)]),
    "eh_pool_assign": (C.c_int, [C.c_void_p, C.POINTER(C.c_size_t)]),
    "eh_pool_slot": (C.c_int, [C.c_void_p, C.c_int32, C.POINTER(C.c_void_p), C.POINTER(C.c_size_t)]),
    "eh_pool_release": (C.c_int, [C.c_void_p, C.c_int32]),
    "eh_pool_destroy": (C.c_int, [C.c_void_p]),
    "eh_stream_create": (C.c_int, [C.POINTER(C.c_void_p)]),
    "eh_stream_destroy": (C.c_int, [C.c_void_p]),
    "eh_stream_sync": (C.c_int, [C.c_void_p]),
    "eh_graph_begin": (C.c_int, [C.c_void_p]),
    "eh_graph_end": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "eh_graph_launch": (C.c_int, [C.c_void_p, C.c_void_p]),
    "eh_graph_destroy": (C.c_int, [C.c_void_p]),
    "eh_last_error": (C.c_char_p, []),
    "eh_transpose_u8_nchw2nhwc": (C.c_int, [C.c_void_p, C.c_void_p] + [C.c_int32] * 4 + [C.c_void_p]),
    "eh_transpose_u8_nhwc2nchw": (C.c_int, [C.c_void_p, C.c_void_p] + [C.c_int32] * 4 + [C.c_void_p]),
    "eh_conv2d_u8_plan": (C.c_int, [C.POINTER(C.c_void_p), C.POINTER(ConvDesc), C.c_void_p, C.c_void_p,
                                    C.POINTER(Requant), C.c_void_p]),
    "eh_conv2d_u8_repack": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(Requant), C.c_void_p]),
    "eh_conv2d_u8_run": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(Requant), C.c_void_p]),
    "eh_conv2d_u8_destroy": (C.c_int, [C.c_void_p]),
    "eh_dwconv2d_u8_plan": (C.c_int, [C.POINTER(C.c_void_p), C.POINTER(ConvDesc), C.c_void_p, C.c_void_p,
                                      C.POINTER(Requant), C.c_void_p]),
    "eh_dwconv2d_u8_repack": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(Requant), C.c_void_p]),
    "eh_dwconv2d_u8_run": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(Requant), C.c_void_p]),
    "eh_dwconv2d_u8_destroy": (C.c_int, [C.c_void_p]),
    "eh_fc_u8_plan": (C.c_int, [C.POINTER(C.c_void_p), C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p,
                                C.POINTER(Requant), C.c_void_p]),
    "eh_fc_q8_plan": (C.c_int, [C.POINTER(C.c_void_p), C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p,
                                C.POINTER(Requant), C.c_void_p]),
    "eh_fc_u8_repack": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(Requant), C.c_void_p]),
    "eh_fc_u8_run": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(Requant), C.c_void_p]),
    "eh_fc_u8_destroy": (C.c_int, [C.c_void_p]),
    "eh_deconv2d_u8_plan": (C.c_int, [C.POINTER(C.c_void_p), C.POINTER(ConvDesc), C.c_void_p, C.c_void_p,
                                      C.POINTER(Requant), C.c_void_p]),
    "eh_deconv2d_u8_repack": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(Requant), C.c_void_p]),
    "eh_deconv2d_u8_run": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(Requant), C.c_void_p]),
    "eh_deconv2d_u8_destroy": (C.c_int, [C.c_void_p]),
    "eh_event_create": (C.c_int, [C.POINTER(C.c_void_p)]),
    "eh_event_record": (C.c_int, [C.c_void_p, C.c_void_p]),
    "eh_stream_wait_event": (C.c_int, [C.c_void_p, C.c_void_p]),
    "eh_event_elapsed_ms": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]),
    "eh_event_destroy": (C.c_int, [C.c_void_p]),
}

_lib = None


def load():
    """Loads libedenhip.so and types every export; raises if the library or a symbol is missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise EdenHipError("%s is not built: run `python cl-eden-kernel_amd/build.py`" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in EXPORTS.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def check(rc):
    if rc != EH_OK:
        raise EdenHipError("eden_hip status %d: %s" % (rc, load().eh_last_error().decode()))


def init(device=0):
    check(load().eh_init(device))


def device_name():
    buf = C.create_string_buffer(256)
    check(load().eh_device_name(buf, 256))
    return buf.value.decode()


def make_requant(s_in, zp_in, s_w, zp_w, s_out, zp_out, act=ACT_NONE, act_enabled=False, s_bias=None):
    if s_bias is None:
        s_bias = float(np.float32(s_in) * np.float32(s_w))
    q = Requant()
    load().eh_make_requant(s_in, zp_in, s_w, zp_w, s_bias, s_out, zp_out, act, int(act_enabled), C.byref(q))
    return q


def make_requant_s8(s_in, zp_in, s_w, zp_w, s_out, zp_out, act=ACT_NONE, act_enabled=False, s_bias=None):
    """INT8 precision (IO_SIGNED plans): zero points and the activation range are int8 values."""
    if s_bias is None:
        s_bias = float(np.float32(s_in) * np.float32(s_w))
    q = Requant()
    load().eh_make_requant_s8(s_in, zp_in, s_w, zp_w, s_bias, s_out, zp_out, act, int(act_enabled), C.byref(q))
    return q


def make_add_requant(s_a, zp_a, s_b, zp_b, s_out, zp_out, act=ACT_NONE, act_enabled=False):
    q = AddRequant()
    load().eh_make_add_requant(s_a, zp_a, s_b, zp_b, s_out, zp_out, act, int(act_enabled), C.byref(q))
    return q


def add_u8(a, b, out, count, q, stream=None):
    """a, b, out: DeviceBuffer or raw device addresses."""
    check(load().eh_add_u8(_addr(a), _addr(b), _addr(out), count, C.byref(q), stream))


def avgpool_u8(src, dst, n, c, h, w, kh, kw, stride=(1, 1), pad=(0, 0, 0, 0), layout=None, act_min=0, act_max=255,
               stream=None):
    """layout | IO_SIGNED: int8 tensors (range within [-128, 127], mean rounded half away from zero)"""
    d = PoolDesc(n, c, h, w, kh, kw, stride[0], stride[1], pad[0], pad[1], pad[2], pad[3],
                 NCHW if layout is None else layout, act_min, act_max)
    check(load().eh_avgpool_u8(_addr(src), _addr(dst), C.byref(d), stream))


def _addr(x):
    return x.ptr if hasattr(x, "ptr") else x


FEED_MIXES = ("dma_alone", "lds_reads_alone", "mfma_alone", "tile_128x128", "tile_64x64_splitk", "tile_256x128", "tile_256x256",
              "tile_128x128_weights_to_registers", "tile_256x256_weights_to_registers")


def probe_feed(mix, workgroups=256, iterations=4000):
    """One feed-probe mix: ns per iteration and what an iteration holds per wave, as rates per CU and as a fraction of
    the 5 POP/s matrix peak.  A workgroup takes a CU's LDS, so 256 workgroups are one per CU and more run in rounds."""
    ns, per = C.c_double(0), (C.c_int32 * 4)()
    check(load().eh_probe_feed(mix, workgroups, iterations, C.byref(ns), per))
    rounds = -(-workgroups // 256)
    ns.value /= rounds
    per_cu = 4   # waves per CU
    mfma, reads, dma, regs = per
    return dict(mix=FEED_MIXES[mix], workgroups=workgroups, ns_per_iteration=round(ns.value, 2), per_wave_iteration=dict(mfma=mfma, lds_reads=reads, dma_1k=dma, register_loads_1k=regs),
                mfma_frac_of_5_pops=round(min(workgroups, 256) * 4 * mfma * 65536 / ns.value / 5e6, 4) if mfma else None,
                lds_read_bytes_per_ns_per_cu=round(per_cu * reads * 1024 / ns.value, 1), dma_bytes_per_ns_per_cu=round(per_cu * dma * 1024 / ns.value, 1),
                register_load_bytes_per_ns_per_cu=round(per_cu * regs * 1024 / ns.value, 1))


def probe_mfma_i8(iterations=100000, toggling_operands=True):
    """Sustained int8 MFMA rate of the device in TOP/s (registers only)."""
    tops = C.c_double(0)
    check(load().eh_probe_mfma_i8(iterations, int(toggling_operands), C.byref(tops)))
    return tops.value


def requant_apply(q, acc, two_step=False, channel_form=None):
    """Host evaluation of the kernels' requantization of int32 accumulators; returns (uint8 array, used_single_shift).
    channel_form: "registers" or "table" evaluates the per-channel single-shift forms with q's pair as the channel's;
    "packed" the per-tensor single-shift form four outputs at a time with a row term folded into the rounding term."""
    acc = np.ascontiguousarray(acc, np.int32)
    out = np.empty(acc.shape, np.uint8)
    used = C.c_int32(0)
    form = {None: 1 if two_step else 0, "registers": 2, "table": 3, "packed": 4}[channel_form]
    check(load().eh_requant_apply(C.addressof(q), acc.ctypes.data, out.ctypes.data, acc.size, form, C.addressof(used)))
    return out, bool(used.value)


def conv_desc(n, c, h, w, cout, kh, kw, stride=(1, 1), pad=(0, 0, 0, 0), dil=(1, 1), groups=1, dm=1,
              layout=NCHW, weight_layout=W_OIHW):
    """pad = (top, bottom, left, right)"""
    return ConvDesc(n, c, h, w, cout, kh, kw, stride[0], stride[1], pad[0], pad[1], pad[2], pad[3],
                    dil[0], dil[1], groups, dm, layout, weight_layout)


KERNEL_NAMES = ("staged", "dma_256x128", "dma_128x128", "dma_128x64", "dma_64x64_splitk", "dma_256x256", "one_tap", "c3k3", "conv3x3_patch", "few_channel_rows", "skinny")


def conv_kernels(desc, deconv=False):
    """Kernel family (a KERNEL_NAMES entry) per part of a convolution / deconvolution plan made from `desc`; no GPU."""
    ids = (C.c_int32 * 64)()
    fn = load().eh_deconv2d_u8_kernels if deconv else load().eh_conv2d_u8_kernels
    count = fn(C.byref(desc), ids, 64)
    if count < 0:
        check(count)
    return [KERNEL_NAMES[ids[i]] for i in range(min(count, 64))]


class DeviceBuffer:
    """A device allocation made through the C ABI, with host copies in and out."""

    def __init__(self, nbytes=None, host=None):
        lib = load()
        if host is not None:
            host = np.ascontiguousarray(host)
            nbytes = host.nbytes
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(lib.eh_malloc(C.byref(p), self.nbytes))
        self.ptr = p
        if host is not None and self.nbytes:
            check(lib.eh_h2d(self.ptr, host.ctypes.data_as(C.c_void_p), self.nbytes, None))
            check(lib.eh_stream_sync(None))

    def download(self, shape, dtype=np.uint8):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        lib = load()
        if out.nbytes:
            check(lib.eh_d2h(out.ctypes.data_as(C.c_void_p), self.ptr, out.nbytes, None))
        check(lib.eh_stream_sync(None))
        return out

    def free(self):
        if self.ptr is not None:
            load().eh_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class BufferView:
    """`base` (a DeviceBuffer or a PooledBuffer) from byte `offset` on; owns nothing."""

    def __init__(self, base, offset):
        self.base, self.offset = base, int(offset)

    @property
    def ptr(self):
        return C.c_void_p(self.base.ptr.value + self.offset)

    @property
    def nbytes(self):
        return self.base.nbytes - self.offset


POOL_INTER_NEW, POOL_INTER_REUSE, POOL_INTRA = 0, 1, 2


class PooledBuffer:
    """One slot of a BufferPool: sized at request time, addressed once the pool is assigned."""

    def __init__(self, pool, slot):
        self.pool, self.slot = pool, slot

    @property
    def ptr(self):
        p = C.c_void_p()
        check(load().eh_pool_slot(self.pool.h, self.slot, C.byref(p), None))
        return p

    @property
    def nbytes(self):
        n = C.c_size_t()
        check(load().eh_pool_slot(self.pool.h, self.slot, None, C.byref(n)))
        return n.value

    def download(self, shape, dtype=np.uint8):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        lib = load()
        if out.nbytes:
            check(lib.eh_d2h(out.ctypes.data_as(C.c_void_p), self.ptr, out.nbytes, None))
        check(lib.eh_stream_sync(None))
        return out


def conv_dw_block_applies(pointwise, depthwise):
    """whether a ConvPlan (1x1) and the DwConvPlan on its output can run as one launch"""
    return bool(load().eh_conv_dw_block_applies(pointwise.handle, depthwise.handle))


def conv_dw_block_preferred(pw, dw):
    """True when the fused launch is also the faster choice for the pair's shape (the library's measured table)."""
    return bool(load().eh_conv_dw_block_preferred(pw.handle, dw.handle))


def conv_dw_block_run(pointwise, depthwise, d_in, d_out, q_pointwise, q_depthwise, rows_per_tile=0, cols_per_tile=0, stream=None):
    """pointwise convolution + 3x3 depthwise convolution as one launch (the expanded tensor stays in LDS)"""
    check(load().eh_conv_dw_block_run(pointwise.handle, depthwise.handle, d_in.ptr, d_out.ptr, C.byref(q_pointwise), C.byref(q_depthwise),
                                      rows_per_tile, cols_per_tile, stream))


class BufferPool:
    """The pooled-buffer protocol of an operator list (eh_pool_*): request / reset while the operators are built,
    then one device allocation for all of them."""

    def __init__(self):
        self.h = C.c_void_p()
        check(load().eh_pool_create(C.byref(self.h)))

    def request(self, kind, nbytes):
        slot = C.c_int32(-1)
        check(load().eh_pool_request(self.h, kind, int(nbytes), C.byref(slot)))
        return PooledBuffer(self, slot.value)

    def reset_inter(self, buf):
        check(load().eh_pool_reset_inter(self.h, buf.slot))

    def reset_intra(self):
        check(load().eh_pool_reset_intra(self.h))

    def layout(self):
        """(bytes an assignment would allocate, slots it would hold)"""
        n, c = C.c_size_t(), C.c_int32()
        check(load().eh_pool_layout(self.h, C.byref(n), C.byref(c)))
        return n.value, c.value

    def assign(self):
        n = C.c_size_t()
        check(load().eh_pool_assign(self.h, C.byref(n)))
        return n.value

    def __del__(self):
        try:
            if self.h:
                load().eh_pool_destroy(self.h)
                self.h = C.c_void_p()
        except Exception:
            pass


class _Plan:
    _kind = ""

    def __init__(self):
        self.handle = C.c_void_p()
        self._keep = []

    def run(self, d_in, d_out, q, stream=None):
        check(getattr(load(), "eh_%s_u8_run" % self._kind)(self.handle, d_in.ptr, d_out.ptr, C.byref(q), stream))

    def repack(self, d_w, d_b, q, stream=None):
        check(getattr(load(), "eh_%s_u8_repack" % self._kind)(self.handle, d_w.ptr, d_b.ptr if d_b else None,
                                                            C.byref(q), stream))

    def destroy(self):
        if self.handle:
            getattr(load(), "eh_%s_u8_destroy" % self._kind)(self.handle)
            self.handle = C.c_void_p()

    def set_perchannel(self, multipliers, shifts, stream=None):
        """One multiplier / shift per output channel from now on (None, None: back to the Requant's pair).
        Convolution, depthwise convolution and deconvolution plans."""
        fn = getattr(load(), "eh_%s_u8_set_perchannel" % self._kind)
        if multipliers is None:
            check(fn(self.handle, None, None, 0, stream))
            return
        m, s = np.ascontiguousarray(multipliers, np.int32), np.ascontiguousarray(shifts, np.int32)
        check(fn(self.handle, m.ctypes.data, s.ctypes.data, m.size, stream))

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class ConvPlan(_Plan):
    _kind = "conv2d"

    def __init__(self, desc, d_w, d_b, q, stream=None):
        super().__init__()
        self.desc = desc
        check(load().eh_conv2d_u8_plan(C.byref(self.handle), C.byref(desc), d_w.ptr, d_b.ptr if d_b else None,
                                       C.byref(q), stream))



def make_requant_perchannel(s_in, zp_in, filter_scales, s_out, zp_out, act=ACT_NONE, act_enabled=False):
    """(Requant, multipliers, shifts) as the per-channel quantized convolution derives them at execute()."""
    scales = np.ascontiguousarray(filter_scales, np.float32)
    mult, shift = np.zeros(scales.size, np.int32), np.zeros(scales.size, np.int32)
    q = Requant()
    load().eh_make_requant_perchannel(s_in, zp_in, scales.ctypes.data, scales.size, s_out, zp_out, act, int(act_enabled),
                                      C.byref(q), mult.ctypes.data, shift.ctypes.data)
    return q, mult, shift


def _conv_run_add(self, d_in, d_residual, d_out, q, aq, stream=None):
    """d_out = add(d_residual, convolution(d_in)) with the add parameters `aq` (the residual is the first operand)"""
    check(load().eh_conv2d_u8_run_add(self.handle, d_in.ptr, d_residual.ptr, d_out.ptr, C.byref(q), C.byref(aq), stream))


def _conv_run_static(self, d_in, d_out, q, stream=None):
    """ConvPlan.run through the entry point that allocates nothing (planar plans stage in the library's static scratch)"""
    check(load().eh_conv2d_u8_run_static(self.handle, d_in.ptr, d_out.ptr, C.byref(q), stream))


STATIC_SCRATCH_BYTES = 32 << 20
ConvPlan.run_static = _conv_run_static
ConvPlan.run_add = _conv_run_add
ConvPlan.fuses_add = lambda self: bool(load().eh_conv2d_u8_fuses_add(self.handle))


class DwConvPlan(_Plan):
    _kind = "dwconv2d"

    def __init__(self, desc, d_w, d_b, q, stream=None):
        super().__init__()
        self.desc = desc
        check(load().eh_dwconv2d_u8_plan(C.byref(self.handle), C.byref(desc), d_w.ptr, d_b.ptr if d_b else None,
                                         C.byref(q), stream))


class DeconvPlan(_Plan):
    _kind = "deconv2d"

    def __init__(self, desc, d_w, d_b, q, stream=None):
        super().__init__()
        self.desc = desc
        check(load().eh_deconv2d_u8_plan(C.byref(self.handle), C.byref(desc), d_w.ptr, d_b.ptr if d_b else None,
                                         C.byref(q), stream))


class FcPlan(_Plan):
    _kind = "fc"

    def __init__(self, m, k, n, d_w, d_b, q, stream=None, flags=0):
        """flags: any of W_SIGNED | IO_SIGNED | EXACT_CHANNELS"""
        super().__init__()
        self.m, self.k, self.n = m, k, n
        if flags:
            check(load().eh_fc_q8_plan(C.byref(self.handle), m, k, n, flags, d_w.ptr, d_b.ptr if d_b else None, C.byref(q), stream))
        else:
            check(load().eh_fc_u8_plan(C.byref(self.handle), m, k, n, d_w.ptr, d_b.ptr if d_b else None, C.byref(q), stream))


class Event:
    def __init__(self):
        self.h = C.c_void_p()
        check(load().eh_event_create(C.byref(self.h)))

    def record(self, stream=None):
        check(load().eh_event_record(self.h, stream))

    def wait_on(self, stream=None):
        """Makes later work on `stream` (a raw handle or None) wait for what this event recorded."""
        check(load().eh_stream_wait_event(stream, self.h))

    def elapsed_ms_since(self, start):
        ms = C.c_float()
        check(load().eh_event_elapsed_ms(start.h, self.h, C.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            load().eh_event_destroy(self.h)
        except Exception:
            pass


class Stream:
    def __init__(self):
        self.h = C.c_void_p()
        check(load().eh_stream_create(C.byref(self.h)))

    def sync(self):
        check(load().eh_stream_sync(self.h))

    def __del__(self):
        try:
            load().eh_stream_destroy(self.h)
        except Exception:
            pass


class Graph:
    """Captures whatever `record(stream_handle)` launches and replays it."""

    def __init__(self, stream, record):
        self.h = C.c_void_p()
        check(load().eh_graph_begin(stream.h))
        try:
            record(stream.h)
        finally:
            rc = load().eh_graph_end(stream.h, C.byref(self.h))
        check(rc)

    def launch(self, stream):
        check(load().eh_graph_launch(self.h, stream.h))

    def __del__(self):
        try:
            load().eh_graph_destroy(self.h)
        except Exception:
            pass


def sync(stream=None):
    check(load().eh_stream_sync(stream))
