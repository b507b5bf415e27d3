"""INT8 precision on the GPU (int8 input, weight and output bytes; zero points and clamp bounds in
[-128, 127]) against the oracle's int8 functions, for every operator and kernel family."""
import numpy as np
import pytest

import oracle_lib as O
from harness import eden, synth

pytestmark = pytest.mark.gpu
SEED = 0xEDE2 + 16 * 11
FLAGS = eden.W_SIGNED | eden.IO_SIGNED


def s8(shape, seed):
    return (synth.fill_u8(shape, seed).astype(np.int16) - 128).astype(np.int8)


def quant_pair(fan, act=eden.ACT_NONE, enabled=False, zp_in=-11, zp_w=3, zp_out=-3):
    s_in, s_w = 0.02, 0.005
    s_out = float(s_in * s_w * 74.0 * 74.0 * np.sqrt(fan) / 50.0)
    return (eden.make_requant_s8(s_in, zp_in, s_w, zp_w, s_out, zp_out, act, enabled),
            O.make_quant_s8(s_in, zp_in, s_w, zp_w, s_out, zp_out, act, enabled))


def run_conv(plan_cls, desc_layouts, x, w, b, s, q, out_shape_nchw, layout, weight_layout, pairs=None):
    n, c, ho, wo = out_shape_nchw
    flags, layout = layout & ~0xFF, layout & 0xFF   # (eden.EXACT_CHANNELS may ride on the layout)
    desc = eden.conv_desc(s.n, s.c, s.h, s.w, c, s.kh, s.kw, (s.stride_h, s.stride_w), (s.pad_t, s.pad_b, s.pad_l, s.pad_r),
                          (s.dil_h, s.dil_w), s.groups if plan_cls is not eden.DwConvPlan else 1, max(s.dm, 1),
                          layout | flags | eden.IO_SIGNED, weight_layout | eden.W_SIGNED)
    x_dev = x if layout == eden.NCHW else x.transpose(0, 2, 3, 1)
    d_x, d_w, d_b = eden.DeviceBuffer(host=x_dev), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    d_o = eden.DeviceBuffer(nbytes=n * c * ho * wo)
    plan = plan_cls(desc, d_w, d_b, q)
    if pairs is not None:
        plan.set_perchannel(*pairs)
    plan.run(d_x, d_o, q)
    raw = d_o.download((n, c, ho, wo)) if layout == eden.NCHW else d_o.download((n, ho, wo, c)).transpose(0, 3, 1, 2)
    plan.destroy()
    return np.ascontiguousarray(raw).view(np.int8)


CONV_CASES = [
    dict(n=2, c=64, h=14, w=14, cout=96, kh=3, kw=3, pad=(1, 1, 1, 1)),                 # direct-to-LDS tiles, padding fill
    dict(n=1, c=3, h=20, w=20, cout=32, kh=3, kw=3, stride=(2, 2), pad=(1, 1, 1, 1)),    # first-layer kernel
    dict(n=2, c=3, h=21, w=20, cout=40, kh=7, kw=7, stride=(2, 2), pad=(3, 3, 3, 3)),    # few-channel kernel-row kernel
    dict(n=2, c=48, h=16, w=16, cout=40, kh=3, kw=3, pad=(1, 1, 1, 1)),                  # patch kernel, channels 16 (mod 32)
    dict(n=2, c=24, h=9, w=9, cout=40, kh=1, kw=1),                                      # one-tap kernel
    dict(n=1, c=20, h=8, w=8, cout=12, kh=3, kw=3, pad=(1, 1, 1, 1), groups=2),          # channel-padded copy (EXACT_CHANNELS: register-staged kernel)
    dict(n=2, c=21, h=9, w=10, cout=21, kh=3, kw=3, pad=(1, 1, 1, 1)),                   # channel-padded copy: int8 padding bytes
    dict(n=2, c=768, h=7, w=7, cout=200, kh=3, kw=3, pad=(1, 1, 1, 1)),                  # reduction sliced over workgroups
    dict(n=2, c=64, h=10, w=10, cout=64, kh=3, kw=3, pad=(1, 1, 1, 1), groups=16),       # block-diagonal bundle of 16 groups
    dict(n=32, c=264, h=28, w=28, cout=256, kh=1, kw=1),                                 # 128 x 128 tiles, no row sums needed? (zp_w != 0: needed)
    dict(n=1, c=200, h=6, w=6, cout=64, kh=3, kw=3, pad=(1, 1, 1, 1)),                   # reduction not a multiple of the slab
]


@pytest.mark.parametrize("layout", [eden.NCHW, eden.NHWC, eden.NHWC | eden.EXACT_CHANNELS], ids=["nchw", "nhwc", "nhwc_exact_channels"])
@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_int8_conv_matches_oracle(case, layout):
    if layout & eden.EXACT_CHANNELS and (case["c"] // case.get("groups", 1)) % 4 == 0:
        pytest.skip("the flag matters for the cases that would stage a padded copy")
    print("int8 conv", case, layout, flush=True)
    s = O.conv_shape(**case)
    x = s8((s.n, s.c, s.h, s.w), SEED + s.c)
    w = s8((s.cout, s.c // s.groups, s.kh, s.kw), SEED + s.cout)
    b = synth.fill_i32((s.cout,), SEED + 2, -500, 500)
    ho, wo = O.conv_out_hw(s)
    for act, enabled in ((eden.ACT_NONE, False), (eden.ACT_RELU6, True)):
        q, oq = quant_pair((s.c // s.groups) * s.kh * s.kw, act, enabled)
        assert q.as_tuple() == oq.as_tuple()
        want = O.conv2d_s8(x, w, b, s, oq)
        got = run_conv(eden.ConvPlan, None, x, w, b, s, q, (s.n, s.cout, ho, wo), layout, eden.W_OIHW)
        assert np.array_equal(got, want), int((got != want).sum())
        assert want.std() > 3   # (the long reductions leave ReLU6 about eight output steps)


def test_int8_conv_perchannel_and_symmetric_weights():
    s = O.conv_shape(2, 64, 14, 14, 96, 3, 3, pad=(1, 1, 1, 1))
    x, w = s8((2, 64, 14, 14), SEED + 41), s8((96, 64, 3, 3), SEED + 42)
    b = synth.fill_i32((96,), SEED + 43, -500, 500)
    w_scales = (0.002 * (1.0 + 29.0 * synth.fill_u8((96,), SEED + 44) / 255.0)).astype(np.float32)
    s_out = float(0.02 * float(w_scales.max()) * 74.0 * 74.0 * 24.0 / 60.0)
    q, mults, shifts = eden.make_requant_perchannel(0.02, -20, w_scales, s_out, 5)
    q.act_min, q.act_max = -128, 127
    oq = O.raw_quant(zp_in=-20, zp_w=0, zp_out=5, act_min=-128, act_max=127)
    want = O.conv2d_s8(x, w, b, s, oq, mults, shifts)
    got = run_conv(eden.ConvPlan, None, x, w, b, s, q, (2, 96, 14, 14), eden.NHWC, eden.W_OIHW, (mults, shifts))
    assert np.array_equal(got, want) and want.std() > 4


DW_CASES = [
    dict(n=2, c=32, h=15, w=14, cout=32, kh=3, kw=3, stride=(1, 1), pad=(1, 1, 1, 1)),
    dict(n=2, c=24, h=15, w=17, cout=24, kh=3, kw=3, stride=(2, 2), pad=(0, 1, 0, 1)),
    dict(n=1, c=16, h=12, w=12, cout=16, kh=5, kw=5, stride=(1, 1), pad=(2, 2, 2, 2)),
    dict(n=2, c=8, h=17, w=15, cout=8, kh=7, kw=7, stride=(2, 2), pad=(3, 3, 3, 3)),
    dict(n=2, c=5, h=9, w=8, cout=10, kh=3, kw=3, stride=(2, 1), pad=(1, 0, 1, 1), dm=2),
    dict(n=2, c=16, h=17, w=14, cout=16, kh=3, kw=3, stride=(1, 1), pad=(2, 2, 2, 2), dil=(2, 2)),   # dilated 3x3 tiles
    dict(n=1, c=8, h=13, w=19, cout=8, kh=3, kw=3, stride=(1, 1), pad=(4, 4, 4, 4), dil=(4, 4)),
    dict(n=1, c=12, h=16, w=15, cout=12, kh=3, kw=3, stride=(1, 1), pad=(5, 5, 5, 5), dil=(5, 5)),
    dict(n=2, c=30, h=11, w=10, cout=30, kh=3, kw=3, stride=(1, 1), pad=(1, 1, 1, 1)),             # 30 channels computed as 32
]


@pytest.mark.parametrize("layout", [eden.NCHW, eden.NHWC, eden.NCHW | eden.EXACT_CHANNELS], ids=["nchw", "nhwc", "nchw_unstaged"])
@pytest.mark.parametrize("case", DW_CASES + [dict(n=2, c=8, h=11, w=10, cout=16, kh=3, kw=3, stride=(1, 1), pad=(1, 1, 1, 1), dm=2)],
                         ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_int8_depthwise_matches_oracle(case, layout):
    if layout & eden.EXACT_CHANNELS and (case["cout"] % 4 != 0 or case.get("dm", 1) != 1):
        pytest.skip("no staging either way")
    print("int8 depthwise", case, layout, flush=True)
    s = O.conv_shape(**case)
    cout = s.c * max(s.dm, 1)
    x, w = s8((s.n, s.c, s.h, s.w), SEED + 51), s8((cout, 1, s.kh, s.kw), SEED + 52)
    b = synth.fill_i32((cout,), SEED + 53, -500, 500)
    ho, wo = O.conv_out_hw(s)
    for act, enabled in ((eden.ACT_NONE, False), (eden.ACT_RELU6, True)):
        q, oq = quant_pair(s.kh * s.kw, act, enabled, zp_out=-128 if enabled else -3)
        want = O.dwconv2d_s8(x, w, b, s, oq)
        got = run_conv(eden.DwConvPlan, None, x, w, b, s, q, (s.n, cout, ho, wo), layout, eden.W_OIHW)
        assert np.array_equal(got, want), int((got != want).sum())
        assert want.std() > 4


@pytest.mark.parametrize("case", [DW_CASES[-1],
                                  dict(n=3, c=7, h=14, w=11, cout=7, kh=3, kw=3, stride=(2, 2), pad=(1, 2, 0, 0)),
                                  dict(n=3, c=7, h=9, w=4, cout=7, kh=3, kw=3, stride=(2, 2), pad=(4, 1, 2, 0), dil=(2, 2))],
                         ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_int8_depthwise_on_ragged_channels_without_staging(case):
    """Channels-last 3x3 with a channel count that is no multiple of four and the plan told not to stage: the kernel
    with one output per thread runs, and reads the weights about the zero point the caller gave (the plan also holds
    the dot-product form of the weights, whose zero point is shifted by 128 for int8 weights)."""
    print("int8 depthwise, ragged channels unstaged", case, flush=True)
    s = O.conv_shape(**case)
    x, w = s8((s.n, s.c, s.h, s.w), SEED + 61), s8((s.c, 1, s.kh, s.kw), SEED + 62)
    b = synth.fill_i32((s.c,), SEED + 63, -500, 500)
    ho, wo = O.conv_out_hw(s)
    q, oq = quant_pair(s.kh * s.kw, eden.ACT_NONE, False, zp_out=-3)
    want = O.dwconv2d_s8(x, w, b, s, oq)
    got = run_conv(eden.DwConvPlan, None, x, w, b, s, q, (s.n, s.c, ho, wo), eden.NHWC | eden.EXACT_CHANNELS, eden.W_OIHW)
    assert np.array_equal(got, want), int((got != want).sum())
    assert want.std() > 4


@pytest.mark.parametrize("case", DW_CASES[:2] + DW_CASES[-4:] + [dict(n=40, c=64, h=64, w=64, cout=64, kh=3, kw=3, stride=(1, 1), pad=(1, 1, 1, 1))],
                         ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_int8_depthwise_weights_within_int8_of_their_zero_point(case):
    """channels-last 3x3 with every w - zp_w inside int8: the 8-bit dot product kernel on int8 tensors"""
    print("int8 depthwise, narrow weights", case, flush=True)
    s = O.conv_shape(**case)
    x = s8((s.n, s.c, s.h, s.w), SEED + 54)
    w = (synth.fill_u8((s.c, 1, 3, 3), SEED + 55).astype(np.int16) % 200 - 100).astype(np.int8)
    w.reshape(-1)[0], w.reshape(-1)[1] = -125, 127    # zp_w - 128 and the top of the range
    b = synth.fill_i32((s.c,), SEED + 56, -500, 500)
    ho, wo = O.conv_out_hw(s)
    for act, enabled in ((eden.ACT_NONE, False), (eden.ACT_RELU6, True)):
        q, oq = quant_pair(9, act, enabled, zp_out=-128 if enabled else -3)
        want = O.dwconv2d_s8(x, w, b, s, oq)
        got = run_conv(eden.DwConvPlan, None, x, w, b, s, q, (s.n, s.c, ho, wo), eden.NHWC, eden.W_OIHW)
        assert np.array_equal(got, want), int((got != want).sum())
        assert want.std() > 4


DW_PC_S8_CASES = DW_CASES[-4:] + [
    dict(n=2, c=32, h=15, w=14, cout=32, kh=3, kw=3, stride=(1, 1), pad=(1, 1, 1, 1)),     # four outputs per thread, stride 1
    dict(n=2, c=24, h=15, w=17, cout=24, kh=3, kw=3, stride=(2, 2), pad=(0, 1, 0, 1)),     # four outputs per thread, stride 2
    dict(n=44, c=32, h=112, w=112, cout=32, kh=3, kw=3, stride=(1, 1), pad=(1, 1, 1, 1)),  # eight outputs per thread
]


@pytest.mark.parametrize("case", DW_PC_S8_CASES, ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_int8_perchannel_depthwise_dot_product_form(case):
    """The full-integer depthwise layer of a TFLite model: int8 tensors, int8 weights at zero point 0 and one
    multiplier / shift per channel.  Every weight fits int8 about its zero point by construction, so channels-last
    3x3 plans run the 8-bit dot product kernel's per-channel variant."""
    print("int8 per-channel depthwise", case, flush=True)
    s = O.conv_shape(**case)
    x, w = s8((s.n, s.c, s.h, s.w), SEED + 91), s8((s.c, 1, 3, 3), SEED + 92)
    w.reshape(-1)[0], w.reshape(-1)[1] = -128, 127
    b = synth.fill_i32((s.c,), SEED + 93, -500, 500)
    w_scales = (0.002 * (1.0 + 29.0 * synth.fill_u8((s.c,), SEED + 94) / 255.0)).astype(np.float32)
    s_out = float(0.02 * float(w_scales.max()) * 74.0 * 74.0 * 3.0 / 60.0)
    q, mults, shifts = eden.make_requant_perchannel(0.02, -20, w_scales, s_out, 5)
    q.act_min, q.act_max = -128, 127
    assert q.zp_w == 0 and len(set(mults.tolist())) > 4
    oq = O.raw_quant(zp_in=-20, zp_w=0, zp_out=5, act_min=-128, act_max=127)
    want = O.dwconv2d_s8(x, w, b, s, oq, mults, shifts)
    ho, wo = O.conv_out_hw(s)
    got = run_conv(eden.DwConvPlan, None, x, w, b, s, q, (s.n, s.c, ho, wo), eden.NHWC, eden.W_OIHW, (mults, shifts))
    assert np.array_equal(got, want), int((got != want).sum())
    assert want.std() > 4


DECONV_CASES = [
    dict(n=2, c=64, h=14, w=14, cout=32, kh=2, kw=2, stride=(2, 2)),
    dict(n=1, c=24, h=7, w=9, cout=40, kh=3, kw=3, stride=(2, 2), pad=(1, 0, 1, 0)),
    dict(n=2, c=12, h=6, w=5, cout=8, kh=4, kw=4, stride=(2, 2), pad=(1, 1, 1, 1), groups=2),
    dict(n=1, c=21, h=6, w=6, cout=21, kh=8, kw=8, stride=(4, 4), pad=(2, 2, 2, 2)),       # merged kernel columns on a channel-padded copy
]


@pytest.mark.parametrize("layout", [eden.NCHW, eden.NHWC], ids=["nchw", "nhwc"])
@pytest.mark.parametrize("case", DECONV_CASES, ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_int8_deconv_matches_oracle(case, layout):
    print("int8 deconvolution", case, layout, flush=True)
    s = O.conv_shape(**case)
    x, w = s8((s.n, s.c, s.h, s.w), SEED + 61), s8((s.c, s.cout // s.groups, s.kh, s.kw), SEED + 62)
    b = synth.fill_i32((s.cout,), SEED + 63, -500, 500)
    taps = max(1, (s.kh // s.stride_h) * (s.kw // s.stride_w))
    q, oq = quant_pair(taps * s.c // s.groups)
    want = O.deconv2d_s8(x, w, b, s, oq)
    ho, wo = O.deconv_out_hw(s)
    got = run_conv(eden.DeconvPlan, None, x, w, b, s, q, (s.n, s.cout, ho, wo), layout, eden.W_IOHW)
    assert np.array_equal(got, want), int((got != want).sum())
    assert want.std() > 4


@pytest.mark.parametrize("m,k,n", [(64, 512, 256), (5, 100, 33), (256, 4096, 512), (3, 1024, 200)])
def test_int8_fc_matches_oracle(m, k, n):
    print("int8 fc", m, k, n, flush=True)
    a, w = s8((m, k), SEED + 71), s8((n, k), SEED + 72)
    b = synth.fill_i32((n,), SEED + 73, -500, 500)
    q, oq = quant_pair(k, eden.ACT_RELU, True)
    want = O.fc_s8(a, w, b, oq)
    d_a, d_w, d_b = eden.DeviceBuffer(host=a), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    d_o = eden.DeviceBuffer(nbytes=m * n)
    plan = eden.FcPlan(m, k, n, d_w, d_b, q, flags=FLAGS)
    plan.run(d_a, d_o, q)
    got = d_o.download((m, n)).view(np.int8)
    plan.destroy()
    assert np.array_equal(got, want), int((got != want).sum())
    assert want.std() > 4


def test_int8_flags_are_independent_and_checked():
    """uint8 weights with int8 activations (and the reverse) are the same arithmetic on shifted bytes."""
    s = O.conv_shape(1, 32, 9, 9, 32, 3, 3, pad=(1, 1, 1, 1))
    x, w = s8((1, 32, 9, 9), SEED + 81), synth.fill_u8((32, 32, 3, 3), SEED + 82)
    b = synth.fill_i32((32,), SEED + 83, -500, 500)
    q = eden.Requant(-5, 120, 9, 1518500250, -9, -128, 127)
    oq = O.raw_quant(zp_in=-5, zp_w=120 - 128, zp_out=9, multiplier=1518500250, shift=-9, act_min=-128, act_max=127)
    want = O.conv2d_s8(x, (w.astype(np.int16) - 128).astype(np.int8), b, s, oq)
    desc = eden.conv_desc(1, 32, 9, 9, 32, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 1, 1, eden.NHWC | eden.IO_SIGNED, eden.W_OIHW)
    d_x, d_w, d_b = eden.DeviceBuffer(host=x.transpose(0, 2, 3, 1)), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    d_o = eden.DeviceBuffer(nbytes=want.size)
    plan = eden.ConvPlan(desc, d_w, d_b, q)
    plan.run(d_x, d_o, q)
    got = d_o.download((1, 9, 9, 32)).transpose(0, 3, 1, 2).view(np.int8)
    assert np.array_equal(got, want) and want.std() > 4
    with pytest.raises(eden.EdenHipError):
        plan.run(d_x, d_o, eden.Requant(-5, 120, 9, 1 << 30, -9, 0, 255))   # uint8 range on an int8 plan
    with pytest.raises(eden.EdenHipError):
        plan.run(d_x, d_o, eden.Requant(200, 120, 9, 1 << 30, -9, -128, 127))  # zero point outside int8
    plan.destroy()
