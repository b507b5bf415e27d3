"""Per-channel quantized convolution (int8 weights, one multiplier and shift per output channel) on the GPU
against the oracle, and the reference's own uint8 known-answer test for it
(src/userdriver/gpu/unittest/gpu_userdriver_test.cc:474-576)."""
import json
import os

import numpy as np
import pytest

import oracle_lib as O
from harness import eden, synth, to_eh_add, to_eh_requant

pytestmark = pytest.mark.gpu

KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))
SEED = 0xEDE2 + 16 * 9


def gpu_conv_perchannel(x_nchw, w_i8_oihw, bias, s, q, mults, shifts, layout, weight_layout=None):
    ho, wo = O.conv_out_hw(s)
    weight_layout = eden.W_OIHW if weight_layout is None else weight_layout
    flags, layout = layout & ~0xFF, layout & 0xFF   # (eden.EXACT_CHANNELS may ride on the layout)
    desc = eden.conv_desc(s.n, s.c, s.h, s.w, s.cout, s.kh, s.kw, (s.stride_h, s.stride_w),
                          (s.pad_t, s.pad_b, s.pad_l, s.pad_r), (s.dil_h, s.dil_w), s.groups, 1, layout | flags,
                          weight_layout | eden.W_SIGNED)
    x_dev = x_nchw if layout == eden.NCHW else x_nchw.transpose(0, 2, 3, 1)
    w_dev = w_i8_oihw if weight_layout == eden.W_OIHW else w_i8_oihw.transpose(0, 2, 3, 1)
    d_x, d_w, d_b = eden.DeviceBuffer(host=x_dev), eden.DeviceBuffer(host=w_dev), eden.DeviceBuffer(host=bias)
    d_o = eden.DeviceBuffer(nbytes=s.n * s.cout * ho * wo)
    plan = eden.ConvPlan(desc, d_w, d_b, q)
    plan.set_perchannel(mults, shifts)
    plan.run(d_x, d_o, q)
    out = d_o.download((s.n, s.cout, ho, wo)) if layout == eden.NCHW else d_o.download((s.n, ho, wo, s.cout)).transpose(0, 3, 1, 2)
    # back to the per-tensor pair of the requant: the plan must follow
    plan.set_perchannel(None, None)
    plan.run(d_x, d_o, q)
    uniform = d_o.download((s.n, s.cout, ho, wo)) if layout == eden.NCHW else d_o.download((s.n, ho, wo, s.cout)).transpose(0, 3, 1, 2)
    plan.destroy()
    return np.ascontiguousarray(out), np.ascontiguousarray(uniform)


def test_reference_uint8_perchannel_kat_on_gpu():
    k = KATS["conv_perchannel_u8"]
    n, c, h, w = k["in_dims_nchw"]
    cout, kh, kw, cin = k["w_dims_ohwi"]
    x = np.array(k["input"], np.uint8).reshape(n, c, h, w)
    wt = np.array(k["weight_i8"], np.int8).reshape(cout, kh, kw, cin).transpose(0, 3, 1, 2)
    q, mults, shifts = eden.make_requant_perchannel(k["in_scale"], k["in_zp"], k["w_scales"], k["out_scale"], k["out_zp"])
    s = O.conv_shape(n, c, h, w, cout, kh, kw)
    for layout in (eden.NCHW, eden.NHWC):
        got, _ = gpu_conv_perchannel(x, wt, np.array(k["bias"], np.int32), s, q, mults, shifts, layout, eden.W_OHWI)
        assert got.reshape(-1).tolist() == k["expect"], layout


PC_CASES = [
    dict(n=2, c=64, h=14, w=14, cout=96, kh=3, kw=3, pad=(1, 1, 1, 1)),                 # direct-to-LDS tiles, k-table
    dict(n=1, c=3, h=20, w=20, cout=32, kh=3, kw=3, stride=(2, 2), pad=(1, 1, 1, 1)),    # first-layer kernel
    dict(n=2, c=3, h=21, w=20, cout=40, kh=7, kw=7, stride=(2, 2), pad=(3, 3, 3, 3)),    # few-channel kernel-row kernel
    dict(n=2, c=48, h=16, w=16, cout=40, kh=3, kw=3, pad=(1, 1, 1, 1)),                  # patch kernel, channels 16 (mod 32)
    dict(n=2, c=24, h=9, w=9, cout=40, kh=1, kw=1),                                      # one-tap kernel, ragged channel blocks
    dict(n=1, c=20, h=8, w=8, cout=12, kh=3, kw=3, groups=2),                            # channel-padded copy (EXACT_CHANNELS: register-staged kernel), groups
    dict(n=2, c=21, h=9, w=10, cout=21, kh=3, kw=3, pad=(1, 1, 1, 1)),                   # channel-padded copy, patch kernel
    dict(n=2, c=768, h=7, w=7, cout=200, kh=3, kw=3, pad=(1, 1, 1, 1)),                  # reduction sliced over workgroups
    dict(n=2, c=64, h=10, w=10, cout=64, kh=3, kw=3, pad=(1, 1, 1, 1), groups=16),       # block-diagonal bundle of 16 groups
    dict(n=4, c=264, h=28, w=28, cout=256, kh=1, kw=1),                                  # few tiles: reduction split over waves
    dict(n=32, c=264, h=28, w=28, cout=256, kh=1, kw=1),                                 # 128 x 128 tiles
    dict(n=33, c=68, h=28, w=28, cout=64, kh=1, kw=1),                                   # 128 x 64 tiles
]


@pytest.mark.parametrize("layout", [eden.NCHW, eden.NHWC, eden.NHWC | eden.EXACT_CHANNELS], ids=["nchw", "nhwc", "nhwc_exact_channels"])
@pytest.mark.parametrize("case", PC_CASES, ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_perchannel_conv_matches_oracle(case, layout):
    if layout & eden.EXACT_CHANNELS and (case["c"] // case.get("groups", 1)) % 4 == 0:
        pytest.skip("the flag matters for the cases that would stage a padded copy")
    print("per-channel conv", case, layout, flush=True)
    s = O.conv_shape(**case)
    x = synth.fill_u8((s.n, s.c, s.h, s.w), SEED + s.c)
    w = (synth.fill_u8((s.cout, s.c // s.groups, s.kh, s.kw), SEED + s.cout).astype(np.int16) - 128).astype(np.int8)
    b = synth.fill_i32((s.cout,), SEED + 2, -500, 500)
    fan = (s.c // s.groups) * s.kh * s.kw
    # channel scales over a 30-fold range; the common output scale keeps every channel inside the uint8 range
    w_scales = (0.002 * (1.0 + 29.0 * synth.fill_u8((s.cout,), SEED + 3) / 255.0)).astype(np.float32)
    s_in = 0.02
    s_out = float(0.02 * float(w_scales.max()) * 74.0 * 74.0 * np.sqrt(fan) / 60.0)
    q, mults, shifts = eden.make_requant_perchannel(s_in, 117, w_scales, s_out, 131, eden.ACT_NONE, False)
    assert q.zp_w == 0 and len(set(mults.tolist())) > 4
    oq = O.raw_quant(zp_in=117, zp_w=0, zp_out=131)
    want = O.conv2d_perchannel(x, w, b, s, oq, mults, shifts)
    got, uniform = gpu_conv_perchannel(x, w, b, s, q, mults, shifts, layout)
    assert np.array_equal(got, want), int((got != want).sum())
    assert want.std() > 4
    # a clamp floor at the output zero point (fused ReLU): the kernels' single-shift form drops its sign test
    q.act_min = 131
    oq_relu = O.raw_quant(zp_in=117, zp_w=0, zp_out=131, act_min=131)
    got, _ = gpu_conv_perchannel(x, w, b, s, q, mults, shifts, layout)
    assert np.array_equal(got, O.conv2d_perchannel(x, w, b, s, oq_relu, mults, shifts))
    # one channel's shift outside the single-shift form's range: the whole launch takes the two-step order
    odd_shifts = shifts.copy()
    odd_shifts[s.cout // 3] = 0
    got, _ = gpu_conv_perchannel(x, w, b, s, q, mults, odd_shifts, layout)
    assert np.array_equal(got, O.conv2d_perchannel(x, w, b, s, oq_relu, mults, odd_shifts))
    q.act_min = 0
    # per-tensor mode on the same plan: int8 weights with the requant's own pair
    q2 = eden.Requant(117, 0, 131, int(mults[0]), int(shifts[0]), 0, 255)
    oq2 = O.raw_quant(zp_in=117, zp_w=0, zp_out=131, multiplier=int(mults[0]), shift=int(shifts[0]))
    want2 = O.conv2d_perchannel(x, w, b, s, oq2, np.full(s.cout, mults[0], np.int32), np.full(s.cout, shifts[0], np.int32))
    _, uniform = gpu_conv_perchannel(x, w, b, s, q2, mults, shifts, layout)
    assert np.array_equal(uniform, want2)


ONE_TAP_PC_CASES = [
    dict(n=3, c=16, h=20, w=21, cout=96, kh=1, kw=1),    # one reduction step, three channel blocks
    dict(n=2, c=64, h=15, w=15, cout=24, kh=1, kw=1),    # two steps, a ragged channel block
    dict(n=2, c=96, h=14, w=14, cout=40, kh=1, kw=1),    # reduction walked in groups of steps
    dict(n=1, c=144, h=9, w=9, cout=200, kh=1, kw=1),    # several channel ranges
]


@pytest.mark.parametrize("case", ONE_TAP_PC_CASES, ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_perchannel_one_tap_kernel_single_shift_forms(case):
    """Channels-last 1x1 layers with every channel's shift in -20 .. -2 requantize from the per-channel tables in LDS:
    with and without the sign test (fused ReLU or not), with and without the row-sum term (zp_w != 0 or 0), with the
    fused residual add, and back on the two-step order when one channel's shift leaves the range."""
    print("per-channel one-tap", case, flush=True)
    s = O.conv_shape(**case)
    ho, wo = O.conv_out_hw(s)
    x = synth.fill_u8((s.n, s.c, s.h, s.w), SEED + 71)
    w = (synth.fill_u8((s.cout, s.c, 1, 1), SEED + 72).astype(np.int16) - 128).astype(np.int8)
    b = synth.fill_i32((s.cout,), SEED + 73, -5000, 5000)
    res = synth.fill_u8((s.n, s.cout, ho, wo), SEED + 74)
    w_scales = (0.002 * (1.0 + 29.0 * synth.fill_u8((s.cout,), SEED + 75) / 255.0)).astype(np.float32)
    s_out = float(0.02 * float(w_scales.max()) * 74.0 * 74.0 * np.sqrt(s.c) / 60.0)
    desc = eden.conv_desc(s.n, s.c, s.h, s.w, s.cout, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), 1, 1, eden.NHWC, eden.W_OIHW | eden.W_SIGNED)
    d_x, d_w, d_b = eden.DeviceBuffer(host=x.transpose(0, 2, 3, 1)), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    d_r = eden.DeviceBuffer(host=np.ascontiguousarray(res.transpose(0, 2, 3, 1)))
    d_o = eden.DeviceBuffer(nbytes=s.n * s.cout * ho * wo)
    aq = O.make_add_quant(0.031, 120, s_out, 131, 0.05, 125, O.ACT_NONE, False)
    plan = None
    for zp_w in (0, -7):
        for act_min, zp_out in ((0, 131), (131, 131), (3, 0)):     # sign test needed / ReLU at the zero point / ReLU6-like floor
            q, mults, shifts = eden.make_requant_perchannel(0.02, 117, w_scales, s_out, zp_out, eden.ACT_NONE, False)
            q.zp_w, q.act_min = zp_w, act_min
            assert shifts.max() <= -2 and shifts.min() >= -20
            oq = O.raw_quant(zp_in=117, zp_w=zp_w, zp_out=zp_out, act_min=act_min)
            want = O.conv2d_perchannel(x, w, b, s, oq, mults, shifts)
            if plan is None:
                plan = eden.ConvPlan(desc, d_w, d_b, q)
            plan.set_perchannel(mults, shifts)
            plan.run(d_x, d_o, q)
            got = d_o.download((s.n, ho, wo, s.cout)).transpose(0, 3, 1, 2)
            assert np.array_equal(got, want), (zp_w, act_min, int((got != want).sum()))
            if zp_out == 131:
                plan.run_add(d_x, d_r, d_o, q, to_eh_add(aq))
                got = d_o.download((s.n, ho, wo, s.cout)).transpose(0, 3, 1, 2)
                assert np.array_equal(got, O.add(res, want, aq))
    assert want.std() > 4
    # shifts the tables do not cover: -1 (the rounding term's low word differs) and 0
    for odd in (-1, 0):
        odd_shifts = shifts.copy()
        odd_shifts[s.cout // 2] = odd
        plan.set_perchannel(mults, odd_shifts)
        plan.run(d_x, d_o, q)
        got = d_o.download((s.n, ho, wo, s.cout)).transpose(0, 3, 1, 2)
        assert np.array_equal(got, O.conv2d_perchannel(x, w, b, s, oq, mults, odd_shifts))
    plan.destroy()


def _pairs_for(s_in, w_scales, s_out):
    q, mults, shifts = eden.make_requant_perchannel(s_in, 117, w_scales, s_out, 131, eden.ACT_NONE, False)
    return q, mults, shifts


DW_PC_CASES = [
    dict(n=2, c=32, h=15, w=14, cout=32, kh=3, kw=3, stride=(1, 1), pad=(1, 1, 1, 1)),              # 3x3 tile kernel, stride 1
    dict(n=2, c=24, h=15, w=17, cout=24, kh=3, kw=3, stride=(2, 2), pad=(0, 1, 0, 1)),              # 3x3 tile kernel, stride 2
    dict(n=1, c=16, h=12, w=12, cout=16, kh=5, kw=5, stride=(1, 1), pad=(2, 2, 2, 2)),              # four-channel kernel
    dict(n=1, c=16, h=12, w=12, cout=16, kh=3, kw=3, stride=(1, 1), pad=(2, 2, 2, 2), dil=(2, 2)),  # 3x3 dilated tile, columns shared
    dict(n=2, c=8, h=14, w=17, cout=8, kh=3, kw=3, stride=(1, 1), pad=(4, 4, 4, 4), dil=(4, 4)),    # 3x3 dilated tile, columns shared
    dict(n=1, c=24, h=13, w=11, cout=24, kh=3, kw=3, stride=(1, 1), pad=(3, 3, 3, 3), dil=(3, 3)),  # 3x3 dilated tile, three column groups
    dict(n=1, c=16, h=12, w=12, cout=16, kh=3, kw=3, stride=(2, 2), pad=(2, 2, 2, 2), dil=(2, 2)),  # four-channel kernel: dilated with stride 2
    dict(n=2, c=5, h=9, w=8, cout=10, kh=3, kw=3, stride=(2, 1), pad=(1, 0, 1, 1), dm=2),           # ten outputs: computed as twelve (planar: one output per thread)
    dict(n=2, c=30, h=11, w=10, cout=30, kh=3, kw=3, stride=(1, 1), pad=(1, 1, 1, 1)),              # 30 channels computed as 32
    dict(n=44, c=32, h=112, w=112, cout=32, kh=3, kw=3, stride=(1, 1), pad=(1, 1, 1, 1)),           # 3x3 tile kernel, eight outputs per thread
]


@pytest.mark.parametrize("layout", [eden.NCHW, eden.NHWC, eden.NCHW | eden.EXACT_CHANNELS], ids=["nchw", "nhwc", "nchw_unstaged"])
@pytest.mark.parametrize("case", DW_PC_CASES, ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_perchannel_depthwise_matches_oracle(case, layout):
    if layout & eden.EXACT_CHANNELS and (case["cout"] % 4 != 0 or case.get("dm", 1) != 1 or case["n"] > 8):
        pytest.skip("no staging either way (or a case too large for the one-output-per-thread kernel to be worth timing)")
    print("per-channel depthwise", case, layout, flush=True)
    flags, layout = layout & ~0xFF, layout & 0xFF
    s = O.conv_shape(**case)
    cout = s.c * max(s.dm, 1)
    x = synth.fill_u8((s.n, s.c, s.h, s.w), SEED + 21)
    w = (synth.fill_u8((cout, 1, s.kh, s.kw), SEED + 22).astype(np.int16) - 128).astype(np.int8)
    b = synth.fill_i32((cout,), SEED + 23, -500, 500)
    w_scales = (0.002 * (1.0 + 29.0 * synth.fill_u8((cout,), SEED + 24) / 255.0)).astype(np.float32)
    s_out = float(0.02 * float(w_scales.max()) * 74.0 * 74.0 * np.sqrt(s.kh * s.kw) / 60.0)
    for zp_w in (0, -9):
        q, mults, shifts = _pairs_for(0.02, w_scales, s_out)
        q.zp_w = zp_w
        oq = O.raw_quant(zp_in=117, zp_w=zp_w, zp_out=131)
        want = O.dwconv2d_perchannel(x, w, b, s, oq, mults, shifts)
        desc = eden.conv_desc(s.n, s.c, s.h, s.w, cout, s.kh, s.kw, (s.stride_h, s.stride_w),
                              (s.pad_t, s.pad_b, s.pad_l, s.pad_r), (s.dil_h, s.dil_w), 1, max(s.dm, 1), layout | flags,
                              eden.W_OIHW | eden.W_SIGNED)
        ho, wo = O.conv_out_hw(s)
        x_dev = x if layout == eden.NCHW else x.transpose(0, 2, 3, 1)
        d_x, d_w, d_b = eden.DeviceBuffer(host=x_dev), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
        d_o = eden.DeviceBuffer(nbytes=s.n * cout * ho * wo)
        plan = eden.DwConvPlan(desc, d_w, d_b, q)
        plan.set_perchannel(mults, shifts)
        plan.run(d_x, d_o, q)
        got = d_o.download((s.n, cout, ho, wo)) if layout == eden.NCHW else d_o.download((s.n, ho, wo, cout)).transpose(0, 3, 1, 2)
        assert np.array_equal(got, want), int((got != want).sum())
        assert want.std() > 4
        # two pairs outside the range of the kernels' single-shift form: the whole plan takes the two-step order
        odd_shifts = shifts.copy()
        odd_shifts[0], odd_shifts[1] = 0, -21
        plan.set_perchannel(mults, odd_shifts)
        plan.run(d_x, d_o, q)
        got = d_o.download((s.n, cout, ho, wo)) if layout == eden.NCHW else d_o.download((s.n, ho, wo, cout)).transpose(0, 3, 1, 2)
        assert np.array_equal(got, O.dwconv2d_perchannel(x, w, b, s, oq, mults, odd_shifts))
        # back to one pair: int8 weights, per-tensor requant
        plan.set_perchannel(None, None)
        q1 = eden.Requant(117, zp_w, 131, int(mults[1]), int(shifts[1]), 0, 255)
        plan.run(d_x, d_o, q1)
        got = d_o.download((s.n, cout, ho, wo)) if layout == eden.NCHW else d_o.download((s.n, ho, wo, cout)).transpose(0, 3, 1, 2)
        want = O.dwconv2d_perchannel(x, w, b, s, oq, np.full(cout, mults[1], np.int32), np.full(cout, shifts[1], np.int32))
        assert np.array_equal(got, want)
        plan.destroy()


DECONV_PC_CASES = [
    dict(n=2, c=64, h=14, w=14, cout=32, kh=2, kw=2, stride=(2, 2)),                       # four equal phases in one launch
    dict(n=1, c=24, h=7, w=9, cout=40, kh=3, kw=3, stride=(2, 2), pad=(1, 0, 1, 0)),       # unequal phases
    dict(n=2, c=12, h=6, w=5, cout=8, kh=4, kw=4, stride=(2, 2), pad=(1, 1, 1, 1), groups=2),
    dict(n=1, c=16, h=8, w=8, cout=16, kh=3, kw=3, stride=(1, 1), pad=(1, 1, 1, 1)),
    dict(n=2, c=16, h=7, w=6, cout=24, kh=6, kw=6, stride=(3, 3)),                         # three kernel columns per problem: the pairs repeat per column
    dict(n=1, c=21, h=6, w=6, cout=21, kh=8, kw=8, stride=(4, 4), pad=(2, 2, 2, 2)),       # ... on a channel-padded copy, two classes of two columns
]


@pytest.mark.parametrize("layout", [eden.NCHW, eden.NHWC], ids=["nchw", "nhwc"])
@pytest.mark.parametrize("case", DECONV_PC_CASES, ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_perchannel_deconv_matches_oracle(case, layout):
    print("per-channel deconvolution", case, layout, flush=True)
    s = O.conv_shape(**case)
    x = synth.fill_u8((s.n, s.c, s.h, s.w), SEED + 31)
    w = (synth.fill_u8((s.c, s.cout // s.groups, s.kh, s.kw), SEED + 32).astype(np.int16) - 128).astype(np.int8)
    b = synth.fill_i32((s.cout,), SEED + 33, -500, 500)
    w_scales = (0.002 * (1.0 + 29.0 * synth.fill_u8((s.cout,), SEED + 34) / 255.0)).astype(np.float32)
    taps = max(1, (s.kh // s.stride_h) * (s.kw // s.stride_w))
    s_out = float(0.02 * float(w_scales.max()) * 74.0 * 74.0 * np.sqrt(taps * s.c // s.groups) / 60.0)
    q, mults, shifts = _pairs_for(0.02, w_scales, s_out)
    oq = O.raw_quant(zp_in=117, zp_w=0, zp_out=131)
    want = O.deconv2d_perchannel(x, w, b, s, oq, mults, shifts)
    ho, wo = O.deconv_out_hw(s)
    desc = eden.conv_desc(s.n, s.c, s.h, s.w, s.cout, s.kh, s.kw, (s.stride_h, s.stride_w),
                          (s.pad_t, s.pad_b, s.pad_l, s.pad_r), (1, 1), s.groups, 1, layout, eden.W_IOHW | eden.W_SIGNED)
    x_dev = x if layout == eden.NCHW else x.transpose(0, 2, 3, 1)
    d_x, d_w, d_b = eden.DeviceBuffer(host=x_dev), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    d_o = eden.DeviceBuffer(nbytes=s.n * s.cout * ho * wo)
    plan = eden.DeconvPlan(desc, d_w, d_b, q)
    plan.set_perchannel(mults, shifts)
    plan.run(d_x, d_o, q)
    got = d_o.download((s.n, s.cout, ho, wo)) if layout == eden.NCHW else d_o.download((s.n, ho, wo, s.cout)).transpose(0, 3, 1, 2)
    plan.destroy()
    assert np.array_equal(got, want), int((got != want).sum())
    assert want.std() > 4


def test_perchannel_argument_errors():
    desc = eden.conv_desc(1, 8, 6, 6, 8, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 1, 1, eden.NHWC, eden.W_OIHW | eden.W_SIGNED)
    w = np.zeros((8, 1, 3, 3), np.int8)
    q = eden.Requant(0, 0, 0, 1 << 30, -3, 0, 255)
    plan = eden.DwConvPlan(desc, eden.DeviceBuffer(host=w), None, q)
    with pytest.raises(eden.EdenHipError):
        plan.set_perchannel(np.ones(7, np.int32), np.zeros(7, np.int32))       # wrong count
    with pytest.raises(eden.EdenHipError):
        plan.set_perchannel(np.full(8, -1, np.int32), np.zeros(8, np.int32))   # negative multiplier
    plan.destroy()
