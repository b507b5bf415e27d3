"""Per-channel quantized convolution (int8 weights, one multiplier and shift per output channel) on the GPU
against the oracle, and the reference's own uint8 known-answer test for it
(src/userdriver/gpu/unittest/gpu_userdriver_test.cc:474-576)."""
import json
import os

import numpy as np
import pytest

import oracle_lib as O
from harness import eden, synth, to_eh_requant

pytestmark = pytest.mark.gpu

KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))
SEED = 0xEDE2 + 16 * 9


def gpu_conv_perchannel(x_nchw, w_i8_oihw, bias, s, q, mults, shifts, layout, weight_layout=None):
    ho, wo = O.conv_out_hw(s)
    weight_layout = eden.W_OIHW if weight_layout is None else weight_layout
    desc = eden.conv_desc(s.n, s.c, s.h, s.w, s.cout, s.kh, s.kw, (s.stride_h, s.stride_w),
                          (s.pad_t, s.pad_b, s.pad_l, s.pad_r), (s.dil_h, s.dil_w), s.groups, 1, layout,
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
    dict(n=2, c=24, h=9, w=9, cout=40, kh=1, kw=1),                                      # one-tap kernel, ragged channel blocks
    dict(n=1, c=20, h=8, w=8, cout=12, kh=3, kw=3, groups=2),                            # register-staged kernel, groups
    dict(n=4, c=264, h=28, w=28, cout=256, kh=1, kw=1),                                  # few tiles: reduction split over waves
    dict(n=32, c=264, h=28, w=28, cout=256, kh=1, kw=1),                                 # 128 x 128 tiles
    dict(n=33, c=68, h=28, w=28, cout=64, kh=1, kw=1),                                   # 128 x 64 tiles
]


@pytest.mark.parametrize("layout", [eden.NCHW, eden.NHWC], ids=["nchw", "nhwc"])
@pytest.mark.parametrize("case", PC_CASES, ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_perchannel_conv_matches_oracle(case, layout):
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
    # per-tensor mode on the same plan: int8 weights with the requant's own pair
    q2 = eden.Requant(117, 0, 131, int(mults[0]), int(shifts[0]), 0, 255)
    oq2 = O.raw_quant(zp_in=117, zp_w=0, zp_out=131, multiplier=int(mults[0]), shift=int(shifts[0]))
    want2 = O.conv2d_perchannel(x, w, b, s, oq2, np.full(s.cout, mults[0], np.int32), np.full(s.cout, shifts[0], np.int32))
    _, uniform = gpu_conv_perchannel(x, w, b, s, q2, mults, shifts, layout)
    assert np.array_equal(uniform, want2)
