"""Pointwise expansion + 3x3 depthwise convolution as one launch (eh_conv_dw_block_run): bit for bit the oracle's
pointwise-then-depthwise chain, and bit for bit what the two stand-alone launches give, over strides, paddings, channel
counts, tile heights, both depthwise dot-product forms, pointwise weights with and without a row-sum term and every
requantization form; BASELINE configs[2] at its full size."""
import numpy as np
import pytest

import oracle_lib as O
from harness import diff_report, eden, synth, to_eh_requant

pytestmark = pytest.mark.gpu
SEED = 0xB10C


def run_block(x, w1, b1, q1, w2, b2, q2, stride, pad, rows=0, separate_too=True):
    """x NHWC uint8; returns (fused NHWC output, stand-alone two-launch output or None)"""
    n, h, w, cin = x.shape
    c = w1.shape[0]
    d1 = eden.conv_desc(n, cin, h, w, c, 1, 1, layout=eden.NHWC)
    d2 = eden.conv_desc(n, c, h, w, c, 3, 3, stride=(stride, stride), pad=pad, dm=1, layout=eden.NHWC)
    ho = (h + pad[0] + pad[1] - 3) // stride + 1
    wo = (w + pad[2] + pad[3] - 3) // stride + 1
    keep = [eden.DeviceBuffer(host=a) for a in (w1, b1, w2, b2)]
    pw = eden.ConvPlan(d1, keep[0], keep[1], q1)
    dw = eden.DwConvPlan(d2, keep[2], keep[3], q2)
    assert eden.conv_dw_block_applies(pw, dw)
    d_x, d_o = eden.DeviceBuffer(host=x), eden.DeviceBuffer(nbytes=n * ho * wo * c)
    eden.conv_dw_block_run(pw, dw, d_x, d_o, q1, q2, rows)
    fused = d_o.download((n, ho, wo, c))
    apart = None
    if separate_too:
        d_mid, d_o2 = eden.DeviceBuffer(nbytes=n * h * w * c), eden.DeviceBuffer(nbytes=n * ho * wo * c)
        pw.run(d_x, d_mid, q1)
        dw.run(d_mid, d_o2, q2)
        apart = d_o2.download((n, ho, wo, c))
    pw.destroy()
    dw.destroy()
    return fused, apart


def oracle_block(x, w1, b1, q1, w2, b2, q2, stride, pad):
    n, h, w, cin = x.shape
    c = w1.shape[0]
    xp = np.ascontiguousarray(x.transpose(0, 3, 1, 2))
    mid = O.conv2d(xp, w1, b1, O.conv_shape(n, cin, h, w, c, 1, 1), q1)
    out = O.dwconv2d(mid, w2, b2, O.conv_shape(n, c, h, w, c, 3, 3, stride=(stride, stride), pad=pad, groups=c), q2)
    return np.ascontiguousarray(out.transpose(0, 2, 3, 1)), mid


def tensors(n, h, w, cin, c, seed, dw_narrow):
    x = synth.fill_u8((n, h, w, cin), seed)
    w1 = synth.fill_u8((c, cin, 1, 1), seed + 1)
    b1 = synth.fill_i32((c,), seed + 2, -1000, 1000)
    # narrow: every w - zp_w fits int8 (the signed dot-product form); else bytes span 0 .. 255 (the unsigned form)
    w2 = synth.fill_u8_normal((c, 1, 3, 3), seed + 3, 128, 20) if dw_narrow else synth.fill_u8((c, 1, 3, 3), seed + 3)
    b2 = synth.fill_i32((c,), seed + 4, -1000, 1000)
    return x, w1, b1, w2, b2


CASES = [
    # n, h, w, cin, c, stride, pad(t, b, l, r), rows, dw_narrow, pointwise zp_w
    (2, 56, 56, 24, 144, 2, (1, 1, 1, 1), 0, False, 131),   # BASELINE configs[2] geometry
    (2, 56, 56, 24, 144, 2, (1, 1, 1, 1), 4, True, 128),    # taller tiles; signed depthwise form; no row-sum term
    (1, 13, 11, 8, 16, 1, (1, 1, 1, 1), 3, False, 120),     # odd extents, stride 1, rows that do not divide the height
    (3, 14, 14, 32, 192, 1, (1, 1, 1, 1), 0, True, 140),
    (1, 15, 17, 16, 96, 2, (0, 1, 0, 1), 2, False, 125),    # TensorFlow SAME at stride 2: padding last only
    (1, 9, 9, 16, 48, 2, (1, 1, 1, 1), 1, True, 128),       # one output row per workgroup
    (2, 28, 28, 32, 192, 2, (1, 1, 1, 1), 7, False, 119),
    (1, 6, 30, 8, 160, 1, (2, 2, 2, 2), 0, False, 133),     # padding 2: two rows and columns of zero-point pixels
    (1, 7, 5, 24, 32, 1, (0, 0, 0, 0), 0, True, 128),       # no padding; output narrower than one tile of four
    # several 32-byte reduction steps and channel ranges per workgroup: MobileNetV2's later expansions
    (3, 14, 14, 64, 384, 1, (1, 1, 1, 1), 0, False, 122),
    (2, 14, 14, 96, 576, 2, (1, 1, 1, 1), 0, True, 128),
    (4, 7, 7, 160, 960, 1, (1, 1, 1, 1), 0, False, 135),
    (1, 28, 28, 32, 192, 2, (1, 1, 1, 1), 5, False, 128),
    (2, 9, 10, 40, 80, 1, (1, 1, 1, 1), 4, True, 119),      # a reduction that ends inside its second step; channels not a multiple of 32
    (1, 12, 12, 256, 48, 1, (1, 1, 1, 1), 0, False, 131),   # eight reduction steps
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(str(v) for v in c[:6]) + ("_r%d" % c[7]))
def test_block_matches_oracle_and_the_two_launches(case):
    n, h, w, cin, c, stride, pad, rows, narrow, zp_w1 = case
    print("block", case, flush=True)
    x, w1, b1, w2, b2 = tensors(n, h, w, cin, c, SEED + 7 * c + h, narrow)
    q1 = O.make_quant(0.02, 117, 0.004, zp_w1, 0.03, 5, O.ACT_RELU6, True)
    q2 = O.make_quant(0.03, 5, 0.006, 128 if narrow else 141, 0.025, 9, O.ACT_RELU6, True)
    want, mid = oracle_block(x, w1, b1, q1, w2, b2, q2, stride, pad)
    fused, apart = run_block(x, w1, b1, to_eh_requant(q1), w2, b2, to_eh_requant(q2), stride, pad, rows)
    assert np.array_equal(apart, want), diff_report(apart, want)
    assert np.array_equal(fused, want), diff_report(fused, want)
    assert want.std() > 1 and mid.std() > 1


@pytest.mark.parametrize("form", ["two_step_left_shift", "single_shift_signed", "single_shift_relu", "two_step_big_shift"])
def test_block_requantization_forms(form):
    """every requantization form of the pointwise stage and of the depthwise stage inside the fused kernel"""
    n, h, w, cin, c = 2, 12, 12, 24, 48
    x, w1, b1, w2, b2 = tensors(n, h, w, cin, c, SEED + 900, False)
    xp = np.ascontiguousarray(x.transpose(0, 3, 1, 2))
    _, acc1 = O.conv2d(xp, w1, b1, O.conv_shape(n, cin, h, w, c, 1, 1), O.raw_quant(zp_in=100, zp_w=127), want_acc=True)
    sd = float(acc1.std())
    if form == "two_step_left_shift":      # multiplier >= 1: a left shift, outside the single-shift form
        m, lo, hi, zp = 2.5, 0, 255, 128
    elif form == "single_shift_signed":    # clamp floor below the zero point: the form with the sign test
        m, lo, hi, zp = 40.0 / sd, 0, 255, 128
    elif form == "single_shift_relu":      # clamp floor at the zero point: the form without it
        m, lo, hi, zp = 40.0 / sd, 20, 230, 20
    else:                                   # right shift beyond 20
        m, lo, hi, zp = 2.0 ** -24, 0, 255, 77
    qm, sh = O.quantize_multiplier(m)
    q1 = O.raw_quant(zp_in=100, zp_w=127, zp_out=zp, multiplier=qm, shift=sh, act_min=lo, act_max=hi)
    mid = O.conv2d(xp, w1, b1, O.conv_shape(n, cin, h, w, c, 1, 1), q1)
    s2 = O.conv_shape(n, c, h, w, c, 3, 3, stride=(1, 1), pad=(1, 1, 1, 1), groups=c)
    _, acc2 = O.dwconv2d(mid, w2, b2, s2, O.raw_quant(zp_in=zp, zp_w=130), want_acc=True)
    sd2 = float(acc2.std()) or 1.0
    m2 = {"two_step_left_shift": 1.5, "two_step_big_shift": 2.0 ** -23}.get(form, 50.0 / sd2)
    qm2, sh2 = O.quantize_multiplier(m2)
    q2 = O.raw_quant(zp_in=zp, zp_w=130, zp_out=zp, multiplier=qm2, shift=sh2, act_min=lo, act_max=hi)
    want = np.ascontiguousarray(O.dwconv2d(mid, w2, b2, s2, q2).transpose(0, 2, 3, 1))
    fused, apart = run_block(x, w1, b1, to_eh_requant(q1), w2, b2, to_eh_requant(q2), 1, (1, 1, 1, 1))
    assert np.array_equal(apart, want), diff_report(apart, want)
    assert np.array_equal(fused, want), diff_report(fused, want)
    if form.startswith("single"):
        assert want.std() > 5


def test_block_config3_full_size():
    """BASELINE configs[2] at N = 32: the fused launch against the two stand-alone launches (each of which the oracle
    checks at this size in test_gpu_parity.py), and against the oracle itself on the first and last two images."""
    n = 32
    x, w1, b1, w2, b2 = tensors(n, 56, 56, 24, 144, SEED + 3000, False)
    q1 = O.make_quant(0.02, 120, 0.004, 131, 0.03, 4, O.ACT_RELU6, True)
    q2 = O.make_quant(0.03, 4, 0.006, 140, 0.025, 9, O.ACT_RELU6, True)
    for rows in (0, 2, 4):
        fused, apart = run_block(x, w1, b1, to_eh_requant(q1), w2, b2, to_eh_requant(q2), 2, (1, 1, 1, 1), rows, separate_too=rows == 0)
        if rows == 0:
            base = apart
            for img in (0, 1, 30, 31):
                want, _ = oracle_block(x[img:img + 1], w1, b1, q1, w2, b2, q2, 2, (1, 1, 1, 1))
                assert np.array_equal(apart[img:img + 1], want), (img, diff_report(apart[img:img + 1], want))
        assert np.array_equal(fused, base), (rows, diff_report(fused, base))
    assert base.std() > 10


def test_block_refuses_what_it_does_not_fit():
    d_w = eden.DeviceBuffer(host=synth.fill_u8((64, 320, 1, 1), 1))
    d_b = eden.DeviceBuffer(host=synth.fill_i32((64,), 2, -10, 10))
    d_w2 = eden.DeviceBuffer(host=synth.fill_u8((64, 1, 3, 3), 3))
    q = eden.make_requant(0.02, 3, 0.004, 120, 0.03, 5)
    wide = eden.ConvPlan(eden.conv_desc(1, 320, 8, 8, 64, 1, 1, layout=eden.NHWC), d_w, d_b, q)   # 320 input channels: more than eight reduction steps
    dw = eden.DwConvPlan(eden.conv_desc(1, 64, 8, 8, 64, 3, 3, pad=(1, 1, 1, 1), dm=1, layout=eden.NHWC), d_w2, d_b, q)
    assert not eden.conv_dw_block_applies(wide, dw)
    d_x, d_o = eden.DeviceBuffer(nbytes=8 * 8 * 320), eden.DeviceBuffer(nbytes=8 * 8 * 64)
    with pytest.raises(eden.EdenHipError):
        eden.conv_dw_block_run(wide, dw, d_x, d_o, q, q)
    wide.destroy()
    # 21 input channels: that plan runs the one-tap kernel too, but on a channel-padded copy of its input, which the
    # fused kernel would not read
    d_w3 = eden.DeviceBuffer(host=synth.fill_u8((64, 21, 1, 1), 4))
    desc = eden.conv_desc(1, 21, 8, 8, 64, 1, 1, layout=eden.NHWC)
    assert eden.conv_kernels(desc) == ["one_tap"]
    ragged = eden.ConvPlan(desc, d_w3, d_b, q)
    assert not eden.conv_dw_block_applies(ragged, dw)
    ragged.destroy()
    dw.destroy()


def test_block_preferred_is_a_subset_of_applies_and_holds_config3():
    """The measured table: BASELINE configs[2]'s pair is in it, a pair of the same family that was measured slower
    (56 x 56 at stride 1) and an unmeasured shape are not; what does not fit is never preferred."""
    def pair(n, cin, c, hw, stride):
        d_w = eden.DeviceBuffer(host=synth.fill_u8((c, cin, 1, 1), 1))
        d_b = eden.DeviceBuffer(host=synth.fill_i32((c,), 2, -10, 10))
        d_w2 = eden.DeviceBuffer(host=synth.fill_u8((c, 1, 3, 3), 3))
        q = eden.make_requant(0.02, 3, 0.004, 120, 0.03, 5)
        pw = eden.ConvPlan(eden.conv_desc(n, cin, hw, hw, c, 1, 1, layout=eden.NHWC), d_w, d_b, q)
        dw = eden.DwConvPlan(eden.conv_desc(n, c, hw, hw, c, 3, 3, stride=(stride, stride), pad=(1, 1, 1, 1), dm=1, layout=eden.NHWC), d_w2, d_b, q)
        return pw, dw, (d_w, d_b, d_w2)
    for shape, applies, preferred in (((32, 24, 144, 56, 2), True, True), ((32, 24, 144, 56, 1), True, False),
                                      ((32, 40, 80, 20, 1), True, False), ((32, 64, 384, 14, 1), True, True),
                                      # below 32 images per launch every fitting pair is preferred (latency), none that does not fit
                                      ((2, 24, 144, 56, 2), True, True), ((8, 40, 80, 20, 1), True, True), ((24, 24, 144, 56, 1), True, True),
                                      ((4, 320, 64, 8, 1), False, False), ((32, 320, 64, 8, 1), False, False)):
        pw, dw, keep = pair(*shape)
        assert eden.conv_dw_block_applies(pw, dw) == applies, shape
        assert eden.conv_dw_block_preferred(pw, dw) == preferred, shape
        pw.destroy()
        dw.destroy()


PC_BLOCK_CASES = [
    # n, h, w, cin, c, stride, rows
    (2, 56, 56, 24, 144, 2, 0),
    (2, 28, 28, 32, 192, 1, 4),
    (3, 14, 14, 64, 384, 1, 0),
    (1, 13, 11, 16, 48, 1, 3),
    (1, 9, 10, 40, 80, 2, 0),      # a reduction that ends inside its second step; channels not a multiple of 32
]


@pytest.mark.parametrize("case", PC_BLOCK_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_block_with_one_pair_per_channel_in_both_operators(case):
    """int8 weights with one multiplier and shift per channel in the pointwise and in the depthwise operator: the fused
    launch against the oracle's per-channel chain and the two stand-alone launches; the single-shift forms with and
    without the sign test, the two-step order once a channel's shift leaves the range, a weight zero point other than 0
    (row-sum term in the pointwise stage, the unsigned dot-product form in the depthwise stage)."""
    n, h, w, cin, c, stride, rows = case
    print("per-channel block", case, flush=True)
    x = synth.fill_u8((n, h, w, cin), SEED + 5000 + c)
    w1 = (synth.fill_u8((c, cin, 1, 1), SEED + 5001).astype(np.int16) - 128).astype(np.int8)
    b1 = synth.fill_i32((c,), SEED + 5002, -500, 500)
    w2 = (synth.fill_u8((c, 1, 3, 3), SEED + 5003).astype(np.int16) - 128).astype(np.int8)
    b2 = synth.fill_i32((c,), SEED + 5004, -500, 500)
    ws1 = (0.002 * (1.0 + 29.0 * synth.fill_u8((c,), SEED + 5005) / 255.0)).astype(np.float32)
    ws2 = (0.002 * (1.0 + 29.0 * synth.fill_u8((c,), SEED + 5006) / 255.0)).astype(np.float32)
    s_mid = float(0.02 * float(ws1.max()) * 74.0 * 74.0 * np.sqrt(cin) / 60.0)
    s_out = float(s_mid * float(ws2.max()) * 74.0 * 74.0 * 3.0 / 60.0)
    pad = (1, 1, 1, 1)
    ho, wo = (h + 2 - 3) // stride + 1, (w + 2 - 3) // stride + 1
    xp = np.ascontiguousarray(x.transpose(0, 3, 1, 2))
    s1 = O.conv_shape(n, cin, h, w, c, 1, 1)
    s2 = O.conv_shape(n, c, h, w, c, 3, 3, stride=(stride, stride), pad=pad, groups=c)
    d1 = eden.conv_desc(n, cin, h, w, c, 1, 1, layout=eden.NHWC, weight_layout=eden.W_OIHW | eden.W_SIGNED)
    d2 = eden.conv_desc(n, c, h, w, c, 3, 3, stride=(stride, stride), pad=pad, dm=1, layout=eden.NHWC, weight_layout=eden.W_OIHW | eden.W_SIGNED)
    keep = [eden.DeviceBuffer(host=a) for a in (w1, b1, w2, b2)]
    d_x, d_o, d_mid, d_o2 = (eden.DeviceBuffer(host=x), eden.DeviceBuffer(nbytes=n * ho * wo * c), eden.DeviceBuffer(nbytes=n * h * w * c),
                             eden.DeviceBuffer(nbytes=n * ho * wo * c))
    variants = 0
    for act_floor, zp_w, odd in ((0, 0, False), (128, 0, False), (0, 0, True), (0, -9, False)):
        q1, m1, sh1 = eden.make_requant_perchannel(0.02, 117, ws1, s_mid, 128, eden.ACT_NONE, False)
        q2, m2, sh2 = eden.make_requant_perchannel(s_mid, 128, ws2, s_out, 128, eden.ACT_NONE, False)
        q1.act_min = q2.act_min = act_floor
        q1.zp_w = q2.zp_w = zp_w
        if odd:   # one channel of each operator outside the single-shift form's range
            sh1, sh2 = sh1.copy(), sh2.copy()
            sh1[c // 3] = 0
            sh2[c // 2] = -21
        oq1 = O.raw_quant(zp_in=117, zp_w=zp_w, zp_out=128, act_min=act_floor)
        oq2 = O.raw_quant(zp_in=128, zp_w=zp_w, zp_out=128, act_min=act_floor)
        mid = O.conv2d_perchannel(xp, w1, b1, s1, oq1, m1, sh1)
        want = np.ascontiguousarray(O.dwconv2d_perchannel(mid, w2, b2, s2, oq2, m2, sh2).transpose(0, 2, 3, 1))
        pw = eden.ConvPlan(d1, keep[0], keep[1], q1)
        dw = eden.DwConvPlan(d2, keep[2], keep[3], q2)
        pw.set_perchannel(m1, sh1)
        assert not eden.conv_dw_block_applies(pw, dw)   # one operator per channel, the other per tensor
        dw.set_perchannel(m2, sh2)
        assert eden.conv_dw_block_applies(pw, dw)
        eden.conv_dw_block_run(pw, dw, d_x, d_o, q1, q2, rows)
        fused = d_o.download((n, ho, wo, c))
        pw.run(d_x, d_mid, q1)
        dw.run(d_mid, d_o2, q2)
        apart = d_o2.download((n, ho, wo, c))
        pw.destroy()
        dw.destroy()
        assert np.array_equal(apart, want), (act_floor, zp_w, odd, diff_report(apart, want))
        assert np.array_equal(fused, want), (act_floor, zp_w, odd, diff_report(fused, want))
        assert want.std() > 4 and mid.std() > 4
        variants += 1
    assert variants == 4
