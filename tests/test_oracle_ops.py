"""Pins the oracle's operators: the reference tests' own known-answer vectors, an
independent numpy formulation (explicit zero-point padding + window view), the
zero-point fold form the GPU kernels use, and structural invariants."""
import json
import os

import numpy as np
import pytest

import oracle_lib as O

KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))
UNIT = dict(multiplier=1 << 30, shift=1)  # real multiplier 1.0


def np_requant(acc, q):
    """Vectorised exact requant in Python integers (independent of the C code)."""
    out = np.empty(acc.shape, np.uint8)
    flat, o = acc.reshape(-1).tolist(), out.reshape(-1)
    ls, rs = max(q.shift, 0), max(-q.shift, 0)
    for i, a in enumerate(flat):
        x = a << ls
        p = x * q.multiplier
        v = (p + (1 << 30)) >> 31                     # round half up
        half = (1 << rs) >> 1
        r = (abs(v) + half) >> rs if rs else abs(v)   # round half away from zero
        r = -r if v < 0 else r
        o[i] = min(max(r + q.zp_out, q.act_min), q.act_max)
    return out


def np_conv_acc(x, w, bias, s, zp_in, zp_w):
    """Pads with zp_in, builds windows, contracts in int64. NCHW, groups supported."""
    xp = np.pad(x.astype(np.int64), ((0, 0), (0, 0), (s.pad_t, s.pad_b), (s.pad_l, s.pad_r)), constant_values=zp_in) - zp_in
    wz = w.astype(np.int64) - zp_w
    ho, wo = O.conv_out_hw(s)
    g, cig, cog = s.groups, s.c // s.groups, s.cout // s.groups
    acc = np.zeros((s.n, s.cout, ho, wo), np.int64)
    for ky in range(s.kh):
        for kx in range(s.kw):
            y0, x0 = ky * s.dil_h, kx * s.dil_w
            win = xp[:, :, y0:y0 + (ho - 1) * s.stride_h + 1:s.stride_h, x0:x0 + (wo - 1) * s.stride_w + 1:s.stride_w]
            for gi in range(g):
                acc[:, gi * cog:(gi + 1) * cog] += np.einsum(
                    "nchw,oc->nohw", win[:, gi * cig:(gi + 1) * cig], wz[gi * cog:(gi + 1) * cog, :, ky, kx])
    return (acc + bias.astype(np.int64)[None, :, None, None]).astype(np.int32)


def rand_case(rng, n, c, h, w, cout, kh, kw, **kw_):
    s = O.conv_shape(n, c, h, w, cout, kh, kw, **kw_)
    x = rng.integers(0, 256, (n, c, h, w), dtype=np.uint8)
    wt = rng.integers(0, 256, (cout, c // s.groups, kh, kw), dtype=np.uint8)
    b = rng.integers(-1000, 1001, cout).astype(np.int32)
    return s, x, wt, b


# --------------------------------------------------------------------- KATs

@pytest.mark.parametrize("kat", KATS["conv"], ids=lambda k: k["name"])
def test_conv_reference_kat(kat):
    n, h, w, c = kat["in_dims"]
    cout, kh, kw, _ = kat["w_dims"]
    x = np.array(kat["input"], np.uint8).reshape(n, h, w, c).transpose(0, 3, 1, 2)
    wt = np.array(kat["weight"], np.uint8).reshape(cout, kh, kw, c).transpose(0, 3, 1, 2)
    bias = np.array(kat["bias"], np.int32)
    t, b, l, r = kat["pad_tblr"]
    s = O.conv_shape(n, c, h, w, cout, kh, kw, stride=tuple(kat["stride"]), pad=(t, b, l, r))
    q = O.raw_quant(**UNIT)
    if kat["relu"]:
        q.act_min, q.act_max = O.act_range_u8(O.ACT_RELU, 1.0, 0)
    out = O.conv2d(x, wt, bias, s, q)
    on, oh, ow, oc = kat["out_dims"]
    want = np.clip(np.array(kat["expect"]).reshape(on, oh, ow, oc).transpose(0, 3, 1, 2), 0, 255)
    assert np.array_equal(out, want.astype(np.uint8))
    # halve the multiplier: every non-negative expected value e becomes (e+1)//2, unsaturated for e <= 510
    qh = O.raw_quant(multiplier=1 << 30, shift=0, act_min=q.act_min, act_max=q.act_max)
    e = np.array(kat["expect"]).reshape(on, oh, ow, oc).transpose(0, 3, 1, 2)
    half = np.sign(e) * ((np.abs(e) + 1) // 2)
    assert np.array_equal(O.conv2d(x, wt, bias, s, qh), np.clip(half, q.act_min, 255).astype(np.uint8))


def test_conv_perchannel_u8_kat():
    k = KATS["conv_perchannel_u8"]
    n, c, h, w = k["in_dims_nchw"]
    cout, kh, kw, cin = k["w_dims_ohwi"]
    x = np.array(k["input"], np.uint8).reshape(n, c, h, w)
    wt = np.array(k["weight_i8"], np.int8).reshape(cout, kh, kw, cin).transpose(0, 3, 1, 2)
    mults, shifts = [], []
    for ws in k["w_scales"]:
        m = float(np.float32(k["in_scale"])) * float(np.float32(ws)) / float(np.float32(k["out_scale"]))
        qm, sh = O.quantize_multiplier(m)
        mults.append(qm)
        shifts.append(sh)
    s = O.conv_shape(n, c, h, w, cout, kh, kw)
    q = O.raw_quant(zp_in=k["in_zp"], zp_w=0, zp_out=k["out_zp"])
    out = O.conv2d_perchannel(x, wt, np.array(k["bias"], np.int32), s, q, mults, shifts)
    assert out.reshape(-1).tolist() == k["expect"]


def test_relu_u8_kat():
    """A quantized ReLU is a clamp at the zero point: values below zp come out as zp."""
    k = KATS["relu_u8"]
    lo, hi = O.act_range_u8(O.ACT_RELU, 1.0, k["zp"])
    q = O.raw_quant(zp_in=k["zp"], zp_w=0, zp_out=k["zp"], act_min=lo, act_max=hi, **UNIT)
    x = np.array(k["input"], np.uint8).reshape(1, 1, 1, 4)
    one = np.array([1], np.uint8).reshape(1, 1, 1, 1)
    out = O.conv2d(x, one, np.zeros(1, np.int32), O.conv_shape(1, 1, 1, 4, 1, 1, 1), q)
    assert out.reshape(-1).tolist() == k["expect"]


@pytest.mark.parametrize("kat", KATS["depthwise"], ids=lambda k: k["name"])
def test_depthwise_reference_kat(kat):
    n, c, h, w = kat["in_dims"]
    cout, _, kh, kw = kat["w_dims"]
    zp_w, zp_out = 16, 40  # weights go down to -16, outputs down to -36
    x = np.array(kat["input"], np.uint8).reshape(n, c, h, w)
    wt = (np.array(kat["weight"]) + zp_w).astype(np.uint8).reshape(cout, 1, kh, kw)
    s = O.conv_shape(n, c, h, w, cout, kh, kw, stride=tuple(kat["stride"]), dm=kat["dm"])
    q = O.raw_quant(zp_w=zp_w, zp_out=zp_out, **UNIT)
    out, acc = O.dwconv2d(x, wt, np.array(kat["bias"], np.int32), s, q, want_acc=True)
    assert list(out.shape) == kat["out_dims"]
    assert acc.reshape(-1).tolist() == kat["expect"]
    assert out.reshape(-1).tolist() == [e + zp_out for e in kat["expect"]]
    # same vector with zp_out = 0: negatives clamp to 0
    q0 = O.raw_quant(zp_w=zp_w, **UNIT)
    assert O.dwconv2d(x, wt, np.array(kat["bias"], np.int32), s, q0).reshape(-1).tolist() == [max(e, 0) for e in kat["expect"]]


@pytest.mark.parametrize("kat", KATS["fc"], ids=lambda k: k["name"])
def test_fc_reference_kat(kat):
    zp_a = 10  # inputs go down to -10
    a = (np.array(kat["input"]) + zp_a).astype(np.uint8).reshape(kat["m"], kat["k"])
    w = np.array(kat["weight"], np.uint8).reshape(kat["n"], kat["k"])
    q = O.raw_quant(zp_in=zp_a, **UNIT)
    out = O.fc(a, w, np.array(kat["bias"], np.int32), q)
    assert out.reshape(-1).tolist() == kat["expect"]


@pytest.mark.parametrize("kat", KATS["deconv_float"], ids=lambda k: k["name"])
def test_deconv_index_math_reference_float_kat(kat):
    n, c, h, w = kat["in_dims"]
    cin, cog, kh, kw = kat["w_dims"]
    g = kat["groups"]
    t, r, b, l = kat["pad_trbl"]
    s = O.conv_shape(n, c, h, w, cog * g, kh, kw, stride=tuple(kat["stride"]), pad=(t, b, l, r), groups=g)
    assert cin == c
    out = O.deconv2d_f64(np.array(kat["input"]).reshape(n, c, h, w), np.array(kat["weight"]).reshape(cin, cog, kh, kw),
                         np.array(kat["bias"]), s)
    assert list(out.shape) == kat["out_dims"]
    # the reference compares at 1e-4 absolute (deconvolution_test.cpp:24); its data carries six digits
    assert np.max(np.abs(out.reshape(-1) - np.array(kat["expect"]))) < 1e-4


# ------------------------------------------------ independent formulations

CONV_CASES = [
    dict(n=2, c=3, h=7, w=9, cout=5, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=1, c=4, h=8, w=8, cout=6, kh=3, kw=3, stride=(2, 2), pad=(0, 1, 0, 1)),
    dict(n=1, c=6, h=9, w=7, cout=4, kh=3, kw=2, dil=(2, 1), pad=(2, 2, 0, 1), groups=2),
    dict(n=3, c=8, h=5, w=5, cout=8, kh=1, kw=1),
    dict(n=1, c=2, h=6, w=6, cout=3, kh=5, kw=5, pad=(2, 2, 2, 2), stride=(1, 2)),
    dict(n=1, c=1, h=3, w=3, cout=1, kh=3, kw=3, pad=(3, 3, 3, 3)),  # windows that lie wholly in the padding
]


@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_conv_vs_numpy_windows_and_fold_form(case):
    rng = np.random.default_rng(11)
    s, x, wt, b = rand_case(rng, **case)
    zp_in, zp_w = int(rng.integers(0, 256)), int(rng.integers(0, 256))
    q = O.make_quant(0.02, zp_in, 0.005, zp_w, 0.05, int(rng.integers(0, 256)), O.ACT_RELU6, True)
    out, acc = O.conv2d(x, wt, b, s, q, want_acc=True)
    want_acc = np_conv_acc(x, wt, b, s, zp_in, zp_w)
    assert np.array_equal(acc, want_acc)
    assert np.array_equal(out, np_requant(want_acc, q))
    # fold form used by the GPU kernels (groups == 1 only): with a' = a-128, w' = w-128,
    # za = zp_in-128, zw = zp_w-128 and padding filled with za:
    # sum (a-zp_in)(w-zp_w) = sum a'w' - zw*sum_k a' - za*sum_k w' + K*za*zw
    if s.groups == 1:
        za, zw = zp_in - 128, zp_w - 128
        s0 = O.conv_shape(s.n, s.c, s.h, s.w, s.cout, s.kh, s.kw, stride=(s.stride_h, s.stride_w),
                          pad=(s.pad_t, s.pad_b, s.pad_l, s.pad_r), dil=(s.dil_h, s.dil_w))
        zero_b = np.zeros(s.cout, np.int32)
        xs, ws = x.astype(np.int64) - 128, wt.astype(np.int64) - 128
        # np_conv_acc with "zero points" za/0 on pre-shifted data gives sum a'w' with za-filled padding
        xp = np.pad(xs, ((0, 0), (0, 0), (s.pad_t, s.pad_b), (s.pad_l, s.pad_r)), constant_values=za)
        ho, wo = O.conv_out_hw(s0)
        dot = np.zeros((s.n, s.cout, ho, wo), np.int64)
        rowsum = np.zeros((s.n, 1, ho, wo), np.int64)
        for ky in range(s.kh):
            for kx in range(s.kw):
                y0, x0 = ky * s.dil_h, kx * s.dil_w
                win = xp[:, :, y0:y0 + (ho - 1) * s.stride_h + 1:s.stride_h, x0:x0 + (wo - 1) * s.stride_w + 1:s.stride_w]
                dot += np.einsum("nchw,oc->nohw", win, ws[:, :, ky, kx])
                rowsum += win.sum(axis=1, keepdims=True)
        k_total = s.c * s.kh * s.kw
        colsum = ws.reshape(s.cout, -1).sum(axis=1)
        folded = dot - zw * rowsum - za * colsum[None, :, None, None] + k_total * za * zw + b[None, :, None, None]
        assert np.array_equal(folded.astype(np.int32), acc)
        del zero_b


def test_depthwise_equals_grouped_conv():
    rng = np.random.default_rng(12)
    for dm, stride, pad in ((1, (1, 1), (1, 1, 1, 1)), (2, (2, 2), (0, 1, 0, 1)), (3, (1, 2), (1, 0, 2, 1))):
        c, h, w = 5, 9, 8
        x = rng.integers(0, 256, (2, c, h, w), dtype=np.uint8)
        wt = rng.integers(0, 256, (c * dm, 1, 3, 3), dtype=np.uint8)
        b = rng.integers(-500, 500, c * dm).astype(np.int32)
        q = O.make_quant(0.1, 7, 0.02, 200, 0.3, 99)
        sd = O.conv_shape(2, c, h, w, c * dm, 3, 3, stride=stride, pad=pad, dm=dm)
        sg = O.conv_shape(2, c, h, w, c * dm, 3, 3, stride=stride, pad=pad, groups=c)
        o1, a1 = O.dwconv2d(x, wt, b, sd, q, want_acc=True)
        o2, a2 = O.conv2d(x, wt, b, sg, q, want_acc=True)
        assert np.array_equal(a1, a2) and np.array_equal(o1, o2)


def test_fc_equals_1x1_conv_and_numpy():
    rng = np.random.default_rng(13)
    m, k, n = 7, 37, 11
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    w = rng.integers(0, 256, (n, k), dtype=np.uint8)
    b = rng.integers(-1000, 1000, n).astype(np.int32)
    q = O.make_quant(0.01, 3, 0.002, 128, 0.08, 0)
    out, acc = O.fc(a, w, b, q, want_acc=True)
    want = (a.astype(np.int64) - 3) @ (w.astype(np.int64) - 128).T + b
    assert np.array_equal(acc, want.astype(np.int32))
    s = O.conv_shape(m, k, 1, 1, n, 1, 1)
    oc = O.conv2d(a.reshape(m, k, 1, 1), w.reshape(n, k, 1, 1), b, s, q)
    assert np.array_equal(oc.reshape(m, n), out)
    # 1x1 conv over pixels == FC over the pixel-major matrix
    x = rng.integers(0, 256, (2, k, 3, 4), dtype=np.uint8)
    s2 = O.conv_shape(2, k, 3, 4, n, 1, 1)
    oc2 = O.conv2d(x, w.reshape(n, k, 1, 1), b, s2, q)
    of = O.fc(O.nchw2nhwc(x).reshape(-1, k), w, b, q).reshape(2, 3, 4, n)
    assert np.array_equal(O.nhwc2nchw(of), oc2)


DECONV_CASES = [
    dict(n=2, c=4, h=3, w=5, cout=6, kh=4, kw=4, stride=(2, 2), pad=(1, 1, 1, 1)),
    dict(n=1, c=6, h=4, w=4, cout=4, kh=3, kw=3, stride=(3, 3), pad=(1, 1, 1, 1), groups=2),
    dict(n=1, c=3, h=5, w=4, cout=2, kh=2, kw=3, stride=(1, 2), pad=(0, 1, 1, 0)),
    dict(n=1, c=2, h=3, w=3, cout=2, kh=3, kw=3, stride=(1, 1), pad=(0, 0, 0, 0)),
]


@pytest.mark.parametrize("case", DECONV_CASES, ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_deconv_gather_equals_scatter(case):
    rng = np.random.default_rng(14)
    s = O.conv_shape(**case)
    x = rng.integers(0, 256, (s.n, s.c, s.h, s.w), dtype=np.uint8)
    wt = rng.integers(0, 256, (s.c, s.cout // s.groups, s.kh, s.kw), dtype=np.uint8)
    b = rng.integers(-1000, 1000, s.cout).astype(np.int32)
    q = O.make_quant(0.03, 131, 0.01, 77, 0.9, 5)
    o1, a1 = O.deconv2d(x, wt, b, s, q, want_acc=True)
    o2, a2 = O.deconv2d(x, wt, b, s, q, want_acc=True, scatter=True)
    assert np.array_equal(a1, a2) and np.array_equal(o1, o2)
    assert a1.std() > 0


def test_deconv_stride1_equals_conv_with_flipped_transposed_kernel():
    rng = np.random.default_rng(15)
    n, c, h, w, cout, k, p = 2, 3, 6, 5, 4, 3, 1
    x = rng.integers(0, 256, (n, c, h, w), dtype=np.uint8)
    wd = rng.integers(0, 256, (c, cout, k, k), dtype=np.uint8)
    b = rng.integers(-100, 100, cout).astype(np.int32)
    q = O.make_quant(0.05, 12, 0.02, 140, 0.7, 33)
    od, ad = O.deconv2d(x, wd, b, O.conv_shape(n, c, h, w, cout, k, k, pad=(p, p, p, p)), q, want_acc=True)
    wc = np.ascontiguousarray(wd.transpose(1, 0, 2, 3)[:, :, ::-1, ::-1])
    pc = k - 1 - p
    oc, ac = O.conv2d(x, wc, b, O.conv_shape(n, c, h, w, cout, k, k, pad=(pc, pc, pc, pc)), q, want_acc=True)
    assert np.array_equal(ad, ac) and np.array_equal(od, oc)


# ------------------------------------------------------------- invariants

def test_input_at_zero_point_gives_requant_of_bias():
    rng = np.random.default_rng(16)
    s, _, wt, b = rand_case(rng, 1, 4, 6, 6, 5, 3, 3, pad=(1, 1, 1, 1))
    q = O.make_quant(0.5, 77, 0.5, 13, 0.25, 100)
    x = np.full((1, 4, 6, 6), 77, np.uint8)
    out, acc = O.conv2d(x, wt, b, s, q, want_acc=True)
    assert np.array_equal(acc, np.broadcast_to(b[None, :, None, None], acc.shape))
    x2 = rng.integers(0, 256, (1, 4, 6, 6), dtype=np.uint8)
    w2 = np.full(wt.shape, 13, np.uint8)
    _, acc2 = O.conv2d(x2, w2, b, s, q, want_acc=True)
    assert np.array_equal(acc2, np.broadcast_to(b[None, :, None, None], acc2.shape))


def test_layout_round_trip_and_index_form():
    rng = np.random.default_rng(17)
    x = rng.integers(0, 256, (3, 5, 4, 7), dtype=np.uint8)
    y = O.nchw2nhwc(x)
    assert np.array_equal(y, x.transpose(0, 2, 3, 1))
    assert np.array_equal(O.nhwc2nchw(y), x)


def test_output_dim_formulas():
    assert O.lib.eo_conv_out_dim(56, 1, 1, 3, 1, 1) == 56
    assert O.lib.eo_conv_out_dim(56, 1, 1, 3, 1, 2) == 28
    assert O.lib.eo_conv_out_dim(224, 0, 1, 3, 1, 2) == 112
    assert O.lib.eo_conv_out_dim(7, 2, 2, 3, 2, 1) == 7
    assert O.lib.eo_deconv_out_dim(32, 1, 1, 4, 2) == 64
    assert O.lib.eo_deconv_out_dim(3, 0, 0, 3, 3) == 9


def test_empty_shapes_do_not_touch_memory():
    s = O.conv_shape(0, 4, 6, 6, 5, 3, 3)
    q = O.raw_quant()
    out = O.conv2d(np.zeros((0, 4, 6, 6), np.uint8), np.zeros((5, 4, 3, 3), np.uint8), np.zeros(5, np.int32), s, q)
    assert out.size == 0
    assert O.fc(np.zeros((0, 8), np.uint8), np.zeros((3, 8), np.uint8), np.zeros(3, np.int32), q).size == 0


def test_add_closed_forms():
    """parity unpinned by reference vectors: equal scales, out scale = in scale -> plain integer add."""
    q = O.make_add_quant(0.5, 10, 0.5, 20, 0.5, 5)
    a = np.arange(0, 200, dtype=np.uint8)
    b = np.arange(200, 0, -1, dtype=np.uint8)
    want = np.clip((a.astype(int) - 10) + (b.astype(int) - 20) + 5, 0, 255)
    assert np.array_equal(O.add(a, b, q), want.astype(np.uint8))
    # out scale twice the input scale halves the sum (ties away from zero after the two-stage rounding)
    q2 = O.make_add_quant(0.5, 0, 0.5, 0, 1.0, 0)
    assert O.add(np.array([4, 5, 7], np.uint8), np.array([2, 2, 2], np.uint8), q2).tolist() == [3, 4, 5]


ADD_UNEQUAL = [
    # scale_a, zp_a, scale_b, zp_b, scale_out, zp_out
    (0.047, 128, 0.0213, 100, 0.0611, 120),
    (0.013, 7, 0.11, 201, 0.09, 64),
    (0.4, 90, 0.031, 33, 0.45, 128),
]


@pytest.mark.parametrize("params", ADD_UNEQUAL, ids=lambda p: "sa%g_sb%g_so%g" % (p[0], p[2], p[4]))
def test_add_unequal_scales_against_exact_rational_arithmetic(params):
    """All 65,536 byte pairs: the three-multiplier fixed-point add stays within one step of the exactly rounded real
    sum round((s_a (a - zp_a) + s_b (b - zp_b)) / s_out) + zp_out, equals it in at least 99 % of the pairs away from
    the clamps, and an add with the two input multipliers exchanged (the mistake this test exists for) does not."""
    from fractions import Fraction
    s_a, zp_a, s_b, zp_b, s_out, zp_out = params
    q = O.make_add_quant(s_a, zp_a, s_b, zp_b, s_out, zp_out)
    a, b = np.meshgrid(np.arange(256, dtype=np.uint8), np.arange(256, dtype=np.uint8), indexing="ij")
    got = O.add(a, b, q).astype(np.int64)
    # exact: the float32 scales as rationals, rounding half away from zero
    fa, fb, fo = (Fraction(float(np.float32(v))) for v in (s_a, s_b, s_out))
    ra, rb = fa / fo, fb / fo
    den = (ra.denominator * rb.denominator)
    num = (a.astype(object) - zp_a) * (ra.numerator * rb.denominator) + (b.astype(object) - zp_b) * (rb.numerator * ra.denominator)  # Python integers
    exact = np.array([[(abs(int(v)) * 2 + den) // (2 * den) * (1 if v >= 0 else -1) for v in row] for row in num], dtype=np.int64) + zp_out
    inside = (exact > 0) & (exact < 255)
    assert inside.mean() > 0.3                      # the case exercises the arithmetic, not the clamps
    err = np.abs(got - np.clip(exact, 0, 255))
    assert err.max() <= 1
    assert (err[inside] == 0).mean() >= 0.99

    # the mutant: multipliers (and shifts) of the two inputs exchanged
    m = O.AddQuant()
    for f, _ in O.AddQuant._fields_:
        setattr(m, f, getattr(q, f))
    m.mult_a, m.mult_b, m.shift_a, m.shift_b = q.mult_b, q.mult_a, q.shift_b, q.shift_a
    bad = np.abs(O.add(a, b, m).astype(np.int64) - np.clip(exact, 0, 255))
    assert bad.max() > 1 and (bad[inside] == 0).mean() < 0.9
    # a second mutant: one more right shift on both inputs
    m2 = O.AddQuant()
    for f, _ in O.AddQuant._fields_:
        setattr(m2, f, getattr(q, f))
    m2.shift_a, m2.shift_b = q.shift_a - 1, q.shift_b - 1
    bad2 = np.abs(O.add(a, b, m2).astype(np.int64) - np.clip(exact, 0, 255))
    assert bad2.max() > 1


def test_avgpool_closed_forms():
    """hand cases of (sum + n/2) / n over the clipped window (AveragepoolKernels.cpp:8-44)"""
    x = np.arange(16, dtype=np.uint8).reshape(1, 1, 4, 4)
    assert O.avgpool(x, 2, 2, stride=(2, 2)).reshape(-1).tolist() == [3, 5, 11, 13]  # 2.5->3, 4.5->5, ...
    assert O.avgpool(x, 4, 4).reshape(-1).tolist() == [8]  # 7.5 -> 8
    # padded window counts only in-image taps
    o = O.avgpool(x, 3, 3, stride=(1, 1), pad=(1, 1, 1, 1))
    assert o[0, 0, 0, 0] == (0 + 1 + 4 + 5 + 2) // 4


@pytest.mark.parametrize("k,stride,pad", [((3, 3), (2, 2), (1, 1, 1, 1)), ((2, 2), (2, 2), (0, 0, 0, 0)), ((3, 2), (1, 2), (0, 2, 1, 0)),
                                          ((7, 7), (1, 1), (0, 0, 0, 0)), ((4, 4), (3, 3), (2, 1, 1, 2))])
def test_avgpool_uint8_against_exact_rational_arithmetic(k, stride, pad):
    """No reference vector exists (the reference's averagepool_test.cpp is float only), so the uint8 pool is pinned by
    what (sum + n / 2) / n has to be: the mean over the in-image taps of the window, rounded to nearest with ties
    upwards, then clamped.  Checked on every output of seeded tensors in exact rational arithmetic; a version that
    divides by the full window size on border windows, one that truncates, and one that rounds ties to even each
    fail the same check."""
    from fractions import Fraction
    import math
    rng = np.random.default_rng(31 + k[0] * 7 + k[1])
    n, c, h, w = 2, 3, 11, 9
    x = rng.integers(0, 256, (n, c, h, w)).astype(np.uint8)
    x[0, 0, :4, :4] = 255   # saturated corner: the clamp's upper bound is reached
    x[1, 2, :2, :2] = np.array([[1, 2], [3, 4]], np.uint8)  # a 2x2 window summing to 10: mean 2.5, a tie
    lo, hi = 7, 240
    got = O.avgpool(x, k[0], k[1], stride=stride, pad=pad, act_min=lo, act_max=hi).astype(np.int64)
    ho = (h + pad[0] + pad[1] - k[0]) // stride[0] + 1
    wo = (w + pad[2] + pad[3] - k[1]) // stride[1] + 1
    assert got.shape == (n, c, ho, wo)
    ties = 0
    mutants = dict(full_window=0, truncating=0, ties_to_even=0)
    for i in range(n):
        for ch in range(c):
            for oy in range(ho):
                for ox in range(wo):
                    ys = [v for v in range(oy * stride[0] - pad[0], oy * stride[0] - pad[0] + k[0]) if 0 <= v < h]
                    xs = [v for v in range(ox * stride[1] - pad[2], ox * stride[1] - pad[2] + k[1]) if 0 <= v < w]
                    total = int(sum(int(x[i, ch, a, b]) for a in ys for b in xs))
                    mean = Fraction(total, len(ys) * len(xs))
                    nearest = math.floor(mean + Fraction(1, 2))   # ties upwards
                    ties += mean.denominator == 2
                    assert got[i, ch, oy, ox] == min(max(nearest, lo), hi), (i, ch, oy, ox, mean)
                    full = math.floor(Fraction(total, k[0] * k[1]) + Fraction(1, 2))
                    mutants["full_window"] += min(max(full, lo), hi) != got[i, ch, oy, ox]
                    mutants["truncating"] += min(max(math.floor(mean), lo), hi) != got[i, ch, oy, ox]
                    mutants["ties_to_even"] += min(max(round(mean), lo), hi) != got[i, ch, oy, ox]
    if k[0] * k[1] <= 9:   # large windows average the clamp's bounds away
        assert got.min() == lo or got.max() == hi
    if any(pad):
        assert mutants["full_window"] > 0
    assert mutants["truncating"] > 0
    if k == (2, 2):
        assert ties > 0 and mutants["ties_to_even"] > 0


def test_avgpool_int8_rounds_half_away_from_zero():
    """parity unpinned by reference vectors.  The int8 pool rounds the signed mean half away from zero, so it is not
    the uint8 pool on bytes + 128: (-1 + 0) / 2 gives -1 there, while (127 + 128 + 1) / 2 - 128 gives 0."""
    x = np.array([-1, 0, 1, 2, -3, -4, -5, -8], np.int8).reshape(1, 1, 2, 4)
    assert O.avgpool_s8(x, 1, 2, stride=(1, 2)).reshape(-1).tolist() == [-1, 2, -4, -7]  # -0.5, 1.5, -3.5, -6.5
    assert O.avgpool_s8(x, 2, 4).reshape(-1).tolist() == [-2]  # -18 / 8 = -2.25
    assert O.avgpool_s8(x, 2, 4, act_min=-1, act_max=5).reshape(-1).tolist() == [-1]
    rng = np.random.default_rng(5)
    y = rng.integers(-128, 128, (2, 3, 9, 7)).astype(np.int8)
    got = O.avgpool_s8(y, 3, 3, stride=(2, 2), pad=(1, 1, 1, 1)).astype(np.int64)
    # against exact rational arithmetic: |got - mean| <= 1/2, ties away from zero
    from fractions import Fraction
    for n in range(2):
        for c in range(3):
            for oy in range(got.shape[2]):
                for ox in range(got.shape[3]):
                    ys = [v for v in range(oy * 2 - 1, oy * 2 + 2) if 0 <= v < 9]
                    xs = [v for v in range(ox * 2 - 1, ox * 2 + 2) if 0 <= v < 7]
                    mean = Fraction(int(sum(int(y[n, c, a, b]) for a in ys for b in xs)), len(ys) * len(xs))
                    g = int(got[n, c, oy, ox])
                    assert abs(g - mean) <= Fraction(1, 2)
                    if abs(g - mean) == Fraction(1, 2):
                        assert abs(g) > abs(mean)


def _perchannel_pairs(rng, cout):
    mults = rng.integers(1 << 30, (1 << 31) - 1, cout).astype(np.int32)
    shifts = rng.integers(-12, -4, cout).astype(np.int32)
    return mults, shifts


@pytest.mark.parametrize("kind", ["conv", "dw", "deconv"])
def test_perchannel_forms_reduce_to_the_per_tensor_functions(kind):
    """Channel c of a per-channel result is channel c of the pinned per-tensor function run on the same weights
    read as uint8 (byte + 128, zero point + 128) with channel c's multiplier and shift."""
    rng = np.random.default_rng(77 + len(kind))
    if kind == "dw":
        s = O.conv_shape(2, 5, 9, 8, 10, 3, 3, stride=(2, 1), pad=(1, 0, 1, 1), dm=2)
        w_shape, fn, fn_pc = (10, 1, 3, 3), O.dwconv2d, O.dwconv2d_perchannel
    elif kind == "deconv":
        s = O.conv_shape(2, 6, 5, 4, 8, 3, 3, stride=(2, 2), pad=(1, 0, 1, 0), groups=2)
        w_shape, fn, fn_pc = (6, 4, 3, 3), O.deconv2d, O.deconv2d_perchannel
    else:
        s = O.conv_shape(2, 6, 7, 6, 8, 3, 2, stride=(1, 2), pad=(1, 1, 0, 1), groups=2)
        w_shape, fn, fn_pc = (8, 3, 3, 2), O.conv2d, O.conv2d_perchannel
    cout = 10 if kind == "dw" else 8
    x = rng.integers(0, 256, (s.n, s.c, s.h, s.w)).astype(np.uint8)
    w = rng.integers(-128, 128, w_shape).astype(np.int8)
    bias = rng.integers(-3000, 3000, cout).astype(np.int32)
    mults, shifts = _perchannel_pairs(rng, cout)
    for zp_w in (0, -7):
        q = O.raw_quant(zp_in=101, zp_w=zp_w, zp_out=120, act_min=3, act_max=250)
        got = fn_pc(x, w, bias, s, q, mults, shifts)
        assert got.std() > 10
        w_u8 = (w.astype(np.int16) + 128).astype(np.uint8)
        for c in range(cout):
            qc = O.raw_quant(zp_in=101, zp_w=zp_w + 128, zp_out=120, multiplier=int(mults[c]), shift=int(shifts[c]),
                             act_min=3, act_max=250)
            assert np.array_equal(got[:, c], fn(x, w_u8, bias, s, qc)[:, c]), (kind, c)


@pytest.mark.parametrize("kind", ["conv", "dw", "deconv", "fc"])
def test_int8_precision_forms_reduce_to_the_uint8_functions(kind):
    """An INT8-precision operator is the uint8 operator on every byte, zero point and clamp bound + 128, with the
    result moved back by 128 (SIGNED_TO_UNSIGNED / UNSIGNED_TO_SIGNED, cl_kernels/DepthwiseconvolutionKernels.cpp:2410-2411)."""
    rng = np.random.default_rng(99 + len(kind))
    q8 = O.raw_quant(zp_in=-20, zp_w=3, zp_out=-7, multiplier=1518500250, shift=-8, act_min=-50, act_max=60)
    qu = O.raw_quant(zp_in=108, zp_w=131, zp_out=121, multiplier=1518500250, shift=-8, act_min=78, act_max=188)
    up = lambda a: (a.astype(np.int16) + 128).astype(np.uint8)
    if kind == "fc":
        a = rng.integers(-128, 128, (7, 40)).astype(np.int8)
        w = rng.integers(-128, 128, (9, 40)).astype(np.int8)
        b = rng.integers(-3000, 3000, 9).astype(np.int32)
        got = O.fc_s8(a, w, b, q8)
        want = O.fc(up(a), up(w), b, qu)
    else:
        if kind == "dw":
            s = O.conv_shape(2, 5, 9, 8, 10, 3, 3, stride=(2, 1), pad=(1, 0, 1, 1), dm=2)
            w_shape, f8, fu = (10, 1, 3, 3), O.dwconv2d_s8, O.dwconv2d
        elif kind == "deconv":
            s = O.conv_shape(2, 6, 5, 4, 8, 3, 3, stride=(2, 2), pad=(1, 0, 1, 0), groups=2)
            w_shape, f8, fu = (6, 4, 3, 3), O.deconv2d_s8, O.deconv2d
        else:
            s = O.conv_shape(2, 6, 7, 6, 8, 3, 2, stride=(1, 2), pad=(1, 1, 0, 1), groups=2)
            w_shape, f8, fu = (8, 3, 3, 2), O.conv2d_s8, O.conv2d
        x = rng.integers(-128, 128, (s.n, s.c, s.h, s.w)).astype(np.int8)
        w = rng.integers(-128, 128, w_shape).astype(np.int8)
        b = rng.integers(-3000, 3000, w_shape[0] if kind != "deconv" else 8).astype(np.int32)
        got = f8(x, w, b, s, q8)
        want = fu(up(x), up(w), b, s, qu)
    assert got.dtype == np.int8 and got.std() > 10
    assert got.min() == -50 and got.max() == 60  # both clamp bounds are reached
    assert np.array_equal(up(got), want)
