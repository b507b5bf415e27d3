"""Randomized differential sweep: a few hundred seeded random operator instances (shapes, strides, paddings, dilations,
groups, layouts, zero points, clamp ranges, requantization scales) through the C ABI against the CPU oracle.  The
hand-picked cases of test_gpu_parity.py aim at each kernel family's corners; this one aims at what nobody thought of.
Bit-exact, as everywhere."""
import numpy as np
import pytest

import oracle_lib as O
from harness import diff_report, eden, gpu_conv, gpu_deconv, gpu_dwconv, gpu_fc, synth, to_eh_add, to_eh_requant

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_operator_instances_match_the_oracle(seed):
    eden.init(0)
    print("random sweep, seed", seed, flush=True)
    rng = np.random.default_rng(seed)
    N = 400
    def centred(acc, zp_in, zp_w, lo, hi):
        sd = float(acc.std()) or 1.0
        qm, sh = O.quantize_multiplier(float(rng.choice([10.0, 40.0, 120.0])) / sd)
        zp_out = int(np.clip(128 - round(float(acc.mean()) * 40.0 / sd), 0, 255))
        return O.raw_quant(zp_in=zp_in, zp_w=zp_w, zp_out=zp_out, multiplier=qm, shift=sh, act_min=lo, act_max=hi)
    ran = {}
    bad = 0
    for it in range(N):
        kind = rng.choice(["conv", "conv1x1", "conv3x3", "dw", "fc", "deconv"], p=[0.25, 0.2, 0.15, 0.2, 0.1, 0.1])
        zp_in, zp_w = int(rng.integers(0, 256)), int(rng.choice([128, int(rng.integers(0, 256))]))
        lo = int(rng.choice([0, 0, int(rng.integers(0, 100))])); hi = int(rng.choice([255, 255, int(rng.integers(150, 256))]))
        layout = eden.NHWC if rng.random() < 0.7 else eden.NCHW
        if rng.random() < 0.2:
            layout |= eden.EXACT_CHANNELS   # no staged copies, no bundled groups: the kernels that read the caller's tensors as they are
        tseed = int(rng.integers(1, 1 << 30))
        try:
            if kind == "fc":
                m, k, n = int(rng.integers(1, 300)), int(rng.choice([8, 16, 24, 37, 40, 64, 100, 128, 192, 256, 260, 512, 1000, 1001, 6200])), int(rng.integers(1, 300))
                a = synth.fill_u8((m, k), tseed); w = synth.fill_u8((n, k), tseed + 1); b = synth.fill_i32((n,), tseed + 2, -1000, 1000)
                _, acc = O.fc(a, w, b, O.raw_quant(zp_in=zp_in, zp_w=zp_w), want_acc=True)
                q = centred(acc, zp_in, zp_w, lo, hi)
                want = O.fc(a, w, b, q); got = gpu_fc(a, w, b, to_eh_requant(q), flags=layout & eden.EXACT_CHANNELS); desc = (kind, m, k, n, layout)
            else:
                n = int(rng.integers(1, 5))
                if kind == "dw":
                    c = int(rng.choice([4, 8, 12, 16, 32, 36, 144, 20, 7, 5, 30])); h, w_ = int(rng.integers(3, 30)), int(rng.integers(3, 30))
                    k = int(rng.choice([3, 3, 3, 5, 2, 7])); st = int(rng.choice([1, 1, 2])); dil = int(rng.choice([1, 1, 1, 2, 3, 4])); dm = int(rng.choice([1, 1, 1, 2, 3]))
                    pads = tuple(int(v) for v in rng.integers(0, dil * (k - 1) + 1, 4))
                    s = O.conv_shape(n, c, h, w_, c * dm, k, k, stride=(st, st), pad=pads, dil=(dil, dil), dm=dm)
                    if min(O.conv_out_hw(s)) < 1: continue
                    x = synth.fill_u8((n, c, h, w_), tseed); w = synth.fill_u8((c * dm, 1, k, k), tseed + 1); b = synth.fill_i32((c * dm,), tseed + 2, -1000, 1000)
                    _, acc = O.dwconv2d(x, w, b, s, O.raw_quant(zp_in=zp_in, zp_w=zp_w), want_acc=True)
                    q = centred(acc, zp_in, zp_w, lo, hi)
                    want = O.dwconv2d(x, w, b, s, q); got = gpu_dwconv(x, w, b, s, to_eh_requant(q), layout=layout); desc = (kind, s, layout)
                elif kind == "deconv":
                    groups = int(rng.choice([1, 1, 1, 2]))
                    c = groups * int(rng.choice([8, 16, 32, 24, 21, 5])); cout = groups * int(rng.choice([8, 16, 20, 32, 21])); h, w_ = int(rng.integers(2, 12)), int(rng.integers(2, 12))
                    k = int(rng.choice([2, 3, 4, 5, 6, 8])); st = int(rng.choice([1, 2, 2, 3, 4])); pads = tuple(int(v) for v in rng.integers(0, k, 4))
                    s = O.conv_shape(n, c, h, w_, cout, k, k, stride=(st, st), pad=pads, groups=groups)
                    if min(O.deconv_out_hw(s)) < 1: continue
                    x = synth.fill_u8((n, c, h, w_), tseed); w = synth.fill_u8((c, cout // groups, k, k), tseed + 1); b = synth.fill_i32((cout,), tseed + 2, -1000, 1000)
                    _, acc = O.deconv2d(x, w, b, s, O.raw_quant(zp_in=zp_in, zp_w=zp_w), want_acc=True)
                    q = centred(acc, zp_in, zp_w, lo, hi)
                    want = O.deconv2d(x, w, b, s, q); got = gpu_deconv(x, w, b, s, to_eh_requant(q), layout=layout); desc = (kind, s, layout)
                else:
                    if kind == "conv1x1":
                        c = int(rng.choice([8, 16, 24, 32, 40, 64, 96, 144, 192, 320])); cout = int(rng.choice([8, 16, 24, 32, 48, 96, 144, 208, 256, 300])); k = 1
                        h, w_ = int(rng.integers(1, 20)), int(rng.integers(1, 20)); st = int(rng.choice([1, 1, 2])); pads = (0, 0, 0, 0) if rng.random() < 0.8 else tuple(int(v) for v in rng.integers(0, 2, 4)); groups = 1; dil = 1
                    elif kind == "conv3x3":
                        c = int(rng.choice([32, 64, 96, 128])); cout = int(rng.choice([16, 32, 40, 64, 100])); k = 3
                        h, w_ = int(rng.integers(6, 24)), int(rng.integers(8, 40)); st = 1; pads = tuple(int(v) for v in rng.integers(0, 3, 4)); groups = 1; dil = 1
                    else:
                        groups = int(rng.choice([1, 1, 1, 2, 4, 8, 16])); c = groups * int(rng.choice([1, 2, 3, 4, 8, 16, 20, 21])); cout = groups * int(rng.choice([1, 3, 4, 8, 10, 16]))
                        k = int(rng.choice([1, 2, 3, 5, 7])); h, w_ = int(rng.integers(k, 20)), int(rng.integers(k, 20)); st = int(rng.choice([1, 2, 3])); pads = tuple(int(v) for v in rng.integers(0, k + 1, 4)); dil = int(rng.choice([1, 1, 2]))
                    s = O.conv_shape(n, c, h, w_, cout, k, k, stride=(st, st), pad=pads, dil=(dil, dil), groups=groups)
                    if min(O.conv_out_hw(s)) < 1: continue
                    x = synth.fill_u8((n, c, h, w_), tseed); w = synth.fill_u8((cout, c // groups, k, k), tseed + 1); b = synth.fill_i32((cout,), tseed + 2, -1000, 1000)
                    _, acc = O.conv2d(x, w, b, s, O.raw_quant(zp_in=zp_in, zp_w=zp_w), want_acc=True)
                    q = centred(acc, zp_in, zp_w, lo, hi)
                    wl = eden.W_OHWI if tseed % 3 == 0 else eden.W_OIHW
                    want = O.conv2d(x, w, b, s, q); got = gpu_conv(x, w, b, s, to_eh_requant(q), layout=layout, weight_layout=wl); desc = (kind, s, layout, wl)
        except Exception as e:
            raise AssertionError(("error", seed, it, kind, repr(e)[:300]))
        ran[kind] = ran.get(kind, 0) + 1
        if not np.array_equal(got, want):
            bad += 1
            print("MISMATCH", it, desc, q.as_tuple(), diff_report(got, want), flush=True)
    assert bad == 0, "%d of %d random instances differ from the oracle (MISMATCH lines above)" % (bad, sum(ran.values()))
    assert sum(ran.values()) > 300 and all(ran.get(k, 0) > 10 for k in ("conv", "conv1x1", "conv3x3", "dw", "fc", "deconv")), ran


@pytest.mark.parametrize("seed", [21, 22])
def test_random_perchannel_instances_match_the_oracle(seed):
    """The same idea for int8 weights with one multiplier and shift per output channel (uint8 tensors): convolution,
    depthwise convolution and deconvolution over random shapes, channel counts off the multiples of 16 and 4, groups,
    depth multipliers, both layouts and EXACT_CHANNELS on a fifth of the instances."""
    eden.init(0)
    print("random per-channel sweep, seed", seed, flush=True)
    rng = np.random.default_rng(seed)
    plans = {"conv": eden.ConvPlan, "dw": eden.DwConvPlan, "deconv": eden.DeconvPlan}
    ran, bad = {}, 0
    for it in range(240):
        kind = str(rng.choice(["conv", "dw", "deconv"]))
        layout = eden.NHWC if rng.random() < 0.7 else eden.NCHW
        flags = eden.EXACT_CHANNELS if rng.random() < 0.2 else 0
        tseed = int(rng.integers(1, 1 << 30))
        n = int(rng.integers(1, 4))
        h, w_ = int(rng.integers(3, 16)), int(rng.integers(3, 16))
        dm = 1
        if kind == "conv":
            groups = int(rng.choice([1, 1, 1, 2, 8])); cig = int(rng.choice([3, 4, 8, 16, 21, 32, 64])); cog = int(rng.choice([3, 8, 16, 24]))
            k = int(rng.choice([1, 1, 3, 3, 5])); st = int(rng.choice([1, 1, 2])); dil = int(rng.choice([1, 1, 2]))
            pads = tuple(int(v) for v in rng.integers(0, dil * (k - 1) + 1, 4))
            s = O.conv_shape(n, groups * cig, h, w_, groups * cog, k, k, stride=(st, st), pad=pads, dil=(dil, dil), groups=groups)
            out_hw, wshape, cout, fan = O.conv_out_hw(s), (groups * cog, cig, k, k), groups * cog, cig * k * k
        elif kind == "dw":
            c = int(rng.choice([4, 8, 16, 30, 7, 32])); dm = int(rng.choice([1, 1, 2])); k = int(rng.choice([3, 3, 5])); st = int(rng.choice([1, 2])); dil = int(rng.choice([1, 1, 2]))
            pads = tuple(int(v) for v in rng.integers(0, dil * (k - 1) + 1, 4))
            s = O.conv_shape(n, c, h, w_, c * dm, k, k, stride=(st, st), pad=pads, dil=(dil, dil), dm=dm)
            out_hw, wshape, cout, fan = O.conv_out_hw(s), (c * dm, 1, k, k), c * dm, k * k
        else:
            c = int(rng.choice([8, 16, 21, 32])); cout = int(rng.choice([8, 16, 21])); k = int(rng.choice([2, 3, 4, 6])); st = int(rng.choice([1, 2, 3]))
            pads = tuple(int(v) for v in rng.integers(0, k, 4))
            s = O.conv_shape(n, c, h // 2 + 1, w_ // 2 + 1, cout, k, k, stride=(st, st), pad=pads)
            out_hw, wshape, fan = O.deconv_out_hw(s), (c, cout, k, k), c * max(1, (k // st) ** 2)
        if min(out_hw) < 1:
            continue
        x = synth.fill_u8((s.n, s.c, s.h, s.w), tseed)
        w = (synth.fill_u8(wshape, tseed + 1).astype(np.int16) - 128).astype(np.int8)
        b = synth.fill_i32((cout,), tseed + 2, -500, 500)
        w_scales = (0.002 * (1.0 + 29.0 * synth.fill_u8((cout,), tseed + 3) / 255.0)).astype(np.float32)
        s_out = float(0.02 * float(w_scales.max()) * 74.0 * 74.0 * np.sqrt(fan) / 60.0)
        zp_in, zp_out = int(rng.integers(0, 256)), int(rng.integers(0, 256))
        q, mults, shifts = eden.make_requant_perchannel(0.02, zp_in, w_scales, s_out, zp_out, eden.ACT_NONE, False)
        oq = O.raw_quant(zp_in=zp_in, zp_w=0, zp_out=zp_out)
        want = {"conv": O.conv2d_perchannel, "dw": O.dwconv2d_perchannel, "deconv": O.deconv2d_perchannel}[kind](x, w, b, s, oq, mults, shifts)
        weight_layout = (eden.W_IOHW if kind == "deconv" else eden.W_OIHW) | eden.W_SIGNED
        desc = eden.conv_desc(s.n, s.c, s.h, s.w, cout, s.kh, s.kw, (s.stride_h, s.stride_w), (s.pad_t, s.pad_b, s.pad_l, s.pad_r),
                              (s.dil_h, s.dil_w), 1 if kind == "dw" else s.groups, dm, layout | flags, weight_layout)
        x_dev = x if layout == eden.NCHW else x.transpose(0, 2, 3, 1)
        d_x, d_w, d_b = eden.DeviceBuffer(host=x_dev), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
        d_o = eden.DeviceBuffer(nbytes=want.size)
        try:
            plan = plans[kind](desc, d_w, d_b, q)
            plan.set_perchannel(mults, shifts)
            plan.run(d_x, d_o, q)
            got = d_o.download(want.shape) if layout == eden.NCHW else d_o.download((s.n, out_hw[0], out_hw[1], cout)).transpose(0, 3, 1, 2)
            plan.destroy()
        except Exception as e:
            raise AssertionError(("error", seed, it, kind, s, layout, flags, repr(e)[:300]))
        ran[kind] = ran.get(kind, 0) + 1
        if not np.array_equal(got, want):
            bad += 1
            print("MISMATCH", it, kind, s, layout, flags, diff_report(np.ascontiguousarray(got), want), flush=True)
    assert bad == 0, "%d of %d random per-channel instances differ from the oracle (MISMATCH lines above)" % (bad, sum(ran.values()))
    assert all(ran.get(k, 0) > 40 for k in plans), ran


@pytest.mark.parametrize("seed", [31, 32])
def test_random_int8_instances_match_the_oracle(seed):
    """And for INT8 precision (int8 tensors and weights, zero points in [-128, 127]): the same kernels behind a sign flip
    on the way in and out, so what has to hold is that every staged copy, padding byte and zero-point constant is
    flipped too.  Convolution, depthwise convolution, deconvolution and fully connected layers over random shapes."""
    eden.init(0)
    print("random int8 sweep, seed", seed, flush=True)
    rng = np.random.default_rng(seed)
    s8 = lambda shape, sd: (synth.fill_u8(shape, sd).astype(np.int16) - 128).astype(np.int8)
    plans = {"conv": eden.ConvPlan, "dw": eden.DwConvPlan, "deconv": eden.DeconvPlan}
    oracles = {"conv": O.conv2d_s8, "dw": O.dwconv2d_s8, "deconv": O.deconv2d_s8}
    ran, bad = {}, 0
    for it in range(240):
        kind = str(rng.choice(["conv", "dw", "deconv", "fc"]))
        layout = eden.NHWC if rng.random() < 0.7 else eden.NCHW
        flags = eden.EXACT_CHANNELS if rng.random() < 0.2 else 0
        tseed = int(rng.integers(1, 1 << 30))
        zp_in, zp_w, zp_out = int(rng.integers(-128, 128)), int(rng.integers(-20, 21)), int(rng.integers(-128, 128))
        act, enabled = (eden.ACT_RELU6, True) if rng.random() < 0.3 else (eden.ACT_NONE, False)
        s_in, s_w = 0.02, 0.005
        if kind == "fc":
            m, k, n = int(rng.integers(1, 200)), int(rng.choice([16, 37, 64, 100, 256, 1001])), int(rng.integers(1, 200))
            s_out = float(s_in * s_w * 74.0 * 74.0 * np.sqrt(k) / 50.0)
            q = eden.make_requant_s8(s_in, zp_in, s_w, zp_w, s_out, zp_out, act, enabled)
            oq = O.make_quant_s8(s_in, zp_in, s_w, zp_w, s_out, zp_out, act, enabled)
            a, w, b = s8((m, k), tseed), s8((n, k), tseed + 1), synth.fill_i32((n,), tseed + 2, -500, 500)
            want = O.fc_s8(a, w, b, oq)
            d_a, d_w, d_b, d_o = eden.DeviceBuffer(host=a), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b), eden.DeviceBuffer(nbytes=m * n)
            plan = eden.FcPlan(m, k, n, d_w, d_b, q, flags=eden.W_SIGNED | eden.IO_SIGNED | flags)
            plan.run(d_a, d_o, q)
            got = d_o.download((m, n)).view(np.int8)
            plan.destroy()
            desc_txt = (m, k, n)
        else:
            n = int(rng.integers(1, 4))
            h, w_ = int(rng.integers(3, 16)), int(rng.integers(3, 16))
            dm = 1
            if kind == "conv":
                groups = int(rng.choice([1, 1, 1, 2, 8])); cig = int(rng.choice([3, 4, 8, 16, 21, 32, 64])); cog = int(rng.choice([3, 8, 16, 24]))
                k = int(rng.choice([1, 1, 3, 3, 5])); st = int(rng.choice([1, 1, 2])); dil = int(rng.choice([1, 1, 2]))
                pads = tuple(int(v) for v in rng.integers(0, dil * (k - 1) + 1, 4))
                s = O.conv_shape(n, groups * cig, h, w_, groups * cog, k, k, stride=(st, st), pad=pads, dil=(dil, dil), groups=groups)
                out_hw, wshape, cout, fan = O.conv_out_hw(s), (groups * cog, cig, k, k), groups * cog, cig * k * k
            elif kind == "dw":
                c = int(rng.choice([4, 8, 16, 30, 7, 32])); dm = int(rng.choice([1, 1, 2])); k = int(rng.choice([3, 3, 5])); st = int(rng.choice([1, 2])); dil = int(rng.choice([1, 1, 2]))
                pads = tuple(int(v) for v in rng.integers(0, dil * (k - 1) + 1, 4))
                s = O.conv_shape(n, c, h, w_, c * dm, k, k, stride=(st, st), pad=pads, dil=(dil, dil), dm=dm)
                out_hw, wshape, cout, fan = O.conv_out_hw(s), (c * dm, 1, k, k), c * dm, k * k
            else:
                c = int(rng.choice([8, 16, 21, 32])); cout = int(rng.choice([8, 16, 21])); k = int(rng.choice([2, 3, 4, 6])); st = int(rng.choice([1, 2, 3]))
                pads = tuple(int(v) for v in rng.integers(0, k, 4))
                s = O.conv_shape(n, c, h // 2 + 1, w_ // 2 + 1, cout, k, k, stride=(st, st), pad=pads)
                out_hw, wshape, fan = O.deconv_out_hw(s), (c, cout, k, k), c * max(1, (k // st) ** 2)
            if min(out_hw) < 1:
                continue
            s_out = float(s_in * s_w * 74.0 * 74.0 * np.sqrt(fan) / 50.0)
            q = eden.make_requant_s8(s_in, zp_in, s_w, zp_w, s_out, zp_out, act, enabled)
            oq = O.make_quant_s8(s_in, zp_in, s_w, zp_w, s_out, zp_out, act, enabled)
            x, w, b = s8((s.n, s.c, s.h, s.w), tseed), s8(wshape, tseed + 1), synth.fill_i32((cout,), tseed + 2, -500, 500)
            want = oracles[kind](x, w, b, s, oq)
            weight_layout = (eden.W_IOHW if kind == "deconv" else eden.W_OIHW) | eden.W_SIGNED
            desc = eden.conv_desc(s.n, s.c, s.h, s.w, cout, s.kh, s.kw, (s.stride_h, s.stride_w), (s.pad_t, s.pad_b, s.pad_l, s.pad_r),
                                  (s.dil_h, s.dil_w), 1 if kind == "dw" else s.groups, dm, layout | flags | eden.IO_SIGNED, weight_layout)
            x_dev = x if layout == eden.NCHW else x.transpose(0, 2, 3, 1)
            d_x, d_w, d_b = eden.DeviceBuffer(host=x_dev), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
            d_o = eden.DeviceBuffer(nbytes=want.size)
            try:
                plan = plans[kind](desc, d_w, d_b, q)
                plan.run(d_x, d_o, q)
                raw = d_o.download(want.shape) if layout == eden.NCHW else d_o.download((s.n, out_hw[0], out_hw[1], cout)).transpose(0, 3, 1, 2)
                plan.destroy()
            except Exception as e:
                raise AssertionError(("error", seed, it, kind, s, layout, flags, repr(e)[:300]))
            got = np.ascontiguousarray(raw).view(np.int8)
            desc_txt = (dict(n=s.n, c=s.c, h=s.h, w=s.w, cout=cout, k=s.kh, stride=s.stride_h, pad=(s.pad_t, s.pad_b, s.pad_l, s.pad_r), dil=s.dil_h, groups=s.groups, dm=dm),
                        layout, flags, (zp_in, zp_w, zp_out), act)
        ran[kind] = ran.get(kind, 0) + 1
        if not np.array_equal(got, want):
            bad += 1
            print("MISMATCH", it, kind, desc_txt, int((got != want).sum()), flush=True)
    assert bad == 0, "%d of %d random int8 instances differ from the oracle (MISMATCH lines above)" % (bad, sum(ran.values()))
    assert all(ran.get(k, 0) > 30 for k in ("conv", "dw", "deconv", "fc")), ran


@pytest.mark.parametrize("seed", [41, 42])
def test_random_network_sized_instances_match_the_oracle(seed):
    """The sweeps above keep to small tensors, which the small tiles serve.  This one draws layer shapes of the sizes image
    networks have (up to 1280 channels, 112 x 112 pixels, batch 32, reductions up to 9216 long), so that every tile
    size, the sliced reductions, the one-tap and patch kernels and the wide depthwise tiles are chosen by the same
    selection code that serves a real model; weight layouts vary too, and a convolution is run in one of four ways: as
    planned, with requantization parameters that differ from the ones it was planned with, with a residual added, or
    through the entry point that allocates nothing."""
    eden.init(0)
    print("random network-sized sweep, seed", seed, flush=True)
    rng = np.random.default_rng(seed)
    pick = lambda *v: v[int(rng.integers(0, len(v)))]
    jitter = lambda v: max(1, v + int(rng.integers(-1, 2)))
    def centred(acc, zp_in, zp_w):
        sd = float(acc.std()) or 1.0
        qm, sh = O.quantize_multiplier(float(pick(20.0, 40.0, 80.0)) / sd)
        zp_out = int(np.clip(128 - round(float(acc.mean()) * 40.0 / sd), 0, 255))
        return O.raw_quant(zp_in=zp_in, zp_w=zp_w, zp_out=zp_out, multiplier=qm, shift=sh, act_min=pick(0, 0, 30), act_max=pick(255, 255, 200))
    ran, kernels, modes, bad = {}, set(), {}, 0
    for it in range(110):
        kind = pick("pw", "pw", "conv3x3", "conv3x3", "convk", "grouped", "dw", "dw", "deconv", "fc")
        zp_in, zp_w = int(rng.integers(0, 256)), int(pick(128, int(rng.integers(100, 160))))
        layout = eden.NHWC if rng.random() < 0.8 else eden.NCHW
        flags = eden.EXACT_CHANNELS if rng.random() < 0.15 else 0
        tseed = int(rng.integers(1, 1 << 30))
        mode = "run"
        if kind == "fc":
            m, k, n = pick(1, 2, 8, 32, 64, 128, 256), pick(256, 1001, 1024, 1280, 2048, 4096, 9216), pick(10, 100, 1000, 1001, 4096)
            a, w, b = synth.fill_u8((m, k), tseed), synth.fill_u8_normal((n, k), tseed + 1, zp_w, 20), synth.fill_i32((n,), tseed + 2, -1000, 1000)
            _, acc = O.fc(a, w, b, O.raw_quant(zp_in=zp_in, zp_w=zp_w), want_acc=True)
            q = centred(acc, zp_in, zp_w)
            want, got, desc_txt = O.fc(a, w, b, q), gpu_fc(a, w, b, to_eh_requant(q), flags=flags), (m, k, n, flags)
        else:
            n = pick(1, 2, 8, 16, 32)
            hw = pick(7, 14, 28, 56, 112)
            groups, dm, dil, st = 1, 1, 1, pick(1, 1, 2)
            if kind == "pw":
                c, cout, k = pick(16, 24, 32, 64, 96, 144, 192, 256, 320, 384, 576, 960, 1280), pick(16, 21, 24, 32, 64, 96, 160, 256, 320, 512, 1001, 1280), 1
            elif kind == "conv3x3":
                c, cout, k, dil = pick(3, 16, 32, 64, 128, 256, 512), pick(16, 32, 64, 128, 256), 3, pick(1, 1, 1, 2)
            elif kind == "convk":
                c, cout, k = pick(3, 16, 64), pick(32, 64, 96), pick(5, 7)
            elif kind == "grouped":
                groups = pick(2, 4, 32); c, cout, k = groups * pick(4, 8, 16, 32), groups * pick(4, 8, 16, 32), pick(1, 3)
            elif kind == "dw":
                c = pick(32, 96, 144, 192, 384, 576, 960); cout, k, dil = c, pick(3, 3, 5), pick(1, 1, 2)
            else:
                c, cout, k = pick(21, 32, 64, 128, 256), pick(21, 32, 64, 128), pick(2, 3, 4, 8, 16)
                st = pick(*[v for v in (1, 2, 4, 8) if v <= k]); hw = pick(4, 7, 14, 28)
            h, w_ = jitter(hw), jitter(hw)
            same = dil * (k - 1)
            pads = (same // 2, same - same // 2, same // 2, same - same // 2) if rng.random() < 0.7 else tuple(int(v) for v in rng.integers(0, same + 1, 4))
            if kind == "deconv":
                pads = tuple(int(v) for v in rng.integers(0, max(1, k - st + 1), 4))
            s = O.conv_shape(n, c, h, w_, cout, k, k, stride=(st, st), pad=pads, dil=(dil, dil), groups=groups, dm=1)
            out_hw = O.deconv_out_hw(s) if kind == "deconv" else O.conv_out_hw(s)
            if min(out_hw) < 1:
                continue
            def work(nn):   # multiply-accumulates and bytes of the instance at batch nn
                px = nn * (s.h * s.w if kind == "deconv" else out_hw[0] * out_hw[1])
                red = k * k if kind == "dw" else (c // groups) * k * k
                return px * (cout if kind != "dw" else c) * red, nn * (c * h * w_ + cout * out_hw[0] * out_hw[1])
            cap = 8e9 if rng.random() < 0.2 else 1.2e9   # (one in five large enough for the 256-row tiles)
            while n > 1 and (work(n)[0] > cap or work(n)[1] > 0.04 * cap):
                n //= 2
            if work(n)[0] > 2 * cap:
                continue
            s = O.conv_shape(n, c, h, w_, cout, k, k, stride=(st, st), pad=pads, dil=(dil, dil), groups=groups, dm=1)
            x, b = synth.fill_u8((n, c, h, w_), tseed), synth.fill_i32((cout,), tseed + 2, -1000, 1000)
            if kind == "dw":
                w = synth.fill_u8((c, 1, k, k), tseed + 1)
                _, acc = O.dwconv2d(x, w, b, s, O.raw_quant(zp_in=zp_in, zp_w=zp_w), want_acc=True)
                q = centred(acc, zp_in, zp_w)
                want, got = O.dwconv2d(x, w, b, s, q), gpu_dwconv(x, w, b, s, to_eh_requant(q), layout=layout | flags)
            elif kind == "deconv":
                w = synth.fill_u8_normal((c, cout, k, k), tseed + 1, zp_w, 20)
                wl = pick(eden.W_IOHW, eden.W_OHWI)
                _, acc = O.deconv2d(x, w, b, s, O.raw_quant(zp_in=zp_in, zp_w=zp_w), want_acc=True)
                q = centred(acc, zp_in, zp_w)
                want, got = O.deconv2d(x, w, b, s, q), gpu_deconv(x, w, b, s, to_eh_requant(q), layout=layout | flags, weight_layout=wl)
                kernels.update(eden.conv_kernels(eden.conv_desc(n, c, h, w_, cout, k, k, (st, st), pads, (1, 1), 1, 1, layout | flags, wl), deconv=True))
            else:
                w = synth.fill_u8_normal((cout, c // groups, k, k), tseed + 1, zp_w, 20)
                wl = pick(eden.W_OIHW, eden.W_OHWI)
                _, acc = O.conv2d(x, w, b, s, O.raw_quant(zp_in=zp_in, zp_w=zp_w), want_acc=True)
                q = centred(acc, zp_in, zp_w)
                want = O.conv2d(x, w, b, s, q)
                mode = pick("run", "run", "other parameters", "residual", "static", "per channel")
                if mode == "per channel":   # int8 weights at zero point 0, one multiplier and shift per output channel
                    w = (w.astype(np.int16) - 128).astype(np.int8)
                    w_scales = (0.002 * (1.0 + 29.0 * synth.fill_u8((cout,), tseed + 4) / 255.0)).astype(np.float32)
                    s_out = float(0.02 * float(w_scales.max()) * 74.0 * 20.0 * np.sqrt((c // groups) * k * k) / 40.0)
                    pq, mults, shifts = eden.make_requant_perchannel(0.02, zp_in, w_scales, s_out, q.zp_out, eden.ACT_NONE, False)
                    q = O.raw_quant(zp_in=zp_in, zp_w=0, zp_out=q.zp_out)
                    want = O.conv2d_perchannel(x, w, b, s, q, mults, shifts)
                    wl |= eden.W_SIGNED
                desc = eden.conv_desc(n, c, h, w_, cout, k, k, (st, st), pads, (dil, dil), groups, 1, layout | flags, wl)
                kernels.update(eden.conv_kernels(desc))
                nhwc = layout == eden.NHWC
                to_dev = (lambda t: np.ascontiguousarray(t.transpose(0, 2, 3, 1))) if nhwc else (lambda t: t)
                d_x, d_w, d_b = eden.DeviceBuffer(host=to_dev(x)), eden.DeviceBuffer(host=w if wl & 0xFF == eden.W_OIHW else w.transpose(0, 2, 3, 1)), eden.DeviceBuffer(host=b)
                d_o = eden.DeviceBuffer(nbytes=want.size)
                planned = q
                if mode == "other parameters":
                    planned = O.raw_quant(zp_in=(zp_in + 77) % 256, zp_w=(zp_w + 9) % 256, zp_out=17, multiplier=q.multiplier // 2 + (1 << 29), shift=q.shift, act_min=0, act_max=255)
                plan = eden.ConvPlan(desc, d_w, d_b, pq if mode == "per channel" else to_eh_requant(planned))
                if mode == "per channel":
                    plan.set_perchannel(mults, shifts)
                    plan.run(d_x, d_o, pq)
                elif mode == "residual":
                    res = synth.fill_u8(want.shape, tseed + 3)
                    aq = O.make_add_quant(0.031, 120, 0.043, q.zp_out, 0.05, 125, O.ACT_NONE, False)
                    want = O.add(res, want, aq)
                    d_r = eden.DeviceBuffer(host=to_dev(res))
                    plan.run_add(d_x, d_r, d_o, to_eh_requant(q), to_eh_add(aq))
                elif mode == "static" and x.size + 2 * want.size < (8 << 20):
                    try:
                        plan.run_static(d_x, d_o, to_eh_requant(q))
                    except eden.EdenHipError as e:   # (its stated limit: the problems of one launch list)
                        assert "at most" in str(e), e
                        plan.run(d_x, d_o, to_eh_requant(q))
                else:
                    plan.run(d_x, d_o, to_eh_requant(q))
                got = d_o.download((n, out_hw[0], out_hw[1], cout)).transpose(0, 3, 1, 2) if nhwc else d_o.download(want.shape)
                plan.destroy()
            desc_txt = (dict(n=n, c=c, h=h, w=w_, cout=cout, k=k, stride=st, pad=pads, dil=dil, groups=groups), layout, flags, mode)
        ran[kind] = ran.get(kind, 0) + 1
        modes[mode] = modes.get(mode, 0) + 1
        if not np.array_equal(got, want):
            bad += 1
            print("MISMATCH", it, kind, desc_txt, q.as_tuple(), diff_report(got, want), flush=True)
    print("kernels chosen:", sorted(kernels), "modes:", modes, "kinds:", ran, flush=True)
    assert bad == 0, "%d of %d network-sized instances differ from the oracle (MISMATCH lines above)" % (bad, sum(ran.values()))
    assert sum(ran.values()) > 80 and len(kernels) >= 5, (ran, kernels)


@pytest.mark.parametrize("seed", [51])
def test_random_add_and_average_pool_instances_match_the_oracle(seed):
    """The two operators between the convolutions: element-wise Add over random lengths, pointer offsets and
    quantization parameters, AveragePool over random windows, strides, paddings, both tensor orders and both
    precisions."""
    eden.init(0)
    print("random add / average pool sweep, seed", seed, flush=True)
    rng = np.random.default_rng(seed)
    bad = 0
    for it in range(150):
        tseed = int(rng.integers(1, 1 << 30))
        count, off = int(rng.choice([1, 7, 16, 63, 1000, 4097, 70001, int(rng.integers(1, 200000))])), int(rng.choice([0, 0, 1, 3, 8]))
        s_a, s_b, s_o = (float(v) for v in rng.uniform(0.002, 0.3, 3))
        zps = [int(v) for v in rng.integers(0, 256, 3)]
        act, en = (O.ACT_NONE, False) if rng.random() < 0.6 else (int(rng.choice([O.ACT_RELU, O.ACT_RELU6])), True)
        q = O.make_add_quant(s_a, zps[0], s_b, zps[1], s_o, zps[2], act, en)
        a, b = synth.fill_u8((count,), tseed), synth.fill_u8((count,), tseed + 1)
        pad = np.zeros(off, np.uint8)
        d_a, d_b = eden.DeviceBuffer(host=np.concatenate([pad, a])), eden.DeviceBuffer(host=np.concatenate([pad, b]))
        d_o = eden.DeviceBuffer(nbytes=count + off + 16)
        eden.add_u8(d_a.ptr.value + off, d_b.ptr.value + off, d_o.ptr.value + off, count, to_eh_add(q))
        if not np.array_equal(d_o.download((count + off,))[off:], O.add(a, b, q)):
            bad += 1
            print("MISMATCH add", it, count, off, (s_a, s_b, s_o), zps, act, flush=True)
    for it in range(150):
        tseed = int(rng.integers(1, 1 << 30))
        n, c = int(rng.integers(1, 5)), int(rng.choice([1, 3, 4, 5, 8, 16, 24, 30, 64, 100, 320]))
        h, w = int(rng.integers(1, 24)), int(rng.integers(1, 24))
        kh, kw = int(rng.integers(1, min(h, 8) + 1)), int(rng.integers(1, min(w, 8) + 1))
        if rng.random() < 0.2:
            kh, kw = h, w   # a global pool
        stride = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        pad = (int(rng.integers(0, kh)), int(rng.integers(0, kh)), int(rng.integers(0, kw)), int(rng.integers(0, kw)))
        lo, hi = int(rng.choice([0, 0, 20])), int(rng.choice([255, 255, 180]))
        nhwc, signed = rng.random() < 0.6, rng.random() < 0.4
        x = synth.fill_u8((n, c, h, w), tseed)
        if signed:
            x = (x.astype(np.int16) - 128).astype(np.int8)
            want = O.avgpool_s8(x, kh, kw, stride, pad, lo - 128, hi - 128)
        else:
            want = O.avgpool(x, kh, kw, stride, pad, lo, hi)
        if want.size == 0:
            continue
        d_in = eden.DeviceBuffer(host=np.ascontiguousarray(x.transpose(0, 2, 3, 1)) if nhwc else x)
        d_out = eden.DeviceBuffer(nbytes=want.size)
        eden.avgpool_u8(d_in, d_out, n, c, h, w, kh, kw, stride, pad, (eden.NHWC if nhwc else eden.NCHW) | (eden.IO_SIGNED if signed else 0),
                        lo - 128 if signed else lo, hi - 128 if signed else hi)
        ho, wo = want.shape[2:]
        got = d_out.download((n, ho, wo, c)).transpose(0, 3, 1, 2) if nhwc else d_out.download(want.shape)
        if not np.array_equal(np.ascontiguousarray(got).view(want.dtype), want):
            bad += 1
            print("MISMATCH avgpool", it, (n, c, h, w), (kh, kw), stride, pad, (lo, hi), "nhwc" if nhwc else "nchw", "int8" if signed else "uint8", flush=True)
    assert bad == 0, "%d random add / average pool instances differ from the oracle (MISMATCH lines above)" % bad


@pytest.mark.parametrize("seed", [61, 62])
def test_random_rectangular_instances_match_the_oracle(seed):
    """Kernels, strides and dilations that differ between rows and columns (the 1 x 7 and 7 x 1 layers of Inception-style
    networks and their like): convolution, depthwise convolution and deconvolution over random shapes, at channel
    counts that reach the patch, row, one-tap and tiled kernels."""
    eden.init(0)
    print("random rectangular sweep, seed", seed, flush=True)
    rng = np.random.default_rng(seed)
    pick = lambda *v: v[int(rng.integers(0, len(v)))]
    ran, bad = {}, 0
    for it in range(300):
        kind = pick("conv", "conv", "dw", "deconv")
        zp_in, zp_w = int(rng.integers(0, 256)), int(pick(128, int(rng.integers(0, 256))))
        layout = (eden.NHWC if rng.random() < 0.7 else eden.NCHW) | (eden.EXACT_CHANNELS if rng.random() < 0.15 else 0)
        tseed = int(rng.integers(1, 1 << 30))
        n, h, w_ = int(rng.integers(1, 4)), int(rng.integers(4, 24)), int(rng.integers(4, 24))
        kh, kw = pick(1, 1, 2, 3, 5, 7), pick(1, 1, 2, 3, 5, 7)
        sh, sw = pick(1, 1, 2, 3), pick(1, 1, 2, 3)
        dh, dw_ = pick(1, 1, 2, 3), pick(1, 1, 2, 3)
        raw = lambda: O.raw_quant(zp_in=zp_in, zp_w=zp_w)
        def centred(acc):
            sd = float(acc.std()) or 1.0
            qm, sh_ = O.quantize_multiplier(float(pick(10.0, 40.0, 120.0)) / sd)
            return O.raw_quant(zp_in=zp_in, zp_w=zp_w, zp_out=int(np.clip(128 - round(float(acc.mean()) * 40.0 / sd), 0, 255)), multiplier=qm, shift=sh_, act_min=0, act_max=255)
        if kind == "deconv":
            c, cout = pick(8, 16, 21, 32, 64), pick(8, 16, 21, 32)
            pads = (int(rng.integers(0, kh)), int(rng.integers(0, kh)), int(rng.integers(0, kw)), int(rng.integers(0, kw)))
            s = O.conv_shape(n, c, h // 2 + 1, w_ // 2 + 1, cout, kh, kw, stride=(sh, sw), pad=pads)
            if min(O.deconv_out_hw(s)) < 1: continue
            x, w, b = synth.fill_u8((n, c, s.h, s.w), tseed), synth.fill_u8((c, cout, kh, kw), tseed + 1), synth.fill_i32((cout,), tseed + 2, -1000, 1000)
            q = centred(O.deconv2d(x, w, b, s, raw(), want_acc=True)[1])
            want, got = O.deconv2d(x, w, b, s, q), gpu_deconv(x, w, b, s, to_eh_requant(q), layout=layout, weight_layout=pick(eden.W_IOHW, eden.W_OHWI))
        else:
            pads = (int(rng.integers(0, dh * (kh - 1) + 1)), int(rng.integers(0, dh * (kh - 1) + 1)), int(rng.integers(0, dw_ * (kw - 1) + 1)), int(rng.integers(0, dw_ * (kw - 1) + 1)))
            if kind == "dw":
                c, dm = pick(4, 8, 16, 30, 32, 7, 144), pick(1, 1, 1, 2)
                s = O.conv_shape(n, c, h, w_, c * dm, kh, kw, stride=(sh, sw), pad=pads, dil=(dh, dw_), dm=dm)
                if min(O.conv_out_hw(s)) < 1: continue
                x, w, b = synth.fill_u8((n, c, h, w_), tseed), synth.fill_u8((c * dm, 1, kh, kw), tseed + 1), synth.fill_i32((c * dm,), tseed + 2, -1000, 1000)
                q = centred(O.dwconv2d(x, w, b, s, raw(), want_acc=True)[1])
                want, got = O.dwconv2d(x, w, b, s, q), gpu_dwconv(x, w, b, s, to_eh_requant(q), layout=layout)
            else:
                groups = pick(1, 1, 1, 2, 8)
                c, cout = groups * pick(1, 3, 4, 8, 16, 21, 32, 64, 128, 192), groups * pick(3, 8, 16, 24, 64, 100)
                s = O.conv_shape(n, c, h, w_, cout, kh, kw, stride=(sh, sw), pad=pads, dil=(dh, dw_), groups=groups)
                if min(O.conv_out_hw(s)) < 1: continue
                x, w, b = synth.fill_u8((n, c, h, w_), tseed), synth.fill_u8((cout, c // groups, kh, kw), tseed + 1), synth.fill_i32((cout,), tseed + 2, -1000, 1000)
                q = centred(O.conv2d(x, w, b, s, raw(), want_acc=True)[1])
                want, got = O.conv2d(x, w, b, s, q), gpu_conv(x, w, b, s, to_eh_requant(q), layout=layout, weight_layout=pick(eden.W_OIHW, eden.W_OHWI))
        ran[kind] = ran.get(kind, 0) + 1
        if not np.array_equal(got, want):
            bad += 1
            print("MISMATCH", it, kind, s, layout, q.as_tuple(), diff_report(got, want), flush=True)
    assert bad == 0, "%d of %d rectangular instances differ from the oracle (MISMATCH lines above)" % (bad, sum(ran.values()))
    assert all(ran.get(k, 0) > 40 for k in ("conv", "dw", "deconv")), ran
