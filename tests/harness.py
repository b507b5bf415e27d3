"""Shared helpers of the GPU parity tests: run one operator through the C ABI and
through the CPU oracle on the same seeded tensors."""
import importlib

import numpy as np

import oracle_lib as O

eden = importlib.import_module("cl-eden-kernel_amd")
synth = importlib.import_module("cl-eden-kernel_amd.synth")
mobilenet = importlib.import_module("cl-eden-kernel_amd.mobilenet")


def to_eh_requant(q):
    return eden.Requant(*q.as_tuple())


def to_eh_add(q):
    r = eden.AddRequant()
    for f, _ in eden.AddRequant._fields_:
        setattr(r, f, getattr(q, f))
    return r


def assert_same_host_quant(args, kwargs):
    """The product's own parameter derivation must agree with the oracle's."""
    a = eden.make_requant(*args, **kwargs).as_tuple()
    b = O.make_quant(*args, **kwargs).as_tuple()
    assert a == b, (a, b)


def gpu_conv(x_nchw, w, bias, s, q, layout=eden.NCHW, weight_layout=eden.W_OIHW, runs=1):
    """x_nchw: uint8 NCHW array; w in OIHW; returns NCHW uint8 output of the GPU path.  `layout` may carry plan flags
    (eden.EXACT_CHANNELS) beside the tensor order."""
    flags, layout = layout & ~0xFF, layout & 0xFF
    ho, wo = O.conv_out_hw(s)
    desc = eden.conv_desc(s.n, s.c, s.h, s.w, s.cout, s.kh, s.kw, (s.stride_h, s.stride_w),
                          (s.pad_t, s.pad_b, s.pad_l, s.pad_r), (s.dil_h, s.dil_w), s.groups, 1, layout | flags, weight_layout)
    x_dev = x_nchw if layout == eden.NCHW else x_nchw.transpose(0, 2, 3, 1)
    w_dev = w if weight_layout == eden.W_OIHW else w.transpose(0, 2, 3, 1)
    d_x, d_w, d_b = eden.DeviceBuffer(host=x_dev), eden.DeviceBuffer(host=w_dev), (eden.DeviceBuffer(host=bias) if bias is not None else None)
    d_o = eden.DeviceBuffer(nbytes=s.n * s.cout * ho * wo)
    plan = eden.ConvPlan(desc, d_w, d_b, q)
    for _ in range(runs):
        plan.run(d_x, d_o, q)
    if layout == eden.NCHW:
        out = d_o.download((s.n, s.cout, ho, wo))
    else:
        out = d_o.download((s.n, ho, wo, s.cout)).transpose(0, 3, 1, 2)
    plan.destroy()
    return np.ascontiguousarray(out)


def gpu_dwconv(x_nchw, w, bias, s, q, layout=eden.NCHW):
    flags, layout = layout & ~0xFF, layout & 0xFF   # (eden.EXACT_CHANNELS: no staging images)
    ho, wo = O.conv_out_hw(s)
    cout = s.c * max(s.dm, 1)
    desc = eden.conv_desc(s.n, s.c, s.h, s.w, cout, s.kh, s.kw, (s.stride_h, s.stride_w),
                          (s.pad_t, s.pad_b, s.pad_l, s.pad_r), (s.dil_h, s.dil_w), 1, max(s.dm, 1), layout | flags, eden.W_OIHW)
    x_dev = x_nchw if layout == eden.NCHW else x_nchw.transpose(0, 2, 3, 1)
    d_x, d_w, d_b = eden.DeviceBuffer(host=x_dev), eden.DeviceBuffer(host=w), (eden.DeviceBuffer(host=bias) if bias is not None else None)
    d_o = eden.DeviceBuffer(nbytes=s.n * cout * ho * wo)
    plan = eden.DwConvPlan(desc, d_w, d_b, q)
    plan.run(d_x, d_o, q)
    if layout == eden.NCHW:
        out = d_o.download((s.n, cout, ho, wo))
    else:
        out = d_o.download((s.n, ho, wo, cout)).transpose(0, 3, 1, 2)
    plan.destroy()
    return np.ascontiguousarray(out)


def gpu_deconv(x_nchw, w_iohw, bias, s, q, layout=eden.NCHW, weight_layout=eden.W_IOHW):
    flags, layout = layout & ~0xFF, layout & 0xFF
    ho, wo = O.deconv_out_hw(s)
    desc = eden.conv_desc(s.n, s.c, s.h, s.w, s.cout, s.kh, s.kw, (s.stride_h, s.stride_w),
                          (s.pad_t, s.pad_b, s.pad_l, s.pad_r), (1, 1), s.groups, 1, layout | flags, weight_layout)
    x_dev = x_nchw if layout == eden.NCHW else x_nchw.transpose(0, 2, 3, 1)
    w_dev = w_iohw if weight_layout == eden.W_IOHW else w_iohw.transpose(1, 2, 3, 0)
    d_x, d_w, d_b = eden.DeviceBuffer(host=x_dev), eden.DeviceBuffer(host=w_dev), (eden.DeviceBuffer(host=bias) if bias is not None else None)
    d_o = eden.DeviceBuffer(nbytes=s.n * s.cout * ho * wo)
    plan = eden.DeconvPlan(desc, d_w, d_b, q)
    plan.run(d_x, d_o, q)
    if layout == eden.NCHW:
        out = d_o.download((s.n, s.cout, ho, wo))
    else:
        out = d_o.download((s.n, ho, wo, s.cout)).transpose(0, 3, 1, 2)
    plan.destroy()
    return np.ascontiguousarray(out)


def gpu_fc(a, w, bias, q, flags=0):
    m, k = a.shape
    n = w.shape[0]
    d_a, d_w, d_b = eden.DeviceBuffer(host=a), eden.DeviceBuffer(host=w), (eden.DeviceBuffer(host=bias) if bias is not None else None)
    d_o = eden.DeviceBuffer(nbytes=m * n)
    plan = eden.FcPlan(m, k, n, d_w, d_b, q, flags=flags)
    plan.run(d_a, d_o, q)
    out = d_o.download((m, n))
    plan.destroy()
    return out


def scattered_batch(batch, distinct=8, seed=2025):
    """Which of `distinct` oracle-evaluated images sits at each of `batch` positions: seeded and without a period, so
    that a kernel reading image i +- 1, 2, 4, 8 ... instead of image i cannot pass; the first two, the middle two and
    the last two positions hold six different images and every image is used."""
    rng = np.random.default_rng(seed)
    while True:
        idx = rng.integers(0, distinct, batch)
        ends = [0, 1, batch // 2 - 1, batch // 2, batch - 2, batch - 1]
        shifted_equal = any(np.array_equal(idx[k:], idx[:-k]) for k in (1, 2, 4, 8, 16, 32) if k < batch)
        if len(set(idx[ends].tolist())) == min(6, distinct) and len(set(idx.tolist())) == distinct and not shifted_equal:
            return idx


def diff_report(got, want):
    bad = np.argwhere(got != want)
    return "%d of %d differ; first at %s: got %s want %s" % (
        len(bad), got.size, bad[0].tolist() if len(bad) else None,
        got[tuple(bad[0])] if len(bad) else None, want[tuple(bad[0])] if len(bad) else None)


def oracle_forward(x_nhwc, image, per_channel=False, weights="minmax"):
    """All tensors of the network, NCHW, computed by the oracle from the same operator list."""
    tensors, ops = mobilenet.layers(image, weights)
    vals = [np.ascontiguousarray(x_nhwc.transpose(0, 3, 1, 2))]
    n = x_nhwc.shape[0]
    for op in ops:
        kind = op["op"]
        if kind == "add":
            a, b, d = (tensors[op[k]] for k in ("a", "b", "dst"))
            q = O.make_add_quant(a["scale"], a["zp"], b["scale"], b["zp"], d["scale"], d["zp"])
            vals.append(O.add(vals[op["a"]], vals[op["b"]], q))
            continue
        s, d = tensors[op["src"]], tensors[op["dst"]]
        x = vals[op["src"]]
        if kind == "avgpool":
            vals.append(O.avgpool(x, op["k"], op["k"]))
            continue
        act = O.ACT_RELU6 if op.get("relu6") else O.ACT_NONE
        if per_channel and kind != "fc":
            w, b, w_scales = mobilenet.op_weights_perchannel(op, s["c"])
            mults, shifts = O.perchannel_pairs(s["scale"], w_scales, d["scale"])
            lo, hi = O.act_range_u8(act if op.get("relu6") else O.ACT_NONE, d["scale"], d["zp"])
            q = O.raw_quant(zp_in=s["zp"], zp_w=0, zp_out=d["zp"], act_min=lo, act_max=hi)
            groups = s["c"] if kind == "dw" else 1
            shape = O.conv_shape(n, s["c"], s["h"], s["w"], op["cout"], op["k"], op["k"], (op["stride"],) * 2, (op["pad"],) * 4,
                                 groups=groups)
            fn = O.dwconv2d_perchannel if kind == "dw" else O.conv2d_perchannel
            vals.append(fn(x, w, b, shape, q, mults, shifts))
            continue
        w, b = mobilenet.op_weights(op, s["c"])
        q = O.make_quant(s["scale"], s["zp"], op["w_scale"], op["w_zp"], d["scale"], d["zp"], act, bool(op.get("relu6")))
        if kind == "fc":
            vals.append(O.fc(x.reshape(n, -1), w, b, q).reshape(n, -1, 1, 1))
        elif kind == "dw":
            shape = O.conv_shape(n, s["c"], s["h"], s["w"], op["cout"], op["k"], op["k"], (op["stride"],) * 2, (op["pad"],) * 4,
                                 groups=s["c"])
            vals.append(O.dwconv2d(x, w, b, shape, q))
        else:
            shape = O.conv_shape(n, s["c"], s["h"], s["w"], op["cout"], op["k"], op["k"], (op["stride"],) * 2, (op["pad"],) * 4)
            vals.append(O.conv2d(x, w, b, shape, q))
    return tensors, ops, vals
