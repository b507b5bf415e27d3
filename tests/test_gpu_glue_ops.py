"""Quantized element-wise Add and AveragePool on the GPU (through the C ABI) against the oracle, bit-exact."""
import numpy as np
import pytest

import oracle_lib as O
from harness import eden, synth, to_eh_add, to_eh_requant

pytestmark = pytest.mark.gpu

SEED = 0xEDE2 + 16 * 7


def gpu_add(a, b, q, offset=0):
    """offset > 0 shifts all three device pointers off 16-byte alignment (byte path)."""
    pad = np.zeros(offset, np.uint8)
    da = eden.DeviceBuffer(host=np.concatenate([pad, a.reshape(-1)]))
    db = eden.DeviceBuffer(host=np.concatenate([pad, b.reshape(-1)]))
    do = eden.DeviceBuffer(nbytes=a.size + offset + 16)
    eden.add_u8(da.ptr.value + offset, db.ptr.value + offset, do.ptr.value + offset, a.size, q)
    return do.download((a.size + offset,))[offset:].reshape(a.shape)


ADD_PARAMS = [
    # s_a, zp_a, s_b, zp_b, s_out, zp_out, act
    (0.02, 128, 0.02, 128, 0.04, 128, None),
    (0.0235, 3, 0.011, 250, 0.03, 77, None),
    (0.5, 0, 0.001, 255, 0.25, 10, O.ACT_RELU6),
    (0.004, 100, 0.3, 17, 0.1, 200, O.ACT_RELU),
]


@pytest.mark.parametrize("params", ADD_PARAMS, ids=lambda p: "-".join(str(v) for v in p[:6]))
@pytest.mark.parametrize("count,offset", [(1, 0), (15, 0), (16, 0), (4099, 0), (64 * 56 * 56 * 24 + 5, 0), (1000, 3)])
def test_add_matches_oracle(params, count, offset):
    print("add", params, count, offset, flush=True)
    s_a, zp_a, s_b, zp_b, s_out, zp_out, act = params
    q = O.make_add_quant(s_a, zp_a, s_b, zp_b, s_out, zp_out, act or O.ACT_NONE, act is not None)
    ge = eden.make_add_requant(s_a, zp_a, s_b, zp_b, s_out, zp_out, act or eden.ACT_NONE, act is not None)
    for f, _ in eden.AddRequant._fields_:
        assert getattr(ge, f) == getattr(q, f), f
    a = synth.fill_u8((count,), SEED + count)
    b = synth.fill_u8((count,), SEED + count + 1)
    want = O.add(a, b, q)
    got = gpu_add(a, b, ge, offset)
    assert np.array_equal(got, want), np.nonzero(got != want)[0][:10]
    if count > 1000:
        assert len(np.unique(want)) > 20


def test_add_every_input_pair():
    """All 65536 (a, b) byte pairs for one parameter set."""
    a, b = np.meshgrid(np.arange(256, dtype=np.uint8), np.arange(256, dtype=np.uint8), indexing="ij")
    q = O.make_add_quant(0.0173, 121, 0.0291, 140, 0.035, 131, O.ACT_NONE, False)
    got = gpu_add(np.ascontiguousarray(a), np.ascontiguousarray(b), to_eh_add(q))
    assert np.array_equal(got, O.add(a, b, q))


POOL_CASES = [
    # n, c, h, w, kh, kw, stride, pad, act range
    (2, 1280, 7, 7, 7, 7, (1, 1), (0, 0, 0, 0), (0, 255)),       # the global pool of the classifier head
    (3, 8, 9, 11, 3, 3, (2, 2), (1, 1, 1, 1), (0, 255)),          # windows clipped at the borders
    (1, 5, 6, 6, 2, 2, (2, 2), (0, 0, 0, 0), (10, 200)),          # odd channel count: scalar kernels
    (2, 16, 8, 8, 5, 3, (1, 2), (2, 2, 1, 1), (0, 255)),
    (1, 4, 3, 3, 3, 3, (1, 1), (2, 2, 2, 2), (0, 255)),           # some windows hold a single pixel
    (2, 24, 13, 12, 13, 12, (1, 1), (0, 0, 0, 0), (0, 255)),      # more window rows than the lanes that share them
    (24, 64, 40, 40, 5, 5, (1, 1), (2, 2, 2, 2), (0, 255)),       # tall windows, many outputs: one lane per output
]


@pytest.mark.parametrize("layout", ["nchw", "nhwc"])
@pytest.mark.parametrize("case", POOL_CASES, ids=lambda c: "x".join(str(v) for v in c[:6]))
def test_avgpool_matches_oracle(case, layout):
    print("avgpool", case, layout, flush=True)
    n, c, h, w, kh, kw, stride, pad, (lo, hi) = case
    x = synth.fill_u8((n, c, h, w), SEED + c + h)
    want = O.avgpool(x, kh, kw, stride, pad, lo, hi)
    nhwc = layout == "nhwc"
    src = np.ascontiguousarray(x.transpose(0, 2, 3, 1)) if nhwc else x
    d_in = eden.DeviceBuffer(host=src)
    d_out = eden.DeviceBuffer(nbytes=want.size)
    eden.avgpool_u8(d_in, d_out, n, c, h, w, kh, kw, stride, pad, eden.NHWC if nhwc else eden.NCHW, lo, hi)
    ho, wo = want.shape[2:]
    got = d_out.download((n, ho, wo, c)).transpose(0, 3, 1, 2) if nhwc else d_out.download(want.shape)
    assert np.array_equal(got, want)
    assert want.std() > 1


@pytest.mark.parametrize("layout", ["nchw", "nhwc"])
@pytest.mark.parametrize("case", POOL_CASES, ids=lambda c: "x".join(str(v) for v in c[:6]))
def test_avgpool_int8_matches_oracle(case, layout):
    print("avgpool int8", case, layout, flush=True)
    n, c, h, w, kh, kw, stride, pad, (lo, hi) = case
    lo, hi = lo - 128, hi - 128
    x = (synth.fill_u8((n, c, h, w), SEED + c + h + 1).astype(np.int16) - 128).astype(np.int8)
    x[0, 0, :2, :2] = np.array([[-1, 0], [0, -1]], np.int8)  # a negative tie in the first window
    want = O.avgpool_s8(x, kh, kw, stride, pad, lo, hi)
    nhwc = layout == "nhwc"
    src = np.ascontiguousarray(x.transpose(0, 2, 3, 1)) if nhwc else x
    d_in = eden.DeviceBuffer(host=src)
    d_out = eden.DeviceBuffer(nbytes=want.size)
    eden.avgpool_u8(d_in, d_out, n, c, h, w, kh, kw, stride, pad, (eden.NHWC if nhwc else eden.NCHW) | eden.IO_SIGNED, lo, hi)
    ho, wo = want.shape[2:]
    got = d_out.download((n, ho, wo, c)).transpose(0, 3, 1, 2) if nhwc else d_out.download(want.shape)
    assert np.array_equal(np.ascontiguousarray(got).view(np.int8), want)
    assert want.std() > 1


RUN_ADD_CASES = [
    # one-tap kernel (fused), split-reduction tiles (fused), 128 x 128 tiles and the register-staged kernel (second launch)
    dict(n=2, c=144, h=14, w=14, cout=24, kh=1, kw=1, fused=True),
    dict(n=2, c=32, h=9, w=9, cout=40, kh=1, kw=1, fused=True),
    # at most 64 pixels under a long reduction (the 7 x 7 stage of an image network at batch 1): the kernel cut along the weights adds the residual too
    dict(n=1, c=960, h=7, w=7, cout=160, kh=1, kw=1, fused=True),
    dict(n=2, c=512, h=5, w=5, cout=50, kh=1, kw=1, fused=True),
    dict(n=4, c=384, h=14, w=14, cout=64, kh=1, kw=1, fused=True),
    dict(n=2, c=576, h=7, w=7, cout=96, kh=1, kw=1, fused=True),
    dict(n=32, c=264, h=28, w=28, cout=256, kh=1, kw=1, fused=False),
    dict(n=1, c=20, h=8, w=8, cout=12, kh=3, kw=3, pad=(1, 1, 1, 1), groups=2, fused=False, exact=True),
    # a reduction sliced over workgroups: the launch that adds the slices up adds the residual
    dict(n=2, c=768, h=7, w=7, cout=72, kh=3, kw=3, pad=(1, 1, 1, 1), fused=True),
    # the same on its channel-padded copy: split-reduction tiles (fused)
    dict(n=1, c=20, h=8, w=8, cout=12, kh=3, kw=3, pad=(1, 1, 1, 1), groups=2, fused=True),
]


@pytest.mark.parametrize("layout", ["nhwc", "nchw"])
@pytest.mark.parametrize("case", RUN_ADD_CASES, ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_conv_with_residual_add_equals_conv_then_add(case, layout):
    print("conv + add", case, layout, flush=True)
    case = dict(case)
    fused = case.pop("fused")
    flags = eden.EXACT_CHANNELS if case.pop("exact", False) else 0
    s = O.conv_shape(**case)
    ho, wo = O.conv_out_hw(s)
    x = synth.fill_u8((s.n, s.c, s.h, s.w), SEED + 500 + s.c)
    w = synth.fill_u8_normal((s.cout, s.c // s.groups, s.kh, s.kw), SEED + 501, 131, 20)
    b = synth.fill_i32((s.cout,), SEED + 502, -500, 500)
    res = synth.fill_u8((s.n, s.cout, ho, wo), SEED + 503)
    fan = (s.c // s.groups) * s.kh * s.kw
    s_out = float(0.02 * 0.005 * 74.0 * 20.0 * np.sqrt(fan) / 30.0)
    for act, en in ((O.ACT_NONE, False), (O.ACT_RELU, True)):
        q = O.make_quant(0.02, 117, 0.005, 131, s_out, 128, act, en)
        aq = O.make_add_quant(0.031, 120, s_out, 128, 0.05, 125, O.ACT_NONE, False)
        want = O.add(res, O.conv2d(x, w, b, s, q), aq)
        nhwc = layout == "nhwc"
        desc = eden.conv_desc(s.n, s.c, s.h, s.w, s.cout, s.kh, s.kw, (s.stride_h, s.stride_w), (s.pad_t, s.pad_b, s.pad_l, s.pad_r),
                              (1, 1), s.groups, 1, (eden.NHWC if nhwc else eden.NCHW) | flags, eden.W_OIHW)
        to_dev = (lambda a: np.ascontiguousarray(a.transpose(0, 2, 3, 1))) if nhwc else (lambda a: a)
        d_x, d_w, d_b = eden.DeviceBuffer(host=to_dev(x)), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
        d_r, d_o = eden.DeviceBuffer(host=to_dev(res)), eden.DeviceBuffer(nbytes=want.size)
        plan = eden.ConvPlan(desc, d_w, d_b, to_eh_requant(q))
        assert plan.fuses_add() == (fused and nhwc)
        plan.run_add(d_x, d_r, d_o, to_eh_requant(q), to_eh_add(aq))
        got = d_o.download((s.n, ho, wo, s.cout)).transpose(0, 3, 1, 2) if nhwc else d_o.download(want.shape)
        assert np.array_equal(got, want), int((got != want).sum())
        # the plan still runs without the add
        plan.run(d_x, d_o, to_eh_requant(q))
        got = d_o.download((s.n, ho, wo, s.cout)).transpose(0, 3, 1, 2) if nhwc else d_o.download(want.shape)
        assert np.array_equal(got, O.conv2d(x, w, b, s, q))
        plan.destroy()
    assert want.std() > 4


def test_streaming_yardsticks_move_what_they_say():
    """eh_probe_stream (the byte-moving kernels the HBM-bound figures are set against): copy, one chunk written six
    times, four chunks folded into one; every 16-byte chunk of the output checked."""
    lib = eden.load()
    chunks = 6 * 1000 + 6          # output chunks; a multiple of 6, not of 256
    out_bytes = chunks * 16
    src = synth.fill_u8((4 * out_bytes,), SEED + 90)
    d_in = eden.DeviceBuffer(host=src)
    d_out = eden.DeviceBuffer(nbytes=out_bytes)
    words = src.view(np.uint32).reshape(-1, 4)
    # copy
    eden.check(lib.eh_probe_stream(d_in.ptr, d_out.ptr, out_bytes, 0, None))
    eden.sync()
    assert np.array_equal(d_out.download((out_bytes,)), src[:out_bytes])
    # 1 -> 6: chunk i of the output is chunk i / 6 of the input with i added to its first word
    eden.check(lib.eh_probe_stream(d_in.ptr, d_out.ptr, out_bytes, 1, None))
    eden.sync()
    want = words[np.arange(chunks) // 6].copy()
    want[:, 0] += np.arange(chunks, dtype=np.uint32)
    assert np.array_equal(d_out.download((out_bytes,)).view(np.uint32).reshape(-1, 4), want)
    # 4 -> 1: the xor of four consecutive input chunks
    eden.check(lib.eh_probe_stream(d_in.ptr, d_out.ptr, out_bytes, 2, None))
    eden.sync()
    want = words[: 4 * chunks].reshape(chunks, 4, 4)
    want = want[:, 0] ^ want[:, 1] ^ want[:, 2] ^ want[:, 3]
    assert np.array_equal(d_out.download((out_bytes,)).view(np.uint32).reshape(-1, 4), want)
    with pytest.raises(eden.EdenHipError):
        eden.check(lib.eh_probe_stream(d_in.ptr, d_out.ptr, out_bytes + 8, 0, None))
