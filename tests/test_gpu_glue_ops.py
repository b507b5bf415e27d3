"""Quantized element-wise Add and AveragePool on the GPU (through the C ABI) against the oracle, bit-exact."""
import numpy as np
import pytest

import oracle_lib as O
from harness import eden, synth

pytestmark = pytest.mark.gpu

SEED = 0xEDE2 + 16 * 7


def to_eh_add(q):
    r = eden.AddRequant()
    for f, _ in eden.AddRequant._fields_:
        setattr(r, f, getattr(q, f))
    return r


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
