"""The entry point that allocates nothing (eh_conv2d_u8_run_static): a planar convolution staged in the library's
static device scratch must give, bit for bit, what eh_conv2d_u8_run gives with the plan's own staging buffers (and
the oracle), on two calls in a row that share the scratch, the second with a smaller input; sizes beyond the scratch
are refused without a launch."""
import numpy as np
import pytest

import oracle_lib as O
from harness import diff_report, eden, synth, to_eh_requant

pytestmark = pytest.mark.gpu

SEED = 0xEDE2 + 700


def planar_conv(case, seed):
    s = O.conv_shape(**case)
    x = synth.fill_u8((s.n, s.c, s.h, s.w), seed)
    w = synth.fill_u8((s.cout, s.c // s.groups, s.kh, s.kw), seed + 1)
    b = synth.fill_i32((s.cout,), seed + 2, -1000, 1000)
    _, acc = O.conv2d(x, w, b, s, O.raw_quant(zp_in=131, zp_w=120), want_acc=True)
    sd = float(acc.std()) or 1.0
    qm, sh = O.quantize_multiplier(40.0 / sd)
    q = O.raw_quant(zp_in=131, zp_w=120, zp_out=int(128 - round(float(acc.mean()) * 40.0 / sd)), multiplier=qm, shift=sh)
    ho, wo = O.conv_out_hw(s)
    desc = eden.conv_desc(s.n, s.c, s.h, s.w, s.cout, s.kh, s.kw, (s.stride_h, s.stride_w), (s.pad_t, s.pad_b, s.pad_l, s.pad_r),
                          (s.dil_h, s.dil_w), s.groups, 1, eden.NCHW, eden.W_OIHW)
    d_x, d_w, d_b = eden.DeviceBuffer(host=x), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    plan = eden.ConvPlan(desc, d_w, d_b, to_eh_requant(q))
    return dict(s=s, q=to_eh_requant(q), want=O.conv2d(x, w, b, s, q), shape=(s.n, s.cout, ho, wo), d_x=d_x, keep=(d_w, d_b), plan=plan)


def test_static_scratch_entry_point_equals_the_allocating_one_on_two_calls_in_a_row():
    eden.init(0)
    big = planar_conv(dict(n=3, c=64, h=40, w=36, cout=96, kh=3, kw=3, pad=(1, 1, 1, 1)), SEED)
    small = planar_conv(dict(n=1, c=16, h=9, w=11, cout=24, kh=3, kw=3, stride=(2, 1), pad=(1, 0, 0, 1)), SEED + 10)
    grouped = planar_conv(dict(n=2, c=32, h=10, w=10, cout=48, kh=3, kw=3, pad=(1, 1, 1, 1), groups=2), SEED + 20)
    # 21 channels: the plan also stages a channel-padded copy of the transposed input, behind the two planar images
    ragged = planar_conv(dict(n=2, c=21, h=17, w=15, cout=21, kh=3, kw=3, pad=(1, 1, 1, 1)), SEED + 25)
    for case in (big, small, grouped, ragged, big, ragged):   # the second call is smaller and finds the first one's bytes in the scratch
        count = int(np.prod(case["shape"]))
        d_ref, d_got = eden.DeviceBuffer(nbytes=count), eden.DeviceBuffer(nbytes=count)
        case["plan"].run(case["d_x"], d_ref, case["q"])
        case["plan"].run_static(case["d_x"], d_got, case["q"])
        eden.sync()
        ref, got = d_ref.download(case["shape"]), d_got.download(case["shape"])
        assert np.array_equal(ref, case["want"]), diff_report(ref, case["want"])
        assert np.array_equal(got, ref), diff_report(got, ref)
        assert case["want"].std() > 10


def test_static_scratch_entry_point_on_a_stream_and_channels_last():
    """Ordered calls on one stream share the scratch safely; a channels-last plan needs no staging at all."""
    eden.init(0)
    a = planar_conv(dict(n=2, c=32, h=20, w=20, cout=64, kh=3, kw=3, pad=(1, 1, 1, 1)), SEED + 30)
    b = planar_conv(dict(n=1, c=24, h=14, w=14, cout=144, kh=1, kw=1), SEED + 40)
    stream = eden.Stream()
    outs = []
    for case in (a, b, a, b):
        d_o = eden.DeviceBuffer(nbytes=int(np.prod(case["shape"])))
        case["plan"].run_static(case["d_x"], d_o, case["q"], stream.h)
        outs.append((case, d_o))
    stream.sync()
    for case, d_o in outs:
        got = d_o.download(case["shape"])
        assert np.array_equal(got, case["want"]), diff_report(got, case["want"])
    # channels-last
    s = a["s"]
    x = synth.fill_u8((s.n, s.c, s.h, s.w), SEED + 30)
    desc = eden.conv_desc(s.n, s.c, s.h, s.w, s.cout, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 1, 1, eden.NHWC, eden.W_OIHW)
    d_x = eden.DeviceBuffer(host=np.ascontiguousarray(x.transpose(0, 2, 3, 1)))
    plan = eden.ConvPlan(desc, a["keep"][0], a["keep"][1], a["q"])
    d_o = eden.DeviceBuffer(nbytes=a["want"].size)
    plan.run_static(d_x, d_o, a["q"])
    eden.sync()
    got = d_o.download((s.n, a["shape"][2], a["shape"][3], s.cout)).transpose(0, 3, 1, 2)
    assert np.array_equal(got, a["want"])
    # channels-last with 21 channels: the channel-padded copy of the input is the one staging image, in the scratch too
    r = planar_conv(dict(n=2, c=21, h=13, w=12, cout=24, kh=3, kw=3, pad=(1, 1, 1, 1)), SEED + 50)
    s = r["s"]
    x = synth.fill_u8((s.n, s.c, s.h, s.w), SEED + 50)
    desc = eden.conv_desc(s.n, s.c, s.h, s.w, s.cout, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 1, 1, eden.NHWC, eden.W_OIHW)
    d_x = eden.DeviceBuffer(host=np.ascontiguousarray(x.transpose(0, 2, 3, 1)))
    plan = eden.ConvPlan(desc, r["keep"][0], r["keep"][1], r["q"])
    for _ in range(2):
        d_o = eden.DeviceBuffer(nbytes=r["want"].size)
        plan.run_static(d_x, d_o, r["q"])
        eden.sync()
        got = d_o.download((s.n, r["shape"][2], r["shape"][3], s.cout)).transpose(0, 3, 1, 2)
        assert np.array_equal(got, r["want"])


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    eden.init(0)
    # staging: 8*64*128*128 = 8 MiB in, 8*256*128*128 = 32 MiB out: more than the 32 MiB scratch
    desc = eden.conv_desc(8, 64, 128, 128, 256, 1, 1, layout=eden.NCHW)
    d_w, d_b = eden.DeviceBuffer(host=synth.fill_u8((256, 64, 1, 1), SEED + 50)), eden.DeviceBuffer(host=synth.fill_i32((256,), SEED + 51, -9, 9))
    q = eden.make_requant(0.02, 128, 0.005, 120, 0.05, 0)
    plan = eden.ConvPlan(desc, d_w, d_b, q)
    d_x, d_o = eden.DeviceBuffer(nbytes=8 * 64 * 128 * 128), eden.DeviceBuffer(nbytes=8 * 256 * 128 * 128)
    with pytest.raises(eden.EdenHipError, match="static scratch holds"):
        plan.run_static(d_x, d_o, q)
    plan.run(d_x, d_o, q)   # the allocating entry point still serves it
    eden.sync()
    # more groups than the entry point's fixed problem table
    desc = eden.conv_desc(1, 36, 6, 6, 36, 3, 3, pad=(1, 1, 1, 1), groups=9, layout=eden.NCHW)
    d_w2 = eden.DeviceBuffer(host=synth.fill_u8((36, 4, 3, 3), SEED + 52))
    d_b2 = eden.DeviceBuffer(host=synth.fill_i32((36,), SEED + 53, -9, 9))
    plan2 = eden.ConvPlan(desc, d_w2, d_b2, q)
    d_x2, d_o2 = eden.DeviceBuffer(nbytes=36 * 36), eden.DeviceBuffer(nbytes=36 * 36)
    with pytest.raises(eden.EdenHipError, match="at most 8"):
        plan2.run_static(d_x2, d_o2, q)
