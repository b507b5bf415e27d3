"""GPU parity: every operator, called through the C ABI, must reproduce the CPU
oracle bit for bit (uint8 outputs; integer work, so the tolerance is zero)."""
import json
import os

import numpy as np
import pytest

import oracle_lib as O
from harness import (diff_report, eden, gpu_conv, gpu_deconv, gpu_dwconv, gpu_fc, scattered_batch, synth, to_eh_requant)

pytestmark = pytest.mark.gpu

KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))
SEED = 0xEDE2


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    eden.init(0)
    print("device:", eden.device_name(), flush=True)


def quant(s_in=0.02, zp_in=128, s_w=0.005, zp_w=120, s_out=0.05, zp_out=0, act=O.ACT_NONE, en=False):
    q = O.make_quant(s_in, zp_in, s_w, zp_w, s_out, zp_out, act, en)
    assert eden.make_requant(s_in, zp_in, s_w, zp_w, s_out, zp_out, act, en).as_tuple() == q.as_tuple()
    return q


def centred_quant(acc, zp_in, zp_w, act_min=0, act_max=255):
    """Integer requant parameters that spread the given accumulators over the uint8 range
    (about 40 output steps per standard deviation, mean at 128), so that a parity case
    exercises rounding and both clamps instead of a saturated constant."""
    sd = float(acc.std()) or 1.0
    qm, sh = O.quantize_multiplier(40.0 / sd)
    zp_out = int(128 - round(float(acc.mean()) * 40.0 / sd))
    return O.raw_quant(zp_in=zp_in, zp_w=zp_w, zp_out=zp_out, multiplier=qm, shift=sh, act_min=act_min, act_max=act_max)


def conv_tensors(s, seed, w_normal=False):
    x = synth.fill_u8((s.n, s.c, s.h, s.w), seed)
    wshape = (s.cout, s.c // s.groups, s.kh, s.kw)
    w = synth.fill_u8_normal(wshape, seed + 1, 128, 20) if w_normal else synth.fill_u8(wshape, seed + 1)
    b = synth.fill_i32((s.cout,), seed + 2, -1000, 1000)
    return x, w, b


# ----------------------------------------------------------------- fully connected

FC_CASES = [
    # m, k, n, zp_a, zp_w
    (1, 64, 16, 3, 128),
    (7, 37, 11, 3, 128),       # byte-granular loads, ragged tiles
    (33, 100, 70, 250, 0),     # 4-byte loads, extreme zero points
    (64, 64, 64, 0, 255),
    (130, 256, 200, 128, 128),  # both shifted zero points vanish
    (256, 1024, 512, 77, 201),
    (300, 4096, 96, 3, 130),
    (5, 4100, 1000, 10, 20),   # classifier-like: k not a multiple of 64, n = 1000
    (1000, 24, 144, 128, 5),   # at most 64 reduction bytes: the fragment-direct kernel
    (129, 56, 17, 250, 128),
    # plain matrices whose reduction ends inside the last 256-byte slab (the dense path with the zero constant)
    (130, 272, 200, 77, 201),
    (64, 1296, 130, 3, 128),
    (200, 528, 64, 131, 120),
    # at most 64 rows and a reduction beyond 256 bytes: the kernel that is cut along the weights (one and two groups of
    # 32 rows, no row-sum term, a reduction that ends inside its last step, fewer steps than waves + 1, eight channels)
    (1, 4096, 1000, 3, 128),
    (1, 1280, 1000, 10, 20),
    (32, 272, 40, 77, 201),
    (33, 2048, 72, 131, 120),
    (64, 9216, 64, 0, 255),
    (17, 304, 8, 5, 100),
    # row lengths that are no multiple of 16 beyond the one-tap kernel's reach: the channel-padded copy of the input
    (1, 1001, 1001, 3, 128),
    (64, 1001, 77, 131, 120),
    (8, 300, 10, 200, 9),
    (300, 90, 40, 17, 250),
    (2, 70, 130, 255, 0),
    # more than 64 rows, few tiles, a long reduction: slices of the reduction on separate workgroups
    (100, 6400, 200, 77, 201),
    (70, 6200, 64, 3, 128),
    (129, 9216, 40, 131, 120),
    # a reduction whose k-table would not fit LDS: as a plain matrix of whole slabs (and sliced, each slice with its
    # part of the table); as a table-driven problem it cannot run on the tiled kernels (the last case: ragged length)
    (40, 25088, 72, 131, 120),
    (70, 25088, 130, 3, 128),
    (300, 25088, 64, 77, 201),
    (66, 25000, 40, 5, 100),
]


@pytest.mark.parametrize("exact_channels", [False, True], ids=["", "exact_channels"])
@pytest.mark.parametrize("m,k,n,zp_a,zp_w", FC_CASES)
def test_fc_matches_oracle(m, k, n, zp_a, zp_w, exact_channels):
    """exact_channels: the plan may not stage a padded copy of its input, which keeps the byte-gathering kernel covered"""
    if exact_channels and k % 16 == 0:
        pytest.skip("the flag changes nothing for whole 16-byte rows")
    print("fc", m, k, n, zp_a, zp_w, exact_channels, flush=True)
    a = synth.fill_u8((m, k), SEED + m)
    w = synth.fill_u8((n, k), SEED + k)
    b = synth.fill_i32((n,), SEED + n, -1000, 1000)
    _, acc = O.fc(a, w, b, O.raw_quant(zp_in=zp_a, zp_w=zp_w), want_acc=True)
    q = centred_quant(acc, zp_a, zp_w)
    want = O.fc(a, w, b, q)
    got = gpu_fc(a, w, b, to_eh_requant(q), flags=eden.EXACT_CHANNELS if exact_channels else 0)
    assert np.array_equal(got, want), diff_report(got, want)
    assert want.std() > 10  # the case exercises the requant range, not a saturated constant


# shapes chosen to land on each large-tile kernel configuration (by tile count), ragged in m and n, and with
# enough multiply-adds (over 1.5e9) that the one-tap latency kernel does not take them
BIG_FC_CASES = [
    (16384 - 37, 128, 1024 - 24, 9, 77),    # 256 x 256 tiles
    (65536 - 5, 256, 128 - 16, 200, 128),   # 256 x 128 tiles
    (16384 - 100, 384, 256, 128, 3),        # 128 x 128 tiles
    (32768 - 3, 896, 64 - 8, 17, 250),      # 128 x 64 tiles
    # more tiles than the device holds workgroups at once, with reductions shorter and longer than the stage count
    (20000 - 3, 128, 1024, 5, 140),         # 256 x 256, one slab per tile
    (80000 - 11, 384, 64, 128, 100),        # 128 x 64, three slabs
    (140000 - 1, 256, 128 - 8, 30, 128),    # 256 x 128, two slabs
    # the one-tap kernel with a long reduction loop and every channel-group width
    (3000, 96, 576, 77, 120),
    (3136 - 7, 256, 320, 0, 131),
    (520, 200, 24, 250, 5),
    (12544, 144, 40, 3, 128),
]


@pytest.mark.parametrize("m,k,n,zp_a,zp_w", BIG_FC_CASES)
def test_fc_large_tile_configurations(m, k, n, zp_a, zp_w):
    print("fc big", m, k, n, flush=True)
    a = synth.fill_u8((m, k), SEED + 7)
    w = synth.fill_u8((n, k), SEED + 8)
    b = synth.fill_i32((n,), SEED + 9, -1000, 1000)
    _, acc = O.fc(a[:512], w, b, O.raw_quant(zp_in=zp_a, zp_w=zp_w), want_acc=True)
    q = centred_quant(acc, zp_a, zp_w)
    want = O.fc(a, w, b, q)
    got = gpu_fc(a, w, b, to_eh_requant(q))
    assert np.array_equal(got, want), diff_report(got, want)
    assert want.std() > 10


def test_conv_batched_large_tiles():
    """3x3 convolution at batch 16 (50176 output pixels): the cooperative-tile kernels with padding taps."""
    s = O.conv_shape(16, 64, 56, 56, 64, 3, 3, pad=(1, 1, 1, 1))
    x, w, b = conv_tensors(s, SEED + 21)
    q = quant(0.02, 128, 0.005, 120, 0.05, 0, O.ACT_RELU, True)
    want = O.conv2d(x, w, b, s, q)
    got = gpu_conv(x, w, b, s, to_eh_requant(q), layout=eden.NHWC)
    assert np.array_equal(got, want), diff_report(got, want)
    s = O.conv_shape(4, 32, 56, 56, 192, 3, 3, stride=(1, 1), pad=(1, 1, 1, 1))
    x, w, b = conv_tensors(s, SEED + 22)
    _, acc = O.conv2d(x[:1], w, b, O.conv_shape(1, 32, 56, 56, 192, 3, 3, pad=(1, 1, 1, 1)), O.raw_quant(zp_in=131, zp_w=120), want_acc=True)
    q = centred_quant(acc, 131, 120)
    want = O.conv2d(x, w, b, s, q)
    got = gpu_conv(x, w, b, s, to_eh_requant(q), layout=eden.NHWC)
    assert np.array_equal(got, want), diff_report(got, want)


@pytest.mark.parametrize("cin,cout", [(16, 64), (32, 64), (64, 128)])
def test_conv_more_tiles_than_workgroups(cin, cout):
    """3x3 convolution at batch 24 (75264 output pixels): more tiles than the device holds workgroups at once, with
    the k-table path and reductions of 2, 3 and 5 slabs against 2 or 3 stages."""
    print("conv many tiles", cin, cout, flush=True)
    s = O.conv_shape(24, cin, 56, 56, cout, 3, 3, pad=(1, 1, 1, 1))
    x, w, b = conv_tensors(s, SEED + 23 + cin)
    _, acc = O.conv2d(x[:1], w, b, O.conv_shape(1, cin, 56, 56, cout, 3, 3, pad=(1, 1, 1, 1)), O.raw_quant(zp_in=131, zp_w=120), want_acc=True)
    q = centred_quant(acc, 131, 120)
    want = O.conv2d(x, w, b, s, q)
    got = gpu_conv(x, w, b, s, to_eh_requant(q), layout=eden.NHWC)
    assert np.array_equal(got, want), diff_report(got, want)
    assert want.std() > 10


def test_fc_config2_full_size():
    """M=256, K=4096, N=4096; uint8 activations zp 3; weights clip(N(128,20)) zp 128; scales 0.01/0.002/0.08."""
    m, k, n = 256, 4096, 4096
    print("fc config2", flush=True)
    a = synth.fill_u8((m, k), SEED + 16 * 2 + 0)
    w = synth.fill_u8_normal((n, k), SEED + 16 * 2 + 1, 128, 20)
    b = synth.fill_i32((n,), SEED + 16 * 2 + 2, -1000, 1000)
    q = quant(0.01, 3, 0.002, 128, 0.08, 0)
    assert (q.multiplier, q.shift) == (1099511680, -11)
    want, acc = O.fc(a, w, b, q, want_acc=True)
    got = gpu_fc(a, w, b, to_eh_requant(q))
    assert np.array_equal(got, want), diff_report(got, want)
    assert O.count_fastpath_overflow(acc, q) == 0
    assert len(np.unique(want)) > 20


@pytest.mark.parametrize("kat", KATS["fc"], ids=lambda k: k["name"])
def test_fc_reference_kat_on_gpu(kat):
    zp_a = 10
    a = (np.array(kat["input"]) + zp_a).astype(np.uint8).reshape(kat["m"], kat["k"])
    w = np.array(kat["weight"], np.uint8).reshape(kat["n"], kat["k"])
    q = O.raw_quant(zp_in=zp_a)
    got = gpu_fc(a, w, np.array(kat["bias"], np.int32), to_eh_requant(q))
    assert got.reshape(-1).tolist() == kat["expect"]


# ----------------------------------------------------------------- convolution

CONV_CASES = [
    # n, c, h, w, cout, kh, kw, kwargs
    dict(n=1, c=64, h=56, w=56, cout=64, kh=3, kw=3, pad=(1, 1, 1, 1)),                    # config 1 shape
    dict(n=2, c=3, h=17, w=19, cout=8, kh=3, kw=3, stride=(2, 2), pad=(0, 1, 0, 1)),       # 3 channels: byte loads
    dict(n=2, c=24, h=14, w=14, cout=144, kh=1, kw=1),                                       # pointwise expand, 4-byte loads
    dict(n=1, c=32, h=9, w=11, cout=20, kh=5, kw=3, pad=(2, 2, 1, 1), dil=(1, 2)),          # dilation, cout % 16 != 0
    dict(n=3, c=16, h=8, w=8, cout=24, kh=3, kw=3, stride=(1, 2), pad=(1, 1, 0, 2)),
    dict(n=1, c=32, h=10, w=10, cout=48, kh=3, kw=3, pad=(1, 1, 1, 1), groups=2),           # grouped
    dict(n=1, c=12, h=6, w=6, cout=12, kh=3, kw=3, pad=(1, 1, 1, 1), groups=3),             # grouped, 4-byte loads
    dict(n=1, c=16, h=3, w=3, cout=16, kh=3, kw=3, pad=(3, 3, 3, 3)),                       # windows wholly in the padding
    dict(n=4, c=128, h=7, w=7, cout=256, kh=1, kw=1),
    dict(n=1, c=160, h=7, w=7, cout=960, kh=1, kw=1),
    # one tap and at most 64 reduction bytes: the fragment-direct kernel
    dict(n=3, c=8, h=9, w=7, cout=20, kh=1, kw=1),                                          # half-filled fragments, ragged channels
    dict(n=2, c=40, h=13, w=13, cout=240, kh=1, kw=1, stride=(2, 2)),                       # two steps, strided rows
    dict(n=2, c=64, h=12, w=12, cout=32, kh=1, kw=1),
    dict(n=1, c=48, h=10, w=10, cout=96, kh=1, kw=1, groups=2),                             # 24-byte rows inside 48-byte pixels
    dict(n=2, c=240, h=14, w=14, cout=120, kh=1, kw=1, groups=6),                            # six groups: one launch of six problems
    dict(n=5, c=16, h=33, w=5, cout=96, kh=1, kw=1, stride=(1, 2)),
    # ... whose output leaves through the per-wave LDS image: one 16-byte chunk per pixel, the widest pixel (256 bytes),
    # a last pixel block of three pixels
    dict(n=1, c=32, h=5, w=7, cout=16, kh=1, kw=1),
    dict(n=2, c=32, h=9, w=9, cout=256, kh=1, kw=1),
    dict(n=1, c=64, h=7, w=5, cout=208, kh=1, kw=1),
    # one tap with bottom / right padding: output pixels whose only tap lies outside the image (they read the zero
    # point); the one-tap kernel must not be chosen
    dict(n=2, c=24, h=14, w=14, cout=144, kh=1, kw=1, pad=(0, 1, 0, 1)),
    dict(n=3, c=16, h=13, w=13, cout=32, kh=1, kw=1, stride=(2, 2), pad=(0, 2, 0, 2)),
    # three channels, 3x3: the first-layer kernel (unaligned 12-byte reads; byte path at the two ends of the tensor)
    dict(n=2, c=3, h=32, w=32, cout=32, kh=3, kw=3, stride=(2, 2), pad=(1, 1, 1, 1)),
    dict(n=1, c=3, h=9, w=10, cout=20, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=3, c=3, h=5, w=3, cout=16, kh=3, kw=3, pad=(2, 0, 0, 2)),
    dict(n=1, c=3, h=3, w=3, cout=5, kh=3, kw=3),
    # 32 channels and more: its matrix-core form (two channel blocks with a ragged second one, a single output pixel)
    dict(n=2, c=3, h=13, w=9, cout=40, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=3, c=3, h=21, w=23, cout=64, kh=3, kw=3, stride=(2, 2), pad=(0, 1, 0, 1)),
    dict(n=1, c=3, h=3, w=3, cout=72, kh=3, kw=3),
    # dilated taps through the direct-to-LDS tiles (16-byte channel units), alone and with stride and groups
    dict(n=2, c=64, h=20, w=20, cout=64, kh=3, kw=3, pad=(2, 2, 2, 2), dil=(2, 2)),
    dict(n=1, c=32, h=15, w=17, cout=32, kh=3, kw=3, stride=(2, 1), pad=(3, 3, 1, 1), dil=(3, 1), groups=2),
    dict(n=3, c=16, h=12, w=9, cout=40, kh=2, kw=3, stride=(1, 2), pad=(0, 2, 2, 0), dil=(2, 3)),
    # 3x3 at stride 1 over 32-byte channel steps: the patch-in-LDS kernel (ragged channel blocks, every padding,
    # widths that are not multiples of 32, tiles whose last rows fall off the image, one and two channel blocks)
    dict(n=2, c=32, h=20, w=17, cout=40, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=3, c=96, h=9, w=30, cout=72, kh=3, kw=3, pad=(0, 2, 2, 0)),
    dict(n=1, c=128, h=16, w=16, cout=100, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=5, c=64, h=33, w=12, cout=64, kh=3, kw=3),
    dict(n=2, c=64, h=14, w=70, cout=32, kh=3, kw=3, pad=(2, 2, 2, 2)),
    dict(n=9, c=64, h=56, w=56, cout=16, kh=3, kw=3, pad=(1, 1, 1, 1)),
    # ... and over channel counts of 16 (mod 32): the reduction ends in half a step of zero weights
    dict(n=2, c=16, h=23, w=40, cout=32, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=3, c=48, h=14, w=19, cout=80, kh=3, kw=3, pad=(1, 0, 2, 1)),
    dict(n=1, c=112, h=12, w=12, cout=40, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=6, c=16, h=64, w=64, cout=16, kh=3, kw=3),
    # one to four input channels, 3 - 11 kernel rows of at most 32 bytes: a kernel row per matrix-instruction step, read
    # straight from the image (channels-last; the NCHW runs of these cases keep the implicit-GEMM kernel's coverage of them)
    dict(n=2, c=3, h=37, w=41, cout=64, kh=7, kw=7, stride=(2, 2), pad=(3, 3, 3, 3)),       # an image network's 7x7 stride-2 stem
    dict(n=1, c=1, h=20, w=33, cout=56, kh=9, kw=9, pad=(4, 4, 4, 4)),                      # grey image, 9x9
    dict(n=2, c=4, h=18, w=18, cout=24, kh=5, kw=5, stride=(1, 2), pad=(2, 2, 2, 2)),       # 20-byte rows: both fragment halves
    dict(n=3, c=3, h=9, w=7, cout=16, kh=5, kw=5, pad=(4, 4, 4, 4)),                        # windows mostly in the padding, some wholly
    dict(n=1, c=2, h=12, w=40, cout=40, kh=3, kw=11, pad=(1, 1, 5, 5)),                     # two channels, wide kernel rows
    dict(n=1, c=3, h=30, w=30, cout=33, kh=11, kw=10, stride=(3, 3)),                       # 30-byte rows, eleven of them; 33 channels
    dict(n=2, c=1, h=64, w=64, cout=32, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=70, c=3, h=24, w=24, cout=96, kh=7, kw=7, stride=(2, 2), pad=(3, 3, 3, 3)),      # many workgroups, three channel blocks
    dict(n=1, c=3, h=10, w=10, cout=8, kh=4, kw=4),                                         # an even number of rows: not that kernel
    # 1x1 on at most 64 pixels with a long reduction: cut along the weights
    dict(n=8, c=1280, h=1, w=1, cout=100, kh=1, kw=1),
    dict(n=2, c=512, h=5, w=5, cout=48, kh=1, kw=1),
    # channels per group that are no multiple of 16 and fit no few-channel kernel: the channel-padded copy of the input
    # (NCHW: after the transposition); with EXACT_CHANNELS the byte-gathering kernel
    dict(n=2, c=21, h=17, w=15, cout=21, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=1, c=6, h=20, w=20, cout=16, kh=5, kw=5),
    dict(n=3, c=68, h=9, w=11, cout=68, kh=1, kw=1, pad=(0, 1, 0, 1)),
    dict(n=2, c=100, h=12, w=12, cout=100, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=1, c=42, h=14, w=9, cout=30, kh=3, kw=2, stride=(2, 1), pad=(1, 0, 1, 1), dil=(1, 2), groups=2),
    dict(n=2, c=30, h=8, w=8, cout=45, kh=1, kw=1, groups=3, stride=(2, 2)),
    dict(n=1, c=17, h=1, w=1, cout=9, kh=1, kw=1),
    # groups of fewer than 16 channels: neighbouring groups as block-diagonal problems over 16 .. 64 adjacent channels
    # (32 groups of 4 -> two bundles of 16; 8 of 8 -> one bundle; 6 groups of 8 -> three bundles of 2; 12 of 4 with a
    # stride and dilation; 1x1 with 4 channels per group and 3 outputs per group)
    dict(n=2, c=128, h=14, w=14, cout=128, kh=3, kw=3, pad=(1, 1, 1, 1), groups=32),
    dict(n=1, c=64, h=9, w=11, cout=96, kh=3, kw=3, pad=(1, 1, 1, 1), groups=8),
    dict(n=2, c=48, h=10, w=10, cout=24, kh=3, kw=3, pad=(1, 0, 0, 1), groups=6),
    dict(n=1, c=48, h=13, w=12, cout=48, kh=3, kw=2, stride=(2, 1), pad=(2, 2, 1, 1), dil=(2, 1), groups=12),
    dict(n=3, c=32, h=6, w=6, cout=24, kh=1, kw=1, groups=8),
    # a table-driven reduction too long for one k-table (7x7 over 512 channels: a fully connected layer written as a
    # convolution): sliced, each slice under its part of the table
    dict(n=2, c=512, h=7, w=7, cout=72, kh=7, kw=7),
    dict(n=1, c=512, h=9, w=8, cout=40, kh=7, kw=7, pad=(1, 0, 0, 1)),
    # few 64 x 64 tiles under a reduction of 24 slabs or more: two to four workgroups share each tile's reduction and
    # a second launch adds their sums up (45 slabs padded to 48 for four slices and 24 channels; 27 slabs and 28 tiles; a
    # stride and three slices; just below the bound: one workgroup per tile)
    dict(n=3, c=1280, h=5, w=5, cout=24, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=2, c=768, h=7, w=7, cout=400, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=1, c=1024, h=14, w=14, cout=200, kh=3, kw=2, stride=(2, 2), pad=(1, 1, 1, 0)),
    dict(n=2, c=512, h=7, w=7, cout=512, kh=3, kw=3, pad=(1, 1, 1, 1)),
]


@pytest.mark.parametrize("layout", [eden.NCHW, eden.NHWC, eden.NHWC | eden.EXACT_CHANNELS], ids=["nchw", "nhwc", "nhwc_exact_channels"])
@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_conv_matches_oracle(case, layout):
    if layout & eden.EXACT_CHANNELS and (case["c"] // case.get("groups", 1)) % 16 == 0:
        pytest.skip("the flag changes nothing for whole 16-byte channel groups")
    print("conv", case, layout, flush=True)
    s = O.conv_shape(**case)
    x, w, b = conv_tensors(s, SEED + s.c + s.cout)
    _, acc = O.conv2d(x, w, b, s, O.raw_quant(zp_in=131, zp_w=120), want_acc=True)
    q = centred_quant(acc, 131, 120, act_min=20, act_max=230)
    want = O.conv2d(x, w, b, s, q)
    got = gpu_conv(x, w, b, s, to_eh_requant(q), layout=layout)
    assert np.array_equal(got, want), diff_report(got, want)
    assert want.std() > 10


def test_conv_config1_exact_and_fastpath_census():
    """N=1, Cin=64, 56x56, Cout=64, 3x3 s1 p1; in zp128 s0.02; w zp120 s0.005; out zp0 s0.05; ReLU."""
    s = O.conv_shape(1, 64, 56, 56, 64, 3, 3, pad=(1, 1, 1, 1))
    x, w, b = conv_tensors(s, SEED + 16 * 1)
    q = quant(0.02, 128, 0.005, 120, 0.05, 0, O.ACT_RELU, True)
    assert (q.multiplier, q.shift) == (1099511562, -8)
    want, acc = O.conv2d(x, w, b, s, q, want_acc=True)
    got = gpu_conv(x, w, b, s, to_eh_requant(q), runs=2)
    assert np.array_equal(got, want), diff_report(got, want)
    # the reference routes this shape to its mul_hi/rhadd kernel; that rounding is the same function
    # unless acc << 2 overflows, which does not happen on these inputs
    assert O.count_fastpath_overflow(acc, q) == 0


@pytest.mark.parametrize("groups,cig,cog", [(1, 16, 32), (2, 16, 8), (8, 4, 4), (4, 5, 3)], ids=["ungrouped", "two_groups", "bundled_groups", "ragged_groups"])
def test_conv_ohwi_weights_equal_oihw(groups, cig, cog):
    """[Cout][kh][kw][Cin / groups] weights give what the same weights in [Cout][Cin / groups][kh][kw] give."""
    s = O.conv_shape(2, groups * cig, 9, 9, groups * cog, 3, 3, pad=(1, 1, 1, 1), groups=groups)
    x, w, b = conv_tensors(s, SEED + 5)
    q = quant(0.02, 100, 0.005, 90, 0.04, 10)
    want = O.conv2d(x, w, b, s, q)
    got = gpu_conv(x, w, b, s, to_eh_requant(q), layout=eden.NHWC, weight_layout=eden.W_OHWI)
    assert np.array_equal(got, want), diff_report(got, want)


@pytest.mark.parametrize("kat", KATS["conv"], ids=lambda k: k["name"])
def test_conv_reference_kat_on_gpu(kat):
    n, h, w, c = kat["in_dims"]
    cout, kh, kw, _ = kat["w_dims"]
    x = np.array(kat["input"], np.uint8).reshape(n, h, w, c).transpose(0, 3, 1, 2)
    wt = np.array(kat["weight"], np.uint8).reshape(cout, kh, kw, c).transpose(0, 3, 1, 2)
    t, b, l, r = kat["pad_tblr"]
    s = O.conv_shape(n, c, h, w, cout, kh, kw, stride=tuple(kat["stride"]), pad=(t, b, l, r))
    q = O.raw_quant()
    got = gpu_conv(np.ascontiguousarray(x), np.ascontiguousarray(wt), np.array(kat["bias"], np.int32), s, to_eh_requant(q))
    on, oh, ow, oc = kat["out_dims"]
    want = np.clip(np.array(kat["expect"]).reshape(on, oh, ow, oc).transpose(0, 3, 1, 2), 0, 255).astype(np.uint8)
    assert np.array_equal(got, want)


def test_requant_edge_multipliers_through_conv():
    """Left shifts (M >= 1), M == 0 and large right shifts through the fused epilogue."""
    s = O.conv_shape(1, 16, 6, 6, 16, 3, 3, pad=(1, 1, 1, 1))
    x, w, b = conv_tensors(s, SEED + 9)
    for m_real, zp_out in ((1.0, 128), (3.0, 128), (0.0, 9), (2.0 ** -20, 100), (0.74, 128), (1e-9, 50)):
        qm, sh = O.quantize_multiplier(m_real)
        q = O.raw_quant(zp_in=130, zp_w=127, zp_out=zp_out, multiplier=qm, shift=max(sh, -31))
        if sh < -31:
            q.multiplier, q.shift = 0, 0
        want = O.conv2d(x, w, b, s, q)
        got = gpu_conv(x, w, b, s, to_eh_requant(q), layout=eden.NHWC)
        assert np.array_equal(got, want), (m_real, diff_report(got, want))


def test_two_step_requant_in_every_kernel_family():
    """Multipliers above 1 and right shifts beyond 20 take the general two-step epilogue: the fragment-direct
    kernel, the direct-to-LDS tiles (whole tiles included), the register-staged kernel and depthwise."""
    for m_real, zp_out in ((1.5, 128), (2.0 ** -24, 77)):
        qm, sh = O.quantize_multiplier(m_real)
        for m, k, n in ((200, 32, 48), (512, 256, 256), (70, 100, 40)):
            a = (synth.fill_u8((m, k), SEED + 31 + m) % 5 + 126).astype(np.uint8)   # small accumulators: outputs spread at M = 1.5
            w = (synth.fill_u8((n, k), SEED + 32 + m) % 5 + 126).astype(np.uint8)
            b = synth.fill_i32((n,), SEED + 33, -20, 20)
            q = O.raw_quant(zp_in=128, zp_w=127, zp_out=zp_out, multiplier=qm, shift=sh)
            want = O.fc(a, w, b, q)
            got = gpu_fc(a, w, b, to_eh_requant(q))
            assert np.array_equal(got, want), (m_real, m, k, n, diff_report(got, want))
            if m_real > 1:
                assert want.std() > 5
        s = O.conv_shape(2, 16, 9, 9, 16, 3, 3, stride=(2, 2), pad=(1, 1, 1, 1), groups=16)
        x = (synth.fill_u8((s.n, s.c, s.h, s.w), SEED + 34) % 5 + 126).astype(np.uint8)
        w = (synth.fill_u8((s.c, 1, 3, 3), SEED + 35) % 5 + 126).astype(np.uint8)
        b = synth.fill_i32((s.c,), SEED + 36, -20, 20)
        q = O.raw_quant(zp_in=128, zp_w=127, zp_out=zp_out, multiplier=qm, shift=sh)
        want = O.dwconv2d(x, w, b, s, q)
        got = gpu_dwconv(x, w, b, s, to_eh_requant(q), layout=eden.NHWC)
        assert np.array_equal(got, want), (m_real, diff_report(got, want))


@pytest.mark.parametrize("rs", [1, 2, 5, 8, 9, 12, 16, 20])
def test_packed_single_shift_epilogue_every_kernel_family(rs):
    """The epilogues' four-at-a-time single-shift form (clamp before the shift, the byte written by the shift, the row
    term inside the rounding term) at small and large shifts, with and without the sign test, through the one-tap
    kernel, the patch-in-LDS 3x3 kernel, the tiled GEMM (whole tiles and its split reduction) and depthwise."""
    print("packed epilogue rs", rs, flush=True)
    for mult, zp_out, lo, hi in ((1 << 30, 0, 0, 255), ((1 << 31) - 1, 131, 0, 255), (1518500250, 17, 17, 200)):
        q = O.raw_quant(zp_in=131, zp_w=121, zp_out=zp_out, multiplier=mult, shift=-rs, act_min=lo, act_max=hi)
        amp = 1 if rs > 6 else 0   # small accumulators for the small shifts, so that the outputs are not all clamped
        def tensor(shape, seed, zp):
            t = synth.fill_u8(shape, seed)
            return t if amp else (t % (3 + rs) + zp - 1 - rs // 2).astype(np.uint8)
        for s in (O.conv_shape(2, 16, 9, 7, 48, 1, 1), O.conv_shape(1, 32, 12, 12, 32, 3, 3, pad=(1, 1, 1, 1))):
            x, w = tensor((s.n, s.c, s.h, s.w), SEED + rs, 131), tensor((s.cout, s.c, s.kh, s.kw), SEED + rs + 1, 121)
            b = synth.fill_i32((s.cout,), SEED + rs + 2, -300, 300)
            want = O.conv2d(x, w, b, s, q)
            got = gpu_conv(x, w, b, s, to_eh_requant(q), layout=eden.NHWC)
            assert np.array_equal(got, want), (rs, mult, s, diff_report(got, want))
        for m, k, n in ((70, 256, 40), (512, 256, 256)):
            a, w = tensor((m, k), SEED + rs + 3, 131), tensor((n, k), SEED + rs + 4, 121)
            b = synth.fill_i32((n,), SEED + rs + 5, -300, 300)
            want = O.fc(a, w, b, q)
            got = gpu_fc(a, w, b, to_eh_requant(q))
            assert np.array_equal(got, want), (rs, mult, m, k, n, diff_report(got, want))
        s = O.conv_shape(2, 16, 9, 9, 16, 3, 3, stride=(2, 2), pad=(1, 1, 1, 1), groups=16)
        x, w = tensor((s.n, s.c, s.h, s.w), SEED + rs + 6, 131), tensor((s.c, 1, 3, 3), SEED + rs + 7, 121)
        b = synth.fill_i32((s.c,), SEED + rs + 8, -300, 300)
        want = O.dwconv2d(x, w, b, s, q)
        got = gpu_dwconv(x, w, b, s, to_eh_requant(q), layout=eden.NHWC)
        assert np.array_equal(got, want), (rs, mult, "dw", diff_report(got, want))
        if rs in (1, 8):
            assert len(np.unique(want)) > 8


def test_negative_half_ties_round_like_the_oracle():
    """Accumulators chosen so that acc * M lands exactly on .5 for both signs and both rounding stages."""
    k, n = 16, 16
    a = np.zeros((64, k), np.uint8)
    a[:, 0] = np.arange(64)              # a - zp_a = -32 .. 31 with zp 32
    w = np.zeros((n, k), np.uint8)
    w[:, 0] = 1
    bias = np.zeros(n, np.int32)
    for m_real in (0.5, 0.25, 0.125, 0.375):
        qm, sh = O.quantize_multiplier(m_real)
        q = O.raw_quant(zp_in=32, zp_w=0, zp_out=128, multiplier=qm, shift=sh)
        want = O.fc(a, w, bias, q)
        got = gpu_fc(a, w, bias, to_eh_requant(q))
        assert np.array_equal(got, want), (m_real, diff_report(got, want))


def test_plan_refolds_when_zero_points_change_and_repacks_new_weights():
    s = O.conv_shape(1, 16, 8, 8, 16, 3, 3, pad=(1, 1, 1, 1))
    x, w, b = conv_tensors(s, SEED + 11)
    desc = eden.conv_desc(1, 16, 8, 8, 16, 3, 3, pad=(1, 1, 1, 1), layout=eden.NCHW)
    d_x, d_w, d_b = eden.DeviceBuffer(host=x), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    d_o = eden.DeviceBuffer(nbytes=16 * 64)
    q1 = quant(0.02, 128, 0.005, 120, 0.05, 0)
    plan = eden.ConvPlan(desc, d_w, d_b, to_eh_requant(q1))
    plan.run(d_x, d_o, to_eh_requant(q1))
    assert np.array_equal(d_o.download((1, 16, 8, 8)), O.conv2d(x, w, b, s, q1))
    q2 = quant(0.02, 7, 0.005, 201, 0.05, 30)  # tensors re-quantized: zero points read at execute time
    plan.run(d_x, d_o, to_eh_requant(q2))
    assert np.array_equal(d_o.download((1, 16, 8, 8)), O.conv2d(x, w, b, s, q2))
    w2 = synth.fill_u8(w.shape, SEED + 99)
    b2 = synth.fill_i32(b.shape, SEED + 98, -50, 50)
    d_w2, d_b2 = eden.DeviceBuffer(host=w2), eden.DeviceBuffer(host=b2)
    plan.repack(d_w2, d_b2, to_eh_requant(q2))  # weights as a run-time input
    plan.run(d_x, d_o, to_eh_requant(q2))
    assert np.array_equal(d_o.download((1, 16, 8, 8)), O.conv2d(x, w2, b2, s, q2))
    plan.destroy()


def test_conv3x3_batch_64_equals_oracle_on_scattered_distinct_images():
    """The benchmark's 3x3 convolution at its batch of 64 (the batch decides the tile height of the patch kernel), on
    eight distinct images scattered over the batch positions without a period: every position must equal the
    oracle's result for the image that sits there."""
    s8 = O.conv_shape(8, 64, 56, 56, 64, 3, 3, pad=(1, 1, 1, 1))
    x, w, b = conv_tensors(s8, SEED + 16)
    q = quant(0.02, 128, 0.005, 120, 0.05, 0, O.ACT_RELU, True)
    want = O.conv2d(x, w, b, s8, q)
    where = scattered_batch(64, 8)
    s64 = O.conv_shape(64, 64, 56, 56, 64, 3, 3, pad=(1, 1, 1, 1))
    got = gpu_conv(x[where], w, b, s64, to_eh_requant(q), layout=eden.NHWC)
    for img in range(64):
        assert np.array_equal(got[img], want[where[img]]), (img, int(where[img]), diff_report(got[img], want[where[img]]))
    assert want.std() > 10
    assert not np.array_equal(want[0], want[1])


# ----------------------------------------------------------------- depthwise

DW_CASES = [
    dict(n=2, c=144, h=56, w=56, cout=144, kh=3, kw=3, stride=(2, 2), pad=(1, 1, 1, 1)),   # config 3 geometry, 2 images
    dict(n=1, c=32, h=12, w=12, cout=32, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=1, c=8, h=9, w=7, cout=16, kh=3, kw=3, pad=(1, 1, 1, 1), dm=2),                  # depth multiplier
    dict(n=2, c=5, h=10, w=10, cout=5, kh=5, kw=5, pad=(2, 2, 2, 2), dil=(1, 1)),           # odd channel count
    dict(n=1, c=16, h=11, w=13, cout=16, kh=3, kw=3, stride=(1, 1), pad=(2, 2, 2, 2), dil=(2, 2)),
    dict(n=1, c=4, h=5, w=5, cout=4, kh=2, kw=2),
    # 3x3 tiles of four output pixels: widths that are not multiples of four, every border, both strides
    dict(n=2, c=16, h=7, w=7, cout=16, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=1, c=24, h=14, w=13, cout=24, kh=3, kw=3, stride=(2, 2), pad=(1, 1, 1, 1)),
    dict(n=1, c=8, h=6, w=9, cout=8, kh=3, kw=3, stride=(2, 2), pad=(0, 1, 0, 1)),
    dict(n=1, c=8, h=5, w=6, cout=8, kh=3, kw=3, pad=(2, 2, 2, 2)),
    dict(n=3, c=960, h=7, w=7, cout=960, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=1, c=12, h=3, w=1, cout=12, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=1, c=6, h=12, w=10, cout=12, kh=3, kw=2, stride=(2, 1), pad=(2, 2, 1, 1), dil=(2, 3), dm=2),   # dilation, stride and depth multiplier
    dict(n=2, c=32, h=16, w=16, cout=32, kh=3, kw=3, stride=(2, 2), pad=(2, 2, 2, 2), dil=(2, 2)),
    # 5x5 and 7x7 tiles of four output pixels (two words per kernel column): both strides, ragged widths, every border,
    # an image smaller than the kernel
    dict(n=2, c=16, h=13, w=11, cout=16, kh=5, kw=5, pad=(2, 2, 2, 2)),
    dict(n=1, c=24, h=14, w=14, cout=24, kh=5, kw=5, stride=(2, 2), pad=(2, 2, 2, 2)),
    dict(n=2, c=8, h=15, w=17, cout=8, kh=7, kw=7, pad=(3, 3, 3, 3)),
    dict(n=1, c=32, h=20, w=18, cout=32, kh=7, kw=7, stride=(2, 2), pad=(3, 2, 3, 2)),
    dict(n=1, c=12, h=4, w=3, cout=12, kh=5, kw=5, pad=(2, 2, 2, 2)),
    dict(n=3, c=144, h=28, w=28, cout=144, kh=5, kw=5, pad=(2, 2, 2, 2)),
    dict(n=1, c=4, h=9, w=9, cout=4, kh=7, kw=7),
    # dilated 3x3 tiles at stride 1: the column-sharing tiles of dilations 2 and 4, the three-group tile of any other
    # dilation; ragged widths, every border, windows wider than the image, uneven padding
    dict(n=2, c=24, h=19, w=21, cout=24, kh=3, kw=3, pad=(2, 2, 2, 2), dil=(2, 2)),
    dict(n=1, c=8, h=17, w=18, cout=8, kh=3, kw=3, pad=(4, 4, 4, 4), dil=(4, 4)),
    dict(n=2, c=16, h=15, w=14, cout=16, kh=3, kw=3, pad=(3, 3, 3, 3), dil=(3, 3)),
    dict(n=1, c=32, h=33, w=33, cout=32, kh=3, kw=3, pad=(6, 6, 6, 6), dil=(6, 6)),
    dict(n=1, c=8, h=5, w=6, cout=8, kh=3, kw=3, pad=(4, 4, 4, 4), dil=(4, 4)),
    dict(n=1, c=12, h=9, w=30, cout=12, kh=3, kw=3, pad=(0, 3, 1, 0), dil=(2, 2)),
    dict(n=1, c=4, h=40, w=41, cout=4, kh=3, kw=3, pad=(12, 12, 12, 12), dil=(12, 12)),
    dict(n=3, c=384, h=33, w=33, cout=384, kh=3, kw=3, pad=(2, 2, 2, 2), dil=(2, 2)),
    # depth multipliers on a copy of the input with every channel repeated (channels-last, outputs a multiple of 4)
    dict(n=2, c=16, h=14, w=13, cout=32, kh=3, kw=3, pad=(1, 1, 1, 1), dm=2),
    dict(n=1, c=3, h=21, w=20, cout=24, kh=3, kw=3, stride=(2, 2), pad=(0, 1, 0, 1), dm=8),
    dict(n=2, c=5, h=9, w=9, cout=20, kh=5, kw=5, pad=(2, 2, 2, 2), dm=4),
    dict(n=1, c=6, h=8, w=8, cout=18, kh=3, kw=3, pad=(1, 1, 1, 1), dm=3),                  # 18 outputs: rounded up to 20 as well
    # channel counts that are no multiple of 4 (channels-last): computed on the count rounded up, the caller's channels copied out
    dict(n=2, c=30, h=15, w=14, cout=30, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=1, c=146, h=20, w=20, cout=146, kh=3, kw=3, stride=(2, 2), pad=(0, 1, 0, 1)),
    dict(n=2, c=7, h=9, w=9, cout=7, kh=5, kw=5, pad=(2, 2, 2, 2)),
    dict(n=1, c=1, h=12, w=13, cout=1, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=1, c=3, h=10, w=10, cout=15, kh=3, kw=3, pad=(1, 1, 1, 1), dm=5),
]


@pytest.mark.parametrize("layout", [eden.NCHW, eden.NHWC, eden.NCHW | eden.EXACT_CHANNELS, eden.NHWC | eden.EXACT_CHANNELS],
                         ids=["nchw", "nhwc", "nchw_unstaged", "nhwc_unstaged"])
@pytest.mark.parametrize("case", DW_CASES, ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_depthwise_matches_oracle(case, layout):
    """Planar tensors run between two transpositions and depth multipliers on a channel-replicated copy of the input;
    EXACT_CHANNELS keeps both on the one-output-per-thread kernels (the `unstaged` runs, where that differs)."""
    if layout == (eden.NCHW | eden.EXACT_CHANNELS) and case["cout"] % 4 != 0:
        pytest.skip("no staging either way")
    if layout == (eden.NHWC | eden.EXACT_CHANNELS) and case.get("dm", 1) == 1 and case["cout"] % 4 == 0:
        pytest.skip("no staging either way")
    if layout == (eden.NCHW | eden.EXACT_CHANNELS) and case.get("dm", 1) != 1:
        pytest.skip("no staging either way")
    print("dw", case, layout, flush=True)
    s = O.conv_shape(**case)
    x = synth.fill_u8((s.n, s.c, s.h, s.w), SEED + 40)
    w = synth.fill_u8((s.cout, 1, s.kh, s.kw), SEED + 41)
    b = synth.fill_i32((s.cout,), SEED + 42, -1000, 1000)
    _, acc = O.dwconv2d(x, w, b, s, O.raw_quant(zp_in=37, zp_w=201), want_acc=True)
    q = centred_quant(acc, 37, 201, act_min=10, act_max=240)
    want = O.dwconv2d(x, w, b, s, q)
    got = gpu_dwconv(x, w, b, s, to_eh_requant(q), layout=layout)
    assert np.array_equal(got, want), diff_report(got, want)
    assert want.std() > 10


DW_INT8_RANGE_CASES = [c for c in DW_CASES if c["kh"] == 3 and c["kw"] == 3 and c.get("dm", 1) == 1] + [
    # large stride-1 layers whose rows are whole eight-pixel tiles: eight outputs per thread
    dict(n=44, c=32, h=112, w=112, cout=32, kh=3, kw=3, pad=(1, 1, 1, 1)),
    dict(n=70, c=16, h=37, w=112, cout=16, kh=3, kw=3, pad=(0, 1, 2, 0)),
]


@pytest.mark.parametrize("case", DW_INT8_RANGE_CASES, ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_depthwise_3x3_weights_within_int8_of_their_zero_point(case):
    """Channels-last 3x3 plans whose w - zp_w all fit int8 run the 8-bit dot product kernel; a zero point that
    pushes one weight out of that range at run time sends the same plan back to the 16-bit form, and back again."""
    print("dw int8 range", case, flush=True)
    s = O.conv_shape(**case)
    zp_w = 140
    x = synth.fill_u8((s.n, s.c, s.h, s.w), SEED + 43)
    w = (12 + synth.fill_u8((s.cout, 1, 3, 3), SEED + 44).astype(np.int32) % 244).astype(np.uint8)   # 12 .. 255
    w.reshape(-1)[0], w.reshape(-1)[1] = 12, 255                                                       # zp_w - 128 and the top
    b = synth.fill_i32((s.cout,), SEED + 45, -1000, 1000)
    quants = []
    for z in (zp_w, zp_w + 1, zp_w):   # 12 - 141 = -129 does not fit
        _, acc = O.dwconv2d(x, w, b, s, O.raw_quant(zp_in=37, zp_w=z), want_acc=True)
        quants.append(centred_quant(acc, 37, z, act_min=5, act_max=250))
    ho, wo = O.conv_out_hw(s)
    desc = eden.conv_desc(s.n, s.c, s.h, s.w, s.cout, 3, 3, (s.stride_h, s.stride_w), (s.pad_t, s.pad_b, s.pad_l, s.pad_r), (s.dil_h, s.dil_w), 1, 1,
                          eden.NHWC, eden.W_OIHW)
    d_x = eden.DeviceBuffer(host=np.ascontiguousarray(x.transpose(0, 2, 3, 1)))
    d_w, d_b, d_o = eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b), eden.DeviceBuffer(nbytes=s.n * s.cout * ho * wo)
    plan = eden.DwConvPlan(desc, d_w, d_b, to_eh_requant(quants[0]))
    for q in quants:
        plan.run(d_x, d_o, to_eh_requant(q))
        got = d_o.download((s.n, ho, wo, s.cout)).transpose(0, 3, 1, 2)
        want = O.dwconv2d(x, w, b, s, q)
        assert np.array_equal(got, want), diff_report(got, want)
        assert want.std() > 10
    plan.destroy()


@pytest.mark.parametrize("kat", KATS["depthwise"], ids=lambda k: k["name"])
def test_depthwise_reference_kat_on_gpu(kat):
    n, c, h, w = kat["in_dims"]
    cout, _, kh, kw = kat["w_dims"]
    zp_w, zp_out = 16, 40
    x = np.array(kat["input"], np.uint8).reshape(n, c, h, w)
    wt = (np.array(kat["weight"]) + zp_w).astype(np.uint8).reshape(cout, 1, kh, kw)
    s = O.conv_shape(n, c, h, w, cout, kh, kw, stride=tuple(kat["stride"]), dm=kat["dm"])
    q = O.raw_quant(zp_w=zp_w, zp_out=zp_out)
    for layout in (eden.NCHW, eden.NHWC):
        got = gpu_dwconv(x, wt, np.array(kat["bias"], np.int32), s, to_eh_requant(q), layout=layout)
        assert got.reshape(-1).tolist() == [e + zp_out for e in kat["expect"]]


@pytest.mark.parametrize("n", [4, 32], ids=["n4", "n32_full_size"])
def test_mobilenet_block_config3(n):
    """Pointwise 24->144 (ReLU6) then depthwise 3x3 s2 p1 (ReLU6), channels-last, zero points drawn from the seed;
    n = 32 is the benchmark's own size (the batch decides tile shapes and the depthwise tile width)."""
    print("config 3 block, n =", n, flush=True)
    zps = synth.fill_u8((6,), SEED + 16 * 3 + 9).tolist()
    x = synth.fill_u8((n, 24, 56, 56), SEED + 16 * 3)
    w1 = synth.fill_u8((144, 24, 1, 1), SEED + 16 * 3 + 1)
    b1 = synth.fill_i32((144,), SEED + 16 * 3 + 2, -1000, 1000)
    w2 = synth.fill_u8((144, 1, 3, 3), SEED + 16 * 3 + 3)
    b2 = synth.fill_i32((144,), SEED + 16 * 3 + 4, -1000, 1000)
    q1 = quant(0.02, zps[0], 0.004, zps[1], 0.03, zps[2] // 4, O.ACT_RELU6, True)
    q2 = quant(0.03, zps[2] // 4, 0.006, zps[3], 0.025, zps[4] // 4, O.ACT_RELU6, True)
    s1 = O.conv_shape(n, 24, 56, 56, 144, 1, 1)
    s2 = O.conv_shape(n, 144, 56, 56, 144, 3, 3, stride=(2, 2), pad=(1, 1, 1, 1))
    mid = O.conv2d(x, w1, b1, s1, q1)
    want = O.dwconv2d(mid, w2, b2, s2, q2)
    got_mid = gpu_conv(x, w1, b1, s1, to_eh_requant(q1), layout=eden.NHWC)
    assert np.array_equal(got_mid, mid), diff_report(got_mid, mid)
    got = gpu_dwconv(got_mid, w2, b2, s2, to_eh_requant(q2), layout=eden.NHWC)
    assert np.array_equal(got, want), diff_report(got, want)
    assert want.std() > 1 and mid.std() > 1


# ----------------------------------------------------------------- deconvolution

DECONV_CASES = [
    dict(n=2, c=16, h=5, w=7, cout=8, kh=4, kw=4, stride=(2, 2), pad=(1, 1, 1, 1)),
    dict(n=1, c=6, h=4, w=4, cout=4, kh=3, kw=3, stride=(3, 3), pad=(1, 1, 1, 1), groups=2),
    dict(n=1, c=3, h=5, w=4, cout=2, kh=2, kw=3, stride=(1, 2), pad=(0, 1, 1, 0)),
    dict(n=1, c=32, h=6, w=6, cout=40, kh=3, kw=3, stride=(2, 2), pad=(0, 0, 0, 0)),       # kernel not a multiple of stride
    dict(n=1, c=16, h=4, w=4, cout=16, kh=2, kw=2, stride=(3, 3), pad=(0, 0, 0, 0)),       # phases without any tap
    dict(n=1, c=8, h=3, w=3, cout=8, kh=3, kw=3, stride=(1, 1), pad=(1, 1, 1, 1)),
    # kernel <= stride (every phase is one tap) with a negative tail padding: phases larger than the input
    dict(n=2, c=16, h=6, w=6, cout=32, kh=2, kw=2, stride=(2, 2), pad=(0, -2, 0, -2)),
    dict(n=2, c=16, h=6, w=6, cout=32, kh=2, kw=2, stride=(2, 2), pad=(0, 0, 0, 0)),
    # nine one-tap phases of equal shape: launches of eight problems and of one problem of the one-tap kernel
    dict(n=2, c=32, h=9, w=7, cout=48, kh=3, kw=3, stride=(3, 3), pad=(0, 0, 0, 0)),
    dict(n=3, c=64, h=20, w=20, cout=32, kh=2, kw=2, stride=(2, 2), pad=(0, 0, 0, 0)),
    # channels per group that are no multiple of 16, several taps per phase: the channel-padded copy of the input
    # (an upsampling layer over 21 class scores, kernel twice the stride; groups; a kernel that is no multiple of the stride)
    dict(n=2, c=21, h=9, w=8, cout=21, kh=4, kw=4, stride=(2, 2), pad=(1, 1, 1, 1)),
    dict(n=1, c=21, h=5, w=6, cout=21, kh=16, kw=16, stride=(8, 8), pad=(4, 4, 4, 4)),
    dict(n=1, c=40, h=7, w=7, cout=12, kh=3, kw=3, stride=(2, 2), pad=(1, 0, 1, 0), groups=2),
    dict(n=2, c=5, h=6, w=6, cout=7, kh=5, kw=5, stride=(2, 2), pad=(2, 2, 2, 2)),
    # output columns whose phases read the same input columns leave as one problem (kernel a multiple of the stride,
    # several taps): three kernel columns in one, two classes of two, a ragged last column group (kept apart), a padding
    # beyond the stride, a kernel three times the stride
    dict(n=2, c=16, h=7, w=6, cout=24, kh=6, kw=6, stride=(3, 3), pad=(0, 0, 0, 0)),
    dict(n=1, c=32, h=9, w=9, cout=20, kh=8, kw=8, stride=(4, 4), pad=(2, 2, 2, 2)),
    dict(n=2, c=16, h=6, w=7, cout=16, kh=6, kw=6, stride=(3, 3), pad=(1, 2, 1, 3)),
    dict(n=1, c=16, h=5, w=8, cout=40, kh=4, kw=8, stride=(2, 4), pad=(1, 1, 5, 5)),
    dict(n=1, c=16, h=6, w=6, cout=8, kh=3, kw=9, stride=(1, 3), pad=(1, 1, 3, 3)),
    dict(n=3, c=48, h=12, w=12, cout=21, kh=16, kw=16, stride=(8, 8), pad=(4, 4, 4, 4)),
    # kernels that are no multiple of the stride over even output extents: phases of 4, 2, 2 and 1 taps (5x5: 9, 6, 6, 4)
    # padded to one length and launched together; 21 channels on their padded copy; odd extents keep a launch per phase
    dict(n=2, c=32, h=6, w=7, cout=24, kh=3, kw=3, stride=(2, 2), pad=(1, 0, 1, 0)),
    dict(n=1, c=64, h=9, w=8, cout=72, kh=5, kw=5, stride=(2, 2), pad=(2, 1, 2, 1)),
    dict(n=2, c=21, h=8, w=8, cout=21, kh=3, kw=3, stride=(2, 2), pad=(1, 0, 1, 0)),
    dict(n=1, c=16, h=7, w=7, cout=16, kh=3, kw=3, stride=(2, 2), pad=(1, 1, 1, 1)),
    dict(n=8, c=256, h=16, w=16, cout=256, kh=3, kw=3, stride=(2, 2), pad=(1, 0, 1, 0)),
]


@pytest.mark.parametrize("layout", [eden.NCHW, eden.NHWC, eden.NHWC | eden.EXACT_CHANNELS], ids=["nchw", "nhwc", "nhwc_exact_channels"])
@pytest.mark.parametrize("case", DECONV_CASES, ids=lambda c: "x".join(str(v) for v in list(c.values())[:7]))
def test_deconv_matches_oracle(case, layout):
    if layout & eden.EXACT_CHANNELS and (case["c"] // case.get("groups", 1)) % 16 == 0:
        pytest.skip("the flag changes nothing for whole 16-byte channel groups")
    print("deconv", case, layout, flush=True)
    s = O.conv_shape(**case)
    x = synth.fill_u8((s.n, s.c, s.h, s.w), SEED + 60)
    w = synth.fill_u8((s.c, s.cout // s.groups, s.kh, s.kw), SEED + 61)
    b = synth.fill_i32((s.cout,), SEED + 62, -1000, 1000)
    _, acc = O.deconv2d(x, w, b, s, O.raw_quant(zp_in=131, zp_w=77), want_acc=True)
    q = centred_quant(acc, 131, 77)
    want = O.deconv2d(x, w, b, s, q)
    got = gpu_deconv(x, w, b, s, to_eh_requant(q), layout=layout)
    assert np.array_equal(got, want), diff_report(got, want)
    assert want.std() > 10


def test_channel_padded_plan_follows_the_input_zero_point():
    """The padding bytes of the staged copy hold the input zero point of the run that reads them: one plan, run with
    two zero points, int8 tensors included."""
    s = O.conv_shape(2, 21, 11, 9, 24, 3, 3, pad=(1, 1, 1, 1))
    x, w, b = conv_tensors(s, SEED + 777)
    ho, wo = O.conv_out_hw(s)
    desc = eden.conv_desc(s.n, s.c, s.h, s.w, s.cout, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 1, 1, eden.NHWC, eden.W_OIHW)
    assert eden.conv_kernels(desc) != ["staged"]
    d_x = eden.DeviceBuffer(host=np.ascontiguousarray(x.transpose(0, 2, 3, 1)))
    d_w, d_b, d_o = eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b), eden.DeviceBuffer(nbytes=s.n * s.cout * ho * wo)
    quants = []
    for zp_in in (131, 7, 255):
        _, acc = O.conv2d(x, w, b, s, O.raw_quant(zp_in=zp_in, zp_w=120), want_acc=True)
        quants.append(centred_quant(acc, zp_in, 120))
    plan = eden.ConvPlan(desc, d_w, d_b, to_eh_requant(quants[0]))
    for q in quants:
        plan.run(d_x, d_o, to_eh_requant(q))
        got = d_o.download((s.n, ho, wo, s.cout)).transpose(0, 3, 1, 2)
        want = O.conv2d(x, w, b, s, q)
        assert np.array_equal(got, want), diff_report(got, want)
    plan.destroy()


def test_bundled_groups_follow_the_weight_zero_point():
    """Groups bundled into block-diagonal problems hold the weight zero point off their blocks: one plan, run with
    three weight zero points (packed again each time), and once more after its weights were replaced."""
    s = O.conv_shape(2, 64, 12, 10, 64, 3, 3, pad=(1, 1, 1, 1), groups=16)
    x, w, b = conv_tensors(s, SEED + 888)
    ho, wo = O.conv_out_hw(s)
    desc = eden.conv_desc(s.n, s.c, s.h, s.w, s.cout, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 16, 1, eden.NHWC, eden.W_OIHW)
    assert len(eden.conv_kernels(desc)) == 1   # sixteen groups, one problem
    d_x = eden.DeviceBuffer(host=np.ascontiguousarray(x.transpose(0, 2, 3, 1)))
    d_w, d_b, d_o = eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b), eden.DeviceBuffer(nbytes=s.n * s.cout * ho * wo)

    def q_for(weights, zp_w):
        _, acc = O.conv2d(x, weights, b, s, O.raw_quant(zp_in=131, zp_w=zp_w), want_acc=True)
        return centred_quant(acc, 131, zp_w)
    plan = eden.ConvPlan(desc, d_w, d_b, to_eh_requant(q_for(w, 120)))
    for zp_w in (120, 7, 255, 120):
        q = q_for(w, zp_w)
        plan.run(d_x, d_o, to_eh_requant(q))
        got = d_o.download((s.n, ho, wo, s.cout)).transpose(0, 3, 1, 2)
        want = O.conv2d(x, w, b, s, q)
        assert np.array_equal(got, want), (zp_w, diff_report(got, want))
        assert want.std() > 10
    w2 = synth.fill_u8(w.shape, SEED + 889)
    d_w2 = eden.DeviceBuffer(host=w2)
    q = q_for(w2, 33)
    plan.repack(d_w2, d_b, to_eh_requant(q))
    plan.run(d_x, d_o, to_eh_requant(q))
    got = d_o.download((s.n, ho, wo, s.cout)).transpose(0, 3, 1, 2)
    assert np.array_equal(got, O.conv2d(x, w2, b, s, q))
    plan.destroy()


@pytest.mark.parametrize("k,stride,pad", [(4, 2, 1), (8, 4, 2), (6, 3, 0)], ids=["k4s2", "k8s4_merged_columns", "k6s3_merged_columns"])
def test_deconv_ohwi_weights(k, stride, pad):
    s = O.conv_shape(1, 16, 5, 5, 12, k, k, stride=(stride, stride), pad=(pad,) * 4)
    x = synth.fill_u8((1, 16, 5, 5), SEED + 63)
    w = synth.fill_u8((16, 12, k, k), SEED + 64)
    b = synth.fill_i32((12,), SEED + 65, -100, 100)
    q = quant(0.03, 131, 0.01, 77, 0.3, 5)
    want = O.deconv2d(x, w, b, s, q)
    got = gpu_deconv(x, w, b, s, to_eh_requant(q), layout=eden.NHWC, weight_layout=eden.W_OHWI)
    assert np.array_equal(got, want), diff_report(got, want)
    assert want.std() > 10


def test_deconv_config4_full_size():
    """N=8, Cin=256, 32x32 -> Cout=128, 4x4 s2 p1 -> 64x64."""
    s = O.conv_shape(8, 256, 32, 32, 128, 4, 4, stride=(2, 2), pad=(1, 1, 1, 1))
    x = synth.fill_u8((8, 256, 32, 32), SEED + 16 * 4)
    w = synth.fill_u8((256, 128, 4, 4), SEED + 16 * 4 + 1)
    b = synth.fill_i32((128,), SEED + 16 * 4 + 2, -1000, 1000)
    q = quant(0.02, 121, 0.005, 133, 0.35, 128)
    assert q.shift < 0
    want = O.deconv2d(x, w, b, s, q)
    got = gpu_deconv(x, w, b, s, to_eh_requant(q))
    assert np.array_equal(got, want), diff_report(got, want)
    assert want.std() > 5


# ----------------------------------------------------------------- layout

@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (2, 3, 5, 7), (1, 64, 56, 56), (3, 24, 17, 9), (2, 144, 28, 28),
                                   (1, 1000, 1, 1), (2, 130, 1, 67),
                                   # extents in 16-byte units on both axes: the three 16 KiB tile shapes, whole and ragged tiles
                                   (2, 96, 16, 24), (3, 32, 20, 20), (2, 16, 8, 10), (1, 144, 28, 28), (2, 48, 4, 4),
                                   (1, 256, 32, 16), (2, 32, 33, 32), (1, 1280, 4, 4),
                                   # multiples of 4 only: rows finished with single dwords, 16-row groups with single row quads
                                   (2, 24, 14, 14), (1, 1000, 2, 2), (2, 40, 6, 6), (1, 36, 5, 4), (3, 20, 2, 2), (1, 4, 1, 4),
                                   # two to four channels over many pixels (images): a dword per plane, C dwords of pixels
                                   (2, 3, 32, 40), (3, 2, 16, 16), (1, 4, 9, 28), (5, 3, 224, 224), (2, 3, 7, 9)])
def test_layout_conversion(shape):
    n, c, h, w = shape
    x = synth.fill_u8(shape, SEED + 70)
    d_x = eden.DeviceBuffer(host=x)
    d_y = eden.DeviceBuffer(nbytes=x.size)
    d_z = eden.DeviceBuffer(nbytes=x.size)
    lib = eden.load()
    eden.check(lib.eh_transpose_u8_nchw2nhwc(d_x.ptr, d_y.ptr, n, c, h, w, None))
    y = d_y.download((n, h, w, c))
    assert np.array_equal(y, O.nchw2nhwc(x))
    eden.check(lib.eh_transpose_u8_nhwc2nchw(d_y.ptr, d_z.ptr, n, c, h, w, None))
    assert np.array_equal(d_z.download(shape), x)


# ----------------------------------------------------------------- size-independent properties at full size

def test_fc_full_size_properties():
    m, k, n = 256, 4096, 4096
    q = quant(0.01, 3, 0.002, 128, 0.08, 0)
    b = synth.fill_i32((n,), SEED + 80, -100000, 100000)
    w = synth.fill_u8((n, k), SEED + 81)
    # inputs at their zero point: every output is requant(bias), whatever the weights
    a = np.full((m, k), 3, np.uint8)
    got = gpu_fc(a, w, b, to_eh_requant(q))
    row = np.array([O.lib.eo_requant(int(v), q) for v in b], np.uint8)
    assert np.array_equal(got, np.broadcast_to(row, (m, n)))
    # weights at their zero point: same
    a = synth.fill_u8((m, k), SEED + 82)
    got = gpu_fc(a, np.full((n, k), 128, np.uint8), b, to_eh_requant(q))
    assert np.array_equal(got, np.broadcast_to(row, (m, n)))
    # permuting the reduction axis of both operands changes nothing
    perm = np.argsort(synth.splitmix64(SEED + 83, k))
    got1 = gpu_fc(a, w, b, to_eh_requant(q))
    got2 = gpu_fc(np.ascontiguousarray(a[:, perm]), np.ascontiguousarray(w[:, perm]), b, to_eh_requant(q))
    assert np.array_equal(got1, got2)


def test_operators_without_a_bias_tensor():
    """A null bias pointer is a bias of zeros in every operator; setting a bias later through repack is honoured."""
    q = O.raw_quant(zp_in=117, zp_w=131, zp_out=128, multiplier=1518500250, shift=-9)
    eq = to_eh_requant(q)
    s = O.conv_shape(2, 32, 9, 9, 48, 3, 3, pad=(1, 1, 1, 1))
    x, w = synth.fill_u8((2, 32, 9, 9), SEED + 901), synth.fill_u8_normal((48, 32, 3, 3), SEED + 902, 131, 20)
    zeros = np.zeros(48, np.int32)
    assert np.array_equal(gpu_conv(x, w, None, s, eq, eden.NHWC), O.conv2d(x, w, zeros, s, q))
    sd = O.conv_shape(2, 16, 9, 9, 16, 3, 3, pad=(1, 1, 1, 1), dm=1)
    wd = synth.fill_u8_normal((16, 1, 3, 3), SEED + 903, 131, 40)
    xd = synth.fill_u8((2, 16, 9, 9), SEED + 904)
    qd = O.raw_quant(zp_in=117, zp_w=131, zp_out=128, multiplier=1518500250, shift=-6)
    for layout in (eden.NHWC, eden.NCHW):
        assert np.array_equal(gpu_dwconv(xd, wd, None, sd, to_eh_requant(qd), layout), O.dwconv2d(xd, wd, np.zeros(16, np.int32), sd, qd))
    st = O.conv_shape(1, 32, 5, 5, 24, 2, 2, stride=(2, 2))
    wt = synth.fill_u8_normal((32, 24, 2, 2), SEED + 905, 131, 20)
    xt = synth.fill_u8((1, 32, 5, 5), SEED + 906)
    assert np.array_equal(gpu_deconv(xt, wt, None, st, eq, eden.NHWC), O.deconv2d(xt, wt, np.zeros(24, np.int32), st, q))
    a, wf = synth.fill_u8((9, 96), SEED + 907), synth.fill_u8_normal((40, 96), SEED + 908, 131, 20)
    assert np.array_equal(gpu_fc(a, wf, None, eq), O.fc(a, wf, np.zeros(40, np.int32), q))
    # repack: none -> some -> none
    b = synth.fill_i32((48,), SEED + 909, -4000, 4000)
    desc = eden.conv_desc(2, 32, 9, 9, 48, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 1, 1, eden.NHWC, eden.W_OIHW)
    d_x, d_w, d_b = eden.DeviceBuffer(host=x.transpose(0, 2, 3, 1)), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    d_o = eden.DeviceBuffer(nbytes=2 * 48 * 81)
    plan = eden.ConvPlan(desc, d_w, None, eq)
    for bias_buf, bias_host in ((d_b, b), (None, zeros)):
        plan.repack(d_w, bias_buf, eq)
        plan.run(d_x, d_o, eq)
        got = d_o.download((2, 9, 9, 48)).transpose(0, 3, 1, 2)
        assert np.array_equal(got, O.conv2d(x, w, bias_host, s, q))
    plan.destroy()
