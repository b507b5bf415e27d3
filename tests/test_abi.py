"""CPU-side checks of the C ABI library: it loads, exports every symbol the
header declares, and its host arithmetic (no GPU involved) matches the golden
vectors written from the reference's own code and the oracle."""
import ctypes as C
import json
import os
import re

import numpy as np
import pytest

import oracle_lib as O
from harness import eden

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = json.load(open(os.path.join(ROOT, "tests", "golden", "arith_vectors.json")))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "eden_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(eh_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = eden.load()
    names = declared_symbols()
    assert len(names) >= 35
    for name in names:
        assert hasattr(lib, name), name
    assert set(names) == set(eden.EXPORTS), set(names) ^ set(eden.EXPORTS)


def test_userdriver_library_exports_every_declared_symbol_and_describes_a_list_without_a_gpu():
    """libedenud.so (include/eden_ud.h): every declared entry point is exported and bound; describing an operator list
    is host work, and its argument checks answer with an error text instead of crashing.  Nothing here computes."""
    import importlib
    ud = importlib.import_module("cl-eden-kernel_amd.userdriver")
    lib = ud.load()
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "eden_ud.h")).read(), flags=re.S)
    names = sorted(set(re.findall(r"\b(eud_[a-z0-9_]+)\s*\(", text)))
    assert len(names) >= 20
    for name in names:
        assert hasattr(lib, name), name
    assert set(names) == set(ud.EXPORTS), set(names) ^ set(ud.EXPORTS)
    ol = ud.OperatorList(5, ud.MODEL_ANDROID_NN)
    x = ol.feature_map(0, (1, 8, 8, 4), 0.1, 3)
    y = ol.feature_map(1, (1, 8, 8, 6), 0.2, 5)
    w = ol.parameter(np.zeros((6, 1, 1, 4), np.uint8), 0.01, 128)
    b = ol.parameter(np.zeros(6, np.int32), 0.001, 0)
    assert (x, y, w, b) == (0, 1, 2, 3)
    ol.operator("CONV_2D", ud.OP_CONV_2D, [x, w, b], [y], ud.options())
    with pytest.raises(ud.EdenUdError, match="unknown tensor"):
        ol.operator("CONV_2D", ud.OP_CONV_2D, [x, 17, b], [y], ud.options())
    with pytest.raises(ud.EdenUdError, match="not offered"):
        ol.operator("SOFTMAX", 25, [x], [y], ud.options())
    with pytest.raises(ud.EdenUdError):
        ol.feature_map(2, (1, 2, 3, 4, 5), 0.1, 0)   # five extents
    mobilenet = importlib.import_module("cl-eden-kernel_amd.mobilenet")
    net, i, o, shape = mobilenet.operator_list(ud, 9, 2, 96)   # 64 operator descriptions, weights copied
    assert (i, o, shape) == (0, 64, (2, 1000))


def test_product_host_arithmetic_matches_golden_vectors():
    lib = eden.load()
    for mhex, q, s in GOLD["quantize_multiplier"]:
        qq, ss = C.c_int32(), C.c_int32()
        lib.eh_quantize_multiplier(float.fromhex(mhex), C.byref(qq), C.byref(ss))
        assert (qq.value, ss.value) == (q, s)
    for a, b, c, d, status, mhex in GOLD["conv_multiplier"]:
        m = C.c_double(-1.0)
        st = lib.eh_conv_multiplier(float.fromhex(a), float.fromhex(b), float.fromhex(c), float.fromhex(d), C.byref(m))
        assert (st != 0) == (status != 0) and m.value.hex() == mhex
    for act, shex, zp, lo, hi in GOLD["act_range_u8"]:
        l, h = C.c_int32(), C.c_int32()
        lib.eh_act_range_u8(act, float.fromhex(shex), zp, C.byref(l), C.byref(h))
        assert (l.value, h.value) == (lo, hi)


def test_make_requant_matches_oracle_and_handles_bias_scale_mismatch():
    rng = np.random.default_rng(21)
    for _ in range(500):
        s_in, s_w, s_out = [float(np.float32(x)) for x in np.exp(rng.uniform(np.log(1e-3), np.log(2.0), 3))]
        zi, zw, zo = [int(v) for v in rng.integers(0, 256, 3)]
        act, en = int(rng.integers(0, 4)), bool(rng.integers(0, 2))
        a = eden.make_requant(s_in, zi, s_w, zw, s_out, zo, act, en).as_tuple()
        b = O.make_quant(s_in, zi, s_w, zw, s_out, zo, act, en).as_tuple()
        assert a == b
        a = eden.make_requant_s8(s_in, zi - 128, s_w, zw - 128, s_out, zo - 128, act, en).as_tuple()
        b = O.make_quant_s8(s_in, zi - 128, s_w, zw - 128, s_out, zo - 128, act, en).as_tuple()
        assert a == b
    lib = eden.load()
    for act, shex, zp, lo, hi in GOLD["act_range_s8"]:
        l, h = C.c_int32(), C.c_int32()
        lib.eh_act_range_s8(act, float.fromhex(shex), zp, C.byref(l), C.byref(h))
        assert (l.value, h.value) == (lo, hi)
    q = eden.make_requant(0.5, 0, 0.5, 0, 1.0, 7, s_bias=1.0)  # bias scale != s_in * s_w
    assert (q.multiplier, q.shift) == (0, 0)


def test_make_requant_perchannel_matches_per_channel_oracle_multipliers():
    """One (multiplier, shift) per filter scale: float(in_scale) * float(filter_scale) / float(out_scale) in double, as
    the per-channel convolution computes them when it runs (cl_operators/CLConvolutionPerChannelQuantized.cpp:96-115)."""
    rng = np.random.default_rng(23)
    for _ in range(50):
        s_in, s_out = [float(np.float32(x)) for x in np.exp(rng.uniform(np.log(1e-3), np.log(2.0), 2))]
        scales = np.exp(rng.uniform(np.log(1e-4), np.log(1.0), int(rng.integers(1, 70)))).astype(np.float32)
        zi, zo = int(rng.integers(0, 256)), int(rng.integers(0, 256))
        act, en = int(rng.integers(0, 4)), bool(rng.integers(0, 2))
        q, mult, shift = eden.make_requant_perchannel(s_in, zi, scales, s_out, zo, act, en)
        want = [O.quantize_multiplier(s_in * float(ws) / s_out) for ws in scales]
        assert list(zip(mult.tolist(), shift.tolist())) == want
        lo, hi = O.act_range_u8(act, s_out, zo) if en else (0, 255)
        assert (q.zp_in, q.zp_w, q.zp_out, q.act_min, q.act_max) == (zi, 0, zo, lo, hi)
        assert (q.multiplier, q.shift) == (0, 0)  # the per-tensor pair is unused in this mode


def test_output_dim_formulas_match_oracle():
    lib = eden.load()
    rng = np.random.default_rng(22)
    for _ in range(300):
        i, pa, pb, k, d, s = [int(v) for v in (rng.integers(1, 300), rng.integers(0, 4), rng.integers(0, 4),
                                                rng.integers(1, 8), rng.integers(1, 3), rng.integers(1, 4))]
        assert lib.eh_conv_out_dim(i, pa, pb, k, d, s) == O.lib.eo_conv_out_dim(i, pa, pb, k, d, s)
        assert lib.eh_deconv_out_dim(i, pa, pb, k, s) == O.lib.eo_deconv_out_dim(i, pa, pb, k, s)


def test_parameter_errors_are_reported_without_a_gpu():
    lib = eden.load()
    plan = C.c_void_p()
    desc = eden.conv_desc(1, 4, 4, 4, 4, 3, 3)
    bad_q = eden.Requant(0, 0, 0, -5, 0, 0, 255)  # negative multiplier
    rc = lib.eh_conv2d_u8_plan(C.byref(plan), C.byref(desc), None, None, C.byref(bad_q), None)
    assert rc == -3 and b"multiplier" in lib.eh_last_error()
    q = eden.Requant(0, 0, 0, 1 << 30, 1, 0, 255)
    desc = eden.conv_desc(1, 4, 4, 4, 6, 3, 3, groups=4)  # groups do not divide cout
    assert lib.eh_conv2d_u8_plan(C.byref(plan), C.byref(desc), None, None, C.byref(q), None) == -3
    desc = eden.conv_desc(1, 4, 4, 4, 9, 3, 3, dm=2)  # cout != c * dm
    assert lib.eh_dwconv2d_u8_plan(C.byref(plan), C.byref(desc), None, None, C.byref(q), None) == -3
    assert lib.eh_fc_u8_plan(C.byref(plan), 4, 0, 4, None, None, C.byref(q), None) == -3
    q = eden.Requant(0, 0, 0, 1 << 30, -40, 0, 255)  # shift out of range
    assert lib.eh_fc_u8_plan(C.byref(plan), 4, 4, 4, None, None, C.byref(q), None) == -3
    q = eden.Requant(300, 0, 0, 1 << 30, 0, 0, 255)  # zero point outside uint8
    assert lib.eh_fc_u8_plan(C.byref(plan), 4, 4, 4, None, None, C.byref(q), None) == -3


def test_synthetic_generators_match_the_c_harness():
    from harness import synth
    assert np.array_equal(synth.fill_u8((4097,), 0xEDE2), O.fill_u8((4097,), 0xEDE2))
    assert np.array_equal(synth.fill_u8((333,), 9, 3, 17), O.fill_u8((333,), 9, 3, 17))
    assert np.array_equal(synth.fill_i32((999,), 0xEDE3, -1000, 1000), O.fill_i32((999,), 0xEDE3, -1000, 1000))
    a = synth.fill_u8_normal((50000,), 0xEDE4, 128, 20)
    assert np.array_equal(a, O.fill_u8_normal((50000,), 0xEDE4, 128, 20))
    assert abs(a.mean() - 128) < 0.5 and abs(a.std() - 20) < 0.5


def test_one_tap_kernel_is_only_chosen_when_every_tap_lies_inside_the_image():
    """The one-tap kernel does not test its pixel against the image, so a 1x1 convolution with bottom / right padding
    and a deconvolution phase that a negative tail padding enlarges beyond the input must go to other kernels."""
    nhwc = eden.NHWC
    assert eden.conv_kernels(eden.conv_desc(2, 24, 14, 14, 144, 1, 1, layout=nhwc)) == ["one_tap"]
    assert eden.conv_kernels(eden.conv_desc(2, 24, 14, 14, 144, 1, 1, stride=(2, 2), layout=nhwc)) == ["one_tap"]
    for pad in ((0, 1, 0, 0), (0, 0, 0, 1), (0, 1, 0, 1), (0, 3, 0, 2)):
        got = eden.conv_kernels(eden.conv_desc(2, 24, 14, 14, 144, 1, 1, pad=pad, layout=nhwc))
        assert got != ["one_tap"], (pad, got)
    # top / left padding never qualified (the tap of the first pixel lies outside)
    assert eden.conv_kernels(eden.conv_desc(2, 24, 14, 14, 144, 1, 1, pad=(1, 0, 0, 0), layout=nhwc)) != ["one_tap"]
    # stride 2 over an odd extent with one row of bottom padding: the last output row reads row 14 of 14
    assert eden.conv_kernels(eden.conv_desc(1, 16, 13, 13, 32, 1, 1, stride=(2, 2), pad=(0, 2, 0, 2), layout=nhwc)) != ["one_tap"]
    # transposed convolution, kernel <= stride: every phase is one tap
    d = eden.conv_desc(1, 16, 6, 6, 32, 2, 2, stride=(2, 2), layout=nhwc, weight_layout=eden.W_IOHW)
    assert eden.conv_kernels(d, deconv=True) == ["one_tap"] * 4
    d = eden.conv_desc(1, 16, 6, 6, 32, 2, 2, stride=(2, 2), pad=(0, -2, 0, -2), layout=nhwc, weight_layout=eden.W_IOHW)
    assert "one_tap" not in eden.conv_kernels(d, deconv=True)


def test_3x3_stride_1_convolutions_take_the_patch_kernel():
    nhwc = eden.NHWC
    assert eden.conv_kernels(eden.conv_desc(1, 64, 56, 56, 64, 3, 3, pad=(1, 1, 1, 1), layout=nhwc)) == ["conv3x3_patch"]
    assert eden.conv_kernels(eden.conv_desc(64, 64, 56, 56, 64, 3, 3, pad=(1, 1, 1, 1), layout=nhwc)) == ["conv3x3_patch"]
    assert eden.conv_kernels(eden.conv_desc(2, 128, 16, 16, 100, 3, 3, layout=eden.NCHW)) == ["conv3x3_patch"]
    # 128 channels over a full round of 128 x 128 tiles and more: the implicit GEMM again
    assert eden.conv_kernels(eden.conv_desc(16, 128, 28, 28, 128, 3, 3, pad=(1, 1, 1, 1), layout=nhwc)) == ["conv3x3_patch"]
    assert eden.conv_kernels(eden.conv_desc(64, 128, 28, 28, 128, 3, 3, pad=(1, 1, 1, 1), layout=nhwc)) == ["dma_128x128"]
    assert eden.conv_kernels(eden.conv_desc(64, 256, 14, 14, 256, 3, 3, pad=(1, 1, 1, 1), layout=nhwc)) == ["dma_128x128"]
    assert eden.conv_kernels(eden.conv_desc(1, 48, 56, 56, 64, 3, 3, pad=(1, 1, 1, 1), layout=nhwc)) == ["conv3x3_patch"]
    assert eden.conv_kernels(eden.conv_desc(1, 16, 112, 112, 32, 3, 3, pad=(1, 1, 1, 1), layout=nhwc)) == ["conv3x3_patch"]
    # stride 2, dilation 2, groups, tiny images: the implicit-GEMM kernels
    for d in (eden.conv_desc(1, 64, 56, 56, 64, 3, 3, stride=(2, 2), pad=(1, 1, 1, 1), layout=nhwc),
              eden.conv_desc(1, 64, 56, 56, 64, 3, 3, pad=(2, 2, 2, 2), dil=(2, 2), layout=nhwc),
              eden.conv_desc(1, 64, 56, 56, 64, 3, 3, pad=(1, 1, 1, 1), groups=2, layout=nhwc),
              eden.conv_desc(4, 64, 7, 7, 64, 3, 3, pad=(1, 1, 1, 1), layout=nhwc)):
        assert "conv3x3_patch" not in eden.conv_kernels(d)


def test_few_channel_convolutions_take_the_kernel_row_kernel():
    nhwc = eden.NHWC
    assert eden.conv_kernels(eden.conv_desc(64, 3, 224, 224, 64, 7, 7, stride=(2, 2), pad=(3, 3, 3, 3), layout=nhwc)) == ["few_channel_rows"]
    assert eden.conv_kernels(eden.conv_desc(1, 1, 64, 64, 56, 9, 9, pad=(4, 4, 4, 4), layout=nhwc)) == ["few_channel_rows"]
    assert eden.conv_kernels(eden.conv_desc(1, 4, 64, 64, 16, 5, 5, layout=nhwc)) == ["few_channel_rows"]
    assert eden.conv_kernels(eden.conv_desc(1, 1, 64, 64, 16, 3, 3, layout=nhwc)) == ["few_channel_rows"]
    # RGB 3x3 keeps its own kernel; rows beyond 32 bytes, an even number of rows, dilation, more channels: the implicit GEMM
    assert eden.conv_kernels(eden.conv_desc(1, 3, 64, 64, 32, 3, 3, layout=nhwc)) == ["c3k3"]
    for d in (eden.conv_desc(1, 3, 64, 64, 32, 11, 11, layout=nhwc), eden.conv_desc(1, 3, 64, 64, 32, 4, 4, layout=nhwc),
              eden.conv_desc(1, 3, 64, 64, 32, 5, 5, dil=(2, 2), layout=nhwc), eden.conv_desc(1, 8, 64, 64, 32, 7, 7, layout=nhwc)):
        assert "few_channel_rows" not in eden.conv_kernels(d)


def test_ragged_channel_counts_run_on_a_padded_copy_unless_told_otherwise():
    """Channels per group that are no multiple of 16 and fit none of the few-channel kernels: the plan is built on
    channels padded to the next multiple of 16 (the wide-load kernels); EXACT_CHANNELS keeps the byte-gathering kernel."""
    nhwc, exact = eden.NHWC, eden.NHWC | eden.EXACT_CHANNELS
    assert eden.conv_kernels(eden.conv_desc(8, 21, 64, 64, 21, 3, 3, pad=(1, 1, 1, 1), layout=nhwc)) == ["conv3x3_patch"]
    assert eden.conv_kernels(eden.conv_desc(8, 21, 64, 64, 21, 3, 3, pad=(1, 1, 1, 1), layout=exact)) == ["staged"]
    assert eden.conv_kernels(eden.conv_desc(8, 100, 32, 32, 100, 3, 3, pad=(1, 1, 1, 1), layout=nhwc)) == ["conv3x3_patch"]
    assert eden.conv_kernels(eden.conv_desc(1, 24, 56, 56, 64, 3, 3, pad=(1, 1, 1, 1), layout=nhwc)) == ["conv3x3_patch"]
    assert eden.conv_kernels(eden.conv_desc(8, 6, 112, 112, 16, 5, 5, layout=nhwc))[0].startswith("dma_")
    assert eden.conv_kernels(eden.conv_desc(1, 20, 8, 8, 12, 3, 3, groups=2, layout=exact)) == ["staged", "staged"]
    assert "staged" not in eden.conv_kernels(eden.conv_desc(1, 20, 8, 8, 12, 3, 3, groups=2, layout=nhwc))
    assert "staged" not in eden.conv_kernels(eden.conv_desc(8, 21, 64, 64, 21, 16, 16, stride=(8, 8), pad=(4, 4, 4, 4), layout=nhwc, weight_layout=eden.W_IOHW), deconv=True)
    # channel counts the one-tap and few-channel kernels take as they are keep them
    assert eden.conv_kernels(eden.conv_desc(32, 24, 56, 56, 144, 1, 1, layout=nhwc)) == ["one_tap"]
    assert eden.conv_kernels(eden.conv_desc(1, 3, 64, 64, 32, 3, 3, layout=nhwc)) == ["c3k3"]


def test_small_groups_are_bundled_into_block_diagonal_problems():
    nhwc = eden.NHWC
    # 32 groups of 4 channels: two problems over 64 adjacent channels each; 8 groups of 8: one; EXACT_CHANNELS: one per group
    assert len(eden.conv_kernels(eden.conv_desc(8, 128, 56, 56, 128, 3, 3, pad=(1, 1, 1, 1), groups=32, layout=nhwc))) == 2
    assert len(eden.conv_kernels(eden.conv_desc(8, 64, 28, 28, 64, 3, 3, pad=(1, 1, 1, 1), groups=8, layout=nhwc))) == 1
    assert len(eden.conv_kernels(eden.conv_desc(8, 128, 56, 56, 128, 3, 3, pad=(1, 1, 1, 1), groups=32, layout=nhwc | eden.EXACT_CHANNELS))) == 32
    # groups of 16 channels or more run one problem each, as before
    assert len(eden.conv_kernels(eden.conv_desc(8, 512, 14, 14, 512, 3, 3, pad=(1, 1, 1, 1), groups=32, layout=nhwc))) == 32
    assert "staged" not in eden.conv_kernels(eden.conv_desc(8, 128, 56, 56, 128, 3, 3, pad=(1, 1, 1, 1), groups=32, layout=nhwc))


def test_reductions_beyond_one_k_table_stay_on_the_tiled_kernels():
    nhwc = eden.NHWC
    assert eden.conv_kernels(eden.conv_desc(8, 512, 7, 7, 4096, 7, 7, layout=nhwc)) == ["dma_64x64_splitk"]     # sliced
    assert eden.conv_kernels(eden.conv_desc(64, 25088, 1, 1, 4096, 1, 1, layout=nhwc))[0].startswith("dma_")   # a plain matrix needs no table


def test_unequal_deconvolution_phases_share_one_configuration():
    """3x3 at stride 2: the four phases (4, 2, 2, 1 taps) are padded to one reduction length and take one tiled
    configuration, the one-tap phase included, over even output extents and over odd ones (phases of 16x16, 16x15,
    15x16 and 15x15 pixels); 24 channels likewise on their padded copy; EXACT_CHANNELS there keeps the byte gathers."""
    for pad in ((1, 0, 1, 0), (1, 1, 1, 1)):
        desc = eden.conv_desc(8, 256, 16, 16, 256, 3, 3, stride=(2, 2), pad=pad, layout=eden.NHWC, weight_layout=eden.W_IOHW)
        kernels = eden.conv_kernels(desc, deconv=True)
        assert len(kernels) == 4 and len(set(kernels)) == 1 and kernels[0].startswith("dma_"), (pad, kernels)
    ragged = eden.conv_desc(8, 24, 16, 16, 24, 3, 3, stride=(2, 2), pad=(1, 0, 1, 0), layout=eden.NHWC, weight_layout=eden.W_IOHW)
    assert len(set(eden.conv_kernels(ragged, deconv=True))) == 1
    ragged.layout |= eden.EXACT_CHANNELS
    assert "staged" in eden.conv_kernels(ragged, deconv=True)


def test_classifier_heads_take_the_kernel_cut_along_the_weights():
    nhwc = eden.NHWC
    assert eden.conv_kernels(eden.conv_desc(1, 1280, 1, 1, 1000, 1, 1, layout=nhwc)) == ["skinny"]
    assert eden.conv_kernels(eden.conv_desc(32, 4096, 1, 1, 4096, 1, 1, layout=nhwc)) == ["skinny"]
    assert eden.conv_kernels(eden.conv_desc(64, 1280, 1, 1, 1000, 1, 1, layout=nhwc)) == ["skinny"]
    assert "skinny" not in eden.conv_kernels(eden.conv_desc(64, 4096, 1, 1, 4096, 1, 1, layout=nhwc))
    assert eden.conv_kernels(eden.conv_desc(2, 512, 5, 5, 48, 1, 1, layout=nhwc)) == ["skinny"]
    # more than 64 pixels, a reduction within the one-tap kernel's, a stride: the other kernels
    assert "skinny" not in eden.conv_kernels(eden.conv_desc(65, 1280, 1, 1, 1000, 1, 1, layout=nhwc))
    assert eden.conv_kernels(eden.conv_desc(1, 256, 1, 1, 1000, 1, 1, layout=nhwc)) == ["one_tap"]
    assert "skinny" not in eden.conv_kernels(eden.conv_desc(1, 512, 9, 9, 48, 1, 1, stride=(2, 2), layout=nhwc))


def test_descriptor_queries_answer_or_refuse_whatever_the_descriptor():
    """Descriptors drawn from edge values (zero, negative, 2^31 - 1, unknown layouts): the kernel query, which runs the
    plan builder's host side, either answers or refuses with a status, and does so quickly; the stated limits (a
    reduction of 2^24 terms, 65536 deconvolution phases) keep absurd descriptors from building tables of that size."""
    import time
    rng = np.random.default_rng(5)
    edge = [0, 1, 2, 3, 7, 16, 17, 64, 255, 1001, 4096, 65536, 1 << 24, (1 << 31) - 1, -1]
    small = [0, 1, 2, 3, 5, 7, 16, 64, -1]
    answered = refused = 0
    start = time.time()
    for it in range(6000):
        p = lambda: int(edge[int(rng.integers(0, len(edge)))]) if rng.random() < 0.4 else int(rng.integers(1, 70))
        k = lambda: int(small[int(rng.integers(0, len(small)))]) if rng.random() < 0.5 else int(rng.integers(1, 8))
        groups = int(rng.choice([1, 1, 1, 2, 4, 32, 1000, 0]))
        c, cout = p(), p()
        if groups > 0 and rng.random() < 0.7:
            c, cout = max(groups, abs(c) // groups * groups), max(groups, abs(cout) // groups * groups)
        kh, kw = k(), k()
        desc = eden.conv_desc(p(), c, p(), p(), cout, kh, kw, (k(), k()), (max(kh, 0) // 2, max(kh, 0) // 2, max(kw, 0) // 2, max(kw, 0) // 2),
                              (int(rng.choice([1, 1, 2, 1000, 0])),) * 2, groups, int(rng.choice([1, 1, 2, 0])),
                              int(rng.choice([0, 1, 1, 0x401, 0x201, 2, 77])), int(rng.choice([0, 0, 1, 2, 0x100, 9])))
        for deconv in (False, True):
            if deconv and desc.weight_layout & 0xFF == 0:
                desc.weight_layout |= eden.W_IOHW
            try:
                assert len(eden.conv_kernels(desc, deconv=deconv)) >= 0
                answered += 1
            except eden.EdenHipError:
                refused += 1
    assert answered > 500 and refused > 500, (answered, refused)
    assert time.time() - start < 60
    for absurd in (eden.conv_desc(1, 1 << 24, 8, 8, 16, 3, 3), eden.conv_desc(1, 4096, 8, 8, 16, 64, 65)):
        with pytest.raises(eden.EdenHipError, match="reductions over"):
            eden.conv_kernels(absurd)
    with pytest.raises(eden.EdenHipError, match="output phases"):
        eden.conv_kernels(eden.conv_desc(1, 1024, 8, 8, 1024, 64, 64, stride=(64, 64), groups=1024, weight_layout=eden.W_IOHW), deconv=True)


def test_buffer_pool_protocol_without_a_gpu():
    """request / reset / layout are host bookkeeping (CLRuntime.cpp:34-118, 147-157): a REUSE request takes over the
    first feature map handed back and grows it, intra-operator scratch is sized to the largest request per slot, and
    the layout is one allocation with 1024 bytes in front of and 32 behind every buffer, rounded to 1024."""
    pool = eden.BufferPool()
    a = pool.request(eden.POOL_INTER_NEW, 128)
    b = pool.request(eden.POOL_INTER_REUSE, 512)          # nothing handed back yet: a new slot
    assert b.slot != a.slot
    pool.reset_inter(a)
    c = pool.request(eden.POOL_INTER_REUSE, 1024)         # takes a over, grown
    assert c.slot == a.slot and a.nbytes == 1024
    d = pool.request(eden.POOL_INTER_REUSE, 16)
    assert d.slot not in (a.slot, b.slot)
    pool.reset_inter(b)
    e = pool.request(eden.POOL_INTER_REUSE, 100)          # smaller than what b holds: b keeps its size
    assert e.slot == b.slot and b.nbytes == 512
    s1 = pool.request(eden.POOL_INTRA, 400)
    s2 = pool.request(eden.POOL_INTRA, 200)
    assert s1.slot != s2.slot
    pool.reset_intra()
    s3 = pool.request(eden.POOL_INTRA, 320)               # the free one that is already large enough
    assert s3.slot == s1.slot and s1.nbytes == 400
    s4 = pool.request(eden.POOL_INTRA, 1200)              # the remaining free one, grown
    assert s4.slot == s2.slot and s2.nbytes == 1200
    nbytes, slots = pool.layout()
    assert slots == 5
    pad = lambda n: (1024 + n + 32 + 1023) // 1024 * 1024
    assert nbytes == pad(1024) + pad(512) + pad(16) + pad(400) + pad(1200)
    assert a.ptr.value is None                            # no memory before the assignment
    with pytest.raises(eden.EdenHipError):
        pool.reset_inter(s1)                              # not a feature map


def test_buffer_pool_release_before_assignment_without_a_gpu():
    """A pooled buffer released before its list is assigned (a tensor destroyed while the list is still being built)
    takes no part in the layout, is not handed to later REUSE / INTRA requests, cannot be reset, and an assignment
    whose every slot was released allocates nothing (so nothing here reaches the device)."""
    lib = eden.load()
    pool = eden.BufferPool()
    a = pool.request(eden.POOL_INTER_NEW, 3000)
    b = pool.request(eden.POOL_INTER_NEW, 500)
    s = pool.request(eden.POOL_INTRA, 700)
    pad = lambda n: (1024 + n + 32 + 1023) // 1024 * 1024
    assert pool.layout() == (pad(3000) + pad(500) + pad(700), 3)
    pool.reset_inter(a)
    eden.check(lib.eh_pool_release(pool.h, a.slot))       # handed back AND released: must not be taken over
    assert pool.layout() == (pad(500) + pad(700), 2)
    c = pool.request(eden.POOL_INTER_REUSE, 100)
    assert c.slot not in (a.slot, b.slot)
    with pytest.raises(eden.EdenHipError):
        pool.reset_inter(a)
    with pytest.raises(eden.EdenHipError):
        eden.check(lib.eh_pool_release(pool.h, a.slot))   # twice
    pool.reset_intra()
    eden.check(lib.eh_pool_release(pool.h, s.slot))
    s2 = pool.request(eden.POOL_INTRA, 50)                # the released scratch slot is not reused either
    assert s2.slot != s.slot
    for buf in (b, c, s2):
        eden.check(lib.eh_pool_release(pool.h, buf.slot))
    assert pool.layout() == (0, 0)
    assert pool.assign() == 0                             # nothing live: no device allocation is made
    assert a.ptr.value is None and b.ptr.value is None


def test_mobilenet_pool_is_a_fraction_of_one_buffer_per_tensor():
    """Liveness reuse over the MobileNetV2 operator list (gpu_op_constructor.cc:2157-2191), on the host: replaying
    the list's requests and releases through the pool gives far fewer buffers than tensors."""
    import importlib
    mobilenet = importlib.import_module("cl-eden-kernel_amd.mobilenet")
    tensors, ops = mobilenet.layers(224)
    batch = 64
    size = lambda i: batch * tensors[i]["h"] * tensors[i]["w"] * tensors[i]["c"]
    readers = {}
    for op in ops:
        for key in ("src", "a", "b"):
            if key in op:
                readers[op[key]] = readers.get(op[key], 0) + 1
    pool = eden.BufferPool()
    bufs = {0: pool.request(eden.POOL_INTER_NEW, size(0))}
    for op in ops:
        bufs[op["dst"]] = pool.request(eden.POOL_INTER_REUSE, size(op["dst"]))
        for t in [op[k] for k in ("src", "a", "b") if k in op]:
            readers[t] -= 1
            if readers[t] == 0:
                pool.reset_inter(bufs[t])
        # an operator's output never shares storage with what it reads
        assert all(bufs[op["dst"]].slot != bufs[op[k]].slot for k in ("src", "a", "b") if k in op)
    nbytes, slots = pool.layout()
    assert slots <= 4
    assert nbytes < 0.45 * sum(size(i) for i in range(len(tensors)))
