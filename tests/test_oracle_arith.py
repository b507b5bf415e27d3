"""Pins the oracle's host arithmetic: closed forms and identities, exact big-integer
brute force, the golden vectors written from the reference's own code, and (where
oracle/_ref was built) the reference's code itself."""
import json
import os
from fractions import Fraction

import numpy as np
import pytest

import oracle_lib as O

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "arith_vectors.json")))
I32MIN, I32MAX = -2 ** 31, 2 ** 31 - 1


def round_half_away(fr):
    """Exact rounding of a Fraction, ties away from zero."""
    sign = -1 if fr < 0 else 1
    fr = abs(fr)
    return sign * int((fr + Fraction(1, 2)).__floor__())


def round_half_up(fr):
    """Exact rounding of a Fraction, ties toward +infinity."""
    return int((fr + Fraction(1, 2)).__floor__())


def test_quantize_multiplier_closed_forms():
    assert O.quantize_multiplier(0.5) == (1 << 30, 0)
    assert O.quantize_multiplier(1.0) == (1 << 30, 1)
    assert O.quantize_multiplier(0.25) == (1 << 30, -1)
    assert O.quantize_multiplier(0.375) == (1610612736, -1)
    assert O.quantize_multiplier(0.0) == (0, 0)
    # rounding up to 2^31 carries into the exponent
    assert O.quantize_multiplier(1.0 - 2.0 ** -40) == (1 << 30, 1)
    # the two multipliers the benchmark configurations use
    f = np.float32
    assert O.quantize_multiplier(float(f(0.02)) * float(f(0.005)) / float(f(0.05))) == (1099511562, -8)
    assert O.quantize_multiplier(float(f(0.01)) * float(f(0.002)) / float(f(0.08))) == (1099511680, -11)


def test_quantize_multiplier_property():
    rng = np.random.default_rng(1)
    for m in np.exp(rng.uniform(np.log(1e-9), np.log(100.0), 2000)):
        q, s = O.quantize_multiplier(float(m))
        assert (1 << 30) <= q < (1 << 31)
        approx = Fraction(q) * Fraction(2) ** (s - 31)
        assert abs(approx - Fraction(float(m))) <= Fraction(2) ** (s - 32)


def test_quantize_multiplier_golden():
    for mhex, q, s in GOLD["quantize_multiplier"]:
        assert O.quantize_multiplier(float.fromhex(mhex)) == (q, s), mhex


def test_conv_multiplier_golden_and_failure_leaves_m_untouched():
    import ctypes as C
    n_fail = 0
    for a, b, c, d, status, mhex in GOLD["conv_multiplier"]:
        m = C.c_double(-1.0)
        st = O.lib.eo_conv_multiplier(float.fromhex(a), float.fromhex(b), float.fromhex(c), float.fromhex(d), C.byref(m))
        assert st == status
        assert m.value.hex() == mhex
        if status:
            n_fail += 1
            assert m.value == -1.0
    assert n_fail >= 2
    # a failed check gives multiplier 0 / shift 0, so every output is clamp(zp_out)
    q = O.make_quant(0.5, 0, 0.5, 0, 1.0, 7, s_bias=1.0)
    assert (q.multiplier, q.shift) == (0, 0)
    assert O.lib.eo_requant(123456, q) == 7


def test_act_range_closed_forms_and_golden():
    assert O.act_range_u8(O.ACT_RELU6, float(np.float32(0.05)), 0) == (0, 120)
    assert O.act_range_u8(O.ACT_RELU, 0.05, 0) == (0, 255)
    assert O.act_range_u8(O.ACT_NONE, 0.05, 0) == (0, 255)
    assert O.act_range_u8(O.ACT_RELU1, 0.0078125, 128) == (0, 255)
    assert O.act_range_u8(O.ACT_RELU1, 0.0625, 128) == (112, 144)
    for act, shex, zp, lo, hi in GOLD["act_range_u8"]:
        assert O.act_range_u8(act, float.fromhex(shex), zp) == (lo, hi)
    # int8 limits: RELU6 at scale 0.05 from zero point -128 ends at -128 + 120
    assert O.act_range_s8(O.ACT_RELU6, float(np.float32(0.05)), -128) == (-128, -8)
    assert O.act_range_s8(O.ACT_NONE, 0.05, 3) == (-128, 127)
    for act, shex, zp, lo, hi in GOLD["act_range_s8"]:
        assert O.act_range_s8(act, float.fromhex(shex), zp) == (lo, hi)
        # the int8 range is the uint8 range of the zero point + 128, moved down by 128
        ulo, uhi = O.act_range_u8(act, float.fromhex(shex), zp + 128)
        assert (ulo - 128, uhi - 128) == (lo, hi)


def test_srdhm_identities():
    L = O.lib
    assert L.eo_srdhm(I32MIN, I32MIN) == I32MAX
    for x in list(range(-50, 51)) + [I32MAX, I32MIN + 1, 12345677, -12345677]:
        # multiplying by 2^30 (i.e. by one half) rounds x/2 with ties toward +infinity:
        # the nudge (1 - 2^30) followed by truncation sends -24.5 to -24, +24.5 to 25
        assert L.eo_srdhm(x, 1 << 30) == round_half_up(Fraction(x, 2)), x
    assert L.eo_srdhm(-1, 1 << 30) == 0 and L.eo_srdhm(1, 1 << 30) == 1
    assert L.eo_srdhm(-3, 1 << 30) == -1 and L.eo_srdhm(3, 1 << 30) == 2


def test_srdhm_bruteforce_exact():
    rng = np.random.default_rng(2)
    a = rng.integers(I32MIN, I32MAX + 1, 20000)
    b = rng.integers(I32MIN, I32MAX + 1, 20000)
    for x, y in zip(a.tolist(), b.tolist()):
        want = round_half_up(Fraction(x * y, 1 << 31))
        want = min(want, I32MAX)
        assert O.lib.eo_srdhm(x, y) == want, (x, y)


def test_rdivpot_identities_and_bruteforce():
    L = O.lib
    assert L.eo_rdivpot(12345, 0) == 12345 and L.eo_rdivpot(-12345, 0) == -12345
    assert L.eo_rdivpot(3, 1) == 2 and L.eo_rdivpot(-3, 1) == -2
    assert L.eo_rdivpot(-1, 1) == -1 and L.eo_rdivpot(1, 1) == 1
    assert L.eo_rdivpot(5, 2) == 1 and L.eo_rdivpot(6, 2) == 2 and L.eo_rdivpot(-6, 2) == -2
    rng = np.random.default_rng(3)
    for x, e in zip(rng.integers(I32MIN, I32MAX + 1, 20000).tolist(), rng.integers(0, 32, 20000).tolist()):
        assert L.eo_rdivpot(x, e) == round_half_away(Fraction(x, 1 << e)), (x, e)


def test_fixed_point_golden():
    for a, b, r in GOLD["srdhm"]:
        assert O.lib.eo_srdhm(a, b) == r, (a, b)
    for x, e, r in GOLD["rdivpot"]:
        assert O.lib.eo_rdivpot(x, e) == r, (x, e)
    for x, q, s, r in GOLD["mbqm"]:
        assert O.lib.eo_mbqm(x, q, s) == r, (x, q, s)


def test_mbqm_perchannel_kat_values():
    # -26 * {0.25, 0.375, 0.5} = -6.5, -9.75, -13 -> -7, -10, -13 (+128 -> 121, 118, 115):
    # the one uint8 known answer of the reference (gpu_userdriver_test.cc:490-494) pins ties away from zero
    for m, want in ((0.25, 121), (0.375, 118), (0.5, 115)):
        q, s = O.quantize_multiplier(m)
        assert O.lib.eo_mbqm(-26, q, s) + 128 == want
    q, s = O.quantize_multiplier(1.0)
    assert O.lib.eo_mbqm(115, q, s) == 115 and O.lib.eo_mbqm(-7, q, s) == -7


def test_mbqm_two_stage_rounding_vs_exact():
    """srdhm then rdivpot is two roundings; it must stay within one unit of the
    exact product and equal it whenever the exact product is far from a tie."""
    rng = np.random.default_rng(4)
    for _ in range(5000):
        q = int(rng.integers(1 << 30, 1 << 31))
        s = int(rng.integers(-20, 1))
        x = int(rng.integers(-(1 << 24), 1 << 24))
        exact = Fraction(x * q, 1 << (31 - s))
        got = O.lib.eo_mbqm(x, q, s)
        assert abs(Fraction(got) - exact) <= Fraction(1, 2) + Fraction(1, 1 << (-s)) if s < 0 else True


def test_fastpath_highmul_is_the_same_function_without_overflow():
    """mul_hi(x << 2, M) + rhadd(., 0) of the reference's hand-optimised kernels equals the
    exact saturating rounding doubling high mul whenever x << 2 stays inside int32."""
    rng = np.random.default_rng(6)
    xs = rng.integers(-(1 << 29), 1 << 29, 30000).tolist() + [-(1 << 29), (1 << 29) - 1, -1, 0, 1, -3, 3]
    ms = rng.integers(1 << 30, 1 << 31, len(xs)).tolist()
    for x, m in zip(xs, ms):
        assert O.lib.eo_srdhm_fastpath(x, m) == O.lib.eo_srdhm(x, m), (x, m)
    # exact ties of either sign
    for x in (-49, 49, -1, 1, -(1 << 20) - 1):
        assert O.lib.eo_srdhm_fastpath(x, 1 << 30) == O.lib.eo_srdhm(x, 1 << 30)
    q = O.raw_quant()
    acc = np.array([0, (1 << 28) - 1, 1 << 28, -(1 << 28), -(1 << 28) - 1], np.int32)
    assert O.count_fastpath_overflow(acc, q) == 2  # shift 1 -> x << 3 overflows from |x| >= 2^28 (positive) / > 2^28 (negative)


def test_requant_clamps():
    q = O.raw_quant(zp_out=10, act_min=20, act_max=100)
    assert O.lib.eo_requant(0, q) == 20
    assert O.lib.eo_requant(50, q) == 60
    assert O.lib.eo_requant(1000, q) == 100
    assert O.lib.eo_requant(-1000, q) == 20


def test_left_shift_multiplier():
    q, s = O.quantize_multiplier(3.0)
    assert s == 2
    for x in (-1000, -7, -1, 0, 1, 5, 33, 100000):
        assert O.lib.eo_mbqm(x, q, s) == 3 * x


@pytest.mark.skipif(O.load_ref() is None, reason="oracle/_ref not built (needs the reference tree)")
def test_against_reference_build_live():
    import ctypes as C
    ref = O.load_ref()
    rng = np.random.default_rng(5)
    for m in np.exp(rng.uniform(np.log(1e-9), np.log(100.0), 3000)):
        q, s = C.c_int32(), C.c_int32()
        ref.ref_quantize_multiplier(float(m), C.byref(q), C.byref(s))
        assert O.quantize_multiplier(float(m)) == (q.value, s.value)
    xs = rng.integers(I32MIN, I32MAX + 1, 30000).tolist()
    ys = rng.integers(I32MIN, I32MAX + 1, 30000).tolist()
    es = rng.integers(0, 32, 30000).tolist()
    for x, y, e in zip(xs, ys, es):
        assert O.lib.eo_srdhm(x, y) == ref.ref_srdhm(x, y)
        assert O.lib.eo_rdivpot(x, e) == ref.ref_rdivpot(x, e)
    for _ in range(20000):
        q = int(rng.integers(1 << 30, 1 << 31))
        s = int(rng.integers(-31, 1))
        x = int(rng.integers(-(1 << 30), 1 << 30))
        assert O.lib.eo_mbqm(x, q, s) == ref.ref_mbqm(x, q, s)
    for _ in range(2000):
        act, zp = int(rng.integers(0, 4)), int(rng.integers(0, 256))
        scale = float(np.float32(np.exp(rng.uniform(np.log(1e-3), 0.0))))
        lo, hi = C.c_int32(), C.c_int32()
        ref.ref_act_range_u8(act, scale, zp, C.byref(lo), C.byref(hi))
        assert O.act_range_u8(act, scale, zp) == (lo.value, hi.value)
        ref.ref_act_range_s8(act, scale, zp - 128, C.byref(lo), C.byref(hi))
        assert O.act_range_s8(act, scale, zp - 128) == (lo.value, hi.value)
