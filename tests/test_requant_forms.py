"""The kernels' requantization, evaluated on the host through the C ABI
(eh_requant_apply compiles the same source the kernels do), against the oracle's
MultiplyByQuantizedMultiplier chain.  Pins the single-shift form the kernels
use for left_shift == 0 and 1 <= right_shift <= 20 on the inputs where a merged
rounding could go wrong: ties of the second rounding on both signs, the band
-2^30 <= x*M < 0 where the first rounding gives 0 for a negative accumulator,
and the int32 extremes."""
import importlib

import numpy as np
import pytest

import oracle_lib as O

eden = importlib.import_module("cl-eden-kernel_amd")


def to_eh(q):
    r = eden.Requant()
    for f in ("zp_in", "zp_w", "zp_out", "multiplier", "shift", "act_min", "act_max"):
        setattr(r, f, getattr(q, f))
    return r


def probe_accumulators(multiplier, rs, rng):
    acc = [0, 1, -1, 2, -2, 3, -3, 2**31 - 1, -2**31, 2**31 - 2, -2**31 + 1, 2**30, -2**30]
    acc += rng.integers(-2**31, 2**31, 1500).tolist()
    acc += rng.integers(-70000, 70000, 1500).tolist()
    if multiplier > 0:
        # accumulators whose first rounding lands on or next to a tie of the second: v = (q << rs) + 2^(rs-1)
        h = 1 << (rs - 1)
        for qv in list(range(-40, 41)) + rng.integers(-2**max(1, 30 - rs), 2**max(1, 30 - rs), 200).tolist():
            v = (int(qv) << rs) + h
            x0 = (v << 31) // multiplier
            acc += [x0 + d for d in range(-3, 4)]
        # negative accumulators whose product stays above -2^30
        lim = (1 << 30) // multiplier
        acc += [-lim - 1, -lim, -lim + 1]
    acc = np.array([a for a in acc if -2**31 <= a < 2**31], np.int64).astype(np.int32)
    return acc


MULTIPLIERS = [1 << 30, (1 << 30) + 1, (1 << 31) - 1, 1099511680, 1518500250, 0, 1, 12345]


@pytest.mark.parametrize("rs", [1, 2, 3, 7, 8, 11, 16, 20])
def test_single_shift_form_equals_oracle(rs):
    rng = np.random.default_rng(1000 + rs)
    for mult in MULTIPLIERS:
        for zp_out, lo, hi in ((0, 0, 255), (128, 0, 255), (255, 20, 230), (3, 3, 3)):
            q = O.raw_quant(zp_out=zp_out, multiplier=mult, shift=-rs, act_min=lo, act_max=hi)
            acc = probe_accumulators(mult, rs, rng)
            want = np.array([O.lib.eo_requant(int(a), q) for a in acc], np.uint8)
            got, single = eden.requant_apply(to_eh(q), acc)
            assert single, "the single-shift form must be the one in use for these parameters"
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, (mult, rs, zp_out, acc[bad[:5]], got[bad[:5]], want[bad[:5]])
            two, single = eden.requant_apply(to_eh(q), acc, two_step=True)
            assert not single and np.array_equal(two, want)
            # the epilogues' packed evaluation: clamp before the shift, a row term inside the rounding term
            near = acc[(acc > -2**31 + 5000) & (acc < 2**31 - 5000)]
            packed, _ = eden.requant_apply(to_eh(q), near, channel_form="packed")
            ref = np.array([O.lib.eo_requant(int(a), q) for a in near], np.uint8)
            bad = np.nonzero(packed != ref)[0]
            assert bad.size == 0, ("packed", mult, rs, zp_out, near[bad[:5]], packed[bad[:5]], ref[bad[:5]])


@pytest.mark.parametrize("shift", [-31, -25, -21, 0, 1, 5])
def test_other_shifts_take_the_two_step_form(shift):
    rng = np.random.default_rng(2000 + shift)
    for mult in (1 << 30, 1099511680, (1 << 31) - 1):
        q = O.raw_quant(zp_out=7, multiplier=mult, shift=shift)
        acc = probe_accumulators(mult, max(1, -shift), rng)
        want = np.array([O.lib.eo_requant(int(a), q) for a in acc], np.uint8)
        got, single = eden.requant_apply(to_eh(q), acc)
        assert not single
        assert np.array_equal(got, want)


@pytest.mark.parametrize("rs", [1, 2, 3, 7, 8, 11, 16, 20])
def test_per_channel_single_shift_forms_equal_oracle(rs):
    """The two per-channel forms (rounding term from the shift in registers; from a table, for rs >= 2), with and
    without the sign test (clamp floor below / at the output zero point)."""
    rng = np.random.default_rng(3000 + rs)
    for mult in MULTIPLIERS:
        for zp_out, lo, hi in ((0, 0, 255), (128, 0, 255), (255, 20, 230), (3, 3, 3), (131, 131, 255), (5, 9, 255)):
            q = O.raw_quant(zp_out=zp_out, multiplier=mult, shift=-rs, act_min=lo, act_max=hi)
            acc = probe_accumulators(mult, rs, rng)
            want = np.array([O.lib.eo_requant(int(a), q) for a in acc], np.uint8)
            for form in ("registers", "table"):
                if form == "table" and rs < 2:
                    with pytest.raises(eden.EdenHipError):
                        eden.requant_apply(to_eh(q), acc, channel_form=form)
                    continue
                got, single = eden.requant_apply(to_eh(q), acc, channel_form=form)
                bad = np.nonzero(got != want)[0]
                assert single and bad.size == 0, (form, mult, rs, zp_out, acc[bad[:5]], got[bad[:5]], want[bad[:5]])


def test_per_channel_forms_refuse_shifts_outside_their_range():
    acc = np.arange(-5, 5, dtype=np.int32)
    for shift in (-21, 0, 1):
        q = O.raw_quant(zp_out=7, multiplier=1 << 30, shift=shift)
        for form in ("registers", "table"):
            with pytest.raises(eden.EdenHipError):
                eden.requant_apply(to_eh(q), acc, channel_form=form)
