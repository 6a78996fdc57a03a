"""CPU oracle against the golden vectors emitted by the reference's compiled CPU extension
(tests/golden/make_golden.py) -- bit-exact."""
import json
import os

import numpy as np
import pytest

import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class _Golden:
    """The fixtures written by the reference's compiled CPU extension: hand-picked cases (make_golden.py),
    seeded random configurations (make_golden_random.py) and operands off the quantisation grid
    (make_golden_offgrid.py), as one key space."""

    def __init__(self):
        self.files = [np.load(os.path.join(ROOT, "tests", "golden", f), allow_pickle=False)
                      for f in ("ref_cpu_ext.npz", "ref_cpu_ext_random.npz", "ref_cpu_ext_offgrid.npz")]
        self.meta = {"conv": [], "linear": [], "fixed": []}
        for f in self.files:
            m = json.loads(bytes(f["meta"]).decode())
            for kind in self.meta:
                self.meta[kind] += m[kind]

    def __getitem__(self, key):
        for f in self.files:
            if key in f.files:
                return f[key]
        raise KeyError(key)


_data = _Golden()
_meta = _data.meta


@pytest.mark.parametrize("case", _meta["conv"], ids=lambda c: c["name"])
def test_conv_golden(case):
    x, w, y = (_data["conv/%s/%s" % (case["name"], k)] for k in ("x", "w", "y"))
    got = orc.conv2d_generic_general(
        x, w, case["bit_length"], case["lfsr_length"], 16, case["padding"], case["stride"], case["prog_load"],
        case["bin_config"], case["gen_config"], True, False,
        channels_last_activation=case["channels_last_activation"],
        channels_last_weight=case["channels_last_weight"])
    assert got.dtype == np.int16 and got.shape == y.shape
    assert np.array_equal(got, y)


@pytest.mark.parametrize("case", _meta["linear"], ids=lambda c: c["name"])
def test_linear_golden(case):
    n = case["name"]
    pos, neg = orc.linear_generic_general(_data["linear/%s/x" % n], _data["linear/%s/w" % n], case["prog_load"],
                                          case["bit_length"], case["lfsr_length"], case["bin_config"],
                                          case["gen_config"], True, False)
    assert np.array_equal(pos, _data["linear/%s/pos" % n])
    assert np.array_equal(neg, _data["linear/%s/neg" % n])


@pytest.mark.parametrize("case", _meta["fixed"], ids=lambda c: c["name"])
def test_fixed_golden(case):
    n = case["name"]
    got = orc.conv2d_saturate(_data["fixed/%s/x" % n], _data["fixed/%s/w" % n], case["add_config"],
                              case["precision_in"], case["precision_out"], case["padding"], case["stride"])
    assert np.array_equal(got, _data["fixed/%s/y" % n])


def _calib_cases():
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_calib.npz"))
    return g, [c.split(",") for c in g["cases"]]


def _poly_values(coef, xs):
    return sum(float(coef[i]) * xs ** i for i in range(len(coef)))


def check_calib_against_reference(fit):
    """fit(or_n, a_bit, a_act, order) -> (bias_coef, std_coef) against the vectors written by the
    reference's own compute_bias_std_coef (tests/golden/make_golden_calib.py).  The reference solves
    its least-squares problems in float32, which leaves the coefficients of the ill-conditioned
    power basis loose in the sixth digit; what is compared is the fitted polynomial over the
    calibrated range, to 2e-5 of its magnitude."""
    g, cases = _calib_cases()
    for name, or_n, order in cases:
        bit, act = g[name + "_bit"], g[name + "_act"]
        b, s = fit(int(or_n), bit, act, int(order))
        b, s = np.asarray(b, np.float64), np.asarray(s, np.float64)
        assert b.shape == g[name + "_bias"].shape and s.shape == g[name + "_std"].shape
        xs = np.linspace(0, float(bit.max()), 64)
        for mine, ref in ((b, g[name + "_bias"]), (s, g[name + "_std"])):
            want = _poly_values(ref, xs)
            assert np.abs(_poly_values(mine, xs) - want).max() <= 2e-5 * np.abs(want).max() + 1e-7, name
        # the suppression rule zeroes the bias fit exactly
        if not g[name + "_bias"].any():
            assert not b.any(), name


def test_calibration_fit_matches_reference_python():
    check_calib_against_reference(orc.compute_bias_std_coef)


def _legacy_linear_cases():
    g = np.load(os.path.join(ROOT, "tests", "golden", "ref_linear_legacy.npz"), allow_pickle=False)
    return g, json.loads(bytes(g["meta"]).decode())


@pytest.mark.parametrize("case", _legacy_linear_cases()[1], ids=lambda c: c["name"])
def test_legacy_linear_generic_matches_reference_python(case):
    """oracle.linear_generic_legacy against the vectors written by the reference's own linear_generic."""
    g, _ = _legacy_linear_cases()
    n = case["name"]
    got = orc.linear_generic_legacy(g[n + "/x"], g[n + "/w"], case["bit_length"], case["forward"],
                                    share=case.get("share", True))
    assert np.abs(g[n + "/y"]).max() > 0
    assert np.array_equal(got, g[n + "/y"])
