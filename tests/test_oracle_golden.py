"""CPU oracle against the golden vectors emitted by the reference's compiled CPU extension
(tests/golden/make_golden.py) -- bit-exact."""
import json
import os

import numpy as np
import pytest

import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_data = np.load(os.path.join(ROOT, "tests", "golden", "ref_cpu_ext.npz"), allow_pickle=False)
_meta = json.loads(bytes(_data["meta"]).decode())


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
