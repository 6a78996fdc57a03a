"""The CPU-named drop-in modules (sc_extension, fixed_extension: sc.cpp:34-37, fixed.cpp:240-242) called the
way the reference's CPU extension is called -- CPU tensors in, CPU tensors out -- on every golden case
written by the reference's compiled CPU extension: same values, dtype, device and memory order."""
import numpy as np
import pytest
import torch

from test_gpu_sc_parity import _data, _meta

pytestmark = pytest.mark.gpu


def _cpu(a, channels_last=False):
    t = torch.from_numpy(np.ascontiguousarray(a))
    return t.contiguous(memory_format=torch.channels_last) if channels_last else t


@pytest.mark.parametrize("case", _meta["conv"], ids=lambda c: c["name"])
def test_sc_extension_conv_cpu_tensors(case):
    import sc_extension
    x, w, y = (_data["conv/%s/%s" % (case["name"], k)] for k in ("x", "w", "y"))
    print("sc_extension conv", case["name"], flush=True)
    xt, wt = _cpu(x, case["channels_last_activation"]), _cpu(w, case["channels_last_weight"])
    out = sc_extension.conv2d_generic_general(xt, wt, case["bit_length"], case["lfsr_length"], 16, tuple(case["padding"]),
                                              tuple(case["stride"]), tuple(case["prog_load"]), case["bin_config"],
                                              case["gen_config"], True, False)
    assert out.device.type == "cpu" and out.dtype == torch.int16 and tuple(out.shape) == y.shape
    st = xt.stride()  # the reference's own layout test (sc_conv.cpp:326-331): a one-channel tensor is never channels-last
    if st[1] == 1 and st[1] * st[2] * st[3] != 1:
        assert out.permute(0, 2, 3, 1).is_contiguous()
    else:
        assert out.is_contiguous()
    assert np.array_equal(out.numpy(), y)


@pytest.mark.parametrize("case", _meta["linear"], ids=lambda c: c["name"])
def test_sc_extension_linear_cpu_tensors(case):
    import sc_extension
    n = case["name"]
    print("sc_extension linear", n, flush=True)
    pos, neg = sc_extension.linear_generic_general(_cpu(_data["linear/%s/x" % n]), _cpu(_data["linear/%s/w" % n]),
                                                   tuple(case["prog_load"]), case["bit_length"], case["lfsr_length"],
                                                   case["bin_config"], case["gen_config"], True, False)
    for t, key in ((pos, "pos"), (neg, "neg")):
        assert t.device.type == "cpu" and t.dtype == torch.int32 and t.is_contiguous()
        assert np.array_equal(t.numpy(), _data["linear/%s/%s" % (n, key)])


@pytest.mark.parametrize("case", _meta["fixed"], ids=lambda c: c["name"])
def test_fixed_extension_cpu_tensors(case):
    import fixed_extension
    n = case["name"]
    print("fixed_extension", n, flush=True)
    out = fixed_extension.conv2d_saturate(_cpu(_data["fixed/%s/x" % n]), _cpu(_data["fixed/%s/w" % n]), case["add_config"],
                                          case["precision_in"], case["precision_out"], tuple(case["padding"]),
                                          tuple(case["stride"]))
    assert out.device.type == "cpu" and out.dtype == torch.int32 and out.is_contiguous()
    assert np.array_equal(out.numpy(), _data["fixed/%s/y" % n])
