"""Drop-in for the reference's CPU-named `sc_extension` module (torch_c/sc-extension/sc.cpp:34-37).

The reference imports this module unconditionally (utils_functional.py:17) but computes on
its CUDA twin.  Here both names are served by the same HIP kernels: tensors on the CPU are
moved to the HIP device of the other operand (or the current one), results come back on the caller's device, with the CPU
module's return conventions (conv: pos-neg int16; linear: [pos, neg] int32).
"""
import torch

import _ops


def _device_for(*tensors):
    """The HIP device the op runs on: the one an operand already lives on, else the current one."""
    for t in tensors:
        if t.is_cuda:
            return t.device
    return torch.device("cuda", torch.cuda.current_device())


def _to_dev(t, device):
    return t if t.device == device else t.to(device)


def conv2d_generic_general(input, weight, bit_length, lfsr_length, z_units, padding, stride, prog_load, bin_config,
                           gen_config, xnor, mux):
    dev = _device_for(input, weight)
    _, _, diff = _ops.sc_conv2d(_to_dev(input, dev), _to_dev(weight, dev), bit_length, lfsr_length, padding, stride, prog_load,
                                bin_config, gen_config, want_split=False, want_diff=True)
    return diff.to(input.device)


def linear_generic_general(input, weight, prog_load, bit_length, lfsr_length, bin_config, gen_config, xnor, mux):
    dev = _device_for(input, weight)
    pos, neg = _ops.sc_linear(_to_dev(input, dev), _to_dev(weight, dev), prog_load, bit_length, lfsr_length, bin_config,
                              gen_config)
    return [pos.to(input.device), neg.to(input.device)]
