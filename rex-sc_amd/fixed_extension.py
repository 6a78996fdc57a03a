"""Drop-in for the reference's CPU-named `fixed_extension` module (torch_c/sc-extension/fixed.cpp:240-242),
served by the HIP kernels (see sc_extension.py for the device handling)."""
import _ops


def conv2d_saturate(input, weight, add_config, precision_in, precision_out, padding, stride):
    x = input if input.is_cuda else input.to("cuda")
    w = weight if weight.is_cuda else weight.to("cuda")
    return _ops.fixed_conv2d(x, w, add_config, precision_in, precision_out, padding, stride).to(input.device)
