"""Drop-in for the reference's CPU-named `fixed_extension` module (torch_c/sc-extension/fixed.cpp:240-242),
served by the HIP kernels (see sc_extension.py for the device handling)."""
import _ops
from sc_extension import _device_for, _to_dev


def conv2d_saturate(input, weight, add_config, precision_in, precision_out, padding, stride):
    dev = _device_for(input, weight)
    x, w = _to_dev(input, dev), _to_dev(weight, dev)
    return _ops.fixed_conv2d(x, w, add_config, precision_in, precision_out, padding, stride).to(input.device)
