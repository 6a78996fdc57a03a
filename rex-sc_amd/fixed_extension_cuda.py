"""Drop-in for the reference's `fixed_extension_cuda` module (torch_c/sc-extension/fixed_cuda.cpp:36-38)."""
import _ops


def conv2d_saturate_acc(input, weight, add_config, precision_in, precision_out, padding, stride):
    """int32 NCHW [N,O,Ho,Wo] = saturating fixed-point conv, positive minus negative part
    (fixed_cuda.cpp:24-34; arithmetic of fixed.cpp:56-238)."""
    return _ops.fixed_conv2d(input, weight, add_config, precision_in, precision_out, padding, stride)
