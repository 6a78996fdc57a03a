"""Drop-in for the reference's `sc_extension_cuda` module (torch_c/sc-extension/sc_cuda.cpp:122-132).

Same function names, positional arguments and return conventions; the work runs on the HIP
kernels of librexsc.so.  Arithmetic follows the reference's CPU extension, which the
bit-exactness contract is defined against: by default `xnor` is accepted and ignored, as
sc_conv.cpp does.  With REXSC_XNOR_MODE=cuda_ref in the environment the conv op honours it the
way the reference's CUDA kernels do (XNOR-feedback LFSR, sc_cuda_conv.cu:28,55-56,139).
"""
import _ops


def conv2d_generic_general_split_acc(input, weight, bit_length, lfsr_length, z_units, padding, stride, prog_load,
                                     bin_config, gen_config, xnor, mux):
    """[pos, neg] int16 [N,O,Ho,Wo]; channels_last iff the input is (sc_cuda.cpp:87-99)."""
    pos, neg, _ = _ops.sc_conv2d(input, weight, bit_length, lfsr_length, padding, stride, prog_load, bin_config,
                                 gen_config, want_split=True, xnor=_ops.honour_xnor(xnor))
    return [pos, neg]


def conv2d_generic_general_acc(input, weight, bit_length, lfsr_length, z_units, padding, stride, prog_load,
                               bin_config, gen_config, xnor, mux):
    """pos - neg, int16 (sc_cuda.cpp:73-85)."""
    _, _, diff = _ops.sc_conv2d(input, weight, bit_length, lfsr_length, padding, stride, prog_load, bin_config,
                                gen_config, want_split=False, want_diff=True, xnor=_ops.honour_xnor(xnor))
    return diff


def linear_generic_general_acc(input, weight, prog_load, bit_length, lfsr_length, bin_config, gen_config, xnor, mux):
    """[pos, neg] int16 [B,O] (sc_cuda.cpp:101-120; the CUDA op's outputs are int16)."""
    pos, neg = _ops.sc_linear(input, weight, prog_load, bit_length, lfsr_length, bin_config, gen_config)
    return [pos.to(dtype=_ops.torch.int16), neg.to(dtype=_ops.torch.int16)]


def or_approx_n_forward_acc(input, or_n):
    """fp32 OR-n activation (sc_cuda_pw.cu:708-746)."""
    return _ops.orn_forward(input, or_n)


def or_approx_n_backward_acc(grad_output, input, or_n):
    """fp32 gradient; the saved sum is rounded to fp16 first (sc_cuda_pw.cu:767-811)."""
    return _ops.orn_backward(grad_output, input, or_n, half_input=True)


def or_approx_n_forward_bias_std_acc(input, bias_coef, std_coef, or_n):
    """Single polarity, fp16 result (sc_cuda_pw.cu:834-861)."""
    return _ops.orn_bias_std_forward_f16(input, bias_coef, std_coef, or_n)


def or_approx_n_backward_bias_std_acc(grad_output, input, bias_coef, or_n):
    """Single polarity (sc_cuda_pw.cu:929-950)."""
    return _ops.orn_bias_std_backward(grad_output, input, bias_coef, or_n, half_input=True)


def or_approx_n_forward_bias_std_both_acc(input_pos, input_neg, bias_coef, std_coef, or_n):
    """Fused OR-n + bias + noise for both polarities and their difference (sc_cuda_pw.cu:863-927)."""
    return _ops.orn_bias_std_both_forward(input_pos, input_neg, bias_coef, std_coef, or_n)


def or_approx_n_backward_bias_std_both_acc(grad_output, input_pos, input_neg, bias_coef, or_n):
    """[grad_pos, grad_neg] (sc_cuda_pw.cu:952-1011)."""
    gp, gn = _ops.orn_bias_std_both_backward(grad_output, input_pos, input_neg, bias_coef, or_n, half_input=True)
    return [gp, gn]
