"""Host-side counterpart of the reference's utils_functional.py for the SC hot path.

Same names and argument meaning as the reference (quantize / QuantizeGrad :93-123, the
autograd wrappers :468-587, compute_bias_std_coef :900-949, conv2d_generic :1083-1317), live
branches only, calling the drop-in extension modules of this package.  What "backward" means
is unchanged: autograd runs through a float surrogate (F.conv2d on the positive / negative
weight parts followed by the OR-n closed form); the integer SC result only replaces the
surrogate's forward values.
"""
import math
import os

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F

import _ops
import fixed_extension_cuda
import sc_extension_cuda

prec_default = 7      # utils_functional.py:31
LFSR_Length = -1      # :44  always the maximal-length LFSR of the stream length
XNOR = True           # :45  passed through; the op follows the CPU extension and ignores it
MUX = False           # :46
Use_Approx = False    # config.py


# ---- small helpers (utils_functional.py:52-91) ----------------------------------------------
def setattr_default(obj, kwargs, att_string, default_value):
    if att_string in kwargs:
        setattr(obj, att_string, kwargs.pop(att_string))
    else:
        setattr(obj, att_string, default_value)


def setdict_default(d, kwargs, att_string, default_value):
    d[att_string] = kwargs.pop(att_string) if att_string in kwargs else default_value


def setvalue_default(kwargs, att_string, default_value):
    return kwargs.pop(att_string) if att_string in kwargs else default_value


def update_sync(model, sync=1):
    for mod in model.modules():
        if isinstance(mod, (nn.Conv2d, nn.Linear)) and hasattr(mod, "run_args"):
            mod.run_args["sync"] = sync


def quantize(input, prec=8):
    """(x * 2^prec).round().clamp(+-(2^prec - 1)) / 2^prec  (utils_functional.py:93-104, prune = 0)."""
    if prec <= 16:
        if (input.is_cuda and prec >= 0 and not torch.is_grad_enabled()
                and (input.dtype == torch.float32 or (input.dtype == torch.float16 and prec <= 10))
                and (input.is_contiguous() or (input.dim() == 4
                                               and input.is_contiguous(memory_format=torch.channels_last)))):
            return _ops.quantize(input, prec)  # the same four passes as one kernel
        prec_2 = 2 ** prec
        return (input * prec_2).round().clamp(-prec_2 + 1, prec_2 - 1) / prec_2
    return input.clamp(-1, 1)


class QuantizeGrad(torch.autograd.Function):
    """Quantise forward, straight-through backward (utils_functional.py:117-123)."""

    @staticmethod
    def forward(ctx, x, prec):
        return quantize(x, prec=prec)

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, None


# ---- OR-n activation and error injection -------------------------------------------------------
def _orn_torch_forward(s, n):
    # utils_functional.py:476-482 (n > 4: no fused kernel)
    e = torch.exp(-s)
    out = n
    for i in range(n):
        out = out - (n - i) * (s ** i) * (1 / math.factorial(i)) * e
    return out


def _orn_torch_backward(g, s, n):
    # utils_functional.py:491-495
    e = torch.exp(-s)
    gi = 0
    for i in range(n):
        gi = gi + (1 / math.factorial(i)) * (s ** i) * e
    return gi * g


class Or_Approx_n_Grad(torch.autograd.Function):
    """y = OR_n(sum); only `sum` is saved (utils_functional.py:468-495)."""

    @staticmethod
    def forward(ctx, sum, n):
        ctx.n = n
        ctx.save_for_backward(sum)
        if n <= 4:
            return sc_extension_cuda.or_approx_n_forward_acc(sum, n)
        return _orn_torch_forward(sum, n)

    @staticmethod
    def backward(ctx, grad_output):
        n = ctx.n
        sum, = ctx.saved_tensors
        if n <= 4:
            return sc_extension_cuda.or_approx_n_backward_acc(grad_output, sum, n), None
        return _orn_torch_backward(grad_output, sum, n), None


class Or_Approx_N_Bias_Correct_Grad_Both(torch.autograd.Function):
    """Fused OR_n + bias/noise injection on both polarities and their difference
    (utils_functional.py:559-575)."""

    @staticmethod
    def forward(ctx, sum_pos, sum_neg, n, bias_coef, std_coef, order):
        ctx.n = n
        ctx.order = order
        ctx.save_for_backward(sum_pos, sum_neg, bias_coef)
        return sc_extension_cuda.or_approx_n_forward_bias_std_both_acc(sum_pos, sum_neg, bias_coef, std_coef, n)

    @staticmethod
    def backward(ctx, grad_output):
        sum_pos, sum_neg, bias_coef = ctx.saved_tensors
        gp, gn = sc_extension_cuda.or_approx_n_backward_bias_std_both_acc(grad_output, sum_pos, sum_neg, bias_coef,
                                                                           ctx.n)
        return gp, gn, None, None, None, None


def _poly5(c, x):
    return c[0] + c[1] * x + c[2] * x ** 2 + c[3] * x ** 3 + c[4] * x ** 4 + c[5] * x ** 5


class Bias_Correct_Grad(torch.autograd.Function):
    """x + poly_bias(x) + poly_std(x) * N(0,1) (utils_functional.py:441-459, 577-587).  Used only at
    calibration steps, so it stays on plain torch ops."""

    @staticmethod
    def forward(ctx, x, bias_coef, std_coef, order):
        ctx.order = order
        ctx.save_for_backward(x, bias_coef)
        x_with_rand = x + _poly5(std_coef, x) * torch.randn_like(x)
        return x_with_rand + _poly5(bias_coef, x)

    @staticmethod
    def backward(ctx, grad_output):
        x, b = ctx.saved_tensors
        x_dot = 1 + b[1] + b[2] * 2 * x + b[3] * 3 * x ** 2 + b[4] * 4 * x ** 3 + b[5] * 5 * x ** 4
        return x_dot * grad_output, None, None, None


def or_approx_no(sum, n):
    """OR-n keeping only the n-th bit (utils_functional.py:590-598)."""
    e = torch.exp(-sum)
    out = 1
    for i in range(n):
        out = out - (sum ** i) * (1 / math.factorial(i)) * e
    return out


def or_approx_2_1(sum, n):
    return (sum / n) ** n + ((sum / n) ** (n - 1)) * (1 - sum / n) * n


def or_approx_2_4(sum, n):
    return 1 - torch.exp(-sum) + (sum / n) ** n


# ---- calibration -----------------------------------------------------------------------------
CALIB_WINDOWS = 30
CALIB_WIDTH = 0.1


def compute_bias_std_coef(or_n, a_bit, a_act, order):
    """Fit the bias / std polynomials of the SC error (utils_functional.py:900-949).

    Windows [s, s+0.1) with s on linspace(0, max(a_bit), 30) are selected on the float surrogate
    a_act; each window with more than one sample contributes the mean and the unbiased std of
    a_bit - a_act.  The reference gathers every window with a boolean mask (60 passes over the
    tensors); here one kernel accumulates count / sum / sum of squares for all windows and the
    two 30 x (order+1) least-squares problems are solved on the host in float64.
    """
    if int(os.environ.get("Weight_Prec", "-1")) > 0:
        or_n = 1
    dev = a_bit.device
    if or_n < 0:
        return torch.zeros(order + 1, device=dev), torch.zeros(order + 1, device=dev)
    output_range = np.linspace(0, a_bit.max().item(), CALIB_WINDOWS)
    lo = [np.float32(s) for s in output_range]
    hi = [np.float32(s + CALIB_WIDTH) for s in output_range]
    stats = _ops.calib_stats(a_bit.reshape(-1), a_act.reshape(-1), lo, hi).cpu().numpy()
    cnt, s1, s2 = stats[:, 0], stats[:, 1], stats[:, 2]
    valid = np.nonzero(cnt > 1)[0]
    n = cnt[valid]
    mean = s1[valid] / n
    var = np.maximum(s2[valid] - s1[valid] * s1[valid] / n, 0.0) / (n - 1)
    bias_bins = mean.astype(np.float32)
    std_bins = np.sqrt(var).astype(np.float32)
    pos = output_range[valid]
    A = np.stack([pos ** i for i in range(order + 1)], axis=1).astype(np.float32).astype(np.float64)
    if order >= len(valid) // 5:
        bias_coef = np.zeros(order + 1, np.float32)
    else:
        bias_coef = np.linalg.lstsq(A, bias_bins.astype(np.float64), rcond=None)[0].astype(np.float32)
    if len(valid) == 0:
        std_coef = np.zeros(order + 1, np.float32)
    else:
        std_coef = np.linalg.lstsq(A, std_bins.astype(np.float64), rcond=None)[0].astype(np.float32)
    return torch.from_numpy(bias_coef).to(dev), torch.from_numpy(std_coef).to(dev)


# ---- merged surrogate ---------------------------------------------------------------------------
def _autocast_dtype():
    """The reduced-precision dtype of an active CUDA autocast region (the reference's half / bfloat16 training,
    utils_own.py:76-80,127-129), else None."""
    return torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled() else None


def merged_surrogate_sums(activation, weight, pad_hw, stride, keep_half=False):
    """One convolution with the 2*O filters [w_pos ; w_neg], written in the activation's memory order (no
    conversion pass inside the convolution): -> (w2, s2, outer, inner, channels_last, xa) with s2 laid out
    [outer][2][inner] in float32.  Inside an autocast region the convolution runs in the region's dtype, as the
    reference's two convolutions do there: w2 and xa (the activation as the convolution took it) are then of that
    dtype, and s2 holds the reduced-precision sums widened to float32 -- or, with keep_half in a float16 region, as
    they are (for the backward kernel that reads and writes float16)."""
    lowp = _autocast_dtype()
    with torch.no_grad():
        w2 = _ops.split_weight(weight, channels_last=_ops.is_channels_last(activation))
        xa = activation.detach()
        if lowp is not None:
            w2 = w2.to(lowp)
            xa = xa.to(lowp)
        with torch.autocast("cuda", enabled=False):
            s2, outer, inner, cl = _ops.pair_layout(F.conv2d(xa, w2, padding=pad_hw, stride=stride),
                                                    keep_half=keep_half and lowp == torch.float16)
    return w2, s2, outer, inner, cl, xa


class Merged_Surrogate_Conv(torch.autograd.Function):
    """The float surrogate of conv2d_generic for forward = 'or_n' (n <= 4) / 'full_or' with its two
    convolutions merged: one conv with the 2*O filters [clamp(w, 0, 100) ; -clamp(w, -100, 0)]
    (utils_functional.py:1204-1211), the OR-n / error-injection kernels reading both halves of its
    output in place, one backward conv pair for both polarities.

    sync = 1: the forward value is the SC result `sc_value` (= pos / L - neg / L, the tensor the
    reference writes into `.data`, :1273-1274) and the OR-n forward is never evaluated;
    sync = 3: the forward value is the fused OR-n + bias/noise kernel's (:1253-1254);
    sync = 2: the caller has fitted the bias / std polynomials to SC result - OR_n(sum) on the sums it
    passes in (`sums`, :1275-1283); the forward value is Bias_Correct(OR_n(sum_pos)) -
    Bias_Correct(OR_n(sum_neg)) with those coefficients (:1284-1285), which is what the sync-3 kernel computes.
    Gradients are those of OR_n(conv(x, w_pos)) - OR_n(conv(x, w_neg)) (sync 2, 3: with the bias
    polynomial's derivative), evaluated on the saved sums rounded to binary16 as the reference's
    backward wrappers do.  Inside an autocast region the forward and backward convolutions run in the region's
    dtype; the pointwise kernels stay in float32 on the widened sums and the value is float32 (the caller casts)."""

    @staticmethod
    def forward(ctx, activation, weight, sc_value, bias_coef, std_coef, or_n, pad_hw, stride, sync, sums):
        if sums is None:
            # sync 1 never evaluates the forward kernels on the sums: they can stay in the convolution's float16
            sums = merged_surrogate_sums(activation, weight, pad_hw, stride, keep_half=(sync == 1))
        w2, s2, outer, inner, cl, xa = sums
        ctx.geom = (outer, inner, cl, or_n, tuple(pad_hw), tuple(stride), sync, activation.dtype)
        if sync >= 2:
            ctx.save_for_backward(xa, weight, w2, s2, bias_coef)
            return _ops.orn_bias_std_pair_forward(s2, outer, inner, cl, bias_coef, std_coef, or_n)
        ctx.save_for_backward(xa, weight, w2, s2)
        return sc_value

    @staticmethod
    def backward(ctx, grad_output):
        outer, inner, cl, or_n, pad_hw, stride, sync, x_dtype = ctx.geom
        if sync >= 2:
            xa, weight, w2, s2, bias_coef = ctx.saved_tensors
            g2 = _ops.orn_bias_std_pair_backward(grad_output, s2, outer, inner, cl, bias_coef, or_n)
        else:
            xa, weight, w2, s2 = ctx.saved_tensors
            g2 = _ops.orn_pair_backward(grad_output, s2, outer, inner, cl, or_n)
        need_x, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        dx = dw = None
        if need_x or need_w:
            if g2.dtype != w2.dtype:  # autocast region: the backward convolutions run in its dtype as well
                g2 = g2.to(w2.dtype)
            dx, dw2, _ = torch.ops.aten.convolution_backward(g2, xa, w2, None, stride, pad_hw, (1, 1), False,
                                                             (0, 0), 1, (need_x, need_w, False))
            if need_x and dx.dtype != x_dtype:
                dx = dx.to(x_dtype)
            if need_w:
                dw = _ops.merge_weight_grad(dw2, weight).to(weight.dtype)
        return dx, dw, None, None, None, None, None, None, None, None


class Merged_Surrogate_Linear(torch.autograd.Function):
    """The same for the linear op: one GEMM with the 2*O rows [w_pos ; w_neg]; the forward value is the
    SC result, the gradient that of OR_n(x w_pos^T) - OR_n(x w_neg^T) on the binary16-rounded sums."""

    @staticmethod
    def forward(ctx, activation, weight, sc_value, or_n):
        w2 = _ops.split_weight(weight)
        s2, outer, inner, _ = _ops.pair_layout(F.linear(activation, w2))
        ctx.geom = (outer, inner, or_n)
        ctx.save_for_backward(activation, w2, weight, s2)
        return sc_value

    @staticmethod
    def backward(ctx, grad_output):
        outer, inner, or_n = ctx.geom
        activation, w2, weight, s2 = ctx.saved_tensors
        g2 = _ops.orn_pair_backward(grad_output, s2, outer, inner, False, or_n)
        dx = g2 @ w2 if ctx.needs_input_grad[0] else None
        dw = _ops.merge_weight_grad(g2.t() @ activation, weight).to(weight.dtype) if ctx.needs_input_grad[1] else None
        return dx, dw, None, None


_side_streams = {}


def _side_stream(device):
    """Second stream (default priority) of a device for the SC forward, or None when overlap is
    switched off (REXSC_OVERLAP_SURROGATE=0) or the caller's stream is being captured."""
    if os.environ.get("REXSC_OVERLAP_SURROGATE", "1") == "0" or torch.cuda.is_current_stream_capturing():
        return None
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if idx not in _side_streams:
        _side_streams[idx] = torch.cuda.Stream(device=idx)
    return _side_streams[idx]


def _merged_surrogate_ok(activation, weight, forward, or_n, sync, sc_on, split_output, stride, pad_hw):
    """Whether conv2d_generic may take the merged path: float32 operands on the GPU (inside a float16 / bfloat16
    autocast region the activation may also be of the region's dtype), OR-n with a fused kernel, a plain forward
    value (no split output), and an output shape with a whole number of float4 vectors per polarity block.
    REXSC_MERGED_SURROGATE=0 switches it off."""
    if os.environ.get("REXSC_MERGED_SURROGATE", "1") == "0" or split_output:
        return False
    lowp = _autocast_dtype()
    if lowp is not None and lowp not in (torch.float16, torch.bfloat16):
        return False
    if not (activation.is_cuda and weight.is_cuda) or weight.dtype != torch.float32:
        return False
    if activation.dtype != torch.float32 and activation.dtype != lowp:
        return False
    if sync == 1:
        if not sc_on or not (forward in ("full_or", "and_2") or (forward[:3] == "or_" and len(forward) == 4)):
            return False
    elif sync == 3:
        if not (forward[:3] == "or_" and len(forward) == 4):
            return False
    elif sync == 2:
        if not sc_on or not (forward[:3] == "or_" and len(forward) == 4):
            return False
    else:
        return False
    n = 1 if forward in ("full_or", "and_2") else or_n
    if not 1 <= n <= 4:
        return False
    O, _, KH, KW = weight.shape
    Ho = (activation.size(2) + 2 * pad_hw[0] - KH) // stride[0] + 1
    Wo = (activation.size(3) + 2 * pad_hw[1] - KW) // stride[1] + 1
    return O % 4 == 0 or (O * Ho * Wo) % 4 == 0


# ---- generic SC layers ------------------------------------------------------------------------
def _parse_forward(forward, generator):
    """forward / generator strings -> (or_n, bin_config, gen_config) (utils_functional.py:1160-1178)."""
    or_n, bin_config = -1, None
    if forward[:3] == "or_":
        if len(forward) == 4:
            or_n = int(forward[-1]); bin_config = or_n - 1
        elif len(forward) == 5:
            or_n = int(forward[3]); bin_config = -or_n + 1
        elif len(forward) == 6:
            or_n = int(forward[-1]); bin_config = or_n
    elif forward == "full_or":
        bin_config = 0
    elif forward == "full_bin":
        bin_config = 51200
    gen_config = None
    if generator in ("lfsr", "lfsr_mult", "lfsr_split"):
        gen_config = 1
    elif generator[:4] == "and_":
        gen_config = int(generator[-1])
    return or_n, bin_config, gen_config


def conv2d_generic(activation, weight, padding, stride, **kwargs):
    """Generic SC conv2d (utils_functional.py:1083-1317).

    sync = 1: SC forward (integer kernels) over the OR-n float surrogate;
    sync = 2: as 1, plus calibration of the bias/std polynomials (returns them as well);
    sync = 3: no SC kernels, fused OR-n + bias/noise error injection on the surrogate;
    sync = 0: surrogate only.
    padding[0] pads the last axis and padding[1] axis 2, as the reference's F.pad call does.
    """
    bit_length = setvalue_default(kwargs, "bit_length", 128)
    generator = setvalue_default(kwargs, "generator", None)
    forward = setvalue_default(kwargs, "forward", "full_or")
    load_unit = setvalue_default(kwargs, "load_unit", 8)
    load_wait_w = setvalue_default(kwargs, "load_wait_w", 1)
    split_output = setvalue_default(kwargs, "split_output", False)
    order = setvalue_default(kwargs, "order", 10)
    z_unit = setvalue_default(kwargs, "z_unit", 16)
    bias_coef = setvalue_default(kwargs, "bias_coef", None)
    std_coef = setvalue_default(kwargs, "std_coef", None)
    sync_override = setvalue_default(kwargs, "sync", 1)
    if bias_coef is None:
        bias_coef = torch.zeros(order + 1, device=activation.device)
    if std_coef is None:
        std_coef = torch.zeros(order + 1, device=activation.device)
    if generator is None:
        raise ValueError("conv2d_generic: a generator must be given ('lfsr', 'and_2', 'fixed')")

    dtype = torch.float16 if torch.is_autocast_enabled() else activation.dtype
    pad_hw = (int(padding[1]), int(padding[0]))  # (axis 2, axis 3) for F.conv2d
    or_n, bin_config, gen_config = _parse_forward(forward, generator)
    global_sync = os.environ.get("Global_Sync", "1") == "1"
    sc_on = global_sync and (not Use_Approx) and 0 < sync_override < 3

    stride = (int(stride[0]), int(stride[1]))
    has_sc_kernel = bin_config is not None and gen_config is not None
    if (sync_override == 3 or has_sc_kernel) and _merged_surrogate_ok(
            activation, weight, forward, or_n, sync_override, sc_on, split_output, stride, pad_hw):
        n = 1 if forward in ("full_or", "and_2") else or_n
        # the kernels' value is float32; inside an autocast region the reference returns float16 (:1148-1150)
        as_dtype = lambda t: t if t.dtype == dtype else t.to(dtype)
        if sync_override == 3:
            return as_dtype(Merged_Surrogate_Conv.apply(activation, weight, None, bias_coef, std_coef, n, pad_hw, stride,
                                                        3, None))
        if sync_override == 2:
            with torch.no_grad():
                pos, neg = sc_extension_cuda.conv2d_generic_general_split_acc(
                    activation.data, weight.data, bit_length, LFSR_Length, z_unit, padding, stride,
                    (prec_default, load_unit, load_wait_w), bin_config, gen_config, XNOR, MUX)
                sums = merged_surrogate_sums(activation, weight, pad_hw, stride)
                _, s2, outer, inner, cl, _ = sums
                # calibration: a_act = OR_n of both sums (one pass over the pair tensor), a_bit = the SC
                # results in the same element order
                a_act = _ops.storage_flat(_ops.orn_forward(s2, n), cl)
                a_bit = _ops.sc_counts_pair(pos, neg, bit_length, outer, inner, cl).reshape(-1)
                bias_new, std_new = compute_bias_std_coef(or_n, a_bit, a_act, order)
                bias_coef[:bias_new.size(0)] = bias_new
                std_coef[:std_new.size(0)] = std_new
            out = Merged_Surrogate_Conv.apply(activation, weight, None, bias_coef, std_coef, n, pad_hw, stride, 2, sums)
            return as_dtype(out), bias_coef, std_coef

        def sc_forward():
            # pos / L - neg / L (:1181-1182, 1273-1274, 1317) comes out of the kernel that produces the sums
            with torch.no_grad():
                return _ops.sc_conv2d(activation.data, weight.data, bit_length, LFSR_Length, padding, stride,
                                      (prec_default, load_unit, load_wait_w), bin_config, gen_config, want_split=False,
                                      xnor=_ops.honour_xnor(XNOR), want_value=True)[3]

        if not (torch.is_grad_enabled() and (activation.requires_grad or weight.requires_grad)):
            return as_dtype(sc_forward())  # inference: the surrogate only ever supplies gradients
        # The integer kernels (VALU-bound) and the surrogate's float convolution (matrix cores) are
        # independent: the SC forward runs on a second stream of default priority and the two overlap.
        side = _side_stream(activation.device)
        # (the value is cast where it is produced, so that the Function's output -- and with it the gradient that
        # comes back -- has the region's dtype without a cast node of autograd's in between)
        if side is None:
            return Merged_Surrogate_Conv.apply(activation, weight, as_dtype(sc_forward()), bias_coef, std_coef, n, pad_hw,
                                               stride, 1, None)
        cur = torch.cuda.current_stream(activation.device)
        side.wait_stream(cur)
        with torch.cuda.stream(side):
            sc_value = as_dtype(sc_forward())
        out = Merged_Surrogate_Conv.apply(activation, weight, sc_value, bias_coef, std_coef, n, pad_hw, stride, 1, None)
        cur.wait_stream(side)
        sc_value.record_stream(cur)  # allocated on the side stream, consumed on the caller's
        return out

    result_pos = result_neg = None
    if sc_on:
        with torch.no_grad():
            if bin_config is not None and gen_config is not None:
                result_pos, result_neg = sc_extension_cuda.conv2d_generic_general_split_acc(
                    activation.data, weight.data, bit_length, LFSR_Length, z_unit, padding, stride,
                    (prec_default, load_unit, load_wait_w), bin_config, gen_config, XNOR, MUX)
                result_pos = result_pos.to(dtype=dtype)
                result_neg = result_neg.to(dtype=dtype)
            if generator == "fixed":
                result_pos = fixed_extension_cuda.conv2d_saturate_acc(
                    activation.data, weight.data, 0, int(np.log2(bit_length)), 24, padding, stride).to(dtype=dtype)
                result_neg = torch.zeros_like(result_pos)
                result_pos = result_pos / bit_length
                result_neg = result_neg / bit_length
            if result_pos is None:
                raise ValueError("conv2d_generic: no SC kernel for forward=%r with generator=%r" % (forward, generator))

    w_pos = weight.clamp(0, 100)
    w_neg = -(weight.clamp(-100, 0))
    activation = activation.to(w_pos.dtype)

    if sync_override >= 0:
        if forward in ("full_or", "and_2"):
            result_pos_value = Or_Approx_n_Grad.apply(F.conv2d(activation, w_pos, padding=pad_hw, stride=stride), 1)
            result_neg_value = Or_Approx_n_Grad.apply(F.conv2d(activation, w_neg, padding=pad_hw, stride=stride), 1)
        elif forward[:3] == "or_":
            conv_pos_normal = F.conv2d(activation, w_pos, padding=pad_hw, stride=stride)
            conv_neg_normal = F.conv2d(activation, w_neg, padding=pad_hw, stride=stride)
            if len(forward) == 4:
                if sync_override == 3:
                    return Or_Approx_N_Bias_Correct_Grad_Both.apply(conv_pos_normal, conv_neg_normal, or_n, bias_coef,
                                                                    std_coef, order).to(dtype)
                result_pos_value = Or_Approx_n_Grad.apply(conv_pos_normal, or_n)
                result_neg_value = Or_Approx_n_Grad.apply(conv_neg_normal, or_n)
            elif len(forward) == 5:
                result_pos_value = or_approx_no(conv_pos_normal, or_n)
                result_neg_value = or_approx_no(conv_neg_normal, or_n)
            else:
                k = weight.size(1) * weight.size(2) * weight.size(3)
                fn = or_approx_2_1 if int(forward[-1]) == 1 else or_approx_2_4
                result_pos_value = fn(conv_pos_normal, k)
                result_neg_value = fn(conv_neg_normal, k)
        elif forward == "full_bin":
            result_pos_value = F.conv2d(activation, weight.clamp(-100, 100), padding=pad_hw, stride=stride)
            result_neg_value = torch.zeros_like(result_pos_value)
        else:
            raise ValueError("conv2d_generic: unknown forward %r" % forward)
    else:
        raise ValueError("conv2d_generic: sync must be >= 0")

    if sc_on and sync_override == 1:
        # the SC result replaces the float forward; gradients still flow through the surrogate
        result_pos_value.data = result_pos / bit_length
        result_neg_value.data = result_neg / bit_length
    elif sync_override == 2:
        with torch.no_grad():
            result_bit = torch.cat([(result_pos / bit_length).reshape(-1), (result_neg / bit_length).reshape(-1)])
            result_act = torch.cat([result_pos_value.reshape(-1), result_neg_value.reshape(-1)])
            bias_coef_new, std_coef_new = compute_bias_std_coef(or_n, result_bit, result_act, order)
            bias_coef[:bias_coef_new.size(0)] = bias_coef_new
            std_coef[:std_coef_new.size(0)] = std_coef_new
        result_pos_value = Bias_Correct_Grad.apply(result_pos_value, bias_coef, std_coef, order)
        result_neg_value = Bias_Correct_Grad.apply(result_neg_value, bias_coef, std_coef, order)

    result_pos_value.data = result_pos_value.data.to(dtype)
    result_neg_value.data = result_neg_value.data.to(dtype)
    if split_output:
        return result_pos_value, result_neg_value
    if sync_override == 2:
        return result_pos_value - result_neg_value, bias_coef, std_coef
    return result_pos_value - result_neg_value


def conv2d_sc_inference(activation, weight, padding, stride, prec, weight_prec, weight_stream_cache=None, **kwargs):
    """What the layer's  conv2d_generic(QuantizeGrad(x, prec), QuantizeGrad(w, weight_prec), sync=1)  returns when no
    gradient is wanted (utils_class.py:54-74 under torch.no_grad()): only the integer SC forward runs, the float
    surrogate exists for gradients alone.  From the UNQUANTISED operands: the fake quantisation is applied inside the
    stream generators (no pass over the tensors of its own), the weight streams are kept in weight_stream_cache while
    `weight` does not change, and pos / L - neg / L is written by the kernel that produces the sums.
    Returns None when this shortcut does not cover the configuration (the caller then takes the general path)."""
    bit_length = kwargs.get("bit_length", 128)
    generator = kwargs.get("generator", None)
    forward = kwargs.get("forward", "full_or")
    if generator is None or kwargs.get("split_output", False) or kwargs.get("sync", 1) != 1:
        return None
    if os.environ.get("Global_Sync", "1") != "1" or Use_Approx or torch.is_autocast_enabled():
        return None
    if not (activation.is_cuda and weight.is_cuda and activation.dtype == torch.float32 and weight.dtype == torch.float32):
        return None
    if not (forward in ("full_or", "and_2") or (forward[:3] == "or_" and len(forward) == 4)):
        return None
    if prec is None or weight_prec is None or not (0 <= prec <= 16 and 0 <= weight_prec <= 16):
        return None
    _, bin_config, gen_config = _parse_forward(forward, generator)
    if bin_config is None or gen_config is None:
        return None
    with torch.no_grad():
        return _ops.sc_conv2d(activation, weight, bit_length, LFSR_Length, padding, stride,
                              (prec_default, kwargs.get("load_unit", 8), kwargs.get("load_wait_w", 1)), bin_config,
                              gen_config, want_split=False, xnor=_ops.honour_xnor(XNOR), want_value=True,
                              weight_cache=weight_stream_cache, act_fake_quant=prec,
                              weight_fake_quant=weight_prec)[3]


def linear_generic_sc(activation, weight, **kwargs):
    """SC linear layer on the extension's semantics (sc_matmul.cpp:576-676): integer SC forward over
    the float surrogate OR_n(x w_pos^T) - OR_n(x w_neg^T).  (The reference's own `linear_generic`
    is a legacy pure-torch simulation with different seeds and never calls the extension.)"""
    bit_length = setvalue_default(kwargs, "bit_length", 128)
    forward = setvalue_default(kwargs, "forward", "or_2")
    generator = setvalue_default(kwargs, "generator", "lfsr")
    load_unit = setvalue_default(kwargs, "load_unit", 8)
    load_wait_w = setvalue_default(kwargs, "load_wait_w", 1)
    sync_override = setvalue_default(kwargs, "sync", 1)
    or_n, bin_config, gen_config = _parse_forward(forward, generator)
    if bin_config is None or gen_config is None:
        raise ValueError("linear_generic_sc: unsupported forward=%r / generator=%r" % (forward, generator))
    merged = (os.environ.get("REXSC_MERGED_SURROGATE", "1") != "0" and sync_override == 1 and forward != "full_bin"
              and 1 <= (or_n if or_n > 0 else 1) <= 4 and activation.is_cuda and activation.dim() == 2
              and activation.dtype == torch.float32 and weight.dtype == torch.float32
              and not torch.is_autocast_enabled() and weight.size(0) % 4 == 0)
    if merged:
        with torch.no_grad():
            pos, neg = sc_extension_cuda.linear_generic_general_acc(
                activation.data, weight.data, (prec_default, load_unit, load_wait_w), bit_length, LFSR_Length,
                bin_config, gen_config, XNOR, MUX)
            sc_value = _ops.sc_counts_to_float(pos, neg, bit_length)
        if not (torch.is_grad_enabled() and (activation.requires_grad or weight.requires_grad)):
            return sc_value
        return Merged_Surrogate_Linear.apply(activation, weight, sc_value, or_n if or_n > 0 else 1)
    w_pos = weight.clamp(0, 100)
    w_neg = -(weight.clamp(-100, 0))
    lin_pos = F.linear(activation, w_pos)
    lin_neg = F.linear(activation, w_neg)
    if forward == "full_bin":
        pos_value, neg_value = lin_pos, lin_neg
    else:
        n = or_n if or_n > 0 else 1
        pos_value = Or_Approx_n_Grad.apply(lin_pos, n)
        neg_value = Or_Approx_n_Grad.apply(lin_neg, n)
    if sync_override == 1:
        with torch.no_grad():
            pos, neg = sc_extension_cuda.linear_generic_general_acc(
                activation.data, weight.data, (prec_default, load_unit, load_wait_w), bit_length, LFSR_Length,
                bin_config, gen_config, XNOR, MUX)
        pos_value.data = pos.to(activation.dtype) / bit_length
        neg_value.data = neg.to(activation.dtype) / bit_length
    return pos_value - neg_value


def linear_sc_inference(activation, weight, prec, weight_stream_cache=None, **kwargs):
    """Forward value of Linear_Or's default path without autograd: the SC linear op on the fake-quantised input and
    weights (the quantisation happens inside the stream generators), returned as pos / L - neg / L.  `weight` is the
    layer's unquantised PARAMETER: with a weight_stream_cache its bitstreams are kept between calls and regenerated
    on the device only when its values have changed."""
    bit_length = setvalue_default(kwargs, "bit_length", 128)
    forward = setvalue_default(kwargs, "forward", "or_2")
    generator = setvalue_default(kwargs, "generator", "lfsr")
    load_unit = setvalue_default(kwargs, "load_unit", 8)
    load_wait_w = setvalue_default(kwargs, "load_wait_w", 1)
    setvalue_default(kwargs, "sync", 1)
    or_n, bin_config, gen_config = _parse_forward(forward, generator)
    if bin_config is None or gen_config is None:
        raise ValueError("linear_sc_inference: unsupported forward=%r / generator=%r" % (forward, generator))
    with torch.no_grad():
        if not 0 <= prec <= 16:  # outside what the generators fold: quantise in passes of their own
            activation, weight, prec = quantize(activation, prec=prec), quantize(weight, prec=prec), None
        pos, neg = _ops.sc_linear(activation, weight, (prec_default, load_unit, load_wait_w), bit_length, LFSR_Length,
                                  bin_config, gen_config, weight_cache=weight_stream_cache, act_fake_quant=prec,
                                  weight_fake_quant=prec)
        # int16 like the CUDA op's outputs (sc_cuda.cpp:101-120), which linear_generic_sc also goes through
        return _ops.sc_counts_to_float(pos.to(torch.int16), neg.to(torch.int16), bit_length)


def linear_or_approx(activation, weight, true_or=False):
    """Float surrogate of OR accumulation for linear layers (utils_functional.py:600-608)."""
    if true_or:
        return 1 - torch.prod(1 - activation.unsqueeze(1) * weight, dim=-1)
    return 1 - torch.exp(-F.linear(activation, weight))


def linear_generic(activation, weight, **kwargs):
    """The reference's legacy generic linear layer (utils_functional.py:955-1081), which its Linear_Or runs
    (utils_class.py:183-208): a bit-by-bit simulation of the SC product in plain torch ops there, the same
    numbers from the HIP kernels here (rexsc_linear_legacy).

    bit_length, prec (128), share (True), generator, forward ('full_or' | 'full_bin') mean what they mean in the
    reference.  generator 'lfsr' with share=True (one generator per input feature) or share=False (one per weight and
    per activation element, :996-998) is built.  The other two generators have no result to reproduce: 'lfsr_split'
    draws its main streams from torch.randint on every cycle (the test at :1017 sends every generator but 'lfsr' to
    rand_init) and the "true random" generator is torch.randint by design; they raise.  The forward value is the SC result
    (sum over the cycles / bit_length, the simulation's `.mean(0)`), gradients are those of the float surrogate
    1 - exp(-x w_pos^T) - (1 - exp(-x w_neg^T)) ('full_or') or x w^T ('full_bin').  The reference's result tensor
    ends up float16 (its compute_type, :28-29); the values here are the same numbers as float32 -- for 'full_bin'
    after the float16 rounding its `.mean(0)` applies."""
    bit_length = setvalue_default(kwargs, "bit_length", 128)
    prec = setvalue_default(kwargs, "prec", 128)
    share = setvalue_default(kwargs, "share", True)
    generator = setvalue_default(kwargs, "generator", None)
    forward = setvalue_default(kwargs, "forward", "full_or")
    if forward not in ("full_or", "full_bin"):
        raise ValueError("linear_generic: forward must be 'full_or' or 'full_bin' (got %r)" % (forward,))
    if generator != "lfsr":
        raise ValueError("linear_generic: only generator='lfsr' is built; the reference's other generators draw from "
                         "torch.randint and have no reproducible result (got generator=%r)" % (generator,))
    bit_range = prec - 1  # taken before prec follows the stream length (:973, :980-981)
    w_pos = weight.clamp(0, 100)
    w_neg = -(weight.clamp(-100, 0))
    activation = activation.to(w_pos.dtype)
    if forward == "full_or":
        result_pos_value = linear_or_approx(activation, w_pos)
        result_neg_value = linear_or_approx(activation, w_neg)
    else:
        result_pos_value = F.linear(activation, w_pos)
        result_neg_value = F.linear(activation, w_neg)
    if os.environ.get("Global_Sync", "1") == "1":
        with torch.no_grad():
            pos, neg = _ops.sc_linear_legacy(activation.data, weight.data, bit_length, 0 if forward == "full_or" else 51200,
                                             weight_clamp=bit_range, share=bool(share))
            mean = lambda t: (t.to(torch.float32) / bit_length).to(torch.float16).to(result_pos_value.dtype)
            result_pos_value.data = mean(pos)
            result_neg_value.data = mean(neg)
    return result_pos_value - result_neg_value
