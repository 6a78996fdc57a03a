"""ctypes/numpy front end of the CPU oracle (TEST INFRASTRUCTURE, not product code).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this module.
The functions take the same arguments as the reference's CPU extension entry points
(sc_extension.conv2d_generic_general, sc_extension.linear_generic_general,
fixed_extension.conv2d_saturate: torch_c/sc-extension/sc.cpp:34-37, fixed.cpp:240-242),
with numpy arrays in place of tensors, so a parity test reads like a call of the reference.

compute_bias_std_coef restates utils_functional.py:900-949 in numpy (float64 statistics
are NOT used: the reference works in float32 tensors, and so does this).

Pinning: the conv / linear / fixed-conv functions against tests/golden/ref_cpu_ext.npz (hand-picked
cases) and ref_cpu_ext_random.npz (96 seeded random configurations), both written by the
reference's compiled CPU extension; compute_bias_std_coef against tests/golden/ref_calib.npz
(written by the reference's own Python function); linear_generic_legacy against tests/golden/ref_linear_legacy.npz
(likewise); the scalar float functions (OR-n, bias/noise,
quantise) against closed forms in tests/test_oracle_invariants.py.

Parity unpinned: the linear op with an 8-bit LFSR (256-bit streams or lfsr_length 8).  The
reference has no defined result there: built with AVX-512 it calls an uninitialised step-function
pointer (sc_matmul.cpp:48-70 has no case for 8 bits) and faults; built without AVX-512 its linear
op returns different numbers on repeated calls with the same operands.  The oracle continues the
7-bit rules with the 8-bit step function that the conv op is pinned on.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# REXSC_ORACLE_SO: another build of the same source (the sanitizer build of tests/test_oracle_sanitizers.py)
_SO = os.environ.get("REXSC_ORACLE_SO") or os.path.join(_HERE, "_build", "librexsc_oracle.so")
_lib = None

_i32p = ctypes.POINTER(ctypes.c_int32)
_i16p = ctypes.POINTER(ctypes.c_int16)
_f32p = ctypes.POINTER(ctypes.c_float)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            raise RuntimeError("oracle library missing: run `python oracle/build.py` "
                               "(or __graft_entry__.build()) first: " + _SO)
        _lib = ctypes.CDLL(_SO)
        _lib.orc_lfsr_step.restype = ctypes.c_int
        _lib.orc_lfsr_bits.restype = ctypes.c_int
        for name in ("orc_orn_forward_s", "orc_orn_backward_s", "orc_bias_forward_s", "orc_bias_backward_s"):
            getattr(_lib, name).restype = ctypes.c_float
    return _lib


def _p(a, typ):
    return a.ctypes.data_as(typ)


def num_threads():
    return int(lib().orc_num_threads())


def lfsr_step(lb, acc, v):
    return lib().orc_lfsr_step(int(lb), int(acc), int(v))


def lfsr_bits(bit_length, lfsr_length=-1):
    return lib().orc_lfsr_bits(int(bit_length), int(lfsr_length))


def quantize_sc(x, scale, which):
    """sc_conv.cpp:318-320.  which 0: ceil(clamp(x*S,0,S-1)); 1: ceil(-clamp(x*S,1-S,0))."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    q = np.empty(x.shape, dtype=np.int32)
    lib().orc_quantize_sc(_p(x, _f32p), _p(q, _i32p), ctypes.c_long(x.size), int(scale), int(which))
    return q


def quantize_fixed(x, scale, which):
    """fixed.cpp:208-210 (round half to even)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    q = np.empty(x.shape, dtype=np.int32)
    lib().orc_quantize_fixed(_p(x, _f32p), _p(q, _i32p), ctypes.c_long(x.size), int(scale), int(which))
    return q


def _pad_hw(x, padding):
    # F::pad(input, {p0,p0,p1,p1}): padding[0] pads the LAST axis (sc_conv.cpp:314)
    p0, p1 = int(padding[0]), int(padding[1])
    return np.pad(x, ((0, 0), (0, 0), (p1, p1), (p0, p0)))


def conv2d_generic_general_split(x, w, bit_length, lfsr_length, z_units, padding, stride, prog_load,
                                 bin_config, gen_config, xnor=False, mux=False,
                                 channels_last_activation=False, channels_last_weight=False, cuda_xnor=False):
    """sc_conv.cpp:301-489, returning (pos, neg) int16 in logical NCHW index order.

    x [N,C,H,W] and w [O,C,KH,KW] are float arrays in logical NCHW/OIHW index order; the two
    flags say which memory order the reference would have seen (they only select the
    operand/ output index formulas, the returned arrays are always logical NCHW).
    xnor and mux are accepted and ignored, as in the reference CPU extension; cuda_xnor=True instead
    restates the stream generators of the reference's CUDA kernels called with xnor=True
    (sc_cuda_conv.cu:28,55-56,139): XNOR-feedback LFSR, seeds lowered by one (no CUDA build or
    fixture exists; pinned by invariants and a per-bit brute force, tests/test_oracle_invariants.py).
    """
    x = np.asarray(x, dtype=np.float32)
    w = np.asarray(w, dtype=np.float32)
    S = (1 << lfsr_length) if lfsr_length > 0 else bit_length
    xq = quantize_sc(_pad_hw(x, padding), S, 0)
    wp = quantize_sc(w, S, 0)
    wn = quantize_sc(w, S, 1)
    N, C, H, W = xq.shape
    O, _, KH, KW = wp.shape
    s0, s1 = int(stride[0]), int(stride[1])
    Ho, Wo = (H - KH) // s0 + 1, (W - KW) // s1 + 1
    if channels_last_activation:
        xq = np.ascontiguousarray(xq.transpose(0, 2, 3, 1))
    if channels_last_weight:
        wp = np.ascontiguousarray(wp.transpose(0, 2, 3, 1))
        wn = np.ascontiguousarray(wn.transpose(0, 2, 3, 1))
    oshape = (N, Ho, Wo, O) if channels_last_activation else (N, O, Ho, Wo)
    pos = np.zeros(oshape, dtype=np.int16)
    neg = np.zeros(oshape, dtype=np.int16)
    rc = lib().orc_conv2d(_p(xq, _i32p), _p(wp, _i32p), _p(wn, _i32p), _p(pos, _i16p), _p(neg, _i16p),
                          N, C, H, W, O, KH, KW, s0, s1, int(bit_length), int(lfsr_length), int(gen_config),
                          int(prog_load[0]), int(prog_load[1]), int(prog_load[2]), int(bin_config),
                          int(channels_last_activation), int(channels_last_weight), int(bool(cuda_xnor)))
    if rc != 0:
        raise ValueError("oracle conv2d: unsupported configuration (rc=%d)" % rc)
    if channels_last_activation:
        pos = pos.transpose(0, 3, 1, 2)
        neg = neg.transpose(0, 3, 1, 2)
    return pos, neg


def conv2d_generic_general(*args, **kwargs):
    """pos - neg in int16 (wrapping), as sc_conv.cpp:488 returns it."""
    pos, neg = conv2d_generic_general_split(*args, **kwargs)
    return (pos.astype(np.int32) - neg.astype(np.int32)).astype(np.int16)


def linear_generic_general(x, w, prog_load, bit_length, lfsr_length, bin_config, gen_config,
                           xnor=False, mux=False):
    """sc_matmul.cpp:576-676 -> (pos, neg) int32 [B,O]."""
    x = np.asarray(x, dtype=np.float32)
    w = np.asarray(w, dtype=np.float32)
    S = (1 << lfsr_length) if lfsr_length > 0 else bit_length
    xq = quantize_sc(x, S, 0)
    wp = quantize_sc(w, S, 0)
    wn = quantize_sc(w, S, 1)
    B, C = xq.shape
    O = wp.shape[0]
    pos = np.zeros((B, O), dtype=np.int32)
    neg = np.zeros((B, O), dtype=np.int32)
    rc = lib().orc_linear(_p(xq, _i32p), _p(wp, _i32p), _p(wn, _i32p), _p(pos, _i32p), _p(neg, _i32p),
                          B, C, O, int(bit_length), int(lfsr_length), int(gen_config),
                          int(prog_load[0]), int(prog_load[1]), int(prog_load[2]), int(bin_config))
    if rc != 0:
        raise ValueError("oracle linear: unsupported configuration (rc=%d)" % rc)
    return pos, neg


def conv2d_saturate(x, w, add_config, precision_in, precision_out, padding, stride):
    """fixed.cpp:197-238 -> int32 [N,O,Ho,Wo]."""
    x = np.asarray(x, dtype=np.float32)
    w = np.asarray(w, dtype=np.float32)
    P2 = 1 << precision_in
    xq = quantize_fixed(_pad_hw(x, padding), P2, 0)
    wp = quantize_fixed(w, P2, 0)
    wn = quantize_fixed(w, P2, 1)
    N, C, H, W = xq.shape
    O, _, KH, KW = wp.shape
    s0, s1 = int(stride[0]), int(stride[1])
    out = np.zeros((N, O, (H - KH) // s0 + 1, (W - KW) // s1 + 1), dtype=np.int32)
    rc = lib().orc_fixed_conv2d(_p(xq, _i32p), _p(wp, _i32p), _p(wn, _i32p), _p(out, _i32p),
                                N, C, H, W, O, KH, KW, s0, s1,
                                int(add_config), int(precision_in), int(precision_out))
    if rc != 0:
        raise ValueError("oracle fixed conv: unsupported configuration (rc=%d)" % rc)
    return out


# ---- pointwise -------------------------------------------------------------------------

def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def or_approx_n_forward(x, or_n):
    """sc_cpu.hpp:192-225 elementwise."""
    x = _f32(x)
    y = np.empty_like(x)
    lib().orc_orn_forward(_p(x, _f32p), _p(y, _f32p), ctypes.c_long(x.size), int(or_n))
    return y


def or_approx_n_backward(g, x, or_n, half_input=True):
    """sc_cpu.hpp:227-262; the saved sum is rounded to fp16 first as sc_cuda_pw.cu:775 does."""
    g, x = _f32(g), _f32(x)
    if half_input:
        x = x.astype(np.float16).astype(np.float32)
    gx = np.empty_like(g)
    lib().orc_orn_backward(_p(g, _f32p), _p(x, _f32p), _p(gx, _f32p), ctypes.c_long(g.size), int(or_n))
    return gx


def or_approx_n_forward_bias_std_both(xp, xn, bias_coef, std_coef, or_n, noise_pos, noise_neg):
    """sc_cuda_pw.cu:219-373 with the N(0,1) draws supplied by the caller."""
    xp, xn, a, b = _f32(xp), _f32(xn), _f32(noise_pos), _f32(noise_neg)
    bc, sc = _f32(bias_coef), _f32(std_coef)
    y = np.empty_like(xp)
    lib().orc_orn_bias_std_both_forward(_p(xp, _f32p), _p(xn, _f32p), _p(a, _f32p), _p(b, _f32p),
                                        _p(bc, _f32p), _p(sc, _f32p), _p(y, _f32p),
                                        ctypes.c_long(xp.size), int(or_n))
    return y


def or_approx_n_backward_bias_std_both(g, xp, xn, bias_coef, or_n, half_input=True):
    """sc_cuda_pw.cu:527-621, 952-1011 (inputs rounded to fp16 by the host wrapper)."""
    g, xp, xn, bc = _f32(g), _f32(xp), _f32(xn), _f32(bias_coef)
    if half_input:
        xp = xp.astype(np.float16).astype(np.float32)
        xn = xn.astype(np.float16).astype(np.float32)
    gp, gn = np.empty_like(g), np.empty_like(g)
    lib().orc_orn_bias_std_both_backward(_p(g, _f32p), _p(xp, _f32p), _p(xn, _f32p), _p(bc, _f32p),
                                         _p(gp, _f32p), _p(gn, _f32p), ctypes.c_long(g.size), int(or_n))
    return gp, gn


def bias_correct_forward(x, bias_coef, std_coef, noise):
    """utils_functional.py:441-447: x + poly_b(x) + poly_s(x)*noise (second return value)."""
    x, nz = _f32(x), _f32(noise)
    b, s = _f32(bias_coef), _f32(std_coef)
    xb = sum(b[k] * x ** k for k in range(6))
    xs = sum(s[k] * x ** k for k in range(6))
    return (x + xs * nz + xb).astype(np.float32)


def bias_correct_backward(g, x, bias_coef):
    """utils_functional.py:456-459."""
    g, x, b = _f32(g), _f32(x), _f32(bias_coef)
    xd = 1 + b[1] + b[2] * 2 * x + b[3] * 3 * x ** 2 + b[4] * 4 * x ** 3 + b[5] * 5 * x ** 4
    return (xd * g).astype(np.float32)


def quantize(x, prec=8):
    """utils_functional.py:93-104 (prune = 0): (x*2^p).round().clamp(+-(2^p-1))/2^p."""
    x = _f32(x)
    if prec <= 16:
        p2 = np.float32(2 ** prec)
        return (np.clip(np.rint(x * p2), -p2 + 1, p2 - 1) / p2).astype(np.float32)
    return np.clip(x, -1, 1)


def compute_bias_std_coef(or_n, a_bit, a_act, order):
    """utils_functional.py:900-949.

    30 windows [s, s+0.1) with s on linspace(0, max(a_bit), 30), selected on the FLOAT
    surrogate a_act; per window with more than one sample: mean and unbiased std of
    a_bit - a_act; polynomial least squares of degree `order` over the start positions of
    the valid windows.  The bias fit is replaced by zeros when order >= n_valid // 5.
    Returns float32 (bias_coef, std_coef), each order+1 long.
    """
    a_bit = _f32(a_bit).reshape(-1)
    a_act = _f32(a_act).reshape(-1)
    if or_n < 0:
        return np.zeros(order + 1, np.float32), np.zeros(order + 1, np.float32)
    output_range = np.linspace(0, float(a_bit.max()), 30)
    bias_bins, std_bins, valid = [], [], []
    for i, start in enumerate(output_range):
        # a_act is float32; the comparison operands are promoted exactly as torch does for a
        # python float against a float32 tensor (the scalar is cast to float32)
        lo = np.float32(start)
        hi = np.float32(start + 0.1)
        sel = (a_act >= lo) & (a_act < hi)
        err = a_bit[sel] - a_act[sel]
        if err.size > 1:
            bias_bins.append(np.float32(err.mean(dtype=np.float32)))
            std_bins.append(np.float32(err.std(ddof=1, dtype=np.float32)))
            valid.append(i)
    pos = output_range[valid]
    A = np.stack([pos ** i for i in range(order + 1)], axis=1).astype(np.float32)
    bias_bins = np.asarray(bias_bins, np.float32)
    std_bins = np.asarray(std_bins, np.float32)
    if order >= len(valid) // 5:
        bias_coef = np.zeros(order + 1, np.float32)
    else:
        bias_coef = np.linalg.lstsq(A.astype(np.float64), bias_bins.astype(np.float64), rcond=None)[0].astype(np.float32)
    std_coef = np.linalg.lstsq(A.astype(np.float64), std_bins.astype(np.float64), rcond=None)[0].astype(np.float32)
    return bias_coef, std_coef


def linear_generic_legacy(x, w, bit_length, forward="full_or", prec=128, share=True):
    """The reference's legacy `linear_generic` (utils_functional.py:955-1081; generator 'lfsr', share=True) with
    its generators (:147-165 lfsr_init, :254-272 lfsr_cont) -> float32 [B,O], pos - neg.

    Restated cycle by cycle in numpy: operands are the float16-rounded products x*L (weights clamped to
    prec-1 per polarity, activations unclamped; :980-995), LFSR states are integers stepped before the compare
    (:1022), seeds c % P + 1 / (67 + c) % P + 1 / (37 + c) % P + 1 with P = L - 1 shared by all rows (:1000-1001),
    per cycle sign(count) ('full_or') or count ('full_bin') (:1031-1036), mean over cycles rounded to float16
    (compute_type, :28; :1067-1068).  share=False (:996-998): one generator per element, the seed index running over
    the whole weight tensor (o * C + c) and the whole activation tensor (b * C + c).  Pinned by
    tests/golden/ref_linear_legacy.npz, written by the reference's own function."""
    x = np.asarray(x, np.float32)
    w = np.asarray(w, np.float32)
    L = int(bit_length)
    lb = {8: 3, 16: 4, 32: 5, 64: 6, 128: 7, 256: 8}[L]
    P = L - 1
    bit_range = np.float32(prec - 1)
    Lf = np.float32(L)
    a = (x * Lf).astype(np.float16).astype(np.float32)
    wp = np.clip(w * Lf, 0, bit_range).astype(np.float16).astype(np.float32)
    wn = (-np.clip(w * Lf, -bit_range, 0)).astype(np.float16).astype(np.float32)
    C = x.shape[1]
    if share:
        c = np.arange(C)
        st_a, st_p, st_n = c % P + 1, (67 + c) % P + 1, (37 + c) % P + 1
    else:
        ia, iw = np.arange(x.size).reshape(x.shape), np.arange(w.size).reshape(w.shape)
        st_a, st_p, st_n = ia % P + 1, (67 + iw) % P + 1, (37 + iw) % P + 1
    step = np.vectorize(lambda v: lfsr_step(lb, 0, int(v)))
    pos = np.zeros((x.shape[0], w.shape[0]), np.float64)
    neg = np.zeros_like(pos)
    for _ in range(L):
        st_a, st_p, st_n = step(st_a), step(st_p), step(st_n)
        ab = (a > st_a).astype(np.float64)
        cp = ab @ (wp > st_p).astype(np.float64).T
        cn = ab @ (wn > st_n).astype(np.float64).T
        if forward == "full_or":
            cp, cn = np.sign(cp), np.sign(cn)
        pos += cp
        neg += cn
    mean = lambda t: (t / L).astype(np.float32).astype(np.float16).astype(np.float32)
    return mean(pos) - mean(neg)
