"""Tensor-level plumbing shared by the drop-in extension modules: layout decisions, workspace,
stream, and the calls into the C ABI.  PyTorch is used for device memory and streams only."""
import ctypes
import os
import warnings

import torch

import _lib

# How the `xnor` argument of the conv op is treated (environment variable REXSC_XNOR_MODE, read at call time):
#   cpu_oracle (default)  ignored, as the reference's CPU extension does (XOR-feedback LFSR, seeds 1..2^lb-1;
#                         sc_conv.cpp:362-425).  Bit-exactness is defined against that extension.
#   cuda_ref              honoured, as the reference's CUDA conv kernels do (XNOR-feedback LFSR, seeds lowered by
#                         one, the same LFSR for the and_2 generator; sc_cuda_conv.cu:28,55-56,139): a caller
#                         coming from the CUDA extension keeps the bit streams it had.  The linear op has no XNOR
#                         generator in either reference extension (sc_cuda_matmul.cu:27-57).
XNOR_MODES = ("cpu_oracle", "cuda_ref")
_warned_xnor_ignored = False


def xnor_mode():
    mode = os.environ.get("REXSC_XNOR_MODE", "cpu_oracle")
    if mode not in XNOR_MODES:
        raise RuntimeError("REXSC_XNOR_MODE must be one of %s (got %r)" % (", ".join(XNOR_MODES), mode))
    return mode


def honour_xnor(xnor):
    """The generator flag for a conv call of the CUDA-named module: True only in cuda_ref mode.  In the default
    mode an xnor=True argument is accepted and not honoured; that is said once per process."""
    global _warned_xnor_ignored
    if not xnor:
        return False
    if xnor_mode() == "cuda_ref":
        return True
    if not _warned_xnor_ignored:
        _warned_xnor_ignored = True
        warnings.warn("sc_extension_cuda: xnor=True is accepted but not honoured: bit streams follow the reference's CPU "
                      "extension (XOR-feedback LFSR).  Set REXSC_XNOR_MODE=cuda_ref for the CUDA extension's XNOR generator.",
                      RuntimeWarning, stacklevel=3)
    return False


def _require_cuda(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("rexsc ops need tensors on a HIP device (got %s)" % t.device)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def is_channels_last(t):
    """The reference's own layout test (sc_conv.cpp:326-331): decided from raw strides."""
    s = t.stride()
    return s[1] == 1 and s[1] * s[2] * s[3] != 1


def _as_layout(t, channels_last, keep_half=False):
    """Dense float32 copy (or t itself) in the requested memory order, 16-byte aligned; keep_half: a float16 tensor
    stays float16."""
    t = t.detach()
    if t.dtype != torch.float32 and not (keep_half and t.dtype == torch.float16):
        t = t.float()
    fmt = torch.channels_last if channels_last else torch.contiguous_format
    t = t.contiguous(memory_format=fmt)
    if channels_last and t.stride(1) != 1:  # size-1 dims make contiguous() ambiguous: force NHWC strides
        t = t.permute(0, 2, 3, 1).contiguous().permute(0, 3, 1, 2)
    if t.data_ptr() % 16:
        t = t.clone(memory_format=torch.preserve_format)
    return t


def _workspace(nbytes, device):
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def _empty_out(shape, dtype, device, channels_last):
    if channels_last:
        n, c, h, w = shape
        return torch.empty((n, h, w, c), dtype=dtype, device=device).permute(0, 3, 1, 2)
    return torch.empty(shape, dtype=dtype, device=device)


class WeightStreamCache:
    """Weight bitstreams of one layer, kept between calls (evaluation, frozen layers) in buffers keyed by the call's
    descriptor.  Whether a kept buffer still belongs to the current weight VALUES is never decided on the host: no
    host-side stamp sees every edit (`p.data.clamp_()`, which the reference's own training loop uses,
    utils_own.py:187-190, changes neither the storage pointer nor the tensor's version counter).  A buffer that
    exists is handed to the library in VERIFY mode: a small kernel compares the weights bit for bit with the copy the
    buffer holds and the generator runs on the device only if something differs -- no synchronisation, and any
    edit of the weights, by any route, is caught.  A new buffer is handed over in FILL mode."""

    def __init__(self, max_entries=4):
        self.entries = {}
        self.max_entries = max_entries
        self.hits = 0    # calls that reused a buffer (the device decided whether to regenerate)
        self.misses = 0  # calls that had to allocate and fill one

    def lookup(self, desc_key, nbytes, device):
        """-> (buffer, mode) with mode one of _lib.WSTREAMS_VERIFY (kept buffer) / _lib.WSTREAMS_FILL (new buffer)."""
        key = (desc_key, str(device), int(nbytes), os.environ.get("REXSC_FOLD_TAPS"), os.environ.get("REXSC_SNG_MODE"))
        buf = self.entries.get(key)
        if buf is not None:
            self.hits += 1
            return buf, _lib.WSTREAMS_VERIFY
        self.misses += 1
        if len(self.entries) >= self.max_entries:
            self.entries.pop(next(iter(self.entries)))
        buf = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)
        self.entries[key] = buf
        return buf, _lib.WSTREAMS_FILL

    def clear(self):
        self.entries.clear()


def _conv_desc(x, w, bit_length, lfsr_length, padding, stride, prog_load, bin_config, gen_config, xnor,
               act_fake_quant, weight_fake_quant):
    """(descriptor, channels-last flags) of a conv call; x may be a tensor or a (shape, channels_last) pair."""
    if isinstance(x, torch.Tensor):
        if x.dim() != 4:
            raise RuntimeError("conv2d: expected input [N,C,H,W], got %s" % (tuple(x.shape),))
        xshape, cl_a = tuple(x.shape), is_channels_last(x)
    else:
        xshape, cl_a = tuple(x[0]), bool(x[1])
    if len(xshape) != 4 or w.dim() != 4 or xshape[1] != w.size(1):
        raise RuntimeError("conv2d: expected input [N,C,H,W] and weight [O,C,KH,KW] with equal C, got %s and %s"
                           % (xshape, tuple(w.shape)))
    cl_w = is_channels_last(w)
    N, C, H, W = xshape
    O, _, KH, KW = w.shape
    fq = lambda p: 0 if p is None else int(p) + 1
    d = _lib.ConvDesc(N, C, H, W, O, KH, KW, int(padding[1]), int(padding[0]), int(stride[0]), int(stride[1]),
                      int(bit_length), int(lfsr_length), int(gen_config), int(bin_config),
                      int(prog_load[0]), int(prog_load[1]), int(prog_load[2]), int(cl_a), int(cl_w), int(bool(xnor)),
                      fq(act_fake_quant), fq(weight_fake_quant))
    return d, cl_a, cl_w


class PreparedWeightStreams:
    """Weight bitstreams generated ahead of the conv call they belong to (sc_conv2d_prepare_weights)."""

    def __init__(self, buf, key):
        self.buf, self.key = buf, key


def sc_conv2d_prepare_weights(x_like, w, bit_length, lfsr_length, padding, stride, prog_load, bin_config, gen_config,
                              xnor=False, act_fake_quant=None, weight_fake_quant=None, into=None, keep_weight_copy=False):
    """Generates the weight bitstreams of the conv call  sc_conv2d(x, w, <same arguments>, prepared=<result>)  on the
    current stream, ahead of that call: a layer's weight streams depend on its weights alone, so they can be made on a
    second stream while the previous layer computes.  x_like: the activation tensor or ((N, C, H, W), channels_last).
    into: a PreparedWeightStreams of an earlier call with the same arguments, whose buffer is then reused.
    keep_weight_copy: also store the copy of w that a WeightStreamCache compares with (not needed for prepared=)."""
    _require_cuda(w)
    d, _, cl_w = _conv_desc(x_like, w, bit_length, lfsr_length, padding, stride, prog_load, bin_config, gen_config, xnor,
                            act_fake_quant, weight_fake_quant)
    wc = _as_layout(w, cl_w)
    L = _lib.lib()
    with torch.cuda.device(w.device):
        nbytes = L.rexsc_conv2d_weight_streams_bytes(ctypes.byref(d))
        if nbytes == 0:
            _lib.check(-1, "rexsc_conv2d (planning)")
        key = d.key()
        if into is not None and into.key == key and into.buf.numel() >= nbytes and into.buf.device == w.device:
            buf = into.buf
        else:
            buf = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
        rc = L.rexsc_conv2d_prepare_weights(ctypes.byref(d), _ptr(wc), _ptr(buf), buf.numel(), int(bool(keep_weight_copy)),
                                            _stream())
        _lib.check(rc, "rexsc_conv2d_prepare_weights")
    return PreparedWeightStreams(buf, key)


def sc_conv2d(x, w, bit_length, lfsr_length, padding, stride, prog_load, bin_config, gen_config,
              want_split=True, want_diff=False, xnor=False, want_value=False, weight_cache=None,
              act_fake_quant=None, weight_fake_quant=None, prepared=None):
    """SC conv2d on the HIP path.  padding=(p0,p1): p0 pads the LAST axis, p1 axis 2, as the
    reference's F::pad call does (sc_conv.cpp:314); stride=(s0,s1): s0 along axis 2.
    -> (pos, neg, diff) int16, plus the float32 tensor pos / L - neg / L as a fourth element when want_value.
    weight_cache: a WeightStreamCache that keeps w's bitstreams between calls (the device checks on every call that
    they still belong to w's values).  act_fake_quant / weight_fake_quant: precision of the layers' fake quantisation
    to apply to the operand inside the generators (None: operand as given).  prepared: the weight streams of exactly
    this call, made by sc_conv2d_prepare_weights on a stream this one is ordered after (the caller's word: no check)."""
    _require_cuda(x, w)
    d, cl_a, cl_w = _conv_desc(x, w, bit_length, lfsr_length, padding, stride, prog_load, bin_config, gen_config, xnor,
                               act_fake_quant, weight_fake_quant)
    xc, wc = _as_layout(x, cl_a), _as_layout(w, cl_w)
    N, C, H, W = xc.shape
    O, _, KH, KW = wc.shape
    L = _lib.lib()
    extended = want_value or weight_cache is not None or prepared is not None
    with torch.cuda.device(x.device):
        Ho = (H + 2 * d.pad_h - KH) // d.stride_h + 1
        Wo = (W + 2 * d.pad_w - KW) // d.stride_w + 1
        shape = (N, O, Ho, Wo)
        mk = lambda want, dt=torch.int16: _empty_out(shape, dt, x.device, cl_a) if want else None
        if N == 0 and Ho > 0 and Wo > 0:  # an empty batch has an empty result; nothing to launch
            res = (mk(want_split), mk(want_split), mk(want_diff))
            return res + (mk(True, torch.float32),) if want_value else res
        ws_bytes = L.rexsc_conv2d_workspace_bytes(ctypes.byref(d))
        if ws_bytes == 0:
            _lib.check(-1, "rexsc_conv2d (planning)")
        pos, neg, diff = mk(want_split), mk(want_split), mk(want_diff)
        ws = _workspace(ws_bytes, x.device)
        if not extended:
            rc = L.rexsc_conv2d_orn(ctypes.byref(d), _ptr(xc), _ptr(wc), _ptr(pos), _ptr(neg), _ptr(diff),
                                    _ptr(ws), ws.numel(), _stream())
            _lib.check(rc, "rexsc_conv2d_orn")
            return pos, neg, diff
        value = mk(want_value, torch.float32)
        wbuf, mode = None, _lib.WSTREAMS_FILL
        if prepared is not None:
            if prepared.key != d.key():
                raise RuntimeError("conv2d: the prepared weight streams belong to another call (descriptor differs)")
            wbuf, mode = prepared.buf, _lib.WSTREAMS_TRUST
        elif weight_cache is not None:
            wbuf, mode = weight_cache.lookup(("conv",) + d.key(), L.rexsc_conv2d_weight_streams_bytes(ctypes.byref(d)),
                                             x.device)
        rc = L.rexsc_conv2d_orn_ex(ctypes.byref(d), _ptr(xc), _ptr(wc), _ptr(pos), _ptr(neg), _ptr(diff), _ptr(value),
                                   _ptr(wbuf), wbuf.numel() if wbuf is not None else 0, mode,
                                   _ptr(ws), ws.numel(), _stream())
        _lib.check(rc, "rexsc_conv2d_orn_ex")
    return (pos, neg, diff, value) if want_value else (pos, neg, diff)


def sc_linear(x, w, prog_load, bit_length, lfsr_length, bin_config, gen_config, weight_cache=None,
              act_fake_quant=None, weight_fake_quant=None):
    """SC linear on the HIP path -> (pos, neg) int32 [B,O].  weight_cache: a WeightStreamCache that keeps w's
    bitstreams between calls (the device checks on every call that they still belong to w's values);
    act_fake_quant / weight_fake_quant: precision of the layers' fake quantisation to apply to the operand inside
    the generators (None: operand as given)."""
    _require_cuda(x, w)
    if x.dim() != 2 or w.dim() != 2 or x.size(1) != w.size(1):
        raise RuntimeError("linear: expected input [B,C] and weight [O,C], got %s and %s"
                           % (tuple(x.shape), tuple(w.shape)))
    xc = x.detach().float().contiguous()
    wc = w.detach().float().contiguous()
    B, C = xc.shape
    O = w.shape[0]
    fq = lambda p: 0 if p is None else int(p) + 1
    d = _lib.LinearDesc(B, C, O, int(bit_length), int(lfsr_length), int(gen_config), int(bin_config),
                        int(prog_load[0]), int(prog_load[1]), int(prog_load[2]), fq(act_fake_quant), fq(weight_fake_quant))
    L = _lib.lib()
    if B == 0:
        return (torch.empty((0, O), dtype=torch.int32, device=x.device),
                torch.empty((0, O), dtype=torch.int32, device=x.device))
    with torch.cuda.device(x.device):
        ws_bytes = L.rexsc_linear_workspace_bytes(ctypes.byref(d))
        if ws_bytes == 0:
            _lib.check(-1, "rexsc_linear (planning)")
        pos = torch.empty((B, O), dtype=torch.int32, device=x.device)
        neg = torch.empty((B, O), dtype=torch.int32, device=x.device)
        ws = _workspace(ws_bytes, x.device)
        if weight_cache is None:
            rc = L.rexsc_linear_orn(ctypes.byref(d), _ptr(xc), _ptr(wc), _ptr(pos), _ptr(neg), _ptr(ws), ws.numel(),
                                    _stream())
            _lib.check(rc, "rexsc_linear_orn")
        else:
            # The batch size is not part of the key: the weight streams do not depend on it.  The buffer's size is:
            # it says whether the buffer also carries the activation generator's table, which small batches go without.
            key = ("linear",) + d.key()[2:]
            wbuf, mode = weight_cache.lookup(key, L.rexsc_linear_weight_streams_bytes(ctypes.byref(d)), x.device)
            rc = L.rexsc_linear_orn_ex(ctypes.byref(d), _ptr(xc), _ptr(wc), _ptr(pos), _ptr(neg), _ptr(wbuf), wbuf.numel(),
                                       mode, _ptr(ws), ws.numel(), _stream())
            _lib.check(rc, "rexsc_linear_orn_ex")
    return pos, neg


def sc_linear_legacy(x, w, bit_length, bin_config, weight_clamp=127, share=True):
    """The reference's legacy `linear_generic` simulation (utils_functional.py:955-1081, generator 'lfsr',
    shared generators, or one per element with share=False) on the HIP kernels -> (pos, neg) int32 [B,O]: per-output
    sums over the bit_length cycles."""
    _require_cuda(x, w)
    if x.dim() != 2 or w.dim() != 2 or x.size(1) != w.size(1):
        raise RuntimeError("linear: expected input [B,C] and weight [O,C], got %s and %s"
                           % (tuple(x.shape), tuple(w.shape)))
    xc = x.detach().float().contiguous()
    wc = w.detach().float().contiguous()
    B, C = xc.shape
    O = wc.shape[0]
    d = _lib.LinearDesc(B, C, O, int(bit_length), -1, 1, int(bin_config), 7, 8, 1)
    L = _lib.lib()
    if B == 0:
        return (torch.empty((0, O), dtype=torch.int32, device=x.device),
                torch.empty((0, O), dtype=torch.int32, device=x.device))
    with torch.cuda.device(x.device):
        ws_bytes = L.rexsc_linear_workspace_bytes(ctypes.byref(d))
        if ws_bytes == 0:
            _lib.check(-1, "rexsc_linear_legacy (planning)")
        pos = torch.empty((B, O), dtype=torch.int32, device=x.device)
        neg = torch.empty((B, O), dtype=torch.int32, device=x.device)
        ws = _workspace(ws_bytes, x.device)
        rc = L.rexsc_linear_legacy(ctypes.byref(d), int(weight_clamp), int(bool(share)), _ptr(xc), _ptr(wc), _ptr(pos), _ptr(neg), _ptr(ws),
                                   ws.numel(), _stream())
        _lib.check(rc, "rexsc_linear_legacy")
    return pos, neg


def fixed_conv2d(x, w, add_config, precision_in, precision_out, padding, stride):
    _require_cuda(x, w)
    if x.dim() != 4 or w.dim() != 4 or x.size(1) != w.size(1):
        raise RuntimeError("conv2d_saturate: expected input [N,C,H,W] and weight [O,C,KH,KW] with equal C")
    xc, wc = _as_layout(x, False), _as_layout(w, False)  # the reference assumes NCHW (fixed.cpp:10-11)
    N, C, H, W = xc.shape
    O, _, KH, KW = wc.shape
    d = _lib.FixedDesc(N, C, H, W, O, KH, KW, int(padding[1]), int(padding[0]), int(stride[0]), int(stride[1]),
                       int(add_config), int(precision_in), int(precision_out))
    L = _lib.lib()
    with torch.cuda.device(x.device):
        Ho = (H + 2 * d.pad_h - KH) // d.stride_h + 1
        Wo = (W + 2 * d.pad_w - KW) // d.stride_w + 1
        if N == 0 and Ho > 0 and Wo > 0:
            return torch.empty((0, O, Ho, Wo), dtype=torch.int32, device=x.device)
        ws_bytes = L.rexsc_fixed_conv2d_workspace_bytes(ctypes.byref(d))
        if ws_bytes == 0:
            _lib.check(-1, "rexsc_fixed_conv2d (planning)")
        out = torch.empty((N, O, Ho, Wo), dtype=torch.int32, device=x.device)
        ws = _workspace(ws_bytes, x.device)
        rc = L.rexsc_fixed_conv2d(ctypes.byref(d), _ptr(xc), _ptr(wc), _ptr(out), _ptr(ws), ws.numel(), _stream())
        _lib.check(rc, "rexsc_fixed_conv2d")
    return out


# ---- pointwise ------------------------------------------------------------------------------

def _dense_f32(t):
    """float32, dense in memory (any permutation of a contiguous block), 16-byte aligned."""
    t = t.detach()
    if t.dtype != torch.float32:
        t = t.float()
    dense = t.is_contiguous() or (t.dim() == 4 and t.is_contiguous(memory_format=torch.channels_last))
    if not dense:
        t = t.contiguous()
    if t.data_ptr() % 16:
        t = t.clone(memory_format=torch.preserve_format)
    return t


def _like_layout(t, ref):
    """Copy of t in ref's dtype (float32, or float16 for the binary16 kernels) laid out with ref's strides (the
    kernels index raw storage)."""
    t = t.detach()
    if t.dtype != ref.dtype:
        t = t.to(ref.dtype)
    if t.stride() != ref.stride() or t.data_ptr() % 16:
        out = torch.empty_like(ref)
        out.copy_(t)
        return out
    return t


def _coef(c, device):
    c = c.detach()
    if c.device != device or c.dtype != torch.float32 or not c.is_contiguous():
        c = c.to(device=device, dtype=torch.float32).contiguous()
    if c.numel() < 6:
        raise RuntimeError("bias/std coefficient vectors need at least 6 entries (got %d)" % c.numel())
    return c


def orn_forward(x, or_n):
    _require_cuda(x)
    xf = _dense_f32(x)
    y = torch.empty_like(xf)
    with torch.cuda.device(x.device):
        rc = _lib.lib().rexsc_orn_forward(_ptr(xf), _ptr(y), xf.numel(), int(or_n), _stream())
        _lib.check(rc, "rexsc_orn_forward")
    return y


def orn_backward(grad_output, x, or_n, half_input=True):
    _require_cuda(grad_output, x)
    g = _dense_f32(grad_output)
    xf = _like_layout(x, g)
    gx = torch.empty_like(g)
    with torch.cuda.device(g.device):
        rc = _lib.lib().rexsc_orn_backward(_ptr(g), _ptr(xf), _ptr(gx), g.numel(), int(or_n), int(half_input),
                                           _stream())
        _lib.check(rc, "rexsc_orn_backward")
    return gx


_capture_counters = {}  # device index -> int64 [1] tensor: noise vectors consumed by captured calls
_CAPTURE_SEED_SALT = 0x9E3779B97F4A7C15  # captured calls draw from a stream of their own


def _next_philox(n_elems, device):
    """(seed, offset, counter) for the next noise draw.

    Eagerly: seed and offset come from the device's torch generator, which is advanced past the
    4-element vectors this call consumes -- the way the reference's kernels consume the generator's
    Philox state (sc_cuda_pw.cu:870-877): torch.manual_seed restarts the stream; counter is None.
    While a stream is being captured the host arguments are frozen into the graph, so the offset lives
    in device memory instead: counter is an int64 tensor the kernel adds to its offset, and
    _advance_philox() records its increment after the launch -- every replay draws new noise."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    used = (n_elems + 3) // 4
    gen = torch.cuda.default_generators[idx]
    if not torch.cuda.is_current_stream_capturing():
        if idx not in _capture_counters:  # allocated and zeroed outside any capture
            _capture_counters[idx] = torch.zeros(1, dtype=torch.int64, device=device)
        seed, off = gen.initial_seed() & 0xFFFFFFFFFFFFFFFF, gen.get_offset()
        gen.set_offset(off + (used + 3) // 4 * 4)  # the generator keeps offsets in multiples of 4
        return seed, off, None
    if idx not in _capture_counters:
        raise RuntimeError("noise kernels need one eager call on this device before they are captured")
    return (torch.initial_seed() ^ _CAPTURE_SEED_SALT) & 0xFFFFFFFFFFFFFFFF, 0, _capture_counters[idx]


def _advance_philox(counter, n_elems):
    if counter is not None:
        counter.add_((n_elems + 3) // 4)  # a kernel on the capturing stream: part of the graph


def orn_bias_std_both_forward(x_pos, x_neg, bias_coef, std_coef, or_n, seed=None, offset=None, return_noise=False):
    _require_cuda(x_pos, x_neg)
    xp = _dense_f32(x_pos)
    xn = _like_layout(x_neg, xp)
    b, s = _coef(bias_coef, xp.device), _coef(std_coef, xp.device)
    y = torch.empty_like(xp)
    n = xp.numel()
    counter = None
    if seed is None:
        seed, offset, counter = _next_philox(n, xp.device)
    np_ = torch.empty_like(xp) if return_noise else None
    nn_ = torch.empty_like(xp) if return_noise else None
    with torch.cuda.device(xp.device):
        rc = _lib.lib().rexsc_orn_bias_std_both_forward(_ptr(xp), _ptr(xn), _ptr(b), _ptr(s), _ptr(y), n, int(or_n),
                                                        int(seed), int(offset), _ptr(counter), _ptr(np_), _ptr(nn_),
                                                        _stream())
        _lib.check(rc, "rexsc_orn_bias_std_both_forward")
        _advance_philox(counter, n)
    return (y, np_, nn_) if return_noise else y


def orn_bias_std_both_backward(grad_output, x_pos, x_neg, bias_coef, or_n, half_input=True):
    _require_cuda(grad_output, x_pos, x_neg)
    g = _dense_f32(grad_output)
    xp, xn = _like_layout(x_pos, g), _like_layout(x_neg, g)
    b = _coef(bias_coef, g.device)
    gp, gn = torch.empty_like(g), torch.empty_like(g)
    with torch.cuda.device(g.device):
        rc = _lib.lib().rexsc_orn_bias_std_both_backward(_ptr(g), _ptr(xp), _ptr(xn), _ptr(b), _ptr(gp), _ptr(gn),
                                                         g.numel(), int(or_n), int(half_input), _stream())
        _lib.check(rc, "rexsc_orn_bias_std_both_backward")
    return gp, gn


def orn_bias_std_forward_f16(x, bias_coef, std_coef, or_n, seed=None, offset=None):
    _require_cuda(x)
    xh = x.detach().to(torch.float16).contiguous()
    b, s = _coef(bias_coef, xh.device), _coef(std_coef, xh.device)
    y = torch.empty_like(xh)
    counter = None
    if seed is None:
        seed, offset, counter = _next_philox(xh.numel(), xh.device)
    with torch.cuda.device(xh.device):
        rc = _lib.lib().rexsc_orn_bias_std_forward_f16(_ptr(xh), _ptr(b), _ptr(s), _ptr(y), xh.numel(), int(or_n),
                                                       int(seed), int(offset), _ptr(counter), _stream())
        _lib.check(rc, "rexsc_orn_bias_std_forward_f16")
        _advance_philox(counter, xh.numel())
    return y


def orn_bias_std_backward(grad_output, x, bias_coef, or_n, half_input=True):
    _require_cuda(grad_output, x)
    g = _dense_f32(grad_output)
    xf = _like_layout(x, g)
    b = _coef(bias_coef, g.device)
    gx = torch.empty_like(g)
    with torch.cuda.device(g.device):
        rc = _lib.lib().rexsc_orn_bias_std_backward(_ptr(g), _ptr(xf), _ptr(b), _ptr(gx), g.numel(), int(or_n),
                                                    int(half_input), _stream())
        _lib.check(rc, "rexsc_orn_bias_std_backward")
    return gx


# ---- merged surrogate (polarity-pair layout) ---------------------------------------------------

def pair_layout(s2, keep_half=False):
    """s2 = conv / linear output with 2*O channels (O positive, then O negative).  Returns
    (s2 dense, outer, inner, channels_last) for the [outer][2][inner] view of its storage, re-laying
    the tensor out if its own layout has no inner % 4 == 0 view; None if neither layout has one.
    The result is float32 unless keep_half and s2 is float16 (for orn_pair_backward's binary16 kernel)."""
    s2 = s2.detach()
    O = s2.size(1) // 2
    if s2.dim() == 2:
        return (s2.contiguous(), s2.size(0), O, False) if O % 4 == 0 else None
    N, _, H, W = s2.shape
    ok_cl, ok_nchw = O % 4 == 0, (O * H * W) % 4 == 0
    is_cl = s2.is_contiguous(memory_format=torch.channels_last) and not s2.is_contiguous()
    if (is_cl and ok_cl) or (not ok_nchw and ok_cl):
        return _as_layout(s2, True, keep_half), N * H * W, O, True
    if ok_nchw:
        return _as_layout(s2, False, keep_half), N, O * H * W, False
    return None


def _pair_result_like(s2, channels_last, dtype=torch.float32):
    if s2.dim() == 2:
        return torch.empty((s2.size(0), s2.size(1) // 2), dtype=dtype, device=s2.device)
    N, O2, H, W = s2.shape
    return _empty_out((N, O2 // 2, H, W), dtype, s2.device, channels_last)


def orn_pair_backward(grad_output, s2, outer, inner, channels_last, or_n, half_input=True):
    """Gradient of the merged convolution's output.  s2 float32: float32 in and out; s2 float16 (pair_layout with
    keep_half, inside a float16 autocast region): the binary16 kernel, float16 in and out."""
    half = s2.dtype == torch.float16
    y_like = _pair_result_like(s2, channels_last, s2.dtype)
    g = _like_layout(grad_output, y_like)
    g2 = torch.empty_like(s2)
    with torch.cuda.device(s2.device):
        if half:
            rc = _lib.lib().rexsc_orn_pair_backward_f16(_ptr(g), _ptr(s2), _ptr(g2), outer, inner, int(or_n), _stream())
        else:
            rc = _lib.lib().rexsc_orn_pair_backward(_ptr(g), _ptr(s2), _ptr(g2), outer, inner, int(or_n), int(half_input),
                                                    _stream())
        _lib.check(rc, "rexsc_orn_pair_backward")
    return g2


def orn_bias_std_pair_forward(s2, outer, inner, channels_last, bias_coef, std_coef, or_n, seed=None, offset=None):
    b, s = _coef(bias_coef, s2.device), _coef(std_coef, s2.device)
    y = _pair_result_like(s2, channels_last)
    counter = None
    if seed is None:
        seed, offset, counter = _next_philox(y.numel(), y.device)
    with torch.cuda.device(s2.device):
        rc = _lib.lib().rexsc_orn_bias_std_pair_forward(_ptr(s2), _ptr(b), _ptr(s), _ptr(y), outer, inner, int(or_n),
                                                        int(seed), int(offset), _ptr(counter), _stream())
        _lib.check(rc, "rexsc_orn_bias_std_pair_forward")
        _advance_philox(counter, y.numel())
    return y


def orn_bias_std_pair_backward(grad_output, s2, outer, inner, channels_last, bias_coef, or_n, half_input=True):
    y_like = _pair_result_like(s2, channels_last)
    g = _like_layout(grad_output, y_like)
    b = _coef(bias_coef, s2.device)
    g2 = torch.empty_like(s2)
    with torch.cuda.device(s2.device):
        rc = _lib.lib().rexsc_orn_bias_std_pair_backward(_ptr(g), _ptr(s2), _ptr(b), _ptr(g2), outer, inner, int(or_n),
                                                         int(half_input), _stream())
        _lib.check(rc, "rexsc_orn_bias_std_pair_backward")
    return g2


def sc_counts_to_float(pos, neg, bit_length):
    """float(pos) / L - float(neg) / L in pos's layout (pos, neg: the int16 results of one SC conv call)."""
    _require_cuda(pos, neg)
    if pos.dtype != torch.int16 or neg.dtype != torch.int16 or pos.stride() != neg.stride():
        raise RuntimeError("sc_counts_to_float: expected two int16 tensors of one layout")
    y = torch.empty_like(pos, dtype=torch.float32)
    if y.stride() != pos.stride():
        raise RuntimeError("sc_counts_to_float: the SC result is not dense")
    with torch.cuda.device(pos.device):
        rc = _lib.lib().rexsc_sc_counts_to_float(_ptr(pos), _ptr(neg), _ptr(y), pos.numel(), int(bit_length),
                                                 _stream())
        _lib.check(rc, "rexsc_sc_counts_to_float")
    return y


def storage_flat(t, channels_last):
    """1-D view of a dense 4-D tensor in the order of its storage (2-D tensors: row major)."""
    if t.dim() == 4 and channels_last:
        return t.permute(0, 2, 3, 1).reshape(-1)
    return t.reshape(-1)


def sc_counts_pair(pos, neg, bit_length, outer, inner, channels_last):
    """float(pos) / L and float(neg) / L of one SC conv call laid out like the merged surrogate's sums,
    [outer][2][inner] (calibration only: plain torch ops)."""
    if channels_last:
        p2, n2 = pos.permute(0, 2, 3, 1).reshape(outer, inner), neg.permute(0, 2, 3, 1).reshape(outer, inner)
    else:
        p2, n2 = pos.reshape(outer, inner), neg.reshape(outer, inner)
    return torch.stack((p2, n2), dim=1).to(torch.float32).div_(bit_length)


def _weight_geometry(w):
    """(dense float32 w, O, C, taps, channels_last) of a conv [O,C,KH,KW] or linear [O,C] weight."""
    wd = _dense_f32(w)
    if wd.dim() == 2:
        return wd, wd.size(0), wd.size(1), 1, False
    O, C, KH, KW = wd.shape
    cl = not wd.is_contiguous()  # _dense_f32 leaves only the two dense orders
    return wd, O, C, KH * KW, cl


def _empty_weight(O, C, KH, KW, channels_last, device):
    if channels_last:
        return torch.empty((O, KH, KW, C), dtype=torch.float32, device=device).permute(0, 3, 1, 2)
    return torch.empty((O, C, KH, KW), dtype=torch.float32, device=device)


def split_weight(w, channels_last=None):
    """[clamp(w, 0, 100) ; -clamp(w, -100, 0)] along dim 0.  channels_last: memory order of the result
    (None: w's own), so that a channels-last convolution needs no filter conversion."""
    _require_cuda(w)
    wd, O, C, taps, w_cl = _weight_geometry(w)
    out_cl = w_cl if channels_last is None or wd.dim() == 2 else bool(channels_last)
    if wd.dim() == 2:
        w2 = torch.empty((2 * O, C), dtype=torch.float32, device=wd.device)
    else:
        w2 = _empty_weight(2 * O, C, wd.size(2), wd.size(3), out_cl, wd.device)
    with torch.cuda.device(wd.device):
        rc = _lib.lib().rexsc_split_weight(_ptr(wd), _ptr(w2), O, C, taps, int(w_cl), int(out_cl), _stream())
        _lib.check(rc, "rexsc_split_weight")
    return w2


def merge_weight_grad(dw2, w):
    """Gradient with respect to w of split_weight, given the gradient of its result (any dense order)."""
    wd, O, C, taps, w_cl = _weight_geometry(w)
    shape = (2 * O,) + tuple(wd.shape[1:])
    if tuple(dw2.shape) != shape:
        raise RuntimeError("merge_weight_grad: gradient shape %s does not match %s" % (tuple(dw2.shape), shape))
    d2 = _dense_f32(dw2)
    d2_cl = d2.dim() == 4 and not d2.is_contiguous()
    dw = torch.empty_like(wd)
    with torch.cuda.device(wd.device):
        rc = _lib.lib().rexsc_merge_weight_grad(_ptr(d2), _ptr(wd), _ptr(dw), O, C, taps, int(d2_cl), int(w_cl),
                                                _stream())
        _lib.check(rc, "rexsc_merge_weight_grad")
    return dw


def quantize(x, prec):
    """clamp(round(x * 2^prec), +-(2^prec - 1)) / 2^prec in one pass, in x's layout (float16 stays float16 for
    prec <= 10; everything else is computed and returned in float32)."""
    _require_cuda(x)
    if x.dtype == torch.float16 and 0 <= int(prec) <= 10:
        xd = x.detach()
        if not (xd.is_contiguous() or (xd.dim() == 4 and xd.is_contiguous(memory_format=torch.channels_last))):
            xd = xd.contiguous()
        if xd.data_ptr() % 8:
            xd = xd.clone(memory_format=torch.preserve_format)
        y = torch.empty_like(xd)
        with torch.cuda.device(xd.device):
            rc = _lib.lib().rexsc_quantize_f16(_ptr(xd), _ptr(y), xd.numel(), int(prec), _stream())
            _lib.check(rc, "rexsc_quantize_f16")
        return y
    xd = _dense_f32(x)
    y = torch.empty_like(xd)
    with torch.cuda.device(xd.device):
        rc = _lib.lib().rexsc_quantize(_ptr(xd), _ptr(y), xd.numel(), int(prec), _stream())
        _lib.check(rc, "rexsc_quantize")
    return y


def calib_stats(a_bit, a_act, win_lo, win_hi):
    """count / sum / sum-of-squares of (a_bit - a_act) per window, float64 [n_win, 3] on device."""
    _require_cuda(a_bit, a_act)
    ab = a_bit.detach().float().contiguous().view(-1)
    aa = a_act.detach().float().contiguous().view(-1)
    n_win = len(win_lo)
    lo = (ctypes.c_float * n_win)(*[float(v) for v in win_lo])
    hi = (ctypes.c_float * n_win)(*[float(v) for v in win_hi])
    stats = torch.empty((n_win, 3), dtype=torch.float64, device=ab.device)
    with torch.cuda.device(ab.device):
        rc = _lib.lib().rexsc_calib_stats(_ptr(ab), _ptr(aa), ab.numel(), lo, hi, n_win, _ptr(stats), _stream())
        _lib.check(rc, "rexsc_calib_stats")
    return stats
