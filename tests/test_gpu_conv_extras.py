"""The extras of rexsc_conv2d_orn_ex around the SC conv (producer / consumer fusion, utils_functional.py:1154,
1181-1182, 1273-1274; utils_class.py:54,62): float output written by the kernel that produces the sums, weight
streams kept while the weights do not change, fake quantisation folded into the stream generators."""
import numpy as np
import pytest
import torch

import oracle as orc

pytestmark = pytest.mark.gpu

CASES = [
    # N, C, H, W, O, K, stride, L, bin_config, cl_act
    (2, 64, 14, 14, 48, 3, 1, 32, 1, True),      # direct store, vector path
    (2, 64, 14, 14, 50, 3, 1, 32, 1, True),      # O % 4 != 0: scalar stores
    (2, 64, 14, 14, 48, 3, 1, 32, 1, False),     # NCHW
    (1, 512, 7, 7, 512, 3, 1, 32, 1, True),      # slot splits: finalize (narrow partials, vector path)
    (1, 512, 7, 7, 510, 3, 1, 64, 3, False),     # finalize, generic path, NCHW
    (1, 24, 10, 10, 20, 2, 1, 32, 1, False),     # no tuned instance: generic compute kernel
    (1, 96, 4, 4, 4, 3, 1, 256, 51200, False),   # sums beyond int16: the float value follows the wrapped int16
]


def _operands(cfg, seed=0):
    N, C, H, W, O, K, stride, L, bc, cla = cfg
    rng = np.random.default_rng(seed + C + O)
    dens = 1.0 if bc > 100 else min(1.0, 60.0 / (C * K * K) + 0.02)
    x = (rng.integers(0, L, size=(N, C, H, W)) / L * (rng.uniform(size=(N, C, H, W)) < dens)).astype(np.float32)
    w = (rng.integers(-L + 1, L, size=(O, C, K, K)) / L * (rng.uniform(size=(O, C, K, K)) < dens)).astype(np.float32)
    if bc > 100:
        w = np.abs(w)  # all weight on one polarity: its sums pass 32767 and wrap
    xt = torch.from_numpy(x).cuda()
    if cla:
        xt = xt.contiguous(memory_format=torch.channels_last)
    return x, w, xt, torch.from_numpy(w).cuda()


@pytest.mark.parametrize("cfg", CASES, ids=lambda c: "_".join(str(v) for v in c))
def test_float_output_equals_counts_over_L(cfg):
    import _ops
    N, C, H, W, O, K, stride, L, bc, cla = cfg
    print("float epilogue", cfg, flush=True)
    x, w, xt, wt = _operands(cfg)
    args = (xt, wt, L, -1, (K // 2, K // 2), (stride, stride), (7, 8, 1), bc, 1)
    pos, neg, diff, value = _ops.sc_conv2d(*args, want_split=True, want_diff=True, want_value=True)
    p0, n0, d0 = _ops.sc_conv2d(*args, want_split=True, want_diff=True)
    assert torch.equal(pos, p0) and torch.equal(neg, n0) and torch.equal(diff, d0)
    assert value.dtype == torch.float32 and value.stride() == pos.stride()
    assert torch.equal(value, pos.float() / L - neg.float() / L)
    assert torch.equal(value, _ops.sc_counts_to_float(pos, neg, L))
    # the float output alone (no int16 tensor is written)
    only = _ops.sc_conv2d(*args, want_split=False, want_value=True)
    assert only[0] is None and only[1] is None and only[2] is None and torch.equal(only[3], value)
    opos, oneg = orc.conv2d_generic_general_split(x, w, L, -1, 16, (K // 2, K // 2), (stride, stride), (7, 8, 1), bc, 1,
                                                  channels_last_activation=cla)
    assert np.array_equal(value.cpu().numpy(), opos.astype(np.float32) / np.float32(L) - oneg.astype(np.float32) / np.float32(L))
    if bc > 100:
        assert int(np.abs(opos.astype(np.int32)).max()) > 0 and (opos < 0).any()  # the 16-bit sums did wrap


def test_weight_stream_cache_reuse_and_invalidation():
    import _ops
    cfg = (2, 128, 14, 14, 64, 3, 1, 32, 1, True)
    x, w, xt, wt = _operands(cfg, seed=5)
    cache = _ops.WeightStreamCache()
    args = (xt, wt, 32, -1, (1, 1), (1, 1), (7, 8, 1), 1, 1)
    want = _ops.sc_conv2d(*args)
    a = _ops.sc_conv2d(*args, weight_cache=cache)
    assert (cache.hits, cache.misses) == (0, 1)
    b = _ops.sc_conv2d(*args, weight_cache=cache)
    assert (cache.hits, cache.misses) == (1, 1)
    for r in (a, b):
        assert torch.equal(r[0], want[0]) and torch.equal(r[1], want[1])
    # other activations, same weights: the kept streams serve
    x2 = torch.roll(xt, 1, 0).contiguous(memory_format=torch.channels_last)
    c = _ops.sc_conv2d(x2, *args[1:], weight_cache=cache)
    assert cache.hits == 2 and torch.equal(c[0], _ops.sc_conv2d(x2, *args[1:])[0])
    # an in-place update of the weights: same buffer, regenerated on the device
    with torch.no_grad():
        wt.mul_(-0.5)
    d = _ops.sc_conv2d(*args, weight_cache=cache)
    assert cache.misses == 1
    want2 = _ops.sc_conv2d(*args)
    assert torch.equal(d[0], want2[0]) and torch.equal(d[1], want2[1]) and not torch.equal(d[0], want[0])
    # in-place edits through .data, which neither move the storage nor bump the version counter
    version = wt._version
    wt.data.clamp_(-0.25, 0.125)
    assert wt._version == version
    d2 = _ops.sc_conv2d(*args, weight_cache=cache)
    want3 = _ops.sc_conv2d(*args)
    assert torch.equal(d2[0], want3[0]) and torch.equal(d2[1], want3[1]) and not torch.equal(d2[0], want2[0])
    # new storage behind the same tensor object
    wt.data = torch.from_numpy(w).cuda()
    e = _ops.sc_conv2d(*args, weight_cache=cache)
    assert cache.misses == 1 and torch.equal(e[0], want[0])
    # another batch size is another descriptor (its own entry); both stay valid
    f = _ops.sc_conv2d(xt[:1].contiguous(memory_format=torch.channels_last), *args[1:], weight_cache=cache)
    assert cache.misses == 2 and torch.equal(f[0], want[0][:1])
    g = _ops.sc_conv2d(*args, weight_cache=cache)
    assert cache.misses == 2 and torch.equal(g[0], want[0])


def test_kept_weight_streams_are_used_until_the_weights_change():
    """The device-side check really skips generation while the weights are unchanged (the streams in the buffer are
    what the call computes with -- shown by wiping them) and regenerates after a single-element edit."""
    import _ops
    cfg = (2, 64, 10, 10, 32, 3, 1, 32, 1, False)
    x, w, xt, wt = _operands(cfg, seed=9)
    cache = _ops.WeightStreamCache()
    args = (xt, wt, 32, -1, (1, 1), (1, 1), (7, 8, 1), 1, 1)
    want = _ops.sc_conv2d(*args)
    assert torch.equal(_ops.sc_conv2d(*args, weight_cache=cache)[0], want[0]) and int(want[0].max()) > 0
    (buf,) = cache.entries.values()
    keep = (wt.numel() * 4 + 255) // 256 * 256 + 256   # the copy of the weights and the change flag close the buffer
    buf[:buf.numel() - keep].zero_()                    # wipe streams and tables
    wiped = _ops.sc_conv2d(*args, weight_cache=cache)
    assert int(wiped[0].abs().max()) == 0 and int(wiped[1].abs().max()) == 0   # nothing was regenerated
    wt.data.view(-1)[-1] += 0.25                        # one element, through .data
    again = _ops.sc_conv2d(*args, weight_cache=cache)
    want2 = _ops.sc_conv2d(*args)
    assert torch.equal(again[0], want2[0]) and torch.equal(again[1], want2[1])
    assert torch.equal(_ops.sc_conv2d(*args, weight_cache=cache)[0], want2[0])


@pytest.mark.parametrize("cfg", [(2, 128, 14, 14, 64, 3, 1, 32, 1, True), (4, 3, 16, 16, 32, 3, 1, 64, 2, False)],
                         ids=["c128", "c3_folded_taps"])
def test_weight_streams_prepared_ahead_on_a_second_stream(cfg):
    """rexsc_conv2d_prepare_weights on a side stream, the conv call proper on the caller's stream after an event:
    same results as the one-call form; the buffer is reused for new weight values; a buffer made for another
    descriptor is refused."""
    import _ops
    x, w, xt, wt = _operands(cfg, seed=21)
    N, C, H, W, O, K, stride, L, bc, cla = cfg
    args = (L, -1, (K // 2, K // 2), (stride, stride), (7, 8, 1), bc, 1)
    want = _ops.sc_conv2d(xt, wt, *args)
    side = torch.cuda.Stream()
    cur = torch.cuda.current_stream()
    prepared = None
    for rnd in range(3):
        if rnd == 2:
            wt.data.mul_(-0.5)
            want = _ops.sc_conv2d(xt, wt, *args)
        side.wait_stream(cur)
        with torch.cuda.stream(side):
            prepared = _ops.sc_conv2d_prepare_weights(((N, C, H, W), cla), wt, *args, into=prepared)
            ev = torch.cuda.Event()
            ev.record(side)
        cur.wait_event(ev)
        got = _ops.sc_conv2d(xt, wt, *args, prepared=prepared)
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]) and int(want[0].max()) > 0
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError, match="another call"):
        _ops.sc_conv2d(xt[:1].contiguous(memory_format=torch.channels_last if cla else torch.contiguous_format), wt, *args,
                       prepared=prepared)


def _oracle_layer_value(x, w, prec, L, padding, stride, cla):
    xq, wq = orc.quantize(x.cpu().numpy(), prec), orc.quantize(w.cpu().numpy(), prec)
    opos, oneg = orc.conv2d_generic_general_split(xq, wq, L, -1, 16, padding, stride, (7, 8, 1), 1, 1,
                                                  channels_last_activation=cla)
    return opos.astype(np.float32) / np.float32(L) - oneg.astype(np.float32) / np.float32(L)


def _edit_weight_data(weight, edit):
    if edit == "clamp":          # literally the reference's line (the layers' quantisation clamps tighter anyway)
        weight.data.clamp_(-1, 0.999)
    elif edit == "clamp_tight":  # a clamp that does change the quantised weights
        weight.data.clamp_(-0.25, 0.125)
    else:
        weight.data.mul_((torch.rand_like(weight) < 0.5).float())


@pytest.mark.parametrize("edit", ["clamp", "clamp_tight", "mask"])
def test_evaluation_after_inplace_data_edit_conv(edit):
    """eval -> weight.data.<op>_() -> eval (the reference's own loop clamps this way, utils_own.py:187-190):
    the second evaluation must be that of the NEW weights, against the oracle."""
    from sc_layers import Conv2d_Add_Partial
    torch.manual_seed(11)
    layer = Conv2d_Add_Partial(40, 24, kernel_size=3, padding=1, bias=False, forward="or_2", err=5).cuda().eval()
    with torch.no_grad():
        layer.weight.mul_(6.0)   # some weights beyond +-1, so that the clamp changes values
    x = (torch.rand(2, 40, 9, 9, device="cuda") * 1.1 - 0.05).contiguous(memory_format=torch.channels_last)
    with torch.no_grad():
        y1 = layer(x)
    assert np.array_equal(y1.cpu().numpy(), _oracle_layer_value(x, layer.weight.data, 7, 32, (1, 1), (1, 1), True))
    version = layer.weight._version
    _edit_weight_data(layer.weight, edit)
    assert layer.weight._version == version
    with torch.no_grad():
        y2 = layer(x)
    assert (layer._weight_streams.hits, layer._weight_streams.misses) == (1, 1)
    assert np.array_equal(y2.cpu().numpy(), _oracle_layer_value(x, layer.weight.data, 7, 32, (1, 1), (1, 1), True))
    assert edit == "clamp" or not torch.equal(y1, y2)


@pytest.mark.parametrize("edit", ["clamp", "clamp_tight", "mask"])
def test_evaluation_after_inplace_data_edit_linear(edit):
    import sc_functional as uf
    from sc_layers import Linear_Or
    torch.manual_seed(12)
    layer = Linear_Or(96, 40, bias=False, forward="or_2", err=6).cuda().eval()
    with torch.no_grad():
        layer.weight.mul_(12.0)
    x = torch.rand(5, 96, device="cuda") * 1.1 - 0.05

    def oracle_value():
        xq = orc.quantize(x.cpu().numpy(), 7)
        wq = orc.quantize(layer.weight.data.cpu().numpy(), 7)
        pos, neg = orc.linear_generic_general(xq, wq, (7, 8, 1), 64, -1, 1, 1, True, False)
        return (pos.astype(np.float32) - neg.astype(np.float32)) / 64

    with torch.no_grad():
        y1 = layer(x)
    assert np.array_equal(y1.cpu().numpy(), oracle_value())
    _edit_weight_data(layer.weight, edit)
    with torch.no_grad():
        y2 = layer(x)
    assert (layer._weight_streams.hits, layer._weight_streams.misses) == (1, 1)
    assert np.array_equal(y2.cpu().numpy(), oracle_value()) and (edit == "clamp" or not torch.equal(y1, y2))
    # entering training mode and loading a state dict give the kept streams back
    layer.train()
    assert not layer._weight_streams.entries
    layer.eval()
    with torch.no_grad():
        layer(x)
    layer.load_state_dict(layer.state_dict())
    assert not layer._weight_streams.entries


@pytest.mark.parametrize("sng_mode", ["1", "2"])
@pytest.mark.parametrize("cla", [False, True])
def test_fake_quantisation_folded_into_the_generators(cla, sng_mode, monkeypatch):
    import _ops
    import sc_functional as uf
    monkeypatch.setenv("REXSC_SNG_MODE", sng_mode)
    g = torch.Generator().manual_seed(3)
    x = (torch.rand(2, 40, 9, 9, generator=g) * 1.3 - 0.15).cuda()      # off-grid, below 0 and above 1
    w = ((torch.rand(24, 40, 3, 3, generator=g) * 2.4 - 1.2) * (torch.rand(24, 40, 3, 3, generator=g) < 0.2)).cuda()
    x[0, 0, 0, :6] = torch.tensor([0.5 / 128, 1.5 / 128, 2.5 / 128, 127.5 / 128, 1.0, -0.5 / 128])  # ties: half to even
    if cla:
        x = x.contiguous(memory_format=torch.channels_last)
    for L, prec in ((32, 7), (64, 7), (32, 3)):
        args = (L, -1, (1, 1), (1, 1), (7, 8, 1), 1, 1)
        want = _ops.sc_conv2d(uf.quantize(x, prec), uf.quantize(w, prec), *args)
        got = _ops.sc_conv2d(x, w, *args, act_fake_quant=prec, weight_fake_quant=prec)
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
        assert int(want[0].max()) > 0
    xq = orc.quantize(x.cpu().numpy(), 7)
    wq = orc.quantize(w.cpu().numpy(), 7)
    opos, oneg = orc.conv2d_generic_general_split(xq, wq, 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 1, channels_last_activation=cla)
    got = _ops.sc_conv2d(x, w, 32, -1, (1, 1), (1, 1), (7, 8, 1), 1, 1, act_fake_quant=7, weight_fake_quant=7)
    assert np.array_equal(got[0].cpu().numpy(), opos) and np.array_equal(got[1].cpu().numpy(), oneg)


def test_layer_evaluation_path_equals_training_forward(monkeypatch):
    from sc_layers import Conv2d_Add_Partial
    torch.manual_seed(4)
    layer = Conv2d_Add_Partial(32, 48, kernel_size=3, padding=1, stride=2, bias=False, forward="or_2", err=5).cuda()
    x = (torch.rand(3, 32, 12, 12, device="cuda") * 1.2 - 0.1).contiguous(memory_format=torch.channels_last)
    y_train = layer(x.clone().requires_grad_(True)).detach()
    with torch.no_grad():
        y1 = layer(x)
        y2 = layer(x)
    assert torch.equal(y1, y_train) and torch.equal(y2, y_train) and y1.stride() == y_train.stride()
    assert (layer._weight_streams.hits, layer._weight_streams.misses) == (1, 1)
    # an optimiser step changes the weights in place: the next evaluation regenerates the streams
    opt = torch.optim.SGD(layer.parameters(), lr=0.5)
    layer(x.clone().requires_grad_(True)).square().sum().backward()
    opt.step()
    with torch.no_grad():
        y3 = layer(x)
    assert layer._weight_streams.misses == 1  # same buffer: the device noticed the new values
    assert torch.equal(y3, layer(x.clone().requires_grad_(True)).detach()) and not torch.equal(y3, y1)
    # switched off: same values, nothing cached
    monkeypatch.setenv("REXSC_WEIGHT_STREAM_CACHE", "0")
    calls = layer._weight_streams.hits + layer._weight_streams.misses
    with torch.no_grad():
        y4 = layer(x)
    assert torch.equal(y4, y3) and layer._weight_streams.hits + layer._weight_streams.misses == calls
    assert "_weight_streams" not in layer.state_dict()


def test_linear_layer_evaluation_path_and_weight_stream_cache(monkeypatch):
    """Linear_Or under no_grad: same values as its training forward, weight bitstreams kept in one buffer for any
    batch size, and straight against the oracle on the quantised operands."""
    import sc_functional as uf
    from sc_layers import Linear_Or
    torch.manual_seed(6)
    layer = Linear_Or(96, 40, bias=False, forward="or_2", err=6).cuda()
    with torch.no_grad():
        layer.weight.mul_(4.0)
    x = torch.rand(5, 96, device="cuda") * 1.1 - 0.05
    y_train = layer(x.clone().requires_grad_(True)).detach()
    with torch.no_grad():
        y1 = layer(x)
        y2 = layer(x)
        y_small = layer(x[:2])          # another batch size shares the entry
    assert torch.equal(y1, y_train) and torch.equal(y2, y_train) and torch.equal(y_small, y_train[:2])
    assert (layer._weight_streams.hits, layer._weight_streams.misses) == (2, 1)
    xq = uf.quantize(x, 7).cpu().numpy()
    wq = uf.quantize(layer.weight.data, 7).cpu().numpy()
    pos, neg = orc.linear_generic_general(xq, wq, (7, 8, 1), 64, -1, 1, 1, True, False)
    assert np.array_equal(y1.cpu().numpy(), (pos.astype(np.float32) - neg.astype(np.float32)) / 64) and np.abs(pos).max() > 0
    opt = torch.optim.SGD(layer.parameters(), lr=0.5)
    layer(x.clone().requires_grad_(True)).square().sum().backward()
    opt.step()
    with torch.no_grad():
        y3 = layer(x)
    assert layer._weight_streams.misses == 1
    assert torch.equal(y3, layer(x.clone().requires_grad_(True)).detach()) and not torch.equal(y3, y1)
    monkeypatch.setenv("REXSC_WEIGHT_STREAM_CACHE", "0")
    calls = layer._weight_streams.hits + layer._weight_streams.misses
    with torch.no_grad():
        y4 = layer(x)
    assert torch.equal(y4, y3) and layer._weight_streams.hits + layer._weight_streams.misses == calls
    assert "_weight_streams" not in layer.state_dict()


FOLD_CASES = [
    # N, C, H, W, O, KH, KW, stride, pad, L, bin_config, gen, cl_act, cl_w
    (4, 3, 32, 32, 32, 3, 3, (1, 1), (1, 1), 64, 2, 1, False, False),   # TinyConv's first layer (OR-3, 64-bit streams)
    (2, 3, 17, 13, 20, 3, 3, (2, 1), (1, 0), 32, 1, 1, True, True),     # strides, asymmetric padding, both channels-last
    (2, 1, 12, 12, 8, 5, 5, (1, 1), (2, 2), 32, 1, 1, False, False),    # 25 taps of one channel
    (1, 2, 9, 9, 5, 4, 4, (1, 1), (1, 1), 16, 0, 1, False, False),      # a kernel width without an unfolded instance, OR-1
    (2, 3, 10, 10, 12, 3, 3, (1, 1), (1, 1), 32, 1, 2, False, False),   # and_2 generator
    (1, 8, 8, 8, 40, 2, 2, (2, 2), (0, 0), 128, 3, 1, False, False),    # exactly 32 bits
    (3, 3, 6, 6, 4, 3, 3, (1, 1), (1, 1), 256, 51200, 1, False, False), # full_bin
]


@pytest.mark.parametrize("cfg", FOLD_CASES, ids=lambda c: "_".join(str(v) for v in c).replace(" ", ""))
def test_tap_folding_is_bit_exact(cfg, monkeypatch):
    """Layers whose receptive field fits one 32-bit word run on regrouped streams (one word per output pixel);
    same sums as the tap-by-tap kernel and as the oracle."""
    import ctypes
    import _lib
    import _ops
    N, C, H, W, O, KH, KW, stride, pad, L, bc, gen, cla, clw = cfg
    print("tap folding", cfg, flush=True)
    rng = np.random.default_rng(hash(cfg) & 0xFFFF)
    x = (rng.integers(0, L, size=(N, C, H, W)) / L).astype(np.float32)
    w = (rng.integers(-L + 1, L, size=(O, C, KH, KW)) / L).astype(np.float32)
    xt, wt = torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()
    if cla:
        xt = xt.contiguous(memory_format=torch.channels_last)
    if clw:
        wt = wt.contiguous(memory_format=torch.channels_last)
    args = (xt, wt, L, -1, pad, stride, (7, 8, 1), bc, gen)
    d = _lib.ConvDesc(N, C, H, W, O, KH, KW, pad[1], pad[0], stride[0], stride[1], L, -1, gen, bc, 7, 8, 1, int(cla), int(clw))
    info = (ctypes.c_int64 * 16)()
    _lib.check(_lib.lib().rexsc_conv2d_plan_info(ctypes.byref(d), info), "plan_info")
    assert info[1] == 1 and info[0] == 1  # planned as a 1x1 layer on a tuned instance
    pos, neg, _, value = _ops.sc_conv2d(*args, want_value=True)
    opos, oneg = orc.conv2d_generic_general_split(x, w, L, -1, 16, pad, stride, (7, 8, 1), bc, gen,
                                                  channels_last_activation=cla, channels_last_weight=clw)
    assert opos.max() > 0
    assert np.array_equal(pos.cpu().numpy(), opos) and np.array_equal(neg.cpu().numpy(), oneg)
    assert torch.equal(value, pos.float() / L - neg.float() / L)
    cache = _ops.WeightStreamCache()
    for _ in range(2):  # folded weight streams are cached with the rest
        p2 = _ops.sc_conv2d(*args, weight_cache=cache)[0]
        assert torch.equal(p2, pos)
    assert cache.hits == 1
    monkeypatch.setenv("REXSC_FOLD_TAPS", "0")
    _lib.check(_lib.lib().rexsc_conv2d_plan_info(ctypes.byref(d), info), "plan_info")
    assert info[1] == KW
    p0, n0, _ = _ops.sc_conv2d(*args)
    assert torch.equal(p0, pos) and torch.equal(n0, neg)
