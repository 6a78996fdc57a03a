"""The ops under HIP graph capture: nothing in the library may synchronise, allocate or memset on
the stream, so a captured call must replay with new operand values and give what the eager call
gives.  Every replay is checked, with eager work and synchronisation between the replays."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _capture(fn, warmup=2):
    """Run fn eagerly on a side stream (first calls build per-device tables), then capture it."""
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(warmup):
            fn()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = fn()
    return g, out


def _check_replays(g, out, eager, refill, n_replays=3):
    outs = out if isinstance(out, (tuple, list)) else (out,)
    for r in range(n_replays):
        refill(r)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want = eager()
        want = want if isinstance(want, (tuple, list)) else (want,)
        torch.cuda.synchronize()
        for a, b in zip(outs, want):
            assert torch.equal(a, b), "replay %d differs from the eager call" % r


@pytest.mark.parametrize("sng", ["1", "2"])
def test_conv_graph(sng, monkeypatch):
    import sc_extension_cuda
    monkeypatch.setenv("REXSC_SNG_MODE", sng)
    print("graph conv", sng, flush=True)
    rng = np.random.default_rng(1)
    x = torch.zeros(4, 48, 12, 12, device="cuda").contiguous(memory_format=torch.channels_last)
    w = torch.zeros(40, 48, 3, 3, device="cuda")

    def refill(r):
        x.copy_(torch.from_numpy((rng.integers(0, 33, size=x.shape) / 32).astype(np.float32)))
        w.copy_(torch.from_numpy((rng.integers(-32, 33, size=w.shape) / 32).astype(np.float32)))

    refill(-1)
    fn = lambda: sc_extension_cuda.conv2d_generic_general_split_acc(x, w, 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 1,
                                                                    True, False)
    g, out = _capture(fn)
    _check_replays(g, out, fn, refill)


def test_linear_graph():
    import sc_extension_cuda
    print("graph linear", flush=True)
    rng = np.random.default_rng(2)
    x = torch.zeros(70, 200, device="cuda")
    w = torch.zeros(33, 200, device="cuda")

    def refill(r):
        x.copy_(torch.from_numpy((rng.integers(0, 65, size=x.shape) / 64).astype(np.float32)))
        w.copy_(torch.from_numpy((rng.integers(-64, 65, size=w.shape) / 64).astype(np.float32)))

    refill(-1)
    fn = lambda: sc_extension_cuda.linear_generic_general_acc(x, w, (7, 8, 1), 64, -1, 1, 1, True, False)
    g, out = _capture(fn)
    _check_replays(g, out, fn, refill)


def test_fixed_conv_and_pointwise_graph():
    import fixed_extension_cuda
    import sc_extension_cuda
    print("graph fixed + pointwise", flush=True)
    rng = np.random.default_rng(3)
    x = torch.zeros(2, 32, 10, 10, device="cuda")
    w = torch.zeros(24, 32, 3, 3, device="cuda")

    def refill(r):
        x.copy_(torch.from_numpy((rng.integers(0, 32, size=x.shape) / 32).astype(np.float32)))
        w.copy_(torch.from_numpy((rng.integers(-31, 32, size=w.shape) / 32).astype(np.float32)))

    refill(-1)

    def fn():
        y = fixed_extension_cuda.conv2d_saturate_acc(x, w, 0, 5, 24, (1, 1), (1, 1))
        return y, sc_extension_cuda.or_approx_n_forward_acc(y.float().abs() / 65536.0, 2)  # keep OR-2 finite

    g, out = _capture(fn)
    _check_replays(g, out, fn, refill)


def test_error_injection_draws_new_noise_on_every_replay():
    """A captured noise kernel has its host arguments frozen; its offset lives in device memory and
    is advanced inside the graph, so replays differ from each other the way eager calls do."""
    import sc_extension_cuda
    print("graph noise", flush=True)
    x = torch.rand(20000, device="cuda")
    coef0 = torch.zeros(6, device="cuda")
    std = torch.tensor([0.25, 0, 0, 0, 0, 0], device="cuda")
    fn = lambda: sc_extension_cuda.or_approx_n_forward_bias_std_both_acc(x, x, coef0, std, 2)
    g, out = _capture(fn)
    seen = []
    for r in range(4):
        g.replay()
        torch.cuda.synchronize()
        seen.append(out.clone())
        _ = fn()                      # eager work between the replays
        torch.cuda.synchronize()
    for i in range(4):
        for j in range(i):
            d = (seen[i] - seen[j]) / 0.25
            assert not torch.equal(seen[i], seen[j])
            assert abs(float(d.var()) - 4.0) < 0.3   # four independent N(0,1) draws per element
        assert abs(float(seen[i].mean())) < 0.02     # same operand on both polarities: zero-mean output
