"""The reference's legacy `linear_generic` simulation (utils_functional.py:955-1081) on the HIP kernels
(rexsc_linear_legacy through the C ABI): against the vectors written by the reference's own function, against
the numpy oracle on larger seeded shapes, gradients of its float surrogate, and the legacy Linear_Or layer."""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle as orc

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_g = np.load(os.path.join(ROOT, "tests", "golden", "ref_linear_legacy.npz"), allow_pickle=False)
_cases = json.loads(bytes(_g["meta"]).decode())


@pytest.mark.parametrize("sng_mode", ["0", "1", "2"])
@pytest.mark.parametrize("case", _cases, ids=lambda c: c["name"])
def test_legacy_linear_golden(case, sng_mode, monkeypatch):
    import sc_functional as uf
    monkeypatch.setenv("REXSC_SNG_MODE", sng_mode)
    n = case["name"]
    print("legacy linear golden", n, "sng mode", sng_mode, flush=True)
    x, w = torch.from_numpy(_g[n + "/x"]).cuda(), torch.from_numpy(_g[n + "/w"]).cuda()
    y = uf.linear_generic(x, w, bit_length=case["bit_length"], forward=case["forward"], generator="lfsr",
                          share=case.get("share", True))
    assert y.dtype == torch.float32
    assert np.array_equal(y.cpu().numpy(), _g[n + "/y"])


SHAPES = [
    # B, C, O, L, forward, kind
    (64, 512, 40, 128, "full_or", "q7"),
    (33, 1000, 17, 32, "full_or", "plain"),
    (256, 4096, 32, 64, "full_or", "q7"),
    (16, 300, 24, 16, "full_bin", "plain"),
    (8, 4096, 12, 128, "full_bin", "q7"),      # sums above 65535: wide accumulators
    (5, 37, 3, 8, "full_or", "q7"),
    (40, 300, 50, 32, "full_or", "q7", False),     # share=False: one generator per element
    (9, 1000, 33, 128, "full_bin", "plain", False),
]


@pytest.mark.parametrize("cfg", SHAPES, ids=lambda c: "_".join(str(v) for v in c))
def test_legacy_linear_vs_oracle(cfg):
    import _ops
    B, C, O, L, forward, kind = cfg[:6]
    share = cfg[6] if len(cfg) > 6 else True
    print("legacy linear", cfg, flush=True)
    rng = np.random.default_rng(hash(cfg) & 0xFFFF)
    dens = 1.0 if forward == "full_bin" else min(1.0, 12.0 / np.sqrt(C) / 4)
    if kind == "plain":
        x = rng.uniform(-0.2, 1.1, size=(B, C))
        w = rng.uniform(-1.2, 1.2, size=(O, C))
    else:
        x = np.round(rng.uniform(0, 1, size=(B, C)) * 128).clip(0, 127) / 128
        w = np.round(rng.uniform(-1, 1, size=(O, C)) * 128).clip(-127, 127) / 128
    x = (x * (rng.uniform(size=x.shape) < dens)).astype(np.float32)
    w = (w * (rng.uniform(size=w.shape) < dens)).astype(np.float32)
    pos, neg = _ops.sc_linear_legacy(torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda(), L,
                                     0 if forward == "full_or" else 51200, share=share)
    assert pos.dtype == torch.int32
    mean = lambda t: (t.float() / L).half().float().cpu().numpy()
    want = orc.linear_generic_legacy(x, w, L, forward, share=share)
    assert np.abs(want).max() > 0
    assert np.array_equal(mean(pos) - mean(neg), want)
    if forward == "full_bin" and C >= 4096:
        assert int(pos.max()) > 65535
    # the positive sums do not depend on the negative weights and vice versa (separate passes, separate seeds)
    p2, _ = _ops.sc_linear_legacy(torch.from_numpy(x).cuda(), torch.from_numpy(np.maximum(w, 0)).cuda(), L,
                                  0 if forward == "full_or" else 51200, share=share)
    assert torch.equal(p2, pos)


def test_legacy_linear_gradients_and_layer():
    import sc_functional as uf
    from sc_layers import Linear_Or
    g = torch.Generator().manual_seed(11)
    x = (torch.rand(12, 96, generator=g) * (torch.rand(12, 96, generator=g) < 0.2)).cuda().requires_grad_(True)
    w = ((torch.rand(10, 96, generator=g) * 2 - 1) * (torch.rand(10, 96, generator=g) < 0.3)).cuda().requires_grad_(True)
    y = uf.linear_generic(x, w, bit_length=64, forward="full_or", generator="lfsr")
    go = torch.randn(12, 10, generator=g)
    y.backward(go.cuda())
    x64, w64 = x.detach().cpu().double().requires_grad_(True), w.detach().cpu().double().requires_grad_(True)
    s = (1 - torch.exp(-F.linear(x64, w64.clamp(0, 100)))) - (1 - torch.exp(-F.linear(x64, -(w64.clamp(-100, 0)))))
    s.backward(go.double())
    assert (x.grad.cpu().double() - x64.grad).abs().max() <= 1e-5 * x64.grad.abs().max()
    assert (w.grad.cpu().double() - w64.grad).abs().max() <= 1e-5 * w64.grad.abs().max()
    with pytest.raises(ValueError, match="generator"):
        uf.linear_generic(x, w, bit_length=64, forward="full_or", generator="rand")
    with pytest.raises(RuntimeError, match="legacy linear"):
        uf.linear_generic(x, w, bit_length=256, forward="full_or", generator="lfsr")
    # the layer: quantise (prec 7) in place, 128-bit streams, full OR
    torch.manual_seed(2)
    layer = Linear_Or(96, 10, bias=False, legacy=True).cuda()
    xin = torch.rand(7, 96, device="cuda") * (torch.rand(7, 96, device="cuda") < 0.3)
    x0 = xin.clone()
    out = layer(xin)
    xq = orc.quantize(x0.cpu().numpy(), 7)
    assert np.array_equal(xin.cpu().numpy(), xq)  # the reference's layer quantises its input in place
    wq = orc.quantize(layer.weight.detach().cpu().numpy(), 7)
    assert np.array_equal(out.detach().cpu().numpy(), orc.linear_generic_legacy(xq, wq, 128, "full_or"))
