"""Host-side logic that needs no GPU: the weight-stream cache's keying, the planner's invariants over many shapes
(through rexsc_conv2d_plan_info, which runs on the host), the legacy linear_generic's argument checks and the
choice between the merged and the two-convolution surrogate."""
import ctypes

import numpy as np
import pytest
import torch

import _lib
import _ops


def test_weight_stream_cache_keys_and_modes(monkeypatch):
    cache = _ops.WeightStreamCache(max_entries=2)
    key_a = ("conv", 1, 2, 3)
    buf, mode = cache.lookup(key_a, 1000, "cpu")
    assert mode == _lib.WSTREAMS_FILL and buf.numel() >= 1000 and cache.misses == 1
    buf2, mode2 = cache.lookup(key_a, 1000, "cpu")
    assert mode2 == _lib.WSTREAMS_VERIFY and buf2 is buf and cache.hits == 1   # never TRUST: the device decides
    # another size, another descriptor, another buffer layout (tap folding, generator choice): other buffers
    assert cache.lookup(key_a, 2000, "cpu")[1] == _lib.WSTREAMS_FILL
    monkeypatch.setenv("REXSC_FOLD_TAPS", "0")
    assert cache.lookup(key_a, 1000, "cpu")[1] == _lib.WSTREAMS_FILL
    monkeypatch.delenv("REXSC_FOLD_TAPS")
    monkeypatch.setenv("REXSC_SNG_MODE", "1")
    assert cache.lookup(key_a, 1000, "cpu")[1] == _lib.WSTREAMS_FILL
    assert len(cache.entries) <= 2                                              # oldest entries were dropped
    cache.clear()
    assert cache.lookup(key_a, 1000, "cpu")[1] == _lib.WSTREAMS_FILL


def test_descriptor_keys_tell_calls_apart():
    a = _lib.ConvDesc(2, 16, 8, 8, 8, 3, 3, 1, 1, 1, 1, 32, -1, 1, 1, 7, 8, 1, 0, 0)
    b = _lib.ConvDesc(2, 16, 8, 8, 8, 3, 3, 1, 1, 1, 1, 32, -1, 1, 1, 7, 8, 1, 0, 0)
    c = _lib.ConvDesc(2, 16, 8, 8, 8, 3, 3, 1, 1, 1, 1, 64, -1, 1, 1, 7, 8, 1, 0, 0)
    assert a.key() == b.key() and a.key() != c.key()
    assert a.struct_size == ctypes.sizeof(_lib.ConvDesc)


NAMES = "tuned KW ZC ZG O_pad px ns splits sps n_slots direct n_chunk M Hp Wp wide".split()


def _plan(d):
    out = (ctypes.c_int64 * 16)()
    rc = _lib.lib().rexsc_conv2d_plan_info(ctypes.byref(d), out)
    return rc, dict(zip(NAMES, out))


def test_planner_invariants_over_random_shapes():
    """Whatever the shape, a plan covers every channel, output and slot exactly once and its workspace is positive."""
    rng = np.random.default_rng(5)
    L_ = _lib.lib()
    for _ in range(400):
        K = int(rng.choice([1, 3, 5, 7, 2]))
        C, O = int(rng.integers(1, 700)), int(rng.integers(1, 600))
        H, W = int(rng.integers(K, 60)), int(rng.integers(K, 60))
        N = int(rng.choice([1, 2, 7, 64, 256]))
        s = int(rng.integers(1, 3))
        L = int(rng.choice([2, 8, 32, 64, 128, 256]))
        if 32 * K * K * ((C + 31) // 32) >= 65536:
            continue
        d = _lib.ConvDesc(N, C, H, W, O, K, K, K // 2, K // 2, s, s, L, -1, 1, int(rng.integers(0, 4)), 7, 8, 1,
                          int(rng.integers(0, 2)), 0)
        rc, p = _plan(d)
        assert rc == 0, (N, C, H, W, O, K, s, L, L_.rexsc_last_error())
        Ho = (H + 2 * (K // 2) - K) // s + 1
        Wo = (W + 2 * (K // 2) - K) // s + 1
        assert 32 * p["ZC"] * p["ZG"] >= (C if p["KW"] == K else 1)        # every channel has a word (folded layers: one word)
        assert p["O_pad"] >= O and p["O_pad"] % 16 == 0
        assert p["px"] in (1, 2) and p["ns"] in (1, 2, 4) and p["splits"] in (1, 2, 4, 8, 16)
        assert p["splits"] * p["sps"] >= p["n_slots"] > (p["splits"] - 1) * p["sps"]  # slot shares tile the stream
        assert bool(p["direct"]) == (p["splits"] == 1) or not p["tuned"]
        assert 1 <= p["n_chunk"] <= N and p["M"] == p["n_chunk"] * Ho * Wo
        assert L_.rexsc_conv2d_workspace_bytes(ctypes.byref(d)) > 0


def test_linear_generic_rejects_what_the_reference_cannot_reproduce():
    import sc_functional as uf
    x, w = torch.zeros(2, 8), torch.zeros(4, 8)
    for gen in ("lfsr_split", "rand", "nonsense"):
        with pytest.raises((ValueError, RuntimeError)) as e:
            uf.linear_generic(x, w, generator=gen)
        assert "generator" in str(e.value)


def test_merged_surrogate_choice_on_the_host(monkeypatch):
    """CPU tensors, other dtypes, split outputs and the switch all take the two-convolution path."""
    import sc_functional as uf
    x, w = torch.zeros(2, 8, 6, 6), torch.zeros(4, 8, 3, 3)
    ok = lambda a, b, **kw: uf._merged_surrogate_ok(a, b, kw.get("forward", "or_2"), 2, kw.get("sync", 1), True,
                                                    kw.get("split", False), (1, 1), (1, 1))
    assert not ok(x, w)                                   # not on the GPU
    assert not ok(x.double(), w)
    assert not ok(x, w, split=True)
    assert not ok(x, w, forward="or_2_1")                 # no fused kernel for the approximations
    monkeypatch.setenv("REXSC_MERGED_SURROGATE", "0")
    assert not ok(x, w)


def test_bench_refuses_more_than_one_gpu():
    """The path has no collectives: bench.py --gpus N > 1 exits with a message instead of printing a number."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode != 0 and "one GPU" in proc.stderr and proc.stdout.strip() == ""
