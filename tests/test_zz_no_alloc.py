"""rexsc_conv2d_orn_noalloc (workspace in the library's static device array) against rexsc_conv2d_orn
(caller-owned workspace), through the C ABI: bit-exact, two calls in a row, the second one smaller; no device memory
is taken by a call; and the use it exists for -- a call recorded into a HIP graph on a non-default stream and replayed."""
import ctypes

import pytest
import torch

import _lib

pytestmark = pytest.mark.gpu


def _p(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _both(N, C, H, W, O, K, stride, L, bin_config, channels_last, seed):
    L_ = _lib.lib()
    g = torch.Generator().manual_seed(seed)
    x = (torch.randint(0, L, (N, C, H, W), generator=g).float() / L).to("cuda")
    w = (torch.randint(-L + 1, L, (O, C, K, K), generator=g).float() / L * (torch.rand(O, C, K, K, generator=g) < 0.3)).to("cuda")
    if channels_last:
        x = x.contiguous(memory_format=torch.channels_last)
    d = _lib.ConvDesc(N, C, H, W, O, K, K, K // 2, K // 2, stride, stride, L, -1, 1, bin_config, 7, 8, 1,
                      int(channels_last), 0)
    Ho = (H + 2 * (K // 2) - K) // stride + 1
    n_out = N * O * Ho * Ho
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ws_bytes = L_.rexsc_conv2d_workspace_bytes(ctypes.byref(d))
    assert 0 < ws_bytes <= _lib.NOALLOC_SCRATCH_BYTES
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    outs = [torch.full((n_out,), -7, dtype=torch.int16, device="cuda") for _ in range(6)]
    print("no-alloc case", (N, C, H, W, O, K, stride, L, bin_config, channels_last, seed), "workspace", ws_bytes, flush=True)
    rc = L_.rexsc_conv2d_orn(ctypes.byref(d), _p(x), _p(w), _p(outs[0]), _p(outs[1]), _p(outs[2]), _p(ws), ws_bytes, stream)
    _lib.check(rc, "rexsc_conv2d_orn")
    rc = L_.rexsc_conv2d_orn_noalloc(ctypes.byref(d), _p(x), _p(w), _p(outs[3]), _p(outs[4]), _p(outs[5]), stream)
    _lib.check(rc, "rexsc_conv2d_orn_noalloc")
    torch.cuda.synchronize()
    for a, b in zip(outs[:3], outs[3:]):
        assert torch.equal(a, b)
    assert int(outs[0].max()) > 0  # the case is not trivially zero


def test_noalloc_matches_workspace_entry_point_twice():
    _lib.check(_lib.lib().rexsc_init(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)), "rexsc_init")
    # first call: split partials and the bit-sliced generator's table in use (ResNet-18 stage-3 shape, batch 2)
    _both(2, 256, 14, 14, 256, 3, 1, 32, 1, True, seed=11)
    # second call, smaller problem in the same (now dirty) scratch array: NCHW, odd channel count, stride 2, OR-1
    _both(1, 33, 9, 9, 20, 3, 2, 16, 0, False, seed=12)
    # and once more the first shape: contents left by the smaller call must not matter
    _both(2, 256, 14, 14, 256, 3, 1, 32, 1, True, seed=13)


def test_noalloc_rejects_oversized_problems():
    L_ = _lib.lib()
    d = _lib.ConvDesc(64, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 32, -1, 1, 1, 7, 8, 1, 1, 0)
    assert L_.rexsc_conv2d_workspace_bytes(ctypes.byref(d)) > _lib.NOALLOC_SCRATCH_BYTES
    x = torch.zeros(1, device="cuda")
    rc = L_.rexsc_conv2d_orn_noalloc(ctypes.byref(d), _p(x), _p(x), _p(x), _p(x), None,
                                     ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == -2 and b"static array" in L_.rexsc_last_error()


def test_noalloc_takes_no_device_memory():
    """Free device memory (hipMemGetInfo, which sees every allocation of the process, torch's included) is the same
    before and after a direct call; torch's own allocator is not touched either."""
    L_ = _lib.lib()
    _lib.check(L_.rexsc_init(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)), "rexsc_init")
    g = torch.Generator().manual_seed(31)
    x = (torch.randint(0, 32, (2, 64, 14, 14), generator=g).float() / 32).to("cuda")
    w = (torch.randint(-31, 32, (48, 64, 3, 3), generator=g).float() / 32).to("cuda")
    d = _lib.ConvDesc(2, 64, 14, 14, 48, 3, 3, 1, 1, 1, 1, 32, -1, 1, 1, 7, 8, 1, 0, 0)
    pos = torch.empty(2 * 48 * 14 * 14, dtype=torch.int16, device="cuda")
    neg = torch.empty_like(pos)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(L_.rexsc_conv2d_orn_noalloc(ctypes.byref(d), _p(x), _p(w), _p(pos), _p(neg), None, stream), "warm-up call")
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    reserved0, allocs0 = torch.cuda.memory_reserved(), torch.cuda.memory_stats()["allocation.all.allocated"]
    for _ in range(3):
        _lib.check(L_.rexsc_conv2d_orn_noalloc(ctypes.byref(d), _p(x), _p(w), _p(pos), _p(neg), None, stream), "rexsc_conv2d_orn_noalloc")
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0
    assert torch.cuda.memory_reserved() == reserved0 and torch.cuda.memory_stats()["allocation.all.allocated"] == allocs0


def test_noalloc_under_graph_capture():
    """rexsc_init, then one rexsc_conv2d_orn_noalloc call captured on a non-default stream (kernels only: no memset node,
    no allocation), replayed with new operand values each time and compared with rexsc_conv2d_orn run eagerly."""
    L_ = _lib.lib()
    _lib.check(L_.rexsc_init(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)), "rexsc_init")
    N, C, H, O = 2, 128, 14, 64
    d = _lib.ConvDesc(N, C, H, H, O, 3, 3, 1, 1, 1, 1, 32, -1, 1, 1, 7, 8, 1, 1, 0)
    gen = torch.Generator().manual_seed(32)
    x = torch.zeros(N, C, H, H, device="cuda").contiguous(memory_format=torch.channels_last)
    w = torch.zeros(O, C, 3, 3, device="cuda")
    n_out = N * O * H * H
    got = [torch.zeros(n_out, dtype=torch.int16, device="cuda") for _ in range(2)]
    want = [torch.zeros(n_out, dtype=torch.int16, device="cuda") for _ in range(2)]
    ws = torch.empty(L_.rexsc_conv2d_workspace_bytes(ctypes.byref(d)), dtype=torch.uint8, device="cuda")

    def refill():
        x.copy_((torch.randint(0, 32, x.shape, generator=gen).float() / 32) * (torch.rand(x.shape, generator=gen) < 0.2))
        w.copy_((torch.randint(-31, 32, w.shape, generator=gen).float() / 32) * (torch.rand(w.shape, generator=gen) < 0.2))

    refill()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    print("no-alloc capture", flush=True)
    with torch.cuda.graph(graph, stream=side):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = L_.rexsc_conv2d_orn_noalloc(ctypes.byref(d), _p(x), _p(w), _p(got[0]), _p(got[1]), None, stream)
    _lib.check(rc, "rexsc_conv2d_orn_noalloc (captured)")
    for replay in range(3):
        refill()
        torch.cuda.synchronize()
        graph.replay()
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = L_.rexsc_conv2d_orn(ctypes.byref(d), _p(x), _p(w), _p(want[0]), _p(want[1]), None, _p(ws), ws.numel(), stream)
        _lib.check(rc, "rexsc_conv2d_orn")
        torch.cuda.synchronize()
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), "replay %d" % replay
        assert int(want[0].max()) > 0
