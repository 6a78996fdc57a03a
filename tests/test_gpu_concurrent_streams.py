"""Calls from two host threads on two streams at once, each with its own workspace: the library keeps no
process-global scratch (the reference's CUDA extension does: one static buffer and the legacy default stream,
sc_cuda_kernel.cu:622-632), so conv, linear and fixed conv may run concurrently.  Every result against the oracle."""
import threading

import numpy as np
import pytest
import torch

import oracle as orc

pytestmark = pytest.mark.gpu


def _case(seed):
    rng = np.random.default_rng(seed)
    L = 32
    x = (rng.integers(0, L, size=(2, 64, 12, 12)) / L * (rng.uniform(size=(2, 64, 12, 12)) < 0.25)).astype(np.float32)
    w = (rng.integers(-L + 1, L, size=(40, 64, 3, 3)) / L * (rng.uniform(size=(40, 64, 3, 3)) < 0.25)).astype(np.float32)
    xl = (rng.integers(0, 64, size=(24, 200)) / 64 * (rng.uniform(size=(24, 200)) < 0.1)).astype(np.float32)
    wl = (rng.integers(-63, 64, size=(48, 200)) / 64 * (rng.uniform(size=(48, 200)) < 0.1)).astype(np.float32)
    xf = (rng.integers(0, 32, size=(2, 40, 9, 9)) / 32).astype(np.float32)
    wf = (rng.integers(-31, 32, size=(24, 40, 3, 3)) / 32).astype(np.float32)
    return x, w, xl, wl, xf, wf


def test_two_threads_two_streams_against_the_oracle():
    import fixed_extension_cuda
    import sc_extension_cuda
    # one eager call first: per-device tables are built (and synchronised) once, outside the threads
    sc_extension_cuda.conv2d_generic_general_split_acc(torch.rand(1, 8, 4, 4, device="cuda"), torch.rand(4, 8, 3, 3, device="cuda"),
                                                       32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 1, True, False)
    torch.cuda.synchronize()
    results, errors = {}, []
    start = threading.Barrier(2)

    def worker(tid):
        try:
            stream = torch.cuda.Stream()
            x, w, xl, wl, xf, wf = _case(100 + tid)
            with torch.cuda.stream(stream):
                dev = lambda a: torch.from_numpy(a).cuda(non_blocking=False)
                xt, wt, xlt, wlt, xft, wft = (dev(a) for a in (x, w, xl, wl, xf, wf))
                start.wait()
                out = []
                for rep in range(6):  # interleaved with the other thread's calls
                    pos, neg = sc_extension_cuda.conv2d_generic_general_split_acc(
                        xt.contiguous(memory_format=torch.channels_last), wt, 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 1,
                        True, False)
                    lp, ln = sc_extension_cuda.linear_generic_general_acc(xlt, wlt, (7, 8, 1), 64, -1, 1, 1, True, False)
                    f = fixed_extension_cuda.conv2d_saturate_acc(xft, wft, 0, 5, 24, (1, 1), (1, 1))
                    out.append((pos, neg, lp, ln, f))
                stream.synchronize()
            results[tid] = [tuple(t.cpu().numpy() for t in o) for o in out]
        except Exception as e:  # surfaces in the main thread
            errors.append((tid, repr(e)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(2)]
    print("two threads, two streams", flush=True)
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    assert sorted(results) == [0, 1]
    for tid in range(2):
        x, w, xl, wl, xf, wf = _case(100 + tid)
        opos, oneg = orc.conv2d_generic_general_split(x, w, 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 1,
                                                      channels_last_activation=True)
        olp, oln = orc.linear_generic_general(xl, wl, (7, 8, 1), 64, -1, 1, 1, True, False)
        of = orc.conv2d_saturate(xf, wf, 0, 5, 24, (1, 1), (1, 1))
        assert opos.max() > 0 and np.abs(olp).max() > 0
        for pos, neg, lp, ln, f in results[tid]:
            assert np.array_equal(pos, opos) and np.array_equal(neg, oneg)
            assert np.array_equal(lp.astype(np.int32), olp) and np.array_equal(ln.astype(np.int32), oln)
            assert np.array_equal(f, of)
