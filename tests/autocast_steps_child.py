"""Child process of tests/test_gpu_z_autocast_steps.py: training steps of one benchmark network under float16
autocast with a gradient scaler (the reference's reduced-precision branch, utils_own.py:127-131,156-165).

    python tests/autocast_steps_child.py tinyconv|resnet18

Prints one line per step and "OK" at the end; any failure is a non-zero exit code with the traceback on stderr
(faulthandler is on, so that a crash inside a native library still names the Python frame it came from)."""
import faulthandler
import os
import sys

faulthandler.enable()
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for sub in ("rex-sc_amd", "oracle", "tests", ""):
    sys.path.insert(0, os.path.join(ROOT, sub) if sub else ROOT)

import numpy as np
import torch
import torch.nn.functional as F

import test_gpu_models as tm


def main(which):
    from sc_models import ResNet18SC, TinyConvSC
    torch.manual_seed(0)
    g = torch.Generator().manual_seed(1)
    if which == "tinyconv":
        net, n_layers = TinyConvSC(forward="or_3", err=6).cuda(), 4
        x = torch.randn(8, 3, 32, 32, generator=g).clamp(-1, 1).cuda()
        y = torch.randint(0, 10, (8,), generator=g).cuda()
    else:
        net, n_layers = ResNet18SC(forward="or_2", err=5).cuda().to(memory_format=torch.channels_last), 19
        x = torch.randn(4, 3, 224, 224, generator=g).clamp(-1, 1).cuda().contiguous(memory_format=torch.channels_last)
        y = torch.randint(0, 1000, (4,), generator=g).cuda()
    opt = torch.optim.Adam(net.parameters(), lr=1e-3)
    scaler = torch.amp.GradScaler("cuda")

    def step(sync):
        print("autocast step, sync", sync, which, flush=True)
        net.sync = sync
        opt.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.float16):
            out = net(x)
        loss = F.cross_entropy(out, y, label_smoothing=0.1)
        scaler.scale(loss).backward()
        scaler.step(opt)
        scaler.update()
        torch.cuda.synchronize()
        return out, loss.item()

    # sync 1: the float convolutions and the wrappers around them run in float16; the integer SC forward must not
    # notice: every SC layer's output equals the oracle's on the layer's own input, bit for bit (pos/L - neg/L is
    # exact in float16 for these stream lengths)
    records, handles = tm._hook_sc_layers(net, [0, x.size(0) - 1])
    out, loss = step(1)
    for h in handles:
        h.remove()
    assert out.dtype == torch.float16 and np.isfinite(loss), (out.dtype, loss)
    assert len(records) == n_layers
    assert any(r["x"].dtype == torch.float16 for r in records), "the half-precision branch was not taken"
    for r in records:
        r["x"], r["y"] = r["x"].float(), r["y"].float()
    print("oracle on", len(records), "layers", flush=True)
    tm._check_records_against_oracle(records)
    for sync in (3, 2, 3):
        _, loss = step(sync)
        assert np.isfinite(loss), (sync, loss)
    assert all(torch.isfinite(p).all() for p in net.parameters())
    print("OK", flush=True)


if __name__ == "__main__":
    main(sys.argv[1])
