"""The two benchmark networks end to end at their full sizes (BASELINE configs 3 and 5): one training
step per step flavour (sync 1 = SC forward, 3 = error injection, 2 = calibration on half a batch), with
forward hooks on every SC layer comparing the values inside the model with the CPU oracle.

What is compared: at sync 1 a layer's output is the integer SC result divided by the stream length
(utils_functional.py:1273-1274, 1317), so output == oracle(quantize(input), quantize(weight)) / L bit for
bit.  The streams are seeded per (channel, y, x), never per image, so image i of a batch equals the oracle
run on image i alone: the hooks keep the first and the last image of the full batch and the oracle runs on
those two (it finishes in seconds), which covers every layer shape at the full batch size.
Step structure: utils_own.py:96-171 (forward, label-smoothed cross entropy, backward, Adam step);
topologies: resnet_sc.py:33-44,246-271 and the TinyConv-style net of the benchmark configuration.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle as orc

pytestmark = pytest.mark.gpu


def _hook_sc_layers(net, keep):
    """Forward hooks on every Conv2d_Add_Partial: records (name, input[keep], weight, output[keep], meta)."""
    import _ops
    from sc_layers import Conv2d_Add_Partial
    records, handles = [], []

    def make(name):
        def hook(mod, inputs, output):
            x = inputs[0]
            out = output[0] if isinstance(output, tuple) else output
            records.append(dict(name=name, x=x.detach()[keep].cpu(), w=mod.weight.detach().cpu(),
                                y=out.detach()[keep].cpu(), cl=bool(_ops.is_channels_last(x)),
                                padding=tuple(mod.padding), stride=tuple(mod.stride), L=mod.run_args["bit_length"],
                                forward=mod.run_args["forward"], prec=mod.run_args["prec"],
                                y_cl=bool(_ops.is_channels_last(out)) if out.dim() == 4 else False))
        return hook

    for name, mod in net.named_modules():
        if isinstance(mod, Conv2d_Add_Partial):
            handles.append(mod.register_forward_hook(make(name)))
    return records, handles


def _check_records_against_oracle(records):
    for r in records:
        n = int(r["forward"][-1])
        xq = orc.quantize(r["x"].numpy(), r["prec"])
        wq = orc.quantize(r["w"].numpy(), r["prec"])
        assert r["padding"][0] == r["padding"][1]
        pos, neg = orc.conv2d_generic_general_split(xq, wq, r["L"], -1, 16, r["padding"], r["stride"], (7, 8, 1), n - 1, 1,
                                                    channels_last_activation=r["cl"])
        want = pos.astype(np.float32) / np.float32(r["L"]) - neg.astype(np.float32) / np.float32(r["L"])
        got = r["y"].numpy()
        assert got.shape == want.shape, r["name"]
        assert np.array_equal(got, want), "SC layer %s differs from the oracle (max |diff| %g)" % (
            r["name"], np.abs(got - want).max())
        assert np.abs(want).max() > 0, r["name"]


def _step(net, opt, x, y, sync):
    net.sync = sync
    opt.zero_grad(set_to_none=True)
    loss = F.cross_entropy(net(x), y, label_smoothing=0.1)
    loss.backward()
    opt.step()
    return loss.item()


def _calib_buffers(net):
    from sc_layers import Conv2d_Add_Partial
    return {n: (m.bias_coef.detach().clone(), m.std_coef.detach().clone()) for n, m in net.named_modules()
            if isinstance(m, Conv2d_Add_Partial)}


def _run_config(make_net, make_batch, batch, lr, n_layers):
    keep = [0, batch - 1]

    def fresh():
        torch.manual_seed(0)
        net = make_net()
        return net, torch.optim.Adam(net.parameters(), lr=lr, weight_decay=1e-4)

    # sync 1: every SC layer against the oracle, loss finite, forward reproducible bit for bit
    net, opt = fresh()
    x, y = make_batch(batch)
    records, handles = _hook_sc_layers(net, keep)
    print("sync 1 step, batch", batch, flush=True)
    loss1 = _step(net, opt, x, y, 1)
    for h in handles:
        h.remove()
    assert len(records) == n_layers
    assert all(r["y_cl"] == r["cl"] for r in records)  # outputs keep the activation's memory order
    print("oracle on", len(records), "layers", flush=True)
    _check_records_against_oracle(records)
    assert np.isfinite(loss1)
    params1 = [p.detach().clone() for p in net.parameters()]
    assert all(torch.isfinite(p).all() for p in params1)
    net_b, opt_b = fresh()
    loss1b = _step(net_b, opt_b, x, y, 1)
    # the forward pass (all integer SC layers) is reproducible bit for bit; the float convolutions' backward is the
    # vendor library's and may accumulate in a different order from run to run
    assert loss1b == loss1

    # sync 2 (calibration, half a batch): the polynomial buffers of every SC layer are refitted in place
    before = _calib_buffers(net)
    assert all(not b.any() and not s.any() for b, s in before.values())
    xh, yh = make_batch(batch // 2)
    print("sync 2 step, batch", batch // 2, flush=True)
    loss2 = _step(net, opt, xh, yh, 2)
    assert np.isfinite(loss2)
    after = _calib_buffers(net)
    for name in before:
        b, s = after[name]
        assert torch.isfinite(b).all() and torch.isfinite(s).all(), name
        assert s.abs().sum() > 0, "std polynomial of %s was not fitted" % name

    # sync 3 (error injection with the fitted polynomials): finite loss and parameters, noise differs per call
    print("sync 3 step, batch", batch, flush=True)
    loss3 = _step(net, opt, x, y, 3)
    assert np.isfinite(loss3)
    assert all(torch.isfinite(p).all() for p in net.parameters())
    net.sync = 3
    with torch.no_grad():
        o1, o2 = net(x[:2]), net(x[:2])
    assert torch.isfinite(o1).all() and not torch.equal(o1, o2)


def test_config5_resnet18_training_step_full_batch():
    from sc_models import ResNet18SC

    def make_net():
        return ResNet18SC(forward="or_2", err=5).cuda().to(memory_format=torch.channels_last)

    g = torch.Generator().manual_seed(5)

    def make_batch(n):
        return (torch.randn(n, 3, 224, 224, generator=g).cuda().contiguous(memory_format=torch.channels_last),
                torch.randint(0, 1000, (n,), generator=g).cuda())

    _run_config(make_net, make_batch, 64, 1e-3, 19)


def test_config3_tinyconv_training_step_full_batch():
    from sc_models import TinyConvSC

    def make_net():
        return TinyConvSC(forward="or_3", err=6).cuda()

    g = torch.Generator().manual_seed(3)

    def make_batch(n):
        return (torch.randn(n, 3, 32, 32, generator=g).clamp(-1, 1).cuda(), torch.randint(0, 10, (n,), generator=g).cuda())

    _run_config(make_net, make_batch, 256, 8e-3, 4)

