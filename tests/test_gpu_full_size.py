"""The benchmark configurations at their full sizes.

Where the oracle finishes in seconds (configs 1 and 2) the comparison is exact over the whole
output.  For the batch-64 ResNet-18 shapes the full-batch GPU result is checked through properties
that do not depend on size -- batch independence (streams are seeded per (c,y,x), never per image),
layout invariance (NCHW and channels_last inputs give the same logical result), OR-n monotonicity
and bounds -- plus an exact oracle comparison of the first and the last image.
"""
import numpy as np
import pytest
import torch

import oracle as orc

pytestmark = pytest.mark.gpu


def test_config1_conv_or1_full_size_exact():
    import sc_extension_cuda
    g = torch.Generator().manual_seed(1)
    x = torch.randint(0, 32, (32, 32, 32, 32), generator=g).float() / 32
    w = ((torch.rand(64, 32, 3, 3, generator=g) * 2 - 1) * 32).round().clamp(-31, 31) / 32
    print("config1 full", flush=True)
    pos, neg = sc_extension_cuda.conv2d_generic_general_split_acc(x.cuda(), w.cuda(), 32, -1, 16, (1, 1), (1, 1),
                                                                  (7, 8, 1), 0, 1, True, False)
    opos, oneg = orc.conv2d_generic_general_split(x.numpy(), w.numpy(), 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 0, 1)
    assert np.array_equal(pos.cpu().numpy(), opos) and np.array_equal(neg.cpu().numpy(), oneg)


def test_config2_linear_or2_full_size_exact():
    import sc_extension
    g = torch.Generator().manual_seed(2)
    x = torch.randint(0, 64, (256, 4096), generator=g).float() / 64
    # sparse weights keep the OR-2 counts away from permanent saturation, so the comparison bites
    w = ((torch.rand(1024, 4096, generator=g) * 2 - 1) * 64).round().clamp(-63, 63) / 64
    w = w * (torch.rand(1024, 4096, generator=g) < 0.002)
    print("config2 full", flush=True)
    pos, neg = sc_extension.linear_generic_general(x.cuda(), w.cuda(), (7, 8, 1), 64, -1, 1, 1, True, False)
    opos, oneg = orc.linear_generic_general(x.numpy(), w.numpy(), (7, 8, 1), 64, -1, 1, 1)
    assert 0 < opos.mean() < 100  # not saturated at 128
    assert np.array_equal(pos.cpu().numpy(), opos) and np.array_equal(neg.cpu().numpy(), oneg)


# all ten distinct SC layer shapes of ResNet-18 at 224x224 (C_in, H_in, C_out, K, stride)
def test_config2_linear_or2_full_size_dense_operands():
    """The benchmark's own operand distribution (dense weights): every OR-2 count saturates, so almost every
    output is 2 * 64 -- the all-saturated path, exact against the oracle."""
    import sc_extension
    g = torch.Generator().manual_seed(2)
    x = torch.randint(0, 64, (256, 4096), generator=g).float() / 64
    w = ((torch.rand(1024, 4096, generator=g) * 2 - 1) * 64).round().clamp(-63, 63) / 64
    print("config2 full, dense", flush=True)
    pos, neg = sc_extension.linear_generic_general(x.cuda(), w.cuda(), (7, 8, 1), 64, -1, 1, 1, True, False)
    opos, oneg = orc.linear_generic_general(x.numpy(), w.numpy(), (7, 8, 1), 64, -1, 1, 1)
    assert opos.max() == 128 and (opos == 128).mean() > 0.5
    assert np.array_equal(pos.cpu().numpy(), opos) and np.array_equal(neg.cpu().numpy(), oneg)


STAGES = [(64, 56, 64, 3, 1), (64, 56, 128, 3, 2), (64, 56, 128, 1, 2), (128, 28, 128, 3, 1),
          (128, 28, 256, 3, 2), (128, 28, 256, 1, 2), (256, 14, 256, 3, 1),
          (256, 14, 512, 3, 2), (256, 14, 512, 1, 2), (512, 7, 512, 3, 1)]


@pytest.mark.parametrize("shape", STAGES, ids=lambda s: "c%d_h%d_o%d_k%d_s%d" % s)
def test_config5_layer_full_batch_properties(shape):
    import sc_extension_cuda
    C, H, O, K, s = shape
    N, L = 64, 32
    print("config5 layer", shape, flush=True)
    g = torch.Generator().manual_seed(C + H)
    dens = 20.0 / (C * K * K)
    x = (torch.randint(0, L, (N, C, H, H), generator=g).float() / L) * (torch.rand(N, C, H, H, generator=g) < 4 * dens)
    w = (torch.randint(-L + 1, L, (O, C, K, K), generator=g).float() / L) * (torch.rand(O, C, K, K, generator=g) < 4 * dens)
    xc = x.cuda().contiguous(memory_format=torch.channels_last)
    wc = w.cuda()
    args = (L, -1, 16, (K // 2, K // 2), (s, s), (7, 8, 1))
    pos, neg = sc_extension_cuda.conv2d_generic_general_split_acc(xc, wc, *args, 1, 1, True, False)
    assert pos.is_contiguous(memory_format=torch.channels_last)
    # batch independence: a slice computed alone equals the slice of the full batch
    for lo, hi in ((0, 3), (61, 64)):
        p2, n2 = sc_extension_cuda.conv2d_generic_general_split_acc(xc[lo:hi].contiguous(memory_format=torch.channels_last),
                                                                    wc, *args, 1, 1, True, False)
        assert torch.equal(p2, pos[lo:hi]) and torch.equal(n2, neg[lo:hi])
    # layout invariance
    p3, n3 = sc_extension_cuda.conv2d_generic_general_split_acc(x.cuda(), wc, *args, 1, 1, True, False)
    assert p3.is_contiguous() and torch.equal(p3, pos.contiguous()) and torch.equal(n3, neg.contiguous())
    # OR-n monotone in n and bounded by n*L; OR-1 <= OR-2 <= OR-3
    p1, _ = sc_extension_cuda.conv2d_generic_general_split_acc(xc, wc, *args, 0, 1, True, False)
    p4, _ = sc_extension_cuda.conv2d_generic_general_split_acc(xc, wc, *args, 2, 1, True, False)
    assert (p1 <= pos).all() and (pos <= p4).all() and pos.max() <= 2 * L and p1.max() <= L and pos.min() >= 0
    assert (pos != p1).any() and pos.float().mean() > 0.5
    # exact against the oracle on the first and the last image
    for i in (0, N - 1):
        opos, oneg = orc.conv2d_generic_general_split(x[i:i + 1].numpy(), w.numpy(), L, -1, 16, (K // 2, K // 2), (s, s),
                                                      (7, 8, 1), 1, 1, channels_last_activation=True)
        assert np.array_equal(pos[i:i + 1].cpu().numpy(), opos) and np.array_equal(neg[i:i + 1].cpu().numpy(), oneg)


@pytest.mark.parametrize("C,H", [(64, 56), (128, 28), (256, 14), (512, 7)])
def test_config4_fixed_conv_full_batch(C, H):
    import fixed_extension_cuda
    print("config4", C, H, flush=True)
    g = torch.Generator().manual_seed(4 + C)
    x = torch.randint(0, 32, (64, C, H, H), generator=g).float() / 32
    w = torch.randint(-31, 32, (C, C, 3, 3), generator=g).float() / 32
    out = fixed_extension_cuda.conv2d_saturate_acc(x.cuda(), w.cuda(), 0, 5, 24, (1, 1), (1, 1))
    assert out.dtype == torch.int32 and out.shape == (64, C, H, H)
    # batch independence
    o2 = fixed_extension_cuda.conv2d_saturate_acc(x[62:64].cuda(), w.cuda(), 0, 5, 24, (1, 1), (1, 1))
    assert torch.equal(o2, out[62:64])
    # the closed form in float64 on the GPU (exact: every term is an integer below 2^53)
    xq = (x.double() * 32).clamp(0, 31).round().cuda()
    wq = (w.double() * 32).round().cuda()
    wp, wn = wq.clamp(min=0), (-wq).clamp(min=0)
    F = torch.nn.functional
    def pol(wpol):
        return F.conv2d(xq, wpol, padding=1) + F.conv2d(xq % 2, wpol % 2, padding=1)
    want = pol(wp).clamp(max=2 ** 24) - pol(wn).clamp(max=2 ** 24)
    assert torch.equal(out.double(), want)
    # and the oracle itself on one image
    o1 = orc.conv2d_saturate(x[:1].numpy(), w.numpy(), 0, 5, 24, (1, 1), (1, 1))
    assert np.array_equal(out[:1].cpu().numpy(), o1)
