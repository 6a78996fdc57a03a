"""What the mathematics fixes about the oracle, independent of the golden vectors: LFSR cycle
structure, stream density, special cases that reduce to library routines, closed forms."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle as orc


@pytest.mark.parametrize("lb", [3, 4, 5, 6, 7, 8])
def test_lfsr_is_maximal_length(lb):
    period = (1 << lb) - 1
    seen, v = [], 1
    for _ in range(period):
        seen.append(v)
        v = orc.lfsr_step(lb, 0, v)
    assert v == 1 and sorted(seen) == list(range(1, period + 1))
    assert orc.lfsr_step(lb, 0, 0) == 0  # zero is a fixed point of the plain LFSR
    # the zero-including flavour visits all 2^lb states
    seen, v = [], 1
    for _ in range(1 << lb):
        seen.append(v)
        v = orc.lfsr_step(lb, 1, v)
    assert v == 1 and sorted(seen) == list(range(1 << lb))


def test_lfsr_bits_fall_through():
    assert [orc.lfsr_bits(b) for b in (2, 4, 8, 16, 32, 64, 128, 256)] == [3, 3, 3, 4, 5, 6, 7, 8]
    assert orc.lfsr_bits(48) == -1 and orc.lfsr_bits(32, 7) == 7


def test_quantize_closed_forms():
    x = np.array([-0.5, 0.0, 1 / 64, 1 / 32, 0.51, 31 / 32, 1.0, 2.0], np.float32)
    assert orc.quantize_sc(x, 32, 0).tolist() == [0, 0, 1, 1, 17, 31, 31, 31]
    assert orc.quantize_sc(-x, 32, 1).tolist() == [0, 0, 1, 1, 17, 31, 31, 31]
    assert orc.quantize_sc(x, 32, 1).tolist() == [16, 0, 0, 0, 0, 0, 0, 0]
    h = np.array([0.5 / 32, 1.5 / 32, 2.5 / 32, 0.49 / 32], np.float32)
    assert orc.quantize_fixed(h, 32, 0).tolist() == [0, 2, 2, 0]  # half to even


def test_single_element_stream_density():
    """One activation against weight 1-1/L: over the L cycles a value v gives v or v-1 ones (the
    LFSR visits every state 1..L-1 once, and one of them twice)."""
    L = 32
    for v in range(L):
        x = np.full((1, 1, 1, 1), v / L, np.float32)
        w = np.full((1, 1, 1, 1), 1.0, np.float32)  # quantises to L-1: its stream is 1 except where state == L-1
        pos, neg = orc.conv2d_generic_general_split(x, w, L, -1, 16, (0, 0), (1, 1), (7, 8, 1), 0, 1)
        assert neg[0, 0, 0, 0] == 0
        assert max(0, v - 2) <= pos[0, 0, 0, 0] <= v


def test_conv_unsaturated_equals_dense_bit_conv():
    """With n_sat above the reduction size nothing saturates: the result is a plain integer conv of
    the {0,1} stream tensors summed over cycles, so pos-neg is linear in the weights' sign pattern:
    flipping every weight's sign swaps pos and neg exactly."""
    rng = np.random.default_rng(3)
    x = (rng.integers(0, 32, size=(2, 40, 6, 6)) / 32).astype(np.float32)
    w = (rng.integers(-31, 32, size=(5, 40, 3, 3)) / 32).astype(np.float32)
    p1, n1 = orc.conv2d_generic_general_split(x, w, 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 10000, 1)
    p2, n2 = orc.conv2d_generic_general_split(x, -w, 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 10000, 1)
    assert np.array_equal(p1, n2) and np.array_equal(n1, p2)
    # additivity over disjoint channel groups holds only without saturation ...
    wa, wb = w.copy(), w.copy()
    wa[:, 20:] = 0
    wb[:, :20] = 0
    pa, _ = orc.conv2d_generic_general_split(x, wa, 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 10000, 1)
    pb, _ = orc.conv2d_generic_general_split(x, wb, 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 10000, 1)
    assert np.array_equal(pa + pb, p1)
    # ... and OR-1 is bounded by it and by the stream length
    po, _ = orc.conv2d_generic_general_split(x, w, 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 0, 1)
    assert (po <= np.minimum(p1, 32)).all() and (po >= (p1 > 0)).all()


def test_linear_matches_conv_1x1_semantics_up_to_seeds():
    """Zero operands give zero; a saturated OR-1 of dense operands gives ~L per output."""
    x = np.zeros((3, 64), np.float32)
    w = np.ones((4, 64), np.float32)
    pos, neg = orc.linear_generic_general(x, w, (7, 8, 1), 32, -1, 0, 1)
    assert not pos.any() and not neg.any()
    x[:] = 31 / 32
    pos, neg = orc.linear_generic_general(x, w, (7, 8, 1), 32, -1, 0, 1)
    assert (pos == 32).all() and not neg.any()


@pytest.mark.parametrize("pin,pout", [(5, 24), (5, 8), (6, 10), (4, 6), (7, 12)])
def test_fixed_conv_closed_form(pin, pout):
    """add_config 0 against the order-independent closed form evaluated with an int64 F.conv2d."""
    rng = np.random.default_rng(pin * 100 + pout)
    P2 = 1 << pin
    x = (rng.integers(0, P2, size=(2, 12, 7, 6)) / P2 * (rng.uniform(size=(2, 12, 7, 6)) < 0.5)).astype(np.float32)
    w = (rng.integers(-P2 + 1, P2, size=(5, 12, 3, 3)) / P2 * (rng.uniform(size=(5, 12, 3, 3)) < 0.5)).astype(np.float32)
    got = orc.conv2d_saturate(x, w, 0, pin, pout, (1, 1), (1, 1))
    xq = torch.from_numpy(orc.quantize_fixed(x, P2, 0)).double()
    wp = torch.from_numpy(orc.quantize_fixed(w, P2, 0)).double()
    wn = torch.from_numpy(orc.quantize_fixed(w, P2, 1)).double()
    d = max(0, 2 * pin - pout)
    pmax = min(31, max(2 * pin, pout))
    max_value = (((1 << pmax) - 1) >> d) << d
    # brute force over products (unfold) so that per-product rounding can be applied
    cols = F.unfold(F.pad(xq, (1, 1, 1, 1)), (3, 3)).long()          # [N, C*9, L]
    res = []
    for wpol in (wp, wn):
        wv = wpol.reshape(5, -1).long()                                   # [O, C*9]
        prod = wv[None, :, :, None] * cols[:, None, :, :]                 # [N, O, C*9, L]
        if d == 0:
            r = (prod + (prod & 1)).sum(2).clamp(max=max_value + 1)
        else:
            r = (((prod + (1 << (d - 1))) >> d) << d).sum(2).clamp(max=max_value)
        res.append(r)
    want = (res[0] - res[1]).reshape(2, 5, 7, 6).numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("n", [1, 2, 3, 4])
def test_orn_closed_forms_against_float64(n):
    x = np.concatenate([np.linspace(0, 12, 4001), [0.0, 1e-4, 30.0]]).astype(np.float32)
    xd = x.astype(np.float64)
    e = np.exp(-xd)
    fact = [1, 1, 2, 6]
    want = n - e * sum((n - i) * xd ** i / fact[i] for i in range(n))
    got = orc.or_approx_n_forward(x, n)
    assert np.allclose(got, want, rtol=2e-6, atol=n * 2.4e-7)
    g = np.linspace(-2, 2, x.size).astype(np.float32)
    dwant = g * e * sum(xd ** i / fact[i] for i in range(n))
    dgot = orc.or_approx_n_backward(g, x, n, half_input=False)
    assert np.allclose(dgot, dwant, rtol=2e-6, atol=1e-7)
    # derivative consistency: d/dx forward == backward (central differences in float64)
    h = 1e-5
    fd = ((n - np.exp(-(xd + h)) * sum((n - i) * (xd + h) ** i / fact[i] for i in range(n))) -
          (n - np.exp(-(xd - h)) * sum((n - i) * (xd - h) ** i / fact[i] for i in range(n)))) / (2 * h)
    assert np.allclose(fd, e * sum(xd ** i / fact[i] for i in range(n)), atol=1e-8)


def test_bias_noise_closed_forms():
    rng = np.random.default_rng(0)
    b = rng.normal(size=6).astype(np.float32) * 0.1
    s = np.abs(rng.normal(size=6)).astype(np.float32) * 0.05
    xp = rng.uniform(0, 4, 1000).astype(np.float32)
    xn = rng.uniform(0, 4, 1000).astype(np.float32)
    zp = rng.normal(size=1000).astype(np.float32)
    zn = rng.normal(size=1000).astype(np.float32)
    for n in (1, 2, 3, 4):
        y = orc.or_approx_n_forward_bias_std_both(xp, xn, b, s, n, zp, zn)
        vp = orc.or_approx_n_forward(xp, n).astype(np.float64)
        vn = orc.or_approx_n_forward(xn, n).astype(np.float64)
        f = lambda v, z: v + sum(b[k] * v ** k for k in range(6)) + sum(s[k] * v ** k for k in range(6)) * z
        assert np.allclose(y, f(vp, zp) - f(vn, zn), rtol=1e-5, atol=1e-5)
        g = rng.normal(size=1000).astype(np.float32)
        gp, gn = orc.or_approx_n_backward_bias_std_both(g, xp, xn, b, n, half_input=False)
        dpoly = lambda v: 1 + sum(k * b[k] * v ** (k - 1) for k in range(1, 6))
        dor = lambda x: np.exp(-x.astype(np.float64)) * sum(x.astype(np.float64) ** i / [1, 1, 2, 6][i] for i in range(n))
        assert np.allclose(gp, g * dpoly(vp) * dor(xp), rtol=1e-4, atol=1e-6)
        assert np.allclose(gn, -g * dpoly(vn) * dor(xn), rtol=1e-4, atol=1e-6)


def test_calibration_recovers_planted_polynomials():
    """Synthetic data with a planted bias polynomial and noise level: the window fit returns them."""
    rng = np.random.default_rng(11)
    n = 400000
    a_act = rng.uniform(0, 2.0, n).astype(np.float32)
    bias = lambda v: 0.05 - 0.04 * v + 0.01 * v ** 2
    std = lambda v: 0.02 + 0.01 * v
    a_bit = (a_act + bias(a_act) + std(a_act) * rng.normal(size=n)).astype(np.float32)
    # max(a_bit) > max(a_act): the last windows are empty, 26 of 30 are valid, so an order-5 bias
    # fit is suppressed (5 >= 26 // 5) while an order-4 fit is kept
    bc5, _ = orc.compute_bias_std_coef(2, a_bit, a_act, 5)
    assert not bc5.any()
    bc, sc = orc.compute_bias_std_coef(2, a_bit, a_act, 4)
    centres = np.linspace(0.2, 1.7, 7)
    fit_b = sum(bc[k] * centres ** k for k in range(5))
    fit_s = sum(sc[k] * centres ** k for k in range(5))
    # a window [s, s+0.1) is attributed to its START s: the fitted curves are the planted ones
    # evaluated ~0.05 to the right
    assert np.allclose(fit_b, bias(centres + 0.05), atol=4e-3)
    assert np.allclose(fit_s, np.sqrt(std(centres + 0.05) ** 2 + (0.04 * 0.1) ** 2 / 12), atol=4e-3)
    # too few valid windows -> bias fit suppressed (order >= n_valid // 5)
    bc2, sc2 = orc.compute_bias_std_coef(2, a_bit[:50] * 0.01, a_act[:50] * 0.01, 5)
    assert not bc2.any()
    z1, z2 = orc.compute_bias_std_coef(-1, a_bit, a_act, 5)
    assert not z1.any() and not z2.any()


def test_quantize_reference_formula():
    x = np.array([-2.0, -0.999, -0.004, 0.0, 0.0039, 0.5, 0.9999, 3.0], np.float32)
    q = orc.quantize(x, 7)
    # x*128 = -256, -127.872, -0.512, 0, 0.4992, 64, 127.987, 384 -> round half to even, clamp to +-127
    assert np.array_equal(q * 128, np.array([-127, -127, -1, 0, 0, 64, 127, 127], np.float32))
    assert q.max() == 127 / 128 and q.min() == -127 / 128
    assert np.array_equal(orc.quantize(q, 7), q)  # idempotent


@pytest.mark.parametrize("g,bc", [(1, 0), (2, 1), (3, 1), (3, -2), (4, 2)])
def test_linear_slot_interleave_brute_force(g, bc):
    """The linear op, gen_config g, against a per-bit Python loop: slot s < L pairs activation cycle
    (s // g^2) * g + s % g with weight cycle s // g (sc_matmul.cpp:422,:667 read only the first L
    of the L*g generated slots), including g that does not divide L."""
    L, B, C, O = 8, 2, 37, 3
    lb, P = 3, 7
    rng = np.random.default_rng(40 + g)
    x = (rng.integers(0, L + 1, size=(B, C)) / L).astype(np.float32)
    w = (rng.integers(-L, L + 1, size=(O, C)) / L).astype(np.float32)
    xq = np.ceil(np.clip(x * L, 0, L - 1)).astype(int)
    wp = np.ceil(np.clip(w * L, 0, L - 1)).astype(int)
    wn = np.ceil(-np.clip(w * L, 1 - L, 0)).astype(int)

    def stream(v, seed):
        bits, state = [], seed
        for _ in range(L):
            state = orc.lfsr_step(lb, 0, state)
            bits.append(int(v > state))
        return bits

    a_bits = [[stream(xq[b, c], c % P + 1) for c in range(C)] for b in range(B)]
    p_bits = [[stream(wp[o, c], (13 + c) % P + 1) for c in range(C)] for o in range(O)]
    n_bits = [[stream(wn[o, c], (13 + c) % P + 1) for c in range(C)] for o in range(O)]
    n_sat = bc + 1 if bc >= 0 else 1 - bc
    exp_p = np.zeros((B, O), np.int32)
    exp_n = np.zeros((B, O), np.int32)
    for b in range(B):
        for o in range(O):
            for s in range(L):
                ta, tw = (s // (g * g)) * g + s % g, s // g
                cp = sum(a_bits[b][c][ta] & p_bits[o][c][tw] for c in range(C))
                cn = sum(a_bits[b][c][ta] & n_bits[o][c][tw] for c in range(C))
                exp_p[b, o] += (cp >= n_sat) if bc < 0 else min(cp, n_sat)
                exp_n[b, o] += (cn >= n_sat) if bc < 0 else min(cn, n_sat)
    pos, neg = orc.linear_generic_general(x, w, (7, 8, 1), L, -1, bc, g)
    assert np.array_equal(pos, exp_p) and np.array_equal(neg, exp_n)


# ---- the XNOR generator of the reference's CUDA conv kernels (no CUDA build or fixture exists) --------------
@pytest.mark.parametrize("lb", [3, 4, 5, 6, 7, 8])
def test_xnor_lfsr_cycle_and_complement_relation(lb):
    """sc_device.cuh:108-286: the XNOR LFSR runs over 0 .. 2^lb-2 with period 2^lb-1 and all-ones as its fixed
    point; every tap set has an even number of taps, so it is the bitwise complement of the plain LFSR:
    xnor_step(~s) == ~xor_step(s)."""
    full = (1 << lb) - 1
    seen, v = [], 0
    for _ in range(full):
        seen.append(v)
        v = orc.lfsr_step(lb, 2, v)
    assert v == 0 and sorted(seen) == list(range(full))
    assert orc.lfsr_step(lb, 2, full) == full
    for s in range(full + 1):
        assert orc.lfsr_step(lb, 2, full ^ s) == full ^ orc.lfsr_step(lb, 0, s)


def _cuda_xnor_step(lb, v):
    """The reference's own arithmetic, d_lfsr_N_xnor (sc_device.cuh:108,147,172,197,224,244)."""
    if lb == 3:
        return 1 - ((v // 4) + (v // 2) % 2) % 2 + 2 * (v % 4)
    if lb == 4:
        return 1 - ((v // 8) + (v // 4) % 2) % 2 + 2 * (v % 8)
    if lb == 5:
        return 1 - ((v // 16) + (v // 4) % 2) % 2 + 2 * (v % 16)
    if lb == 6:
        return 1 - ((v // 32) + (v // 16) % 2) % 2 + 2 * (v % 32)
    if lb == 7:
        return 1 - ((v // 64) + (v // 32) % 2) % 2 + 2 * (v % 64)
    return 1 - ((v // 128) + (v // 32) % 2 + (v // 16) % 2 + (v // 8) % 2) % 2 + 2 * (v % 128)


@pytest.mark.parametrize("L,gen,bc", [(8, 1, 0), (16, 1, 1), (32, 1, 1), (32, 2, 1), (64, 1, 2), (16, 2, 0)])
def test_cuda_xnor_conv_brute_force(L, gen, bc):
    """The oracle's cuda_xnor mode against a per-bit Python model written from sc_cuda_conv.cu:3-166 (seeds
    (13 + c*KH*KW + ky*KW + kx) % P + 1 - 1 and (c*Hp*Wp + y*Wp + x) % P + 1 - 1, state stepped before the
    compare, the same LFSR for gen_config 2, slot interleave :90-93,160-162) and the per-slot saturating sum."""
    rng = np.random.default_rng(L + gen)
    N, C, H, W, O, K = 1, 5, 4, 5, 3, 3
    lb = orc.lfsr_bits(L)
    P = (1 << lb) - 1
    for s in range(P + 1):  # the step the model uses is the reference's own formula
        assert _cuda_xnor_step(lb, s) == orc.lfsr_step(lb, 2, s)
    x = (rng.integers(0, L, size=(N, C, H, W)) / L).astype(np.float32)
    w = (rng.integers(-L + 1, L, size=(O, C, K, K)) / L).astype(np.float32)
    got_p, got_n = orc.conv2d_generic_general_split(x, w, L, -1, 16, (1, 1), (1, 1), (7, 8, 1), bc, gen, cuda_xnor=True)
    xq = np.pad(orc.quantize_sc(x, L, 0), ((0, 0), (0, 0), (1, 1), (1, 1)))
    wq = (orc.quantize_sc(w, L, 0), orc.quantize_sc(w, L, 1))
    Hp, Wp, T = H + 2, W + 2, L * gen

    def stream(value, seed):
        bits, st = [], seed
        for _ in range(L):
            st = _cuda_xnor_step(lb, st)
            bits.append(int(value > st))
        return bits

    a_slots = np.zeros((T, C, Hp, Wp), np.int64)
    for c in range(C):
        for y in range(Hp):
            for xx in range(Wp):
                b = stream(xq[0, c, y, xx], (c * Hp * Wp + y * Wp + xx) % P + 1 - 1)
                for t in range(L):
                    for j in range(gen):
                        a_slots[(t // gen) * gen * gen + j * gen + t % gen, c, y, xx] = b[t]
    w_slots = np.zeros((2, T, O, C, K, K), np.int64)
    for pol in range(2):
        for o in range(O):
            for c in range(C):
                for ky in range(K):
                    for kx in range(K):
                        b = stream(wq[pol][o, c, ky, kx], (13 + c * K * K + ky * K + kx) % P + 1 - 1)
                        for t in range(L):
                            for j in range(gen):
                                w_slots[pol, t * gen + j, o, c, ky, kx] = b[t]
    n_sat = bc + 1
    for pol, got in ((0, got_p), (1, got_n)):
        want = np.zeros((N, O, H, W), np.int64)
        for t in range(T):
            cnt = F.conv2d(torch.from_numpy(a_slots[t][None].astype(np.float64)),
                           torch.from_numpy(w_slots[pol, t].astype(np.float64))).numpy()
            want += np.minimum(cnt.astype(np.int64), n_sat)
        assert want.max() > 0
        assert np.array_equal(got.astype(np.int64), want)
    # and it is a different generator: the CPU-extension result differs
    cpu_p, _ = orc.conv2d_generic_general_split(x, w, L, -1, 16, (1, 1), (1, 1), (7, 8, 1), bc, gen)
    assert not np.array_equal(cpu_p, got_p)


def test_cuda_xnor_refuses_8_bit_lfsrs():
    x = np.zeros((1, 4, 4, 4), np.float32)
    w = np.zeros((2, 4, 3, 3), np.float32)
    with pytest.raises(ValueError):
        orc.conv2d_generic_general_split(x, w, 256, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 1, cuda_xnor=True)
