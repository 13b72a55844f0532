"""Pins of the norm_multiply_dropout oracle against library routines and autograd."""
import torch
import torch.nn.functional as F

from oracle import layer_oracle as LO


def _inputs(seed, rows=7, cols=512):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: torch.rand(*s, generator=g, dtype=torch.float64) * 2 - 1
    return mk(rows, cols), mk(rows, cols), mk(cols), mk(cols), mk(rows, cols)


def test_forward_is_layer_norm_times_u():
    x, u, w, b, _ = _inputs(0)
    y, mean, var = LO.nmd_forward(x, u, w, b, 1e-5)
    assert torch.allclose(y, F.layer_norm(x, [512], w, b, 1e-5) * u, rtol=1e-12, atol=1e-12)
    assert torch.allclose(mean, x.mean(1)) and torch.allclose(var, x.var(1, unbiased=False))


def test_dropout_follows_the_mask_with_the_usual_scale():
    x, u, w, b, _ = _inputs(1)
    keep = torch.rand(x.shape, generator=torch.Generator().manual_seed(2)) >= 0.3
    y0 = LO.nmd_forward(x, u, w, b, 1e-5)[0]
    y = LO.nmd_forward(x, u, w, b, 1e-5, 0.3, keep)[0]
    assert torch.equal(y == 0, ~keep | (y0 == 0)) and torch.allclose(y[keep], y0[keep] / 0.7)
    assert not LO.nmd_forward(x, u, w, b, 1e-5, 1.0, keep)[0].any()
    # mask bytes: bit e % 8 of byte e / 8
    packed = torch.zeros(((keep.numel() + 127) // 128) * 16, dtype=torch.uint8)
    flat = keep.reshape(-1)
    for e in range(0, flat.numel(), 97):
        if flat[e]:
            packed[e // 8] |= 1 << (e % 8)
    got = LO.unpack_mask(packed, flat.numel())
    assert torch.equal(got[::97], flat[::97])


def test_backward_matches_autograd_through_the_library_forward():
    for ratio in (0.0, 0.25):
        x, u, w, b, dy = _inputs(3, rows=5, cols=1024)
        keep = torch.rand(x.shape, generator=torch.Generator().manual_seed(4)) >= ratio
        leaves = [t.clone().requires_grad_(True) for t in (x, u, w, b)]
        y = F.layer_norm(leaves[0], [1024], leaves[2], leaves[3], 1e-5) * leaves[1]
        if ratio:
            y = y * keep / (1 - ratio)
        auto = torch.autograd.grad(y, leaves, grad_outputs=dy)
        _, mean, var = LO.nmd_forward(x, u, w, b, 1e-5)
        got = LO.nmd_backward(dy, x, u, w, b, mean, var, 1e-5, ratio, keep)
        for name, a, wnt in zip(("dx", "du", "dw", "db"), got, auto):
            assert torch.allclose(a, wnt, rtol=1e-9, atol=1e-11), (ratio, name)


def test_in_linear_silu_is_addmm_silu_split():
    """Small integers and dyadic weights: every product and sum is exact in fp32, so the library routines in fp32 and the
    oracle's fp64 agree to the last bit before and after the roundings."""
    g = torch.Generator().manual_seed(6)
    x = torch.randint(-8, 9, (37, 32), generator=g).to(torch.bfloat16)
    w = (torch.randint(-4, 5, (128, 32), generator=g).float() / 8).to(torch.bfloat16)
    b = torch.randint(-3, 4, (128,), generator=g).float()
    split = [16, 48, 32, 32]
    lin = torch.addmm(b, x.float(), w.float().t()).to(torch.bfloat16)
    want = list(torch.split(F.silu(lin.float()).to(torch.bfloat16), split, dim=-1)) + [lin]
    got = LO.in_linear_silu(x, w, b, split)
    for a, wnt in zip(got, want):
        assert a.dtype == torch.bfloat16 and torch.equal(a, wnt)
    assert [t.shape[1] for t in got] == split + [128]
    assert torch.equal(LO.in_linear_silu(x, w, None, split)[4], (x.float() @ w.float().t()).to(torch.bfloat16))


def test_in_linear_silu_backward_is_autograd_of_linear_silu():
    """fp64 autograd through F.linear and F.silu: an independent derivation of all three gradients (no closed-form
    silu' anywhere in it), unequal splits; and central differences of the loss for a few coordinates."""
    g = torch.Generator().manual_seed(8)
    m, k, split = 23, 16, [16, 32, 48, 32]
    n = sum(split)
    x = torch.randn(m, k, generator=g, dtype=torch.float64)
    w = torch.randn(n, k, generator=g, dtype=torch.float64) * 0.3
    b = torch.randn(n, generator=g, dtype=torch.float64)
    grads = [torch.randn(m, s_, generator=g, dtype=torch.float64) for s_ in split]
    xa, wa, ba = (t.clone().requires_grad_() for t in (x, w, b))
    lin = F.linear(xa, wa, ba)
    outs = torch.split(F.silu(lin), split, dim=-1)
    loss = sum((o * g_).sum() for o, g_ in zip(outs, grads))
    loss.backward()
    gx, gw, gb = LO.in_linear_silu_backward(grads, x, w, lin.detach(), with_bias=True, round_dlin=False)
    for a, wnt in ((gx, xa.grad), (gw, wa.grad), (gb, ba.grad)):
        assert torch.allclose(a, wnt, rtol=1e-11, atol=1e-12)
    assert LO.in_linear_silu_backward(grads, x, w, lin.detach(), with_bias=False)[2] is None

    def f(x_, w_, b_):
        o = F.silu(F.linear(x_, w_, b_))
        return float((o * torch.cat(grads, dim=-1)).sum())
    h = 1e-6
    for (i, j) in ((0, 0), (5, 7), (22, 15)):
        d = torch.zeros_like(x); d[i, j] = h
        assert abs((f(x + d, w, b) - f(x - d, w, b)) / (2 * h) - float(gx[i, j])) < 1e-6
    for (i, j) in ((0, 0), (100, 3), (127, 15)):
        d = torch.zeros_like(w); d[i, j] = h
        assert abs((f(x, w + d, b) - f(x, w - d, b)) / (2 * h) - float(gw[i, j])) < 1e-6
    # rounding dlin to the I/O dtype only moves the products by that rounding
    xb, wb = x.to(torch.bfloat16), w.to(torch.bfloat16)
    lb = lin.detach().to(torch.bfloat16)
    gb16 = [t.to(torch.bfloat16) for t in grads]
    r0 = LO.in_linear_silu_backward(gb16, xb, wb, lb, round_dlin=False)
    r1 = LO.in_linear_silu_backward(gb16, xb, wb, lb, round_dlin=True)
    assert torch.equal(r0[2], r1[2])
    for a, c in zip(r0[:2], r1[:2]):
        assert 0 < float((a - c).abs().max()) < 2.0 ** -7 * float(a.abs().max())
