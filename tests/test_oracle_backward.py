"""Pins of the oracle's backward restatement: it is checked against derivations that share no formula with it."""
import pytest
import torch

from oracle import hstu_oracle as O


def _case(seed, lens_q, lens_k, nq, nk, d, dv, *, bias=False, ctx=None, tgt=None):
    g = torch.Generator().manual_seed(seed)
    tq, tk = sum(lens_q), sum(lens_k)
    q = torch.randn(tq, nq, d, generator=g, dtype=torch.float64) * 0.7
    k = torch.randn(tk, nk, d, generator=g, dtype=torch.float64) * 0.7
    v = torch.randn(tk, nk, dv, generator=g, dtype=torch.float64)
    grad = torch.randn(tq, nq, dv, generator=g, dtype=torch.float64)
    off_q = torch.tensor([0] + list(torch.tensor(lens_q).cumsum(0)))
    off_k = torch.tensor([0] + list(torch.tensor(lens_k).cumsum(0)))
    mq, mk = max(lens_q), max(lens_k)
    kw = dict(max_seq_len_q=mq, max_seq_len_k=mk, alpha=0.37, silu_scale=0.0, num_context=ctx, num_target=tgt,
              target_group_size=1 if tgt else 0)
    if bias:
        kw["attn_bias"] = torch.randn(len(lens_q), nq, mq, mk, generator=g, dtype=torch.float64) * 0.3
    return grad, q, k, v, off_q, off_k, kw


CASES = [
    dict(lens_q=[5, 9, 1], lens_k=[5, 9, 1], nq=2, nk=2, d=4, dv=16),
    dict(lens_q=[3, 7], lens_k=[6, 11], nq=4, nk=2, d=8, dv=16, bias=True),                      # delta-q, GQA, bias
    dict(lens_q=[12, 8], lens_k=[12, 8], nq=2, nk=1, d=4, dv=16, ctx=[2, 0], tgt=[4, 3], bias=True),
]


@pytest.mark.parametrize("c", CASES)
def test_backward_matches_autograd_of_the_forward(c):
    grad, q, k, v, off_q, off_k, kw = _case(1, **c)
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v)]
    fkw = dict(kw)
    if "attn_bias" in kw:
        fkw["attn_bias"] = kw["attn_bias"].clone().requires_grad_(True)
        leaves.append(fkw["attn_bias"])
    out = O.hstu_jagged_forward(leaves[0], leaves[1], leaves[2], off_q, off_k, mode="exact", compute_dtype=torch.float64, **fkw)
    auto = torch.autograd.grad(out, leaves, grad_outputs=grad)
    dq, dk, dv, db = O.hstu_jagged_backward(grad, q, k, v, off_q, off_k, **kw)
    for name, got, want in zip(("dq", "dk", "dv"), (dq, dk, dv), auto):
        assert torch.allclose(got, want, rtol=1e-10, atol=1e-12), name
    if "attn_bias" in kw:
        assert torch.allclose(db, auto[3], rtol=1e-10, atol=1e-12)
    else:
        assert db is None


def test_backward_matches_finite_differences():
    grad, q, k, v, off_q, off_k, kw = _case(2, lens_q=[4, 3], lens_k=[4, 3], nq=2, nk=1, d=3, dv=16, bias=True)
    dq, dk, dv, db = O.hstu_jagged_backward(grad, q, k, v, off_q, off_k, **kw)

    def loss(q_, k_, v_, b_):
        kk = dict(kw, attn_bias=b_)
        return (O.hstu_jagged_forward(q_, k_, v_, off_q, off_k, mode="exact", compute_dtype=torch.float64, **kk) * grad).sum()

    eps = 1e-6
    g = torch.Generator().manual_seed(3)
    for which, (t, d) in enumerate(((q, dq), (k, dk), (v, dv), (kw["attn_bias"], db))):
        for _ in range(6):
            idx = tuple(int(torch.randint(0, n, (1,), generator=g)) for n in t.shape)
            args = [q, k, v, kw["attn_bias"]]
            hi, lo = t.clone(), t.clone()
            hi[idx] += eps
            lo[idx] -= eps
            args[which] = hi
            f1 = loss(*args)
            args[which] = lo
            f0 = loss(*args)
            fd = float(f1 - f0) / (2 * eps)
            assert abs(fd - float(d[idx])) <= 1e-6 * max(1.0, abs(fd)), (which, idx, fd, float(d[idx]))


def test_gqa_gradients_are_summed_over_the_query_heads_of_a_kv_head():
    grad, q, k, v, off_q, off_k, kw = _case(4, lens_q=[6, 5], lens_k=[6, 5], nq=4, nk=2, d=4, dv=16)
    dq, dk, dv, _ = O.hstu_jagged_backward(grad, q, k, v, off_q, off_k, **kw)
    kr, vr = k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1)
    dq2, dk2, dv2, _ = O.hstu_jagged_backward(grad, q, kr, vr, off_q, off_k, **kw)
    assert torch.allclose(dq, dq2)
    assert torch.allclose(dk, dk2.reshape(dk.shape[0], 2, 2, -1).sum(2))
    assert torch.allclose(dv, dv2.reshape(dv.shape[0], 2, 2, -1).sum(2))


def test_bias_gradient_is_zero_outside_the_sequences():
    grad, q, k, v, off_q, off_k, kw = _case(5, lens_q=[2, 6], lens_k=[2, 6], nq=1, nk=1, d=4, dv=16, bias=True)
    _, _, _, db = O.hstu_jagged_backward(grad, q, k, v, off_q, off_k, **kw)
    assert float(db[0, :, 2:, :].abs().max()) == 0.0 and float(db[0, :, :, 2:].abs().max()) == 0.0
    assert float(db[1].abs().max()) > 0.0
    # masked (non-causal) entries carry no gradient either
    assert float(torch.triu(db[1, 0], diagonal=1).abs().max()) == 0.0


def test_dense_backward_matches_autograd_of_the_dense_forward():
    g = torch.Generator().manual_seed(5)
    b, s_, n, d = 2, 7, 2, 16
    q, k, v, grad = (torch.randn(b, s_, n, d, generator=g, dtype=torch.float64) * 0.6 for _ in range(4))
    bias = torch.randn(b, n, s_, s_, generator=g, dtype=torch.float64) * 0.3
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v, bias)]
    out = O.hstu_dense_forward(leaves[0], leaves[1], leaves[2], max_seq_len=s_, attn_bias=leaves[3], mode="exact",
                               compute_dtype=torch.float64)
    auto = torch.autograd.grad(out, leaves, grad_outputs=grad)
    got = O.hstu_dense_backward(grad, q, k, v, max_seq_len=s_, attn_bias=bias)
    for name, a, w in zip(("dq", "dk", "dv", "dbias"), got, auto):
        assert a.shape == w.shape and torch.allclose(a, w, rtol=1e-10, atol=1e-12), name
