"""Pins of the bias-producer oracle against derivations that share no formula with it."""
import math

import numpy as np
import torch

from oracle import bias_oracle as BO


def test_rab_time_against_an_element_loop():
    g = torch.Generator().manual_seed(0)
    ts = torch.randint(0, 5000, (2, 5), generator=g, dtype=torch.int32)
    w = torch.randn(3, 129, generator=g)
    out, ids = BO.rab_time(ts, w)
    assert out.shape == (3, 2, 10, 10) and ids.shape == (2, 5, 5) and ids.dtype == torch.int32
    cmax = math.exp(128 * 0.301)
    for b in range(2):
        for i in range(5):
            for j in range(5):
                d = float(np.float32(abs(int(ts[b, i]) - int(ts[b, j]))))
                k = int(np.float32(np.log(np.float32(min(max(d, 1.0), cmax)))) / np.float32(0.301))
                assert int(ids[b, i, j]) == k
                for n in range(3):
                    assert torch.equal(out[n, b, 2 * i:2 * i + 2, 2 * j:2 * j + 2], w[n, k].expand(2, 2))


def test_rab_time_closed_forms():
    w = torch.arange(3 * 129, dtype=torch.float32).reshape(3, 129)
    same = torch.full((1, 4), 77, dtype=torch.int64)
    out, ids = BO.rab_time(same, w)
    assert not ids.any() and torch.equal(out, w[:, 0].reshape(3, 1, 1, 1).expand(3, 1, 8, 8))
    # |dt| = 1 is still bucket 0; the first |dt| of bucket k is ceil(e^(k * 0.301)) for integer timestamps
    for k in (3, 10, 27):       # (bucket 1 holds no integer: e^0.301 = 1.35 .. e^0.602 = 1.83)
        first = math.ceil(math.exp(k * 0.301))
        ts = torch.tensor([[0, first - 1, first]], dtype=torch.int64)
        ids = BO.rab_time(ts, w)[1]
        assert int(ids[0, 0, 2]) == k and int(ids[0, 0, 1]) == k - 1 and int(ids[0, 2, 0]) == k
    huge = torch.tensor([[0, 2 ** 62]], dtype=torch.int64)
    assert int(BO.rab_time(huge, w)[1][0, 0, 1]) in (127, 128)          # clamped at e^(128 * divisor)


def test_rab_time_backward_is_the_adjoint_of_the_forward_and_matches_a_loop():
    g = torch.Generator().manual_seed(1)
    ts = torch.randint(0, 3000, (2, 6), generator=g, dtype=torch.int64)
    w = torch.randn(2, 129, generator=g, dtype=torch.float64)
    grad = torch.randn(2, 2, 12, 12, generator=g, dtype=torch.float64)
    out, ids = BO.rab_time(ts, w)
    gw = BO.rab_time_backward(grad, ids, 129)
    assert abs(float((out * grad).sum() - (w * gw).sum())) < 1e-9
    want = torch.zeros(2, 129, dtype=torch.float64)
    for n in range(2):
        for b in range(2):
            for r in range(12):
                for c in range(12):
                    want[n, int(ids[b, r // 2, c // 2])] += grad[n, b, r, c]
    assert torch.allclose(gw, want, rtol=0, atol=1e-12)
    # ids outside the table are ignored (the reference's test draws them modulo 128 for a 128-column result)
    assert torch.allclose(BO.rab_time_backward(grad, ids, 4), want[:, :4], rtol=0, atol=1e-12)


def test_rab_pos_against_an_element_loop_and_closed_forms():
    g = torch.Generator().manual_seed(2)
    s2 = 6
    rel = torch.randn(s2, s2, generator=g)
    ident = (torch.rand(s2, s2, generator=g) < 0.3).float()
    lens = [0, 3, 5]
    out = BO.rab_pos(rel, ident, lens)
    for u, v in enumerate(lens):
        for i in range(s2):
            for j in range(s2):
                want = rel[0, 0] if ident[i, j] == 1 else rel[min(i, v), j]
                assert out[u, i, j] == want
    assert torch.equal(BO.rab_pos(rel, torch.ones(s2, s2), lens), rel[0, 0].expand(3, s2, s2))
    assert torch.equal(BO.rab_pos(rel, torch.zeros(s2, s2), [s2 - 1])[0], rel)
