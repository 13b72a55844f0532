"""Pins ``oracle.builtin_mask`` against the reference-held 65x65 fixture
(cust_op/test/hstu_dense/torch/target_mask_tesnor_example.txt), the independent point
predicate and the tril special cases."""
import itertools
import os

import pytest
import torch

from oracle import hstu_oracle as O


def _load_fixture(golden_dir):
    rows = []
    with open(os.path.join(golden_dir, "target_mask_65x65.txt")) as f:
        for line in f:
            line = line.strip()
            if line:
                rows.append([int(x) for x in line.split(",")])
    return torch.tensor(rows, dtype=torch.float32)


def test_fixture_is_ctx17_tgt31_tgs5(golden_dir):
    fx = _load_fixture(golden_dir)
    assert fx.shape == (65, 65)
    # the fixture's parameters are recovered by search, not assumed
    hits = [(c, t, g) for c in range(0, 33) for t in range(0, 49) for g in range(0, 9)
            if torch.equal(O.builtin_mask(65, 65, c, t, g), fx)]
    assert (17, 31, 5) in hits
    assert all(h[0] == 17 and h[1] == 31 for h in hits)


def test_fixture_matches_point_predicate(golden_dir):
    fx = _load_fixture(golden_dir)
    for i in range(65):
        for j in range(65):
            assert O.mask_point(i, j, 65, 65, 17, 31, 5) == int(fx[i, j]), (i, j)


@pytest.mark.parametrize("lq,lk", [(1, 1), (7, 7), (16, 16), (5, 9), (33, 64), (64, 64), (40, 41)])
@pytest.mark.parametrize("ctx,tgt,tgs", [(0, 0, 0), (3, 0, 0), (0, 4, 1), (2, 5, 3), (0, 5, 0), (4, 4, 2), (0, 1, 1)])
def test_closed_form_vs_point(lq, lk, ctx, tgt, tgs):
    if ctx + tgt > lq:
        pytest.skip("context+target longer than the sequence")
    m = O.builtin_mask(lq, lk, ctx, tgt, tgs)
    ref = torch.tensor([[O.mask_point(i, j, lq, lk, ctx, tgt, tgs) for j in range(lk)] for i in range(lq)],
                       dtype=torch.float32)
    assert torch.equal(m, ref)


def test_special_cases():
    for lq, lk in [(5, 5), (4, 9), (9, 9)]:
        assert torch.equal(O.builtin_mask(lq, lk), torch.tril(torch.ones(lq, lk), diagonal=lk - lq))
    # tgs == 1: the trailing square is the identity
    m = O.builtin_mask(12, 12, 0, 5, 1)
    assert torch.equal(m[-5:, -5:], torch.eye(5))
    assert torch.equal(m[-5:, :7], torch.ones(5, 7))
    assert torch.equal(m[:7, :7], torch.tril(torch.ones(7, 7)))
    # num_target without a group size leaves plain causal
    assert torch.equal(O.builtin_mask(12, 12, 0, 5, 0), torch.tril(torch.ones(12, 12)))
    # context rows see every history column, no target column
    m = O.builtin_mask(10, 10, 3, 2, 1)
    assert torch.equal(m[:3, :8], torch.ones(3, 8)) and m[:3, 8:].sum() == 0


def test_valid_batch_rule():
    assert O.valid_batch(torch.tensor([0, 3, 5, 5, 5])) == 2
    assert O.valid_batch(torch.tensor([0, 3, 3, 5])) == 3
    assert O.valid_batch(torch.tensor([0, 0])) == 1
