"""Seeded random geometries: the matrix-core kernels against the plain-FMA kernels (both on the GPU, through the C ABI),
forward and backward.  Head dims 32 .. 256, both 16-bit dtypes, GQA, empty and one-row sequences, longer K than Q,
context / target rows with groups, no mask, dense bias on aligned and unaligned rows, rows behind the last offset."""
import random

import pytest
import torch

from tests import hstu_testlib as T
from tests.test_backward_gpu import _case
from tests.test_parity_gpu import say

pytestmark = pytest.mark.gpu


def _random_case(seed, it):
    rnd = random.Random(seed * 100000 + it)
    d = rnd.choice([32, 64, 128, 128, 128, 256])
    dtype = rnd.choice([torch.bfloat16, torch.float16])
    nk = rnd.choice([1, 2, 3, 4])
    ratio = rnd.choice([1, 1, 1, 2, 4])
    nq = nk * ratio
    if nq > 16:
        nq, nk = 16, 16 // ratio
    nseq = rnd.choice([1, 2, 3, 5, 9])
    maxl = rnd.choice([40, 130, 300, 700])
    lens_q = [rnd.choice([0, 1, rnd.randint(1, maxl), rnd.randint(1, maxl), rnd.randint(maxl // 2, maxl)]) for _ in range(nseq)]
    if sum(lens_q) == 0:
        lens_q[0] = 5
    lens_k = [l + rnd.randint(0, 150) for l in lens_q] if rnd.random() < 0.3 else None
    mode = rnd.choice(["plain", "plain", "tgt", "none", "bias", "bias", "bias_tgt"])
    kw = {}
    if "tgt" in mode:
        kw["ctx"] = [rnd.randint(0, min(l, 9)) for l in lens_q]
        kw["tgt"] = [rnd.randint(0, max(0, min(l - c, 70))) for l, c in zip(lens_q, kw["ctx"])]
        kw["tgs"] = rnd.choice([0, 1, 2, 5])
    if mode == "none":
        kw["mask"] = "none"
    if "bias" in mode:
        kw["bias"] = True
    cfg, grad = _case(seed * 1000 + it, lens_q, nq, nk, d, d, dtype, lens_k=lens_k, extra_rows=rnd.choice([0, 0, 3]), **kw)
    if "bias" in mode and rnd.random() < 0.7:
        # rows of the bias on 16-byte boundaries (what the matrix-core paths with a bias ask for): pad the attribute to a multiple of 8
        b = cfg["attn_bias"]
        mk = (cfg["max_seq_len_k"] + 7) // 8 * 8
        mq = mk if lens_k is None else b.shape[2]
        nb = torch.zeros(b.shape[0], b.shape[1], mq, mk, dtype=b.dtype)
        nb[:, :, :b.shape[2], :b.shape[3]] = b
        cfg["attn_bias"], cfg["max_seq_len_k"] = nb, mk
        if lens_k is None:
            cfg["max_seq_len"] = mk
    return cfg, grad, dtype, dict(d=d, nq=nq, nk=nk, lens_q=lens_q, lens_k=lens_k, mode=mode, **kw)


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_geometries_matrix_core_kernels_against_plain_kernels(seed):
    for it in range(40):
        cfg, grad, dtype, desc = _random_case(seed, it)
        say("random", seed, it, dtype, desc)
        out, name = T.run_capi(cfg)
        assert name.startswith("mfma_"), name
        gen, _ = T.run_capi(cfg, flags=2)
        T.assert_parity(out, gen.float(), dtype, what=f"forward {desc}")
        got = T.run_capi_backward(cfg, grad)
        ref = T.run_capi_backward(cfg, grad, flags=2)
        names = ("dq", "dk", "dv", "dbias") if cfg.get("attn_bias") is not None else ("dq", "dk", "dv")
        for n, g, r in zip(names, got, ref):
            T.assert_parity(g, r.double(), dtype, what=f"backward {n} {desc}")
