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


def _random_forward_case(seed, it):
    """Paged history (pages in the dtype of q or fp8 with scales, page sizes that do and do not divide the tile), bias
    tables, dense bias and / or custom mask on aligned and unaligned rows."""
    import numpy as np
    from recsdk_amd import workloads as W
    from tests.test_parity_gpu import _jag
    rnd = random.Random(seed * 100000 + it)
    kind = rnd.choice(["paged", "paged8", "table", "xmask"])
    dtype = rnd.choice([torch.bfloat16, torch.float16])
    kw = {}
    if kind in ("paged", "paged8"):
        d = rnd.choice([64, 128, 128])
        ps = rnd.choice([4, 8, 10, 12, 16, 32, 64, 7])
        users, heads = rnd.randint(1, 6), rnd.choice([1, 2, 4])
        cand, new_hist = rnd.choice([1, 17, 40, 130]), rnd.choice([0, 0, 3, 33])
        lo = new_hist + 1
        hi = rnd.choice([lo + 5, 200, 900])
        if kind == "paged8":
            dtype = torch.bfloat16
        cfg = W.paged_config(seed * 1000 + it, users, heads, d, lo, hi, cand, ps, dtype, new_hist=new_hist)
        kw["op"] = "paged"
        if kind == "paged8":
            cfg["kv_cache_fp8"], cfg["kv_scales"] = W.quantize_pages_fp8(cfg["kv_cache"])
            kw["use_fp8"] = True
        return cfg, dtype, kw, f"{kind} d={d} page_size={ps} users={users} heads={heads} cand={cand} new_hist={new_hist} hist={cfg['hist']}"
    d = rnd.choice([32, 64, 128, 256])
    nseq, maxl = rnd.randint(1, 4), rnd.choice([50, 200, 500])
    lens = [rnd.randint(1, maxl) for _ in range(nseq)]
    lens_k = [l + rnd.randint(0, 100) for l in lens] if rnd.random() < 0.4 else None
    nq = rnd.choice([1, 2, 4]) if kind == "table" else rnd.choice([1, 2])
    cfg, rng = _jag(seed * 1000 + it, lens, nq, nq, d, d, dtype, lens_k=lens_k)
    mq, mk = cfg["max_seq_len"], cfg.get("max_seq_len_k") or cfg["max_seq_len"]
    if kind == "table":
        which = rnd.choice(["pos", "ts", "both"])
        if which != "ts":
            cfg["pos_table"] = torch.from_numpy(rng.normal(0, 0.5, 2 * mk - 1).astype(np.float32))
        if which != "pos":
            nb = rnd.choice([16, 40, 128])
            cfg["ts_table"] = torch.from_numpy(rng.normal(0, 0.5, nb + 1).astype(np.float32))
            cfg["bucket_divisor"] = rnd.choice([0.301, 0.301, 0.2, 0.7])
            gap = rnd.choice([1.0, 60.0, 6000.0, 1e9])
            lk = lens if lens_k is None else lens_k
            cfg["timestamps"] = torch.from_numpy(np.concatenate([1_700_000_000 + np.cumsum(rng.exponential(gap, l).astype(np.int64)) for l in lk]))
        if rnd.random() < 0.5:
            cfg["num_target"] = torch.tensor([rnd.randint(0, min(l, 30)) for l in lens])
            cfg["target_group_size"] = rnd.choice([0, 1, 3])
        return cfg, dtype, kw, f"table {which} d={d} lens={lens} lens_k={lens_k} divisor={cfg.get('bucket_divisor')}"
    if rnd.random() < 0.7:   # rows on 16-byte boundaries: the variants that copy the blocks straight into LDS
        mk = (mk + 7) // 8 * 8
        if lens_k is None:
            mq = cfg["max_seq_len"] = mk
        else:
            cfg["max_seq_len_k"] = mk
    which = rnd.choice(["bias", "mask", "both"])
    if which != "mask":
        cfg["attn_bias"] = torch.from_numpy(rng.normal(0, 0.3, (nseq, nq, mq, mk)).astype(np.float32)).to(dtype)
    if which != "bias":
        cfg["mask_type"] = 3
        cfg["mask"] = (torch.from_numpy(rng.random((nseq, nq, mq, mk))) < 0.6).to(dtype)
    return cfg, dtype, kw, f"dense {which} d={d} lens={lens} lens_k={lens_k} max_q={mq} max_k={mk}"


@pytest.mark.parametrize("seed", [21, 22, 23])
def test_random_forward_variants_against_plain_kernels(seed):
    for it in range(40):
        cfg, dtype, kw, desc = _random_forward_case(seed, it)
        say("random forward", seed, it, dtype, desc)
        out, name = T.run_capi(cfg, **kw)
        assert name.startswith("mfma_"), name
        gen, _ = T.run_capi(cfg, flags=2, **kw)
        T.assert_parity(out, gen.float(), dtype, what=desc)
