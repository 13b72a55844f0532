"""GPU parity tests: the HIP path (through the C ABI) against the CPU oracle on the same seeded inputs.

Sizes are chosen so that the oracle finishes in seconds.  Every case prints its name before
touching the GPU so that a fault names its case.
"""
import math
import sys

import numpy as np
import pytest
import torch

from oracle import hstu_oracle as O
from recsdk_amd import workloads as W
from tests import hstu_testlib as T

pytestmark = pytest.mark.gpu
FORCE_GENERIC = 2


def say(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def _jag(seed, lens_q, nq, nk, dqk, dv, dtype, lens_k=None, index_dtype=torch.int64, extra_rows=0):
    rng = np.random.default_rng(seed)
    lens_k = lens_q if lens_k is None else lens_k
    tq, tk = sum(lens_q) + extra_rows, sum(lens_k)
    mk = lambda shape: torch.from_numpy(rng.normal(0, 0.5, shape).astype(np.float32)).to(dtype)
    c = dict(q=mk((tq, nq, dqk)), k=mk((tk, nk, dqk)), v=mk((tk, nk, dv)), seq_offset=W.offsets(lens_q, index_dtype),
             max_seq_len=max(max(lens_q), 1), alpha=1.0 / math.sqrt(dqk), mask_type=0, lens=lens_q)
    if lens_k is not lens_q:
        c["seq_offset_k"] = W.offsets(lens_k, index_dtype)
        c["max_seq_len_k"] = max(max(lens_k), 1)
    return c, rng


DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def test_config1_fp32_plumbing():
    """B=4, h=2, d=32, L in [16,128], fp32, alpha=1/sqrt(d), causal: 1e-5 relative against the fp64 oracle."""
    cfg = W.config1()
    say("config1", cfg["lens"])
    ref = T.oracle_jagged(cfg, compute_dtype=torch.float64)
    out, name = T.run_capi(cfg)
    assert name == "generic_f32"
    T.assert_parity(out, ref, torch.float32, what="config1 capi")
    out2 = T.run_op(cfg)
    assert torch.equal(out, out2), "torch op and direct C-ABI call disagree"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", [
    dict(lens=[1], nq=1, nk=1, dqk=16, dv=16),
    dict(lens=[15, 16, 17, 1, 64, 65], nq=2, nk=2, dqk=32, dv=32),
    dict(lens=[33, 0, 70, 0], nq=4, nk=2, dqk=24, dv=48),                       # interior + trailing empty, GQA, Dqk != Dv
    dict(lens=[100, 257], nq=8, nk=1, dqk=64, dv=16, index_dtype=torch.int32),
    dict(lens=[40, 90], lens_k=[75, 90], nq=2, nk=2, dqk=64, dv=64),             # delta-q
    dict(lens=[130], nq=1, nk=1, dqk=256, dv=256),
    dict(lens=[50, 20], nq=2, nk=2, dqk=128, dv=128, extra_rows=5),              # rows past the last offset -> zeros
    dict(lens=[70, 45], nq=3, nk=3, dqk=40, dv=80, mask_type=2),
])
def test_generic_shapes(case, dtype):
    c = dict(case)
    lens = c.pop("lens")
    say("generic_shapes", dtype, case)
    cfg, rng = _jag(11, lens, c["nq"], c["nk"], c["dqk"], c["dv"], dtype, c.get("lens_k"),
                    c.get("index_dtype", torch.int64), c.get("extra_rows", 0))
    cfg["mask_type"] = c.get("mask_type", 0)
    ref = T.oracle_jagged(cfg, compute_dtype=torch.float64)
    out, name = T.run_capi(cfg, flags=FORCE_GENERIC)
    assert name.startswith("generic")
    T.assert_parity(out, ref, dtype, what=str(case))
    if c.get("extra_rows"):
        assert torch.equal(out[-c["extra_rows"]:], torch.zeros_like(out[-c["extra_rows"]:]))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("ctx,tgt,tgs", [(0, 0, 0), (3, 0, 0), (0, 6, 1), (4, 9, 3), (2, 7, 0), (5, 5, 5)])
def test_generic_builtin_masks(ctx, tgt, tgs, dtype):
    say("builtin_masks", dtype, ctx, tgt, tgs)
    lens = [40, 71, 129]
    cfg, rng = _jag(12, lens, 2, 2, 32, 32, dtype)
    cfg["num_context"] = torch.tensor([ctx, ctx + 1 if ctx else 0, ctx])
    cfg["num_target"] = torch.tensor([tgt, tgt, tgt + 2 if tgt else 0])
    cfg["target_group_size"] = tgs
    ref = T.oracle_jagged(cfg, compute_dtype=torch.float64)
    out, _ = T.run_capi(cfg, flags=FORCE_GENERIC)
    T.assert_parity(out, ref, dtype)
    # delta-q with targets: Q rows are the last rows of the K timeline
    cfg2, _ = _jag(13, [30, 50], 2, 1, 32, 32, dtype, lens_k=[64, 50])
    cfg2["num_target"] = torch.tensor([tgt, tgt])
    cfg2["num_context"] = torch.tensor([ctx, ctx])
    cfg2["target_group_size"] = tgs
    ref2 = T.oracle_jagged(cfg2, compute_dtype=torch.float64)
    out2, _ = T.run_capi(cfg2, flags=FORCE_GENERIC)
    T.assert_parity(out2, ref2, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_generic_custom_mask_and_dense_bias(dtype):
    say("custom_mask_bias", dtype)
    lens = [37, 64, 90]
    cfg, rng = _jag(14, lens, 2, 2, 32, 48, dtype)
    b, n, m = len(lens), 2, max(lens)
    cfg["attn_bias"] = torch.from_numpy(rng.random((b, n, m, m)).astype(np.float32)).to(dtype)
    ref = T.oracle_jagged(cfg, compute_dtype=torch.float64)
    out, _ = T.run_capi(cfg, flags=FORCE_GENERIC)
    T.assert_parity(out, ref, dtype, what="bias + tril")
    cfg["mask"] = torch.from_numpy(rng.integers(0, 2, (b, n, m, m)).astype(np.float32)).to(dtype)
    cfg["mask_type"] = 3
    ref = T.oracle_jagged(cfg, compute_dtype=torch.float64)
    out, _ = T.run_capi(cfg, flags=FORCE_GENERIC)
    T.assert_parity(out, ref, dtype, what="bias + custom mask")
    # explicit tril mask == built-in
    tril = torch.tril(torch.ones(m, m)).expand(b, n, m, m).to(dtype).contiguous()
    out_t, _ = T.run_capi(cfg, mask=tril, flags=FORCE_GENERIC)
    out_b, _ = T.run_capi(cfg, mask=None, mask_type=0, flags=FORCE_GENERIC)
    assert torch.equal(out_t, out_b)


def test_repeat_offset_and_permutation():
    """Trailing duplicate offset changes nothing (test_hstu_jagged_forward.py:44-47); permuting the
    sequences permutes the outputs."""
    say("repeat_offset")
    cfg, _ = _jag(15, [20, 35, 9], 2, 2, 32, 32, torch.float32)
    cfg["num_target"] = torch.tensor([2, 3, 1]); cfg["target_group_size"] = 1
    base, _ = T.run_capi(cfg)
    rep = dict(cfg, seq_offset=torch.cat([cfg["seq_offset"], cfg["seq_offset"][-1:]]),
               num_target=torch.tensor([2, 3, 1, 1]))
    out, _ = T.run_capi(rep)
    assert torch.equal(out, base)
    o = cfg["seq_offset"].tolist()
    perm = [2, 0, 1]
    seg = lambda x: [x[o[i]:o[i + 1]] for i in range(3)]
    pc = dict(cfg, q=torch.cat([seg(cfg["q"])[i] for i in perm]), k=torch.cat([seg(cfg["k"])[i] for i in perm]),
              v=torch.cat([seg(cfg["v"])[i] for i in perm]), seq_offset=W.offsets([cfg["lens"][i] for i in perm]),
              num_target=torch.tensor([1, 2, 3]))
    outp, _ = T.run_capi(pc)
    assert torch.equal(outp, torch.cat([seg(base)[i] for i in perm]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dense_layout(dtype):
    say("dense", dtype)
    rng = np.random.default_rng(16)
    b, s, n, d = 3, 45, 2, 32
    mk = lambda: torch.from_numpy(rng.normal(0, 0.5, (b, s, n, d)).astype(np.float32)).to(dtype)
    cfg = dict(q=mk(), k=mk(), v=mk(), max_seq_len=s, mask_type=0)
    cfg["attn_bias"] = torch.from_numpy(rng.random((b, n, s, s)).astype(np.float32)).to(dtype)
    ref = O.hstu_dense_forward(cfg["q"], cfg["k"], cfg["v"], max_seq_len=s, attn_bias=cfg["attn_bias"],
                               compute_dtype=torch.float64)
    out, _ = T.run_capi(cfg, op="dense")
    T.assert_parity(out, ref, dtype)
    assert torch.equal(T.run_op(cfg, op="dense"), out)
    # B=1 dense == jagged
    one = dict(q=cfg["q"][:1], k=cfg["k"][:1], v=cfg["v"][:1], max_seq_len=s, mask_type=0)
    od, _ = T.run_capi(one, op="dense")
    jag = dict(q=one["q"][0], k=one["k"][0], v=one["v"][0], seq_offset=W.offsets([s]), max_seq_len=s, mask_type=0)
    oj, _ = T.run_capi(jag)
    assert torch.equal(od[0], oj)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_table_bias_equals_dense_bias(dtype):
    """Fused table gather == the dense-bias op fed with the tables expanded by the reference formulas
    (the fused variant has no reference counterpart; this pins it by construction), and == oracle."""
    say("table_bias", dtype)
    rng = np.random.default_rng(17)
    lens, lens_k = [50, 77, 20], [50, 90, 20]
    cfg, _ = _jag(17, lens, 2, 2, 32, 32, dtype, lens_k=lens_k)
    mq, mk = cfg["max_seq_len"], cfg["max_seq_len_k"]
    cfg["pos_table"] = torch.from_numpy(rng.normal(0, 0.5, 2 * mk - 1).astype(np.float32))
    cfg["ts_table"] = torch.from_numpy(rng.normal(0, 0.5, 129).astype(np.float32))
    ts = [1_700_000_000 + np.cumsum(rng.exponential(600.0, l).astype(np.int64)) for l in lens_k]
    ts[1][5:9] = ts[1][5]                                                     # equal timestamps -> dt = 0
    cfg["timestamps"] = torch.from_numpy(np.concatenate(ts))
    cfg["num_target"] = torch.tensor([4, 4, 4]); cfg["target_group_size"] = 1
    ref = T.oracle_jagged(cfg, compute_dtype=torch.float64)
    out, _ = T.run_capi(cfg, flags=FORCE_GENERIC)
    T.assert_parity(out, ref, dtype, what="fused tables vs oracle")
    assert torch.equal(T.run_op(cfg, op="table"), T.run_capi(cfg)[0])
    if dtype == torch.float32:
        dense = O.dense_bias_from_tables(cfg["seq_offset"], cfg["seq_offset_k"], 2, mq, mk, pos_table=cfg["pos_table"],
                                         ts_table=cfg["ts_table"], timestamps=cfg["timestamps"])
        d2 = dict(cfg, attn_bias=dense, pos_table=None, ts_table=None, timestamps=None)
        out_d, _ = T.run_capi(d2, flags=FORCE_GENERIC)
        assert torch.allclose(out, out_d, rtol=1e-6, atol=1e-9)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("page_size,new_hist", [(32, 0), (64, 7), (8, 3)])
def test_paged_matches_oracle(dtype, page_size, new_hist):
    say("paged", dtype, page_size, new_hist)
    cfg = W.paged_config(18, 5, 2, 32, new_hist + 1, 150, 6, page_size, dtype, new_hist=new_hist)
    ref = T.oracle_paged(cfg, compute_dtype=torch.float64)
    out, _ = T.run_capi(cfg, op="paged", flags=FORCE_GENERIC)
    T.assert_parity(out, ref, dtype)
    assert torch.equal(T.run_op(cfg, op="paged"), T.run_capi(cfg, op="paged")[0])


def test_paged_fp8_cache():
    """fp8 cache == bf16 op on the dequantised cache (construction), and within 5e-2 of the unquantised oracle."""
    say("paged_fp8")
    cfg = W.paged_config(19, 4, 2, 64, 40, 300, 16, 64, torch.bfloat16)
    cfg["kv_cache_fp8"], cfg["kv_scales"] = W.quantize_pages_fp8(cfg["kv_cache"])
    u8, sc = O.quantize_kv_cache_fp8(cfg["kv_cache"])
    assert torch.equal(u8, cfg["kv_cache_fp8"].view(torch.uint8)) and torch.equal(sc, cfg["kv_scales"])
    out8, _ = T.run_capi(cfg, op="paged", use_fp8=True, flags=FORCE_GENERIC)
    deq = O.dequantize_kv_cache_fp8(u8, sc, torch.bfloat16)
    out16, _ = T.run_capi(dict(cfg, kv_cache=deq), op="paged", flags=FORCE_GENERIC)
    assert torch.equal(out8, out16)
    ref = T.oracle_paged(cfg, compute_dtype=torch.float64)
    T.assert_parity(out8, ref, torch.bfloat16, tol=5e-2, what="fp8 cache vs unquantised oracle")
    assert torch.equal(T.run_op(cfg, op="paged_fp8"), T.run_capi(cfg, op="paged", use_fp8=True)[0])


def test_buffers_off_a_16_byte_boundary_take_the_plain_kernel():
    """q (or any of k, v, out) starting 2 bytes past a 16-byte boundary: the MFMA kernels' 16-byte accesses do not apply,
    the call is routed to the plain kernel and the result is the same."""
    say("misaligned")
    from recsdk_amd import _capi
    dtype = torch.bfloat16
    cfg, _ = _jag(81, [70, 200, 33], 2, 2, 128, 128, dtype)
    q = cfg["q"].cuda()
    buf = torch.empty(q.numel() + 8, dtype=dtype, device="cuda")
    q_off = buf[1:1 + q.numel()].view_as(q)
    q_off.copy_(q)
    assert q_off.data_ptr() % 16 == 2
    out = torch.full_like(q, float("nan"))
    p, keep = _capi.make_params(q_off, cfg["k"].cuda(), cfg["v"].cuda(), out, seq_offset_q=cfg["seq_offset"].cuda(),
                                max_seq_len_q=cfg["max_seq_len"], alpha=cfg["alpha"])
    assert _capi.describe_kernel(p) == "generic_bf16"
    _capi.run("jagged", p)
    torch.cuda.synchronize()
    T.assert_parity(out.cpu(), T.oracle_jagged(cfg), dtype, what="misaligned q")


def test_error_paths_on_device():
    """Host rejections surface as RuntimeError with the reference's messages (test_hstu_jagged_forward.py:508-711)."""
    say("errors")
    import recsdk_amd  # noqa: F401
    q = torch.randn(10, 2, 32, device="cuda")
    off = torch.tensor([0, 4, 10], device="cuda")
    m = torch.ops.mxrec
    with pytest.raises(RuntimeError, match="The q should be 3D in jagged layout"):
        m.hstu_jagged(q[0], q, q, None, None, 0, 8, 0.0, off)
    with pytest.raises(RuntimeError, match=r"maxSeqLen expect in \[1, 20480\]"):
        m.hstu_jagged(q, q, q, None, None, 0, 20481, 0.0, off)
    with pytest.raises(RuntimeError, match="should have at least two element"):
        m.hstu_jagged(q, q, q, None, None, 0, 8, 0.0, off[:1])
    bad = torch.randn(10, 2, 24, device="cuda")
    with pytest.raises(RuntimeError, match="V dim size"):
        m.hstu_jagged(bad, bad, bad, None, None, 0, 8, 0.0, off)
    with pytest.raises(RuntimeError, match="divisible"):
        m.hstu_jagged(torch.randn(10, 3, 32, device="cuda"), q, q, None, None, 0, 8, 0.0, off)
