"""GPU parity of the jagged backward (through the C ABI) against the oracle's float64 restatement of the reference
golden (build/presmoke/hstu/hstu_common.py:387-476) on the same seeded inputs."""
import math
import sys

import numpy as np
import pytest
import torch

from oracle import hstu_oracle as O
from recsdk_amd import workloads as W
from tests import hstu_testlib as T

pytestmark = pytest.mark.gpu


def say(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def _case(seed, lens_q, nq, nk, dqk, dv, dtype, lens_k=None, bias=False, ctx=None, tgt=None, tgs=0, mask=None,
          index_dtype=torch.int64, extra_rows=0):
    rng = np.random.default_rng(seed)
    lens_k = lens_q if lens_k is None else lens_k
    tq, tk = sum(lens_q) + extra_rows, sum(lens_k) + extra_rows
    mk = lambda shape, std=0.5: torch.from_numpy(rng.normal(0, std, shape).astype(np.float32)).to(dtype)
    mq, mkk = max(max(lens_q), 1), max(max(lens_k), 1)
    c = dict(q=mk((tq, nq, dqk)), k=mk((tk, nk, dqk)), v=mk((tk, nk, dv)), seq_offset=W.offsets(lens_q, index_dtype),
             seq_offset_k=W.offsets(lens_k, index_dtype), max_seq_len=mq, max_seq_len_k=mkk, alpha=1.0 / math.sqrt(dqk),
             mask_type=0, silu_scale=1.0 / 8)
    if bias:
        c["attn_bias"] = mk((len(lens_q), nq, mq, mkk), 0.3)
    if ctx is not None:
        c["num_context"] = torch.tensor(ctx, dtype=index_dtype)
        c["num_target"] = torch.tensor(tgt, dtype=index_dtype)
        c["target_group_size"] = tgs
    if mask == "custom":
        c["mask_type"] = 3
        c["mask"] = (torch.from_numpy(rng.random((len(lens_q), nq, mq, mkk))) < 0.6).to(dtype)
    elif mask == "none":
        c["mask_type"] = 2
    grad = mk((tq, nq, dv), 1.0)
    return c, grad


def _oracle(c, grad):
    return O.hstu_jagged_backward(grad, c["q"], c["k"], c["v"], c["seq_offset"], c["seq_offset_k"],
                                  max_seq_len_q=c["max_seq_len"], max_seq_len_k=c["max_seq_len_k"], mask_type=c["mask_type"],
                                  mask=c.get("mask"), attn_bias=c.get("attn_bias"), silu_scale=c["silu_scale"], alpha=c["alpha"],
                                  num_context=c.get("num_context"), num_target=c.get("num_target"),
                                  target_group_size=c.get("target_group_size", 0))


def _check(c, grad, dtype, what):
    got = T.run_capi_backward(c, grad)
    want = _oracle(c, grad)
    nq_rows, nk_rows = int(c["seq_offset"][-1]), int(c["seq_offset_k"][-1])
    for name, g, w in zip(("dq", "dk", "dv", "dbias"), got, want):
        if w is None:
            assert g is None
            continue
        T.assert_parity(g, w, dtype, what=f"{what} {name}")
    # rows past the last offset carry zeros
    assert float(got[0][nq_rows:].abs().max() if got[0][nq_rows:].numel() else 0.0) == 0.0
    assert float(got[1][nk_rows:].abs().max() if got[1][nk_rows:].numel() else 0.0) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_backward_plain_causal(dtype):
    say("backward causal", dtype)
    c, grad = _case(1, [37, 5, 64, 0, 129], 2, 2, 32, 32, dtype)
    _check(c, grad, dtype, "causal")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_backward_delta_q_gqa_bias(dtype):
    say("backward delta-q gqa bias", dtype)
    c, grad = _case(2, [20, 7, 33], 4, 2, 64, 48, dtype, lens_k=[52, 30, 33], bias=True)
    _check(c, grad, dtype, "delta-q gqa bias")


def test_backward_context_and_targets_with_bias():
    say("backward ctx/tgt")
    c, grad = _case(3, [70, 40], 2, 1, 32, 16, torch.float32, bias=True, ctx=[3, 0], tgt=[9, 6], tgs=3)
    _check(c, grad, torch.float32, "ctx/tgt")


@pytest.mark.parametrize("mask", ["custom", "none"])
def test_backward_custom_and_no_mask(mask):
    say("backward mask", mask)
    c, grad = _case(4, [33, 18], 2, 2, 16, 16, torch.float32, mask=mask, bias=(mask == "custom"))
    _check(c, grad, torch.float32, mask)


def test_backward_large_head_dim_int32_offsets_and_tail_rows():
    say("backward d=256, int32 offsets, rows past the last offset")
    c, grad = _case(5, [50, 31], 2, 2, 256, 128, torch.bfloat16, index_dtype=torch.int32, extra_rows=5)
    _check(c, grad, torch.bfloat16, "d=256")


def test_backward_matches_autograd_of_our_forward_oracle_at_training_shape():
    """A slice of the headline shape (d=128, 4 heads, bf16) against torch.autograd of the forward oracle in float64."""
    say("backward headline slice")
    c, grad = _case(6, [300, 257, 512], 4, 4, 128, 128, torch.bfloat16)
    got = T.run_capi_backward(c, grad)
    leaves = [c[n].double().requires_grad_(True) for n in ("q", "k", "v")]
    out = O.hstu_jagged_forward(leaves[0], leaves[1], leaves[2], c["seq_offset"], c["seq_offset_k"], max_seq_len_q=c["max_seq_len"],
                                max_seq_len_k=c["max_seq_len_k"], silu_scale=c["silu_scale"], alpha=c["alpha"], mode="exact",
                                compute_dtype=torch.float64)
    auto = torch.autograd.grad(out, leaves, grad_outputs=grad.double())
    for name, g, w in zip(("dq", "dk", "dv"), got, auto):
        T.assert_parity(g, w, torch.bfloat16, what=f"headline slice {name}")


def test_backward_torch_ops_equal_and_delta_overloads():
    """The drop-in entries: torch.ops.mxrec.hstu_jagged_backward with the reference's two schemas."""
    say("backward torch ops")
    import recsdk_amd  # noqa: F401
    dev = lambda t: None if t is None else t.cuda()
    c, grad = _case(7, [40, 23], 2, 2, 64, 64, torch.bfloat16, bias=True)
    want = T.run_capi_backward(c, grad)
    got = torch.ops.mxrec.hstu_jagged_backward(dev(grad), dev(c["q"]), dev(c["k"]), dev(c["v"]), None, dev(c["attn_bias"]), 0,
                                               c["max_seq_len"], c["silu_scale"], dev(c["seq_offset"]), None, None, 0, c["alpha"])
    for g, w in zip(got, want):
        assert torch.equal(g.cpu(), w)
    c, grad = _case(8, [12, 9], 4, 2, 32, 32, torch.float32, lens_k=[30, 9])
    want = T.run_capi_backward(c, grad)
    got = torch.ops.mxrec.hstu_jagged_backward(dev(grad), dev(c["q"]), dev(c["k"]), dev(c["v"]), None, None, 0, c["max_seq_len"],
                                               c["max_seq_len_k"], c["silu_scale"], dev(c["seq_offset"]), dev(c["seq_offset_k"]),
                                               None, None, 0, c["alpha"])
    for g, w in zip(got[:3], want[:3]):
        assert torch.equal(g.cpu(), w)
    assert got[3] is None or got[3].numel() == 0


MFMA_CASES = [
    # lens_q, nq, nk, d, dtype, extras
    dict(lens_q=[300, 129, 64, 1, 0, 257], nq=2, nk=2, d=128, dtype=torch.bfloat16),
    dict(lens_q=[515, 31, 128, 2], nq=3, nk=3, d=128, dtype=torch.float16),                            # (dV by the forward's kernel on reversed rows)
    dict(lens_q=[300, 129, 64, 1, 0, 257], nq=2, nk=2, d=64, dtype=torch.bfloat16),                   # (the same at head dim 64)
    dict(lens_q=[200, 77], nq=4, nk=2, d=64, dtype=torch.float16),                                    # GQA
    dict(lens_q=[130, 40], nq=2, nk=1, d=128, dtype=torch.bfloat16, lens_k=[333, 40]),                 # delta-q + GQA
    dict(lens_q=[260, 150], nq=2, nk=2, d=64, dtype=torch.bfloat16, ctx=[5, 0], tgt=[40, 17], tgs=3),  # context rows + target groups
    dict(lens_q=[190, 33], nq=1, nk=1, d=128, dtype=torch.float16, mask="none"),
    dict(lens_q=[515], nq=2, nk=2, d=64, dtype=torch.bfloat16, ctx=[130], tgt=[0], tgs=1),             # context rows across tiles
    # dense attn_bias (rows of max_seq_len_k % 8 == 0 elements): the scores take it in, the dQ kernel writes dBias
    dict(lens_q=[296, 129, 64, 1, 0, 257], nq=2, nk=2, d=128, dtype=torch.bfloat16, bias=True),
    dict(lens_q=[200, 77], nq=4, nk=2, d=64, dtype=torch.float16, bias=True),                          # GQA
    dict(lens_q=[130, 40], nq=2, nk=1, d=128, dtype=torch.bfloat16, lens_k=[336, 40], bias=True),      # delta-q + GQA
    dict(lens_q=[264, 150], nq=2, nk=2, d=64, dtype=torch.bfloat16, ctx=[5, 0], tgt=[40, 17], tgs=3, bias=True),
    dict(lens_q=[192, 33], nq=1, nk=1, d=128, dtype=torch.float16, mask="none", bias=True),
    # the ends of the reference's head-dim sweep (test_backward_op_benchmark.py: head_dims 32 .. 256)
    dict(lens_q=[300, 129, 64, 1, 0, 257], nq=2, nk=2, d=32, dtype=torch.bfloat16),
    dict(lens_q=[200, 77], nq=4, nk=2, d=32, dtype=torch.float16, ctx=[3, 0], tgt=[20, 9], tgs=2),
    dict(lens_q=[264, 150], nq=2, nk=1, d=32, dtype=torch.bfloat16, bias=True),
    dict(lens_q=[300, 129, 64, 1, 0, 257], nq=2, nk=2, d=256, dtype=torch.bfloat16),
    dict(lens_q=[130, 40], nq=2, nk=1, d=256, dtype=torch.float16, lens_k=[333, 40]),
    dict(lens_q=[200, 72], nq=2, nk=2, d=256, dtype=torch.bfloat16, bias=True),
    # custom mask (mask_type 3, rows of max_seq_len_k % 8 == 0 elements): read like a bias, multiplies P and dS
    dict(lens_q=[296, 129, 64, 1, 0, 257], nq=2, nk=2, d=128, dtype=torch.bfloat16, mask="custom"),
    dict(lens_q=[200, 77], nq=4, nk=2, d=64, dtype=torch.float16, mask="custom"),                      # GQA
    dict(lens_q=[130, 40], nq=2, nk=1, d=128, dtype=torch.float16, lens_k=[336, 40], mask="custom"),   # delta-q + GQA
    dict(lens_q=[264, 150], nq=2, nk=2, d=32, dtype=torch.bfloat16, mask="custom"),
    dict(lens_q=[136, 72], nq=2, nk=2, d=256, dtype=torch.bfloat16, mask="custom"),
]


@pytest.mark.parametrize("c", MFMA_CASES)
def test_backward_mfma_kernels(c):
    say("backward mfma", {k: v for k, v in c.items() if k != "dtype"}, c["dtype"])
    c = dict(c)
    dtype, d = c.pop("dtype"), c.pop("d")
    cfg, grad = _case(11, c.pop("lens_q"), c.pop("nq"), c.pop("nk"), d, d, dtype, **c)
    got = T.run_capi_backward(cfg, grad)
    assert T.last_backward_kernel.startswith("mfma_bwd_"), T.last_backward_kernel
    want = _oracle(cfg, grad)
    gen = T.run_capi_backward(cfg, grad, flags=2)   # the plain-FMA kernels
    assert T.last_backward_kernel.startswith("generic_bwd_"), T.last_backward_kernel
    names = ("dq", "dk", "dv", "dbias") if cfg.get("attn_bias") is not None else ("dq", "dk", "dv")
    for name, g, w, x in zip(names, got, want, gen):
        T.assert_parity(g, w, dtype, what=f"mfma backward {name}")
        T.assert_parity(g, x.double(), dtype, what=f"mfma vs plain kernels {name}")
    if cfg.get("attn_bias") is not None:
        # dBias is written completely: exact zeros wherever the oracle has none (behind the sequences, under the mask)
        assert bool((got[3][want[3] == 0] == 0).all())


@pytest.mark.parametrize("d", [64, 128])
def test_backward_mfma_sequences_longer_than_the_attribute(d):
    """max_seq_len smaller than the longest sequence: the tiles behind the attribute are still covered."""
    say("backward mfma, rows behind max_seq_len", d)
    cfg, grad = _case(12, [400, 90], 2, 2, d, d, torch.bfloat16)
    cfg["max_seq_len"] = cfg["max_seq_len_k"] = 128
    got = T.run_capi_backward(cfg, grad)
    want = _oracle(cfg, grad)
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        T.assert_parity(g, w, torch.bfloat16, what=f"long {name}")


def test_hstu_jagged_is_differentiable_like_the_reference_op():
    """out.backward() through torch.ops.mxrec.hstu_jagged (.equal and .delta) gives the backward op's gradients."""
    say("autograd through the torch op")
    import recsdk_amd  # noqa: F401
    dev = lambda t: None if t is None else t.cuda()
    for lens_k, bias in (([60, 35], True), ([90, 35], False)):
        c, grad = _case(9, [60, 35], 2, 2, 64, 64, torch.bfloat16, lens_k=lens_k, bias=bias)
        want = T.run_capi_backward(c, grad)
        q, k, v = (dev(c[n]).requires_grad_(True) for n in ("q", "k", "v"))
        b = dev(c.get("attn_bias"))
        if b is not None:
            b.requires_grad_(True)
        if lens_k == [60, 35]:
            out = torch.ops.mxrec.hstu_jagged(q, k, v, None, b, 0, c["max_seq_len"], c["silu_scale"], dev(c["seq_offset"]), None, None, 0,
                                              c["alpha"])
        else:
            out = torch.ops.mxrec.hstu_jagged(q, k, v, None, b, 0, c["max_seq_len"], c["max_seq_len_k"], c["silu_scale"],
                                              dev(c["seq_offset"]), dev(c["seq_offset_k"]), None, None, 0, c["alpha"])
        out.backward(dev(grad))
        assert torch.equal(q.grad.cpu(), want[0]) and torch.equal(k.grad.cpu(), want[1]) and torch.equal(v.grad.cpu(), want[2])
        if b is not None:
            assert torch.equal(b.grad.cpu(), want[3])
    # no gradient requested: the plain forward
    with torch.no_grad():
        c, _ = _case(10, [20], 1, 1, 64, 64, torch.bfloat16)
        out = torch.ops.mxrec.hstu_jagged(dev(c["q"]), dev(c["k"]), dev(c["v"]), None, None, 0, 20, c["silu_scale"], dev(c["seq_offset"]),
                                          None, None, 0, c["alpha"])
        assert not out.requires_grad


def _dense_case(seed, b, s, n, d, dtype, bias=False, mask=None):
    rng = np.random.default_rng(seed)
    mk = lambda shape, std=0.5: torch.from_numpy(rng.normal(0, std, shape).astype(np.float32)).to(dtype)
    sd = d ** -0.25   # the dense op has no alpha: scores of unit variance
    c = dict(q=mk((b, s, n, d), sd), k=mk((b, s, n, d), sd), v=mk((b, s, n, d)), max_seq_len=s, mask_type=0, silu_scale=1.0 / 8)
    if bias:
        c["attn_bias"] = mk((b, n, s, s), 0.3)
    if mask == "custom":
        c["mask_type"] = 3
        c["mask"] = (torch.from_numpy(rng.random((b, n, s, s))) < 0.6).to(dtype)
    return c, mk((b, s, n, d), 1.0)


@pytest.mark.parametrize("kind", ["mfma_bf16", "mfma_f16_d64", "mfma_bias_bf16", "bias_f32", "custom_mask_bf16"])
def test_dense_backward(kind):
    """hstu_hip_dense_backward ([B, S, N, D] layout, no offsets) against the oracle, for the MFMA and the plain kernels."""
    say("dense backward", kind)
    c, grad = {"mfma_bf16": lambda: _dense_case(21, 3, 200, 2, 128, torch.bfloat16),
               "mfma_f16_d64": lambda: _dense_case(22, 2, 130, 3, 64, torch.float16),
               "mfma_bias_bf16": lambda: _dense_case(25, 2, 168, 2, 128, torch.bfloat16, bias=True),
               "bias_f32": lambda: _dense_case(23, 2, 45, 2, 32, torch.float32, bias=True),
               "custom_mask_bf16": lambda: _dense_case(24, 2, 70, 2, 64, torch.bfloat16, bias=True, mask="custom")}[kind]()
    dtype = c["q"].dtype
    got = T.run_capi_backward(c, grad, op="dense")
    want = O.hstu_dense_backward(grad, c["q"], c["k"], c["v"], max_seq_len=c["max_seq_len"], mask_type=c["mask_type"],
                                 mask=c.get("mask"), attn_bias=c.get("attn_bias"), silu_scale=c["silu_scale"])
    for name, g, w in zip(("dq", "dk", "dv", "dbias"), got, want):
        if w is None:
            assert g is None
            continue
        T.assert_parity(g, w, dtype, what=f"dense backward {kind} {name}")
    if kind.startswith("mfma"):
        gen = T.run_capi_backward(c, grad, op="dense", flags=2)
        assert T.last_backward_kernel.startswith("generic_bwd_")
        for name, g, x in zip(("dq", "dk", "dv", "dbias"), got, gen):
            if x is not None:
                T.assert_parity(g, x.double(), dtype, what=f"dense mfma vs plain kernels {name}")
        # the same rows as a jagged batch of equal lengths give the same bits
        b, s, n, d = c["q"].shape
        j = dict(c, q=c["q"].reshape(b * s, n, d), k=c["k"].reshape(b * s, n, d), v=c["v"].reshape(b * s, n, d),
                 seq_offset=W.offsets([s] * b, torch.int64), seq_offset_k=None, max_seq_len_k=s)
        jag = T.run_capi_backward(j, grad.reshape(b * s, n, d))
        for g, x in zip(got[:3], jag[:3]):
            assert torch.equal(g.reshape(b * s, n, d), x)


def test_hstu_dense_backward_op_and_autograd():
    """torch.ops.mxrec.hstu_dense_backward with the reference's schema, and out.backward() through hstu_dense."""
    say("dense backward torch op + autograd")
    import recsdk_amd  # noqa: F401
    dev = lambda t: None if t is None else t.cuda()
    for bias in (True, False):
        c, grad = _dense_case(25, 2, 96, 2, 64, torch.bfloat16, bias=bias)
        want = T.run_capi_backward(c, grad, op="dense")
        got = torch.ops.mxrec.hstu_dense_backward(dev(grad), dev(c["q"]), dev(c["k"]), dev(c["v"]), None, dev(c.get("attn_bias")), 0,
                                                  c["max_seq_len"], c["silu_scale"])
        for g, w in zip(got[:3], want[:3]):
            assert torch.equal(g.cpu(), w)
        if bias:
            assert torch.equal(got[3].cpu(), want[3])
        else:   # the reference returns zeros with the sequence dimension rounded up to 256 (hstu_dense.cpp:131-136)
            assert tuple(got[3].shape) == (2, 2, 256, 256) and float(got[3].abs().max()) == 0.0
        q, k, v = (dev(c[n]).requires_grad_(True) for n in ("q", "k", "v"))
        b = dev(c.get("attn_bias"))
        if b is not None:
            b.requires_grad_(True)
        out = torch.ops.mxrec.hstu_dense(q, k, v, None, b, 0, c["max_seq_len"], c["silu_scale"])
        out.backward(dev(grad))
        assert torch.equal(q.grad.cpu(), want[0]) and torch.equal(k.grad.cpu(), want[1]) and torch.equal(v.grad.cpu(), want[2])
        if b is not None:
            assert torch.equal(b.grad.cpu(), want[3])


def test_backward_serial_flag_gives_the_same_bits():
    """HSTU_FLAG_SERIAL_BACKWARD keeps a large backward (more than 3000 items per kernel: normally three streams) on the
    caller's stream: same sums in the same order, so the same bits."""
    say("backward serial flag")
    from recsdk_amd import _capi
    cfg, grad = _case(31, [1300] * 36, 8, 8, 128, 128, torch.bfloat16)
    forked = T.run_capi_backward(cfg, grad)
    assert T.last_backward_kernel.startswith("mfma_bwd_")
    serial = T.run_capi_backward(cfg, grad, flags=_capi.FLAG_SERIAL_BACKWARD)
    for a, b in zip(forked[:3], serial[:3]):
        assert torch.equal(a, b)
