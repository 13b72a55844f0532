"""GPU parity tests of float8_e4m3fn q / k / v (fp16 output) through the C ABI and the torch op, against the CPU oracle's
restatement of the reference's fp8 golden (test_hstu_jagged_forward.py:150-189: fp32 scores, P through e4m3, fp32 P V).

Tolerance: 5e-2 of the tensor's scale on every element (the bound stated for fp8 work), and 99.8 % of the elements within
2e-3 of the scale: apart from scores that sit within an fp32 rounding of an e4m3 tie (P then moves by one e4m3 step) the
two sides compute the same numbers."""
import math

import numpy as np
import pytest
import torch

from recsdk_amd import workloads as W
from tests import hstu_testlib as T
from tests.test_parity_gpu import say, FORCE_GENERIC

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


def _jag8(seed, lens_q, nq, nk, dqk, dv, lens_k=None, index_dtype=torch.int64, extra_rows=0, silu_scale=1.0):
    rng = np.random.default_rng(seed)
    lens_k = lens_q if lens_k is None else lens_k
    tq, tk = sum(lens_q) + extra_rows, sum(lens_k)
    mk = lambda shape: torch.from_numpy(rng.uniform(-1, 1, shape).astype(np.float32)).to(FP8)   # the reference's data: uniform(-1, 1)
    c = dict(q=mk((tq, nq, dqk)), k=mk((tk, nk, dqk)), v=mk((tk, nk, dv)), seq_offset=W.offsets(lens_q, index_dtype),
             max_seq_len=max(max(lens_q), 1), alpha=1.0 / math.sqrt(dqk), mask_type=0, lens=lens_q, silu_scale=silu_scale)
    if lens_k is not lens_q:
        c["seq_offset_k"] = W.offsets(lens_k, index_dtype)
        c["max_seq_len_k"] = max(max(lens_k), 1)
    return c, rng


def _close(out, ref, what, tol=5e-2, tight=2e-3, frac=2e-3):
    assert out.dtype == torch.float16 and out.shape == ref.shape, (out.dtype, out.shape, ref.shape)
    assert torch.isfinite(out.float()).all(), f"{what}: non-finite output"
    o, r = out.double(), ref.double()
    scale = max(r.abs().max().item(), 1e-30)
    err = (o - r).abs()
    assert err.max().item() <= tol * scale, f"{what}: max err {err.max().item():.3e} vs scale {scale:.3e}"
    off = (err > tight * scale).double().mean().item()
    assert off <= frac, f"{what}: {off:.2e} of the elements are off by more than {tight} of the scale"


def _check(cfg, what, mfma, op="jagged"):
    ref = T.oracle_jagged(cfg, mode="lowp")
    assert ref.dtype == torch.float16
    out, name = T.run_capi(cfg, op=op)
    assert name.startswith("mfma_fp8_d") if mfma else name == "generic_fp8", name
    _close(out, ref, what + " vs oracle")
    if mfma:
        gen, gname = T.run_capi(cfg, op=op, flags=FORCE_GENERIC)
        assert gname == "generic_fp8", gname
        _close(gen, ref, what + " plain kernel vs oracle")
    return out


@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("lens", [[1], [31, 32, 33], [63, 64, 65, 127, 128, 129], [300, 0, 17, 0], [513, 257]])
def test_fp8_mfma_causal_shapes(lens, d):
    say("fp8_causal", d, lens)
    cfg, _ = _jag8(71, lens, 4, 4, d, d)
    _check(cfg, f"fp8 causal d={d} lens={lens}", True)


@pytest.mark.parametrize("d", [64, 128, 256])
def test_fp8_mfma_gqa_delta_int32_tail(d):
    say("fp8_gqa_delta", d)
    cfg, _ = _jag8(72, [70, 200, 33], 8, 2, d, d, lens_k=[130, 200, 97], index_dtype=torch.int32, extra_rows=7)
    out = _check(cfg, "fp8 gqa+delta", True)
    assert torch.equal(out[-7:], torch.zeros_like(out[-7:]))
    cfg["mask_type"] = 2
    _check(cfg, "fp8 no mask", True)
    cfg2, _ = _jag8(73, [300, 140], 2, 2, d, d)
    cfg2["max_seq_len"] = 100          # attribute smaller than the longest sequence: every row must still be produced
    _check(cfg2, "fp8 short max_seq_len attr", True)


@pytest.mark.parametrize("ctx,tgt,tgs", [(3, 0, 0), (0, 6, 1), (40, 70, 3), (2, 7, 0), (0, 64, 1), (33, 33, 33), (6, 30, 3)])
def test_fp8_mfma_builtin_masks(ctx, tgt, tgs):
    say("fp8_masks", ctx, tgt, tgs)
    cfg, _ = _jag8(74, [140, 271, 129], 2, 2, 64, 64)
    cfg["num_context"] = torch.tensor([ctx, ctx, ctx])
    cfg["num_target"] = torch.tensor([tgt, tgt + 1 if tgt else 0, tgt])
    cfg["target_group_size"] = tgs
    _check(cfg, "fp8 builtin masks", True)
    cfg2, _ = _jag8(75, [90, 150], 2, 1, 128, 128, lens_k=[190, 150])
    cfg2["num_target"] = torch.tensor([tgt, tgt]); cfg2["num_context"] = torch.tensor([ctx, ctx])
    cfg2["target_group_size"] = tgs
    _check(cfg2, "fp8 builtin masks + delta", True)


@pytest.mark.parametrize("case", [
    dict(lens=[15, 9, 1], nq=8, nk=8, dqk=64, dv=16),                 # the reference's fp8 sweep: Dqk in {64, 96, 128}, Dv in {16..80}
    dict(lens=[256, 100, 31], nq=8, nk=2, dqk=96, dv=80),
    dict(lens=[200, 77], nq=8, nk=1, dqk=128, dv=48, mask_type=2),
    dict(lens=[40, 90], lens_k=[75, 90], nq=6, nk=3, dqk=72, dv=32),   # its delta-q sweep (test_hstu_deltaqk_forward.py:420-440)
])
@pytest.mark.parametrize("bias", [False, True])
def test_fp8_plain_kernel_reference_sweep(case, bias):
    """Shapes of the reference's (switched-off) fp8 tests: Dqk != Dv (the padded matrix-core variant where both are
    multiples of 16 and there is no bias), attn_bias and custom mask in float8_e4m3fn (its op definition makes both follow
    the dtype of q: hstu_jagged_forward.cpp:79-86; the plain kernel)."""
    c = dict(case)
    say("fp8_plain", c, bias)
    lens = c.pop("lens")
    mask_type = c.pop("mask_type", 0)
    cfg, rng = _jag8(76, lens, c["nq"], c["nk"], c["dqk"], c["dv"], lens_k=c.get("lens_k"), silu_scale=1 / 16)
    cfg["mask_type"] = mask_type
    b, n, mq, mk = len(lens), c["nq"], cfg["max_seq_len"], cfg.get("max_seq_len_k") or cfg["max_seq_len"]
    if bias:
        cfg["attn_bias"] = torch.from_numpy(rng.random((b, n, mq, mk)).astype(np.float32)).to(FP8)
    # without a bias, head dims that are multiples of 16 run on the matrix cores (the padded variant); 72 does not
    padded = not bias and c["dqk"] % 16 == 0
    out = _check(cfg, "fp8 sweep shape", padded)
    if padded:
        assert T.run_capi(cfg)[1].endswith("_padded") and out.shape[2] == c["dv"]
    cfg["mask"] = torch.from_numpy(rng.integers(0, 2, (b, n, mq, mk)).astype(np.float32)).to(FP8)
    cfg["mask_type"] = 3
    _check(cfg, "fp8 plain kernel, custom mask", False)


def test_fp8_bias_takes_the_plain_kernel_and_default_scale():
    """attn_bias is not specialised for fp8: same shape with and without it; and the default silu_scale = 1 / max_seq_len,
    which puts P among the subnormals of e4m3 (steps of 2^-9), as in the reference's own sweep."""
    say("fp8_bias_default_scale")
    cfg, rng = _jag8(77, [137, 64, 290], 2, 2, 128, 128, silu_scale=0.0)
    out = _check(cfg, "fp8 default scale", True)
    assert float(out.float().abs().max()) > 0
    cfg["attn_bias"] = torch.from_numpy(rng.random((3, 2, 290, 290)).astype(np.float32)).to(FP8)
    _check(cfg, "fp8 dense bias", False)


def test_fp8_dense_layout_and_torch_op():
    say("fp8_dense_and_op")
    rng = np.random.default_rng(78)
    b, s, n, d = 3, 200, 4, 64
    mk = lambda: torch.from_numpy(rng.uniform(-1, 1, (b, s, n, d)).astype(np.float32)).to(FP8)
    q, k, v = mk(), mk(), mk()
    cfg = dict(q=q, k=k, v=v, max_seq_len=s, mask_type=0, silu_scale=1.0, alpha=1.0)
    jag = dict(q=q.reshape(b * s, n, d), k=k.reshape(b * s, n, d), v=v.reshape(b * s, n, d), seq_offset=W.offsets([s] * b),
               max_seq_len=s, mask_type=0, silu_scale=1.0, alpha=1.0)
    ref = T.oracle_jagged(jag, mode="lowp").reshape(b, s, n, d)
    out, name = T.run_capi(cfg, op="dense")
    assert name == "mfma_fp8_d64", name
    _close(out, ref, "fp8 dense layout")
    op_out = T.run_op(cfg, op="dense")
    assert op_out.dtype == torch.float16 and torch.equal(op_out, out)
    jout, _ = T.run_capi(jag)
    assert torch.equal(jout.reshape(b, s, n, d), out), "dense and jagged layouts of one problem disagree"
    op_j = T.run_op(jag)
    assert op_j.dtype == torch.float16 and torch.equal(op_j, jout), "torch op and direct C-ABI call disagree"


def test_fp8_rejected_where_the_reference_has_no_fp8_path():
    from recsdk_amd import _capi
    cfg, _ = _jag8(79, [40, 20], 2, 2, 64, 64)
    q, k, v = (cfg[x].cuda() for x in "qkv")
    with pytest.raises(RuntimeError, match="float32, float16 or bfloat16"):
        torch.ops.mxrec.hstu_jagged_backward(torch.zeros(60, 2, 64, dtype=FP8, device="cuda"), q, k, v, None, None, 0, 40, 0.0,
                                             cfg["seq_offset"].cuda(), None, None, 0, 1.0)
    out = torch.empty(60, 2, 64, dtype=torch.float16, device="cuda")
    p, keep = _capi.make_params(q, k, v, out, seq_offset_q=cfg["seq_offset"].cuda(), max_seq_len_q=40)
    bp = _capi.make_backward_params(p, out, out, out, out)
    with pytest.raises(_capi.HstuError, match="forward only"):
        _capi.run_backward(bp)


def test_fp8_full_size_training_batch():
    """The headline batch (B=64, h=4, d=128, L in [256, 1024]) in fp8: matrix-core kernel against the plain kernel on every row,
    determinism, and isolation of the sequences (changing one sequence's K changes only its rows)."""
    say("fp8_config2")
    cfg = W.config2()
    g = torch.Generator().manual_seed(5)
    for x in "qkv":
        cfg[x] = (torch.rand(cfg[x].shape, generator=g) * 2 - 1).to(FP8)
    cfg["silu_scale"] = 1.0 / 64
    out, name = T.run_capi(cfg)
    assert name == "mfma_fp8_d128_selfsched", name
    again, _ = T.run_capi(cfg, reuse_from=cfg)      # the same launch over the list that the first call left in the workspace
    assert torch.equal(out, again)
    gen, gname = T.run_capi(cfg, flags=FORCE_GENERIC)
    assert gname == "generic_fp8"
    _close(out, gen, "fp8 config 2, matrix-core vs plain kernel")
    out2, _ = T.run_capi(cfg)
    assert torch.equal(out, out2), "two runs differ"
    off = cfg["seq_offset"].tolist()
    b = 17
    k2 = cfg["k"].clone()
    k2[off[b]:off[b + 1]] = (torch.rand(k2[off[b]:off[b + 1]].shape, generator=g) * 2 - 1).to(FP8)
    out3, _ = T.run_capi(cfg, k=k2)
    same = torch.ones(out.shape[0], dtype=torch.bool)
    same[off[b]:off[b + 1]] = False
    assert torch.equal(out3[same], out[same]) and not torch.equal(out3[~same], out[~same])


def test_fp8_self_derived_launches_match_the_list_driven_launch_on_random_batches():
    """Random batches of up to 128 sequences at head dims 64 / 128 / 256 (uniform, heavy-tailed, half-empty, equal and
    tile-aligned lengths, attributes below / at / above the longest sequence, both offset dtypes, target rows): the launch
    that derives its items gives the same bits as the same call made ineligible by a num_context of zeros (which runs over
    the schedule kernel's list), and as a second call over the list it left."""
    rng = np.random.default_rng(6)
    taken = 0
    for it in range(50):
        B = int(rng.choice([1, 2, 3, 7, 16, 33, 63, 64, 65, 100, 127, 128])) if rng.random() < 0.5 else int(rng.integers(1, 129))
        H = int(rng.choice([1, 2, 3, 4, 5, 8, 16]))
        d = int(rng.choice([64, 128, 256]))
        kind = int(rng.integers(0, 5))
        cap = max(1, min(8064, 40000 // B))
        if kind == 0: lens = rng.integers(0, cap + 1, B)
        elif kind == 1: lens = np.minimum((rng.pareto(1.1, B) * 64).astype(np.int64), cap)
        elif kind == 2: lens = np.where(rng.random(B) < 0.5, 0, rng.integers(0, cap + 1, B))
        elif kind == 3: lens = np.full(B, int(rng.integers(1, cap + 1)))
        else: lens = (rng.integers(0, max(2, cap // 128 + 1), B) * 128 + rng.choice([-1, 0, 1], B)).clip(0, cap)
        lens = [int(x) for x in lens]
        if sum(lens) == 0: lens[0] = 5
        idt = torch.int64 if rng.random() < 0.5 else torch.int32
        cfg, _ = _jag8(6000 + it, lens, H, H, d, d, index_dtype=idt, silu_scale=1.0 / 64)
        mx, r = max(lens), rng.random()
        cfg["max_seq_len"] = mx if r < 0.6 else (max(1, mx // 2) if r < 0.8 else min(8064, mx + int(rng.integers(0, 700))))
        if rng.random() < 0.4:
            cfg["num_target"] = torch.tensor([min(l, int(t)) for l, t in zip(lens, rng.integers(0, 50, B))], dtype=idt)
            cfg["target_group_size"] = int(rng.integers(1, 4))
        if rng.random() < 0.3:
            cfg["mask_type"] = 2
        say("fp8_self_derived_random", it, B, H, d, kind, sum(lens), mx, cfg["max_seq_len"], cfg["mask_type"])
        out, name = T.run_capi(cfg)
        if not name.endswith("_selfsched"):
            continue
        taken += 1
        again, _ = T.run_capi(cfg, reuse_from=cfg)
        assert torch.equal(out, again), "the list left behind gives other bits"
        listed, name2 = T.run_capi(dict(cfg, num_context=torch.zeros(B, dtype=idt)))
        assert name2.startswith("mfma_fp8_d") and not name2.endswith("_selfsched"), name2
        assert torch.equal(torch.isnan(out), torch.isnan(listed)), "other rows produced"
        assert torch.equal(torch.nan_to_num(out.float()), torch.nan_to_num(listed.float())), "other bits than over the schedule kernel's list"
    assert taken >= 40, taken


@pytest.mark.parametrize("d", [64, 128, 256])
def test_fp8_self_derived_launch_with_k_offsets_in_a_tensor_of_their_own(d):
    """seq_offset_k given next to seq_offset_q with as many K rows in total: still no schedule kernel; same bits as with one
    tensor for both, and with other lengths per sequence the plain kernel's rows."""
    say("fp8_self_derived_own_k_offsets", d)
    cfg, _ = _jag8(7, [700, 0, 129, 513, 64, 300], 4, 4, d, d, silu_scale=1.0 / 64)
    out0, name0 = T.run_capi(cfg)
    out1, name1 = T.run_capi(dict(cfg, seq_offset_k=cfg["seq_offset"].clone(), max_seq_len_k=cfg["max_seq_len"]))
    assert name0.endswith("_selfsched") and name1.endswith("_selfsched"), (name0, name1)
    assert torch.equal(out0, out1)
    c3, _ = _jag8(8, [300, 100, 513, 8], 4, 4, d, d, lens_k=[100, 513, 300, 8], silu_scale=1.0 / 64)
    out3, name3 = T.run_capi(c3)
    assert name3.endswith("_selfsched"), name3
    gen, gname = T.run_capi(c3, flags=FORCE_GENERIC)
    assert gname == "generic_fp8"
    _close(out3, gen, "fp8, own K offsets, other lengths: matrix-core vs plain kernel")
