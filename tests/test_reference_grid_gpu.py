"""The grids of the reference's own operator tests for the attention, judged by the reference's own rule.

cust_op/test/hstu_v2/test_forward_op_precision.py (forward: batch sizes, head dims, head counts, dense bias, sequence
lengths, the two lists of user shapes), test_backward_op_precision.py (the same grids for the gradients) and
test_backward_op_precision_mask.py:331-351 (backward under the causal mask with context rows and target groups) draw their inputs with utils/data.py:85-143 -- q / k / v / bias / grad uniform in (-1, 1),
alpha 0.5, silu_scale 1/1024, lengths either random in [1 + context + targets, S] with lq <= lk or all int(0.9 S) -- and
accept a kernel when its largest error against the golden evaluated in fp32 is at most five times the largest error of
the same golden evaluated in the I/O dtype (backend/pytorch_native_backend.py:138-220).  The same grids (the larger ones
thinned: one seed, goldens over the first sequences of the big batches) run here through the C ABI; the goldens are
plain torch on the CPU in one dtype throughout, as the reference's are.  Their window_size (-1, -1) is no mask at all
(mask_type NONE here); (-1, 0), which only the masked backward tests use, is the built-in causal mask.
"""
import numpy as np
import pytest
import torch

from oracle import hstu_oracle as O
from recsdk_amd import workloads as W
from tests import hstu_testlib as T
from tests.test_parity_gpu import say

pytestmark = pytest.mark.gpu
F16, BF16 = torch.float16, torch.bfloat16


def _draw(seed, batch, heads, dqk, dv, sq, sk, rab, dtype, all_equal, ctx=0, tgt=0, tgs=0, causal=False):
    rng = np.random.default_rng(seed)
    if all_equal:
        lq, lk = [int(0.9 * sq)] * batch, [int(0.9 * sk)] * batch
    else:
        lo = 1 + ctx + tgt
        a, b = rng.integers(lo, sq + 1, batch), rng.integers(lo, sk + 1, batch)
        lq, lk = [int(x) for x in np.minimum(a, b)], [int(x) for x in b]
    uni = lambda shape: torch.from_numpy(rng.random(shape, dtype=np.float32) * 2 - 1).to(dtype)
    c = dict(q=uni((sum(lq), heads, dqk)), k=uni((sum(lk), heads, dqk)), v=uni((sum(lk), heads, dv)),
             seq_offset=W.offsets(lq, torch.int32), seq_offset_k=W.offsets(lk, torch.int32), max_seq_len=sq, max_seq_len_k=sk,
             alpha=0.5, silu_scale=1.0 / 1024, mask_type=0 if causal else 2, lens=lq, lens_k=lk)
    if rab:
        c["attn_bias"] = uni((batch, heads, sq, sk))
    if ctx:
        c["num_context"] = torch.full((batch,), ctx, dtype=torch.int32)
    if tgt:
        c["num_target"] = torch.full((batch,), tgt, dtype=torch.int32)
        c["target_group_size"] = tgs
    c["_mask"] = (ctx, tgt, tgs) if causal else None
    return c, uni((sum(lq), heads, dv))


def _golden(c, dt, nseq, grad=None):
    """Output (and, with `grad`, the gradients) of the first `nseq` sequences in dtype `dt` throughout."""
    oq, ok = c["seq_offset"].tolist(), c["seq_offset_k"].tolist()
    outs, dqs, dks, dvs, dbs = [], [], [], [], []
    for b in range(nseq):
        q, k, v = (c[x][(oq if x == "q" else ok)[b]:(oq if x == "q" else ok)[b + 1]].to(dt).transpose(0, 1).contiguous().requires_grad_(grad is not None)
                   for x in "qkv")
        lq, lk = q.shape[1], k.shape[1]
        s = q @ k.transpose(1, 2)
        rab = None
        if "attn_bias" in c:
            rab = c["attn_bias"][b, :, :lq, :lk].to(dt).requires_grad_(grad is not None)
            s = s + rab
        p = torch.nn.functional.silu(s * c["alpha"]) * c["silu_scale"]
        if c["_mask"] is not None:
            p = p * O.builtin_mask(lq, lk, *c["_mask"]).to(dt)
        o = p @ v
        outs.append(o.detach().transpose(0, 1))
        if grad is not None:
            g = torch.autograd.grad(o, (q, k, v) + ((rab,) if rab is not None else ()), grad[oq[b]:oq[b + 1]].to(dt).transpose(0, 1))
            dqs.append(g[0].transpose(0, 1)); dks.append(g[1].transpose(0, 1)); dvs.append(g[2].transpose(0, 1))
            if rab is not None:
                dbs.append(g[3])
    if grad is None:
        return torch.cat(outs)
    return torch.cat(outs), torch.cat(dqs), torch.cat(dks), torch.cat(dvs), dbs


def _forward_case(what, *a, nseq=None, **kw):
    say("reference_grid_forward", what, a, kw)
    c, _ = _draw(*a, **kw)
    n = min(nseq or len(c["lens"]), len(c["lens"]))
    out, name = T.run_capi(c)
    assert torch.isfinite(out.float()).all(), name
    rows = int(c["seq_offset"][n])
    g32, glow = _golden(c, torch.float32, n), _golden(c, c["q"].dtype, n)
    assert O.double_benchmark_close(out[:rows], glow, g32, multiplier=5), (what, name, (out[:rows].float() - g32).abs().max().item(), (glow.float() - g32).abs().max().item())


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("rab", [True, False])
@pytest.mark.parametrize("batch", [1, 4, 16, 32])
def test_generic_batch_size(batch, rab, dtype):          # test_forward_op_precision.py:224-236
    _forward_case("batch_size", 123, batch, 1, 32, 32, 256, 256, rab, dtype, False)


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("d", [32, 64, 128, 256])
def test_generic_head_dim(d, dtype):                     # :277-289
    _forward_case("head_dim", 123, 1, 1, d, d, 256, 256, False, dtype, False)


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("heads", [1, 4, 8, 16])
def test_generic_head_num(heads, dtype):                 # :330-342
    _forward_case("head_num", 123, 1, heads, 32, 32, 256, 256, False, dtype, False)


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("rab", [True, False])
@pytest.mark.parametrize("batch,heads", [(1, 1), (1, 4), (4, 1), (4, 4)])
def test_generic_rab(batch, heads, rab, dtype):          # :383-395
    _forward_case("rab", 123, batch, heads, 32, 32, 256, 256, rab, dtype, False)


@pytest.mark.parametrize("rab", [True, False])
@pytest.mark.parametrize("d", [32, 128])
@pytest.mark.parametrize("s", [512, 1024, 2048])
@pytest.mark.parametrize("heads", [1, 4])
def test_generic_sequence(heads, s, d, rab):             # :436-447 (ten seeds there; one here, the dtypes in turn)
    _forward_case("sequence", s + d, 8, heads, d, d, s, s, rab, F16 if (s // 512 + d // 32 + heads) % 2 else BF16, False)


@pytest.mark.parametrize("batch,heads,dims,lens,dtype,nseq", [
    (2048, 4, (64, 64), (52, 1000), F16, 24), (16, 4, (64, 64), (501, 1000), F16, 16), (2048, 2, (256, 256), (32, 32), F16, 64),
    (96, 2, (256, 256), (512, 3072), F16, 4), (16, 4, (64, 32), (32, 499), F16, 16), (4, 4, (128, 48), (1001, 901), F16, 4),
    (96, 3, (256, 256), (674, 674), BF16, 6)])
def test_user_case_1(batch, heads, dims, lens, dtype, nseq):    # :488-499: every sequence 0.9 of the attribute
    _forward_case("user_case_1", 123, batch, heads, dims[0], dims[1], lens[0], lens[1], False, dtype, True, nseq=nseq)


@pytest.mark.parametrize("s,dtype,d,rab", [(512, dt, d, rab) for dt in (F16, BF16) for d in (32, 64, 128, 256) for rab in (True, False)] +
                         [(2048, BF16, d, False) for d in (32, 64, 128, 256)] + [(2048, BF16, 128, True)])
def test_user_case_2(s, dtype, d, rab):                  # :542-553 (B = 32, h = 8; S = 1024 left out, S = 2048 thinned)
    _forward_case("user_case_2", 123, 32, 8, d, d, s, s, rab, dtype, True, nseq=2)


MASKS = [(128, None, None, None), (128, 64, None, None), (512, None, None, None), (512, 128, None, None), (512, None, 66, 1),
         (512, 128, 66, 1), (512, 66, 128, 1), (1234, None, None, None), (1234, 501, 257, 3)]


@pytest.mark.parametrize("rab", [True, False])
@pytest.mark.parametrize("d", [32, 128, 256])
@pytest.mark.parametrize("s,ctx,tgt,tgs", MASKS)
@pytest.mark.parametrize("batch,heads", [(4, 4)])
def test_backward_has_mask(batch, heads, s, ctx, tgt, tgs, d, rab):   # test_backward_op_precision_mask.py:331-351
    _backward_case(batch, heads, s, ctx, tgt, tgs, d, rab, BF16 if rab else F16)


@pytest.mark.parametrize("batch,heads,mask,d,dtype", [(1, 8, MASKS[6], 128, BF16), (16, 8, MASKS[5], 128, F16), (16, 1, MASKS[8], 32, BF16),
                                                      (128, 1, MASKS[3], 32, F16), (128, 4, MASKS[4], 128, BF16)])
def test_backward_has_mask_other_batches(batch, heads, mask, d, dtype):
    _backward_case(batch, heads, *mask, d, False, dtype, nseq=8)


# test_backward_op_precision.py:228-240, 281-293, 334-346, 387-399, 440-451, 492-503, 552-563: the forward's grids again,
# gradients under no mask (window_size (-1, -1))
@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("rab", [True, False])
@pytest.mark.parametrize("batch", [1, 4, 16, 32])
def test_backward_generic_batch_size(batch, rab, dtype):
    _backward_case(batch, 1, 256, None, None, None, 32, rab, dtype, causal=False)


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("d", [32, 64, 128, 256])
def test_backward_generic_head_dim(d, dtype):
    _backward_case(1, 1, 256, None, None, None, d, False, dtype, causal=False)


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("heads", [1, 4, 8, 16])
def test_backward_generic_head_num(heads, dtype):
    _backward_case(1, heads, 256, None, None, None, 32, False, dtype, causal=False)


@pytest.mark.parametrize("rab", [True, False])
@pytest.mark.parametrize("d", [32, 128])
@pytest.mark.parametrize("s", [512, 1024, 2048])
@pytest.mark.parametrize("heads", [1, 4])
def test_backward_generic_sequence(heads, s, d, rab):    # one seed of the ten, the dtypes in turn
    _backward_case(8, heads, s, None, None, None, d, rab, BF16 if (s // 512 + d // 32 + heads) % 2 else F16, causal=False, seed=s + d, nseq=4)


@pytest.mark.parametrize("batch,heads,dims,lens,dtype,nseq", [
    (2048, 4, (64, 64), (52, 1000), F16, 16), (16, 4, (64, 64), (501, 1000), F16, 8), (2048, 2, (256, 256), (32, 32), F16, 64),
    (96, 2, (256, 256), (512, 3072), F16, 2), (16, 4, (64, 32), (32, 499), F16, 16), (4, 4, (128, 48), (1001, 901), F16, 4),
    (96, 3, (256, 256), (674, 674), BF16, 4)])
def test_backward_user_case_1(batch, heads, dims, lens, dtype, nseq):
    _backward_case(batch, heads, lens[0], None, None, None, dims[0], False, dtype, causal=False, nseq=nseq, dv=dims[1], sk=lens[1], all_equal=True)


@pytest.mark.parametrize("s,dtype,d", [(512, F16, 32), (512, BF16, 64), (512, F16, 128), (512, BF16, 256), (2048, BF16, 128)])
def test_backward_user_case_2(s, dtype, d):              # B = 32, h = 8, every sequence 0.9 S; thinned
    _backward_case(32, 8, s, None, None, None, d, False, dtype, causal=False, nseq=2, all_equal=True)


def _backward_case(batch, heads, s, ctx, tgt, tgs, d, rab, dtype, nseq=None, causal=True, seed=123, dv=None, sk=None, all_equal=False):
    say("reference_grid_backward", batch, heads, s, ctx, tgt, tgs, d, rab, dtype, causal, dv, sk)
    c, grad = _draw(seed, batch, heads, d, dv or d, s, sk or s, rab, dtype, all_equal, ctx=ctx or 0, tgt=tgt or 0, tgs=tgs or 0, causal=causal)
    n = min(nseq or batch, batch)
    rows_q, rows_k = int(c["seq_offset"][n]), int(c["seq_offset_k"][n])
    out, name = T.run_capi(c)
    dq, dk, dv, db = T.run_capi_backward(c, grad)
    g32, glow = _golden(c, torch.float32, n, grad), _golden(c, dtype, n, grad)
    got = [out[:rows_q], dq[:rows_q], dk[:rows_k], dv[:rows_k]]
    for i, what in enumerate(["out", "dq", "dk", "dv"]):
        assert O.double_benchmark_close(got[i], glow[i], g32[i], multiplier=5), \
            (what, name, T.last_backward_kernel, (got[i].float() - g32[i]).abs().max().item(), (glow[i].float() - g32[i]).abs().max().item())
    if rab:
        oq, ok = c["seq_offset"].tolist(), c["seq_offset_k"].tolist()
        mine = max((db[b, :, :oq[b + 1] - oq[b], :ok[b + 1] - ok[b]].float() - g32[4][b]).abs().max().item() for b in range(n))
        theirs = max((glow[4][b].float() - g32[4][b]).abs().max().item() for b in range(n))
        assert mine <= 5 * theirs, ("dbias", mine, theirs)
