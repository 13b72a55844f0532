"""GPU parity of the standalone bias producers against the oracle, on the reference's own test generators
(cust_op/test/relative_attn_bias/torch/utils.py:29-97, test_relative_attn_bias.py) at sizes the oracle finishes in seconds.
Bucket ids and the gathered / selected values are integer and copy work: bit-exact.  The weight gradient is a
floating-point sum: the reference's own tolerances (1e-5 for fp32, 1e-3 for fp16; test_relative_attn_bias.py:101-103)."""
import sys

import pytest
import torch
import torch.nn.functional as F

import recsdk_amd  # noqa: F401
from oracle import bias_oracle as BO

pytestmark = pytest.mark.gpu
NUM_BUCKETS, DIV = 128, 0.301


def say(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def _timestamps(train_len, candidate_len, valid_lens, dtype):
    """utils.py:70-81: 1..valid_len, zero padding, candidates at train_len + 1."""
    ts = torch.zeros(len(valid_lens), train_len + candidate_len // 2)
    for i, v in enumerate(valid_lens):
        if v > 0:
            ts[i, :v] = torch.arange(1, v + 1)
    if candidate_len > 0:
        ts[:, -(candidate_len // 2):] = train_len + 1
    return ts.to(dtype)


@pytest.mark.parametrize("num_layers,train_len,candidate_len,bs,dtype,tsdtype", [
    (1, 500, 600, 2, torch.float16, torch.int32), (8, 300, 0, 3, torch.float32, torch.int32), (3, 257, 90, 2, torch.bfloat16, torch.int64),
    (2, 31, 0, 1, torch.float16, torch.int32),
    # rows of whole 16-byte chunks (s a multiple of 4) take the variant that stores whole cache lines: 8-byte ids, more
    # layers than one table read holds, more than one workgroup per row (s / 4 > 248), fp32 chunks of 32 bytes
    (3, 256, 96, 2, torch.bfloat16, torch.int64), (20, 36, 0, 2, torch.float16, torch.int64), (2, 1000, 200, 1, torch.float16, torch.int32),
    (5, 1020, 0, 1, torch.float32, torch.int64)])
def test_rab_time_with_index(num_layers, train_len, candidate_len, bs, dtype, tsdtype):
    say("rab_time", num_layers, train_len, candidate_len, bs, dtype, tsdtype)
    g = torch.Generator().manual_seed(7)
    lens = torch.randint(0, train_len, (bs,), generator=g).tolist()
    ts = _timestamps(train_len, candidate_len, lens, tsdtype)
    w = torch.arange(NUM_BUCKETS + 1, dtype=torch.float32).repeat(num_layers).reshape(num_layers, -1)      # utils.py:84-89
    w = (w + torch.randn(w.shape, generator=g)).to(dtype)
    want, ids = BO.rab_time(ts, w, DIV)
    out, got_ids = torch.ops.mxrec.relative_attn_bias_time_with_index(ts.cuda(), w.cuda(), DIV)
    assert got_ids.dtype == tsdtype and torch.equal(got_ids.cpu(), ids)
    assert out.dtype == dtype and torch.equal(out.cpu(), want)
    assert torch.equal(torch.ops.mxrec.relative_attn_bias_time(ts.cuda(), w.cuda(), DIV), out)


def test_rab_time_random_timestamps_and_a_narrow_table():
    """Real-looking second-resolution timestamps (differences up to 10^8), and a 17-column table (16 buckets)."""
    say("rab_time random")
    g = torch.Generator().manual_seed(8)
    ts = torch.randint(1_600_000_000, 1_700_000_000, (2, 150), generator=g, dtype=torch.int64).sort(dim=1).values
    for cols in (129, 17):
        w = torch.randn(2, cols, generator=g)
        want, ids = BO.rab_time(ts, w, DIV)
        out, got = torch.ops.mxrec.relative_attn_bias_time_with_index(ts.cuda(), w.cuda(), DIV)
        assert torch.equal(got.cpu(), ids) and torch.equal(out.cpu(), want)


@pytest.mark.parametrize("num_layers,s,bs,dtype", [(1, 550, 2, torch.float32), (8, 200, 3, torch.float16), (2, 37, 2, torch.bfloat16)])
def test_rab_time_backward(num_layers, s, bs, dtype):
    say("rab_time_backward", num_layers, s, bs, dtype)
    g = torch.Generator().manual_seed(9)
    grad = (torch.randn(num_layers, bs, 2 * s, 2 * s, generator=g) * 1e-5).to(dtype)      # utils.py:92-93
    ids = (torch.arange(bs * s) % NUM_BUCKETS).reshape(bs, s, 1).repeat(1, 1, s).to(torch.int32)    # utils.py:96-99
    want = BO.rab_time_backward(grad, ids, NUM_BUCKETS)
    got = torch.ops.mxrec.relative_attn_bias_time_backward(grad.cuda(), ids.cuda(), NUM_BUCKETS)
    assert got.dtype == dtype and got.shape == (num_layers, NUM_BUCKETS)
    tol = 1e-5 if dtype == torch.float32 else 1e-3
    assert torch.allclose(got.cpu().double(), want, rtol=tol, atol=tol)
    # random ids, some outside the table
    ids2 = torch.randint(-2, NUM_BUCKETS + 3, (bs, s, s), generator=g, dtype=torch.int32)
    grad2 = torch.randn(num_layers, bs, 2 * s, 2 * s, generator=g).to(dtype)
    want = BO.rab_time_backward(grad2, ids2, NUM_BUCKETS)
    got = torch.ops.mxrec.relative_attn_bias_time_backward(grad2.cuda(), ids2.cuda(), NUM_BUCKETS).cpu().double()
    scale = float(want.abs().max())
    assert float((got - want).abs().max()) <= (1e-5 if dtype == torch.float32 else 4e-3) * scale


def test_rab_time_is_differentiable_like_the_reference_op():
    say("rab_time autograd")
    g = torch.Generator().manual_seed(10)
    ts = torch.randint(0, 4000, (2, 60), generator=g, dtype=torch.int32)
    w = torch.randn(3, 129, generator=g).cuda().requires_grad_(True)
    out = torch.ops.mxrec.relative_attn_bias_time(ts.cuda(), w, DIV)
    grad = torch.randn(out.shape, generator=g)
    out.backward(grad.cuda())
    ids = BO.rab_time(ts, w.detach().cpu(), DIV)[1]
    want = BO.rab_time_backward(grad, ids, 129)
    assert torch.allclose(w.grad.cpu().double(), want, rtol=1e-5, atol=1e-5 * float(want.abs().max()))


def _rel_pos_tables(train_len, candidate_len, dtype):
    """utils.py:38-66 for one layer: Toeplitz table padded for the candidates, every entry repeated 2x2; identity marks
    the 2x2 blocks on the diagonal."""
    pos_w = torch.arange(0, 2 * train_len + 1, dtype=torch.float32)
    max_len = train_len + candidate_len // 2
    t = F.pad(pos_w[:2 * train_len - 1], [0, train_len]).repeat(train_len)
    t = t[..., :-train_len].reshape(1, train_len, 3 * train_len - 2)
    r = (2 * train_len - 1) // 2
    rel = F.pad(t[:, :, r:-r], (0, candidate_len // 2, 0, candidate_len // 2), "constant", 0.0)
    rel = rel.unsqueeze(-1).repeat(1, 1, 2, 2).reshape(2 * max_len, 2 * max_len)
    idx = torch.arange(max_len).repeat(max_len).view(max_len, max_len).unsqueeze(-1).repeat(1, 2, 2).reshape(2 * max_len, 2 * max_len)
    return rel.to(dtype), (idx.t() == idx).float().to(dtype)


@pytest.mark.parametrize("train_len,candidate_len,bs,dtype", [(300, 60, 3, torch.float16), (129, 0, 70, torch.float32), (50, 10, 2, torch.bfloat16)])
def test_rab_pos(train_len, candidate_len, bs, dtype):
    say("rab_pos", train_len, candidate_len, bs, dtype)
    g = torch.Generator().manual_seed(11)
    rel, ident = _rel_pos_tables(train_len, candidate_len, dtype)
    lens = torch.randint(0, train_len, (bs,), generator=g).tolist()
    want = BO.rab_pos(rel, ident, lens)
    got = torch.ops.mxrec.relative_attn_bias_pos(rel.cuda(), ident.cuda(), lens)
    assert got.dtype == dtype and torch.equal(got.cpu(), want)
    # an identity that is not 0/1 (the reference never builds one): the same expression, a blend, to within the roundings
    # of the dtype
    frac = torch.rand(ident.shape, generator=g).to(dtype)
    relr = (rel.float() * 0.37 + torch.randn(rel.shape, generator=g)).to(dtype)
    want = BO.rab_pos(relr.double(), frac.double(), lens[:2])
    got = torch.ops.mxrec.relative_attn_bias_pos(relr.cuda(), frac.cuda(), lens[:2])
    eps = {torch.float16: 2 ** -10, torch.bfloat16: 2 ** -7, torch.float32: 2 ** -22}[dtype]
    assert torch.allclose(got.cpu().double(), want, rtol=4 * eps, atol=4 * eps * float(relr.abs().max()))


def test_rab_time_feeds_hstu_jagged_as_attn_bias():
    """The dense tensor the producer writes is what the attention takes as attn_bias: same output as the fused-table path
    of the attention on the same timestamps (items and actions interleaved: every timestamp twice)."""
    say("rab_time -> hstu_jagged")
    from tests import hstu_testlib as T
    from recsdk_amd import workloads as W
    g = torch.Generator().manual_seed(12)
    s, heads, d = 48, 2, 64
    ts = torch.randint(0, 100000, (2, s), generator=g, dtype=torch.int64).sort(dim=1).values
    w = (torch.randn(1, 129, generator=g) * 0.2)
    bias = torch.ops.mxrec.relative_attn_bias_time(ts.cuda(), w.cuda(), DIV)[0]           # [b, 2s, 2s]
    L = 2 * s
    mk = lambda: (torch.randn(2 * L, heads, d, generator=g) * 0.5).to(torch.bfloat16)
    q, k, v = mk(), mk(), mk()
    off = W.offsets([L, L])
    dense = bias[:, None].expand(2, heads, L, L).to(torch.bfloat16).contiguous()
    out_dense = torch.ops.mxrec.hstu_jagged(q.cuda(), k.cuda(), v.cuda(), None, dense, 0, L, 0.0, off.cuda(), None, None, 0, 0.125)
    out_fused = torch.ops.mxrec.hstu_jagged_table_bias(q.cuda(), k.cuda(), v.cuda(), None, w[0].cuda(), ts.repeat_interleave(2, dim=1).reshape(-1).cuda(),
                                                       None, 0, L, L, 0.0, off.cuda(), off.cuda(), None, None, 0, 0.125, DIV)
    # the dense path rounds the bias to bf16 first, the fused path adds the fp32 table entry
    T.assert_parity(out_dense.cpu(), out_fused.cpu().double(), torch.bfloat16, what="dense bias from the producer vs fused table")


def test_rab_time_at_the_evaluation_shape():
    """8 layers, 4 users, s = 2300 (train 2000 + 600 candidates), fp16 (test_relative_attn_bias.py:106-113): too large for
    the oracle's Python-side repeat in a test, so checked through what must hold at any size -- the output is the table
    gathered at the returned ids and repeated 2 x 2, the ids are symmetric with a zero diagonal and equal the oracle's on
    a slice; the weight gradient equals an index_add over the same ids (torch on the GPU, fp32)."""
    say("rab_time at the evaluation shape")
    n, bs, train, cand = 8, 4, 2000, 600
    s = train + cand // 2
    g = torch.Generator().manual_seed(0)
    lens = torch.randint(0, train, (bs,), generator=g).tolist()
    ts = _timestamps(train, cand, lens, torch.int32)
    w = (torch.arange(NUM_BUCKETS + 1, dtype=torch.float32).repeat(n).reshape(n, -1) + torch.randn(n, NUM_BUCKETS + 1, generator=g)).half()
    out, ids = torch.ops.mxrec.relative_attn_bias_time_with_index(ts.cuda(), w.cuda(), DIV)
    assert out.shape == (n, bs, 2 * s, 2 * s) and ids.shape == (bs, s, s)
    assert torch.equal(ids, ids.transpose(1, 2)) and not bool(torch.diagonal(ids, dim1=1, dim2=2).any())
    assert int(ids.min()) >= 0 and int(ids.max()) <= NUM_BUCKETS
    _, want_ids = BO.rab_time(ts[:1, :300], w[:1], DIV)
    assert torch.equal(ids[:1, :300, :300].cpu(), want_ids)
    wd = w.cuda()
    for layer in range(n):
        gathered = wd[layer][ids.long()]                                   # [bs, s, s]
        for a in (0, 1):
            for c in (0, 1):
                assert torch.equal(out[layer, :, a::2, c::2], gathered)
    grad = (torch.randn(n, bs, 2 * s, 2 * s, generator=g, dtype=torch.float16) * 1e-2).cuda()
    gw = torch.ops.mxrec.relative_attn_bias_time_backward(grad, ids, NUM_BUCKETS + 1)
    summed = (grad[:, :, 0::2, 0::2].float() + grad[:, :, 0::2, 1::2].float()) + (grad[:, :, 1::2, 0::2].float() + grad[:, :, 1::2, 1::2].float())
    want = torch.zeros(n, NUM_BUCKETS + 1, device="cuda", dtype=torch.float64)
    flat = ids.reshape(-1).long()
    for layer in range(n):
        want[layer].index_add_(0, flat, summed[layer].reshape(-1).double())
    assert float((gw.double() - want).abs().max()) <= 1e-3 * float(want.abs().max())
