"""CPU oracle for the HSTU fused attention forward.  TEST INFRASTRUCTURE ONLY.

This module restates, from scratch, the algorithm of the reference's own
PyTorch/NumPy goldens for ``mxrec::hstu_jagged`` / ``hstu_paged`` /
``hstu_dense``.  It is the checker used by ``tests/``, by
``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``.
Nothing in the shipped package imports it and the HIP path never routes
through it.

Definition followed (reference file:line):

* element-wise order ``x = alpha*(S + bias); p = x*sigmoid(x); p *= silu_scale*mask``
  -- cust_op/ascendc_op/ai_core_op/hstu_dense_forward/v220/op_kernel/vector_score_inter.h:299-323,186-212
  and cust_op/test/hstu_v2/backend/pytorch_native_backend.py:62-76
* pad jagged -> dense, matmul, fp32 score math, cast, matmul, un-pad
  -- cust_op/test/hstu_dense/torch/test_hstu_jagged_forward.py:126-192
* rounding points of the low-precision golden (S rounded to the I/O dtype
  before the fp32 math, P rounded to the I/O dtype before PV)
  -- test_hstu_jagged_forward.py:163,182
* built-in mask (causal with delta = Lk-Lq, context rows, target groups)
  -- cust_op/test/hstu_dense/torch/test_target_mask.py:260-288 and
  .../op_kernel/hstu_dense_causal_mask.h:63-117,204-237
* fp8 inputs (float8_e4m3fn q/k/v, the reference's Ascend-950 path): operands up-cast to fp32, score math in
  fp32, P (after silu_scale and mask) rounded to e4m3 and back, PV in fp32, fp16 out
  -- test_hstu_jagged_forward.py:150-189 (``use_float8``), plugin hstu_jagged.cpp:53-54
* GQA = repeat_interleave of K/V heads -- test_hstu_jagged_forward.py:155-159
* defaults ``silu_scale==0 -> 1/max_seq_len_q``, ``alpha -> 1.0``
  -- cust_op/framework/torch_plugin/torch_library/hstu/hstu_jagged.cpp:43-61
* paged K/V assembly (de-paged history followed by the candidate rows of the
  input k/v) -- cust_op/test/hstu_dense/torch/test_hstu_paged_forward.py:216-292
  and test_common_utils.py:217-262
* bias formulas: time buckets -- cust_op/test/relative_attn_bias/torch/utils.py:26-27,99-129;
  Toeplitz relative position -- utils.py:38-51

* backward: explicit gradient formulas of the reference golden -- build/presmoke/hstu/hstu_common.py:387-476

Pinning status (what fixes each function independently of this file's own
formulas; the checks live in tests/test_oracle_*.py):

* ``builtin_mask``: the reference's checked-in 65x65 fixture
  (tests/golden/target_mask_65x65.txt) + the independent point predicate
  ``mask_point`` + tril special cases.                                  PINNED
* ``hstu_jagged_forward`` / ``hstu_dense_forward``: brute-force fp64 triple
  loop on tiny inputs, reduction to torch.matmul/F.silu, invariants
  (linearity in V and silu_scale, alpha=0, batch permutation, causality,
  B=1 dense==jagged, explicit tril mask == mask_type 0, GQA ==
  repeat_interleave).                                                     PINNED
* fp8 branch of ``hstu_jagged_forward`` (mode "lowp" on float8_e4m3fn inputs): brute-force loop whose e4m3
  rounding is an independent numpy implementation (round to nearest even on the 3-bit mantissa grid,
  subnormals below 2^-6), tests/test_oracle_forward.py.                    PINNED
* ``hstu_paged_forward``: equivalence with the delta-q jagged op on the
  de-paged K/V.                                                           PINNED
* ``hstu_jagged_backward``: torch.autograd of ``hstu_jagged_forward`` in
  float64 (an independent derivation: no gradient formula is shared), central
  finite differences on tiny inputs, and the GQA sum against explicitly
  repeated K/V heads (tests/test_oracle_backward.py).                     PINNED
* ``time_bucket_ids`` / ``rel_pos_bias``: closed forms with the reference's
  constants; integer ids compared exactly against a float64 evaluation away
  from bucket edges and at the documented edge cases.                    PINNED
* fp8-e4m3 KV cache with per-(page, k|v, head) scales and the fused table
  bias: no counterpart in the reference -- PARITY UNPINNED (build-defined;
  pinned by construction only: fused == dense-bias op, fp8 == bf16 op on the
  dequantised cache).
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import torch
import torch.nn.functional as F

MASK_TRIL = 0
MASK_TRIU = 1
MASK_NONE = 2
MASK_CUSTOM = 3

NUM_BUCKETS = 128          # utils.py:26
BUCKET_DIVISOR = 0.301     # utils.py:27
FP8_E4M3_MAX = 448.0


# --------------------------------------------------------------------------
# masks
# --------------------------------------------------------------------------
def builtin_mask(lq: int, lk: Optional[int] = None, num_context: int = 0, num_target: int = 0,
                 target_group_size: int = 0) -> torch.Tensor:
    """Closed-form built-in mask, ``[lq, lk]`` float32 of 0/1.

    Q row i sits at position i + (lk - lq) of the K timeline.  Follows
    test_target_mask.py:272-288; for lq != lk the target square is anchored
    at the bottom-right corner exactly as hstu_dense_causal_mask.h:204-237
    does (rows >= lq - num_target, columns >= lk - num_target).
    """
    if lk is None:
        lk = lq
    m = torch.tril(torch.ones(lq, lk), diagonal=lk - lq)
    if num_context > 0:
        m[:num_context, : max(lk - num_target, 0)] = 1
    if target_group_size > 0 and num_target > 0:
        idx = torch.arange(num_target)
        grp = idx // target_group_size
        sq = ((grp[:, None] == grp[None, :]) & (idx[None, :] <= idx[:, None])).float()
        r0, c0 = max(lq - num_target, 0), max(lk - num_target, 0)
        m[r0:, c0:] = sq[r0 - (lq - num_target):, c0 - (lk - num_target):]
    return m


def mask_point(i: int, j: int, lq: int, lk: int, num_context: int = 0, num_target: int = 0,
               target_group_size: int = 0) -> int:
    """Independent per-point formulation (the ``GPUSmit`` predicates of
    test_target_mask.py:51-73,166-192, extended with delta = lk - lq)."""
    delta = lk - lq
    hist_k = lk - num_target
    hist_q = lq - num_target
    if num_context > 0 and i < num_context and j < hist_k:
        return 1
    if j > i + delta:
        return 0
    if num_target > 0 and target_group_size > 0 and i >= hist_q and j >= hist_k:
        left = hist_k + ((i - hist_q) // target_group_size) * target_group_size
        if j < left:
            return 0
    return 1


# --------------------------------------------------------------------------
# jagged helpers (harness side of the reference tests)
# --------------------------------------------------------------------------
def lengths_from_offsets(offsets: torch.Tensor) -> list:
    o = offsets.tolist()
    return [int(o[i + 1] - o[i]) for i in range(len(o) - 1)]


def valid_batch(offsets: torch.Tensor) -> int:
    """Trailing sequences whose end offset equals the final offset are dropped
    (hstu_common_const.h:125-148); interior empty sequences stay."""
    o = offsets.tolist()
    b = len(o) - 1
    while b > 1 and o[b - 1] == o[b]:
        b -= 1
    return b


# --------------------------------------------------------------------------
# bias producers
# --------------------------------------------------------------------------
def rel_pos_bias(pos_table: torch.Tensor, lq: int, lk: int, max_seq_len_k: int) -> torch.Tensor:
    """``bias[i, j] = pos_table[(max_seq_len_k - 1) + j - (i + lk - lq)]`` (utils.py:38-51:
    Toeplitz matrix of a ``2n-1`` table with n = max_seq_len_k)."""
    assert pos_table.numel() == 2 * max_seq_len_k - 1
    i = torch.arange(lq)[:, None] + (lk - lq)
    j = torch.arange(lk)[None, :]
    return pos_table.float()[(max_seq_len_k - 1) + j - i]


def time_bucket_ids(ts_q: torch.Tensor, ts_k: torch.Tensor, num_buckets: int = NUM_BUCKETS,
                    bucket_divisor: float = BUCKET_DIVISOR) -> torch.Tensor:
    """``trunc(log(clamp(|t_i - t_j|, 1, e^(num_buckets*divisor))) / divisor)`` in fp32
    (utils.py:115-123).  The difference is taken in the integer domain first when
    the timestamps are integers, then converted to fp32."""
    d = (ts_q[:, None] - ts_k[None, :]).abs()
    d = d.to(torch.float32)
    clamp_max = torch.exp(torch.tensor(num_buckets * bucket_divisor))
    x = torch.log(d.clamp(1, clamp_max.item())) / bucket_divisor
    return x.long()


def time_bias(ts_table: torch.Tensor, ts_q: torch.Tensor, ts_k: torch.Tensor, **kw) -> torch.Tensor:
    ids = time_bucket_ids(ts_q, ts_k, **kw)
    return ts_table.float()[ids]


def dense_bias_from_tables(seq_offset_q, seq_offset_k, heads_q: int, max_q: int, max_k: int,
                           pos_table: Optional[torch.Tensor] = None, ts_table: Optional[torch.Tensor] = None,
                           timestamps: Optional[torch.Tensor] = None, dtype=torch.float32, **bucket_kw) -> torch.Tensor:
    """The dense ``[B, Nq, max_q, max_k]`` tensor the reference op would be fed:
    position bias + time bias, zero outside ``[:Lq, :Lk]``.  ``timestamps`` is
    indexed on the K timeline (one value per K row); ``num_buckets`` / ``bucket_divisor``
    go to :func:`time_bucket_ids`."""
    lq = lengths_from_offsets(seq_offset_q)
    lk = lengths_from_offsets(seq_offset_k)
    ok = seq_offset_k.tolist()
    out = torch.zeros(len(lq), heads_q, max_q, max_k, dtype=torch.float32)
    for b, (a, c) in enumerate(zip(lq, lk)):
        if a == 0 or c == 0:
            continue
        bias = torch.zeros(a, c)
        if pos_table is not None:
            bias = bias + rel_pos_bias(pos_table, a, c, max_k)
        if ts_table is not None:
            t = timestamps[ok[b]: ok[b] + c]
            bias = bias + time_bias(ts_table, t[c - a:], t, **bucket_kw)
        out[b, :, :a, :c] = bias
    return out.to(dtype)


# --------------------------------------------------------------------------
# the forward
# --------------------------------------------------------------------------
def _score_to_p(s: torch.Tensor, bias, alpha: float, silu_scale: float, mask) -> torch.Tensor:
    x = s if bias is None else s + bias
    x = x * alpha
    p = F.silu(x) * silu_scale
    if mask is not None:
        p = p * mask
    return p


def hstu_jagged_forward(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, seq_offset_q: torch.Tensor,
                        seq_offset_k: Optional[torch.Tensor] = None, *, max_seq_len_q: int,
                        max_seq_len_k: Optional[int] = None, mask_type: int = MASK_TRIL,
                        mask: Optional[torch.Tensor] = None, attn_bias: Optional[torch.Tensor] = None,
                        silu_scale: float = 0.0, alpha: float = 1.0,
                        num_context: Optional[Sequence[int]] = None, num_target: Optional[Sequence[int]] = None,
                        target_group_size: int = 0, mode: str = "exact",
                        compute_dtype: torch.dtype = torch.float32,
                        out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """HSTU attention forward over packed sequences.

    q ``[Tq, Nq, Dqk]``, k ``[Tk, Nk, Dqk]``, v ``[Tk, Nk, Dv]``; returns ``[Tq, Nq, Dv]``.

    mode ``"exact"``: every operand is up-cast to ``compute_dtype`` first and
    nothing is rounded until the end (the fp32 leg of the reference's
    double-benchmark, pytorch_native_backend.py:36-45).
    mode ``"lowp"``: the reference golden's rounding points -- matmuls in the
    I/O dtype, score math in fp32, P rounded to the I/O dtype.
    ``out_dtype`` None keeps ``compute_dtype`` for "exact" and the I/O dtype
    for "lowp".
    """
    assert q.dim() == 3 and k.dim() == 3 and v.dim() == 3
    if seq_offset_k is None:
        seq_offset_k = seq_offset_q
    if max_seq_len_k is None:
        max_seq_len_k = max_seq_len_q
    if mask_type == MASK_TRIU or not (0 <= mask_type <= 3):
        raise ValueError("unsupported mask_type")
    if mask_type == MASK_CUSTOM and mask is None:
        raise ValueError("custom mask needs a mask tensor")
    io_dtype = q.dtype
    fp8 = io_dtype == torch.float8_e4m3fn
    if fp8:
        # the reference's use_float8 golden: fp32 operands, P through e4m3, fp16 out (test_hstu_jagged_forward.py:150-189)
        q, k, v = q.to(torch.float32), k.to(torch.float32), v.to(torch.float32)
        if attn_bias is not None:
            attn_bias = attn_bias.to(torch.float32)
    nq, nk, dv = q.shape[1], k.shape[1], v.shape[2]
    assert nq % nk == 0
    ratio = nq // nk
    scale = (1.0 / max_seq_len_q) if silu_scale == 0.0 else silu_scale
    oq, okk = seq_offset_q.tolist(), seq_offset_k.tolist()
    nb = len(oq) - 1
    ctx = [0] * nb if num_context is None else [int(x) for x in num_context]
    tgt = [0] * nb if num_target is None else [int(x) for x in num_target]

    exact = mode == "exact"
    cd = compute_dtype if exact else torch.float32
    out = torch.zeros(q.shape[0], nq, dv, dtype=cd if exact else (torch.float32 if fp8 else io_dtype))
    for b in range(nb):
        lq, lk = int(oq[b + 1] - oq[b]), int(okk[b + 1] - okk[b])
        if lq == 0 or lk == 0:
            continue
        qb = q[oq[b]: oq[b] + lq].permute(1, 0, 2)                       # [Nq, lq, D]
        kb = k[okk[b]: okk[b] + lk].repeat_interleave(ratio, dim=1).permute(1, 0, 2)
        vb = v[okk[b]: okk[b] + lk].repeat_interleave(ratio, dim=1).permute(1, 0, 2)
        if mask_type == MASK_TRIL:
            m = builtin_mask(lq, lk, ctx[b], tgt[b], target_group_size).to(cd)
        elif mask_type == MASK_CUSTOM:
            m = mask[b, :, :lq, :lk].to(cd)
        else:
            m = None
        bias = None if attn_bias is None else attn_bias[b, :, :lq, :lk].to(cd)
        if exact:
            s = torch.matmul(qb.to(cd), kb.to(cd).transpose(1, 2))
            p = _score_to_p(s, bias, alpha, scale, m)
            ob = torch.matmul(p, vb.to(cd))
        else:
            s = torch.matmul(qb, kb.transpose(1, 2)).to(torch.float32)
            p = _score_to_p(s, bias, alpha, scale, m).to(io_dtype)
            if fp8:
                p = p.to(torch.float32)
            ob = torch.matmul(p, vb)
        out[oq[b]: oq[b] + lq] = ob.permute(1, 0, 2)
    if out_dtype is not None:
        out = out.to(out_dtype)
    elif fp8 and not exact:
        out = out.to(torch.float16)
    return out


def hstu_jagged_backward(grad: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                         seq_offset_q: torch.Tensor, seq_offset_k: Optional[torch.Tensor] = None, *,
                         max_seq_len_q: int, max_seq_len_k: Optional[int] = None, mask_type: int = MASK_TRIL,
                         mask: Optional[torch.Tensor] = None, attn_bias: Optional[torch.Tensor] = None,
                         silu_scale: float = 0.0, alpha: float = 1.0,
                         num_context: Optional[Sequence[int]] = None, num_target: Optional[Sequence[int]] = None,
                         target_group_size: int = 0, compute_dtype: torch.dtype = torch.float64):
    """Gradients of ``hstu_jagged_forward`` for an upstream gradient ``grad`` ``[Tq, Nq, Dv]``.

    Restates the reference golden ``hstu_bwd_gold`` (build/presmoke/hstu/hstu_common.py:387-476) per sequence,
    without the padding to dense tensors and without intermediate rounding:

        x  = alpha * (Q K^T + bias)          P  = silu(x) * silu_scale * mask
        dS = (dO V^T) * silu_scale * mask * sigmoid(x) * (1 + x * (1 - sigmoid(x))) * alpha
        dQ = dS K      dK = dS^T Q      dV = P^T dO      dBias = dS

    With GQA the K/V gradients of the query heads that share a K/V head are summed (hstu_common.py:457-463).
    Returns ``(dq, dk, dv, dbias)`` in ``compute_dtype``; ``dbias`` is ``None`` without ``attn_bias`` and is zero
    outside the sequences' own ``[:lq, :lk]`` corners (the op allocates it with zeros, hstu_jagged.cpp:121-123).
    """
    if seq_offset_k is None:
        seq_offset_k = seq_offset_q
    if max_seq_len_k is None:
        max_seq_len_k = max_seq_len_q
    cd = compute_dtype
    nq, nk = q.shape[1], k.shape[1]
    ratio = nq // nk
    scale = (1.0 / max_seq_len_q) if silu_scale == 0.0 else silu_scale
    oq, okk = seq_offset_q.tolist(), seq_offset_k.tolist()
    nb = len(oq) - 1
    ctx = [0] * nb if num_context is None else [int(x) for x in num_context]
    tgt = [0] * nb if num_target is None else [int(x) for x in num_target]
    dq = torch.zeros(q.shape, dtype=cd)
    dk = torch.zeros(k.shape, dtype=cd)
    dv = torch.zeros(v.shape, dtype=cd)
    dbias = None if attn_bias is None else torch.zeros(attn_bias.shape, dtype=cd)
    for b in range(nb):
        lq, lk = int(oq[b + 1] - oq[b]), int(okk[b + 1] - okk[b])
        if lq == 0 or lk == 0:
            continue
        qb = q[oq[b]: oq[b] + lq].to(cd).permute(1, 0, 2)                                   # [Nq, lq, D]
        gb = grad[oq[b]: oq[b] + lq].to(cd).permute(1, 0, 2)                                # [Nq, lq, Dv]
        kb = k[okk[b]: okk[b] + lk].to(cd).repeat_interleave(ratio, dim=1).permute(1, 0, 2)  # [Nq, lk, D]
        vb = v[okk[b]: okk[b] + lk].to(cd).repeat_interleave(ratio, dim=1).permute(1, 0, 2)
        if mask_type == MASK_TRIL:
            m = builtin_mask(lq, lk, ctx[b], tgt[b], target_group_size).to(cd)
        elif mask_type == MASK_CUSTOM:
            m = mask[b, :, :lq, :lk].to(cd)
        else:
            m = torch.ones(lq, lk, dtype=cd)
        x = torch.matmul(qb, kb.transpose(1, 2))
        if attn_bias is not None:
            x = x + attn_bias[b, :, :lq, :lk].to(cd)
        x = x * alpha
        sg = torch.sigmoid(x)
        p = x * sg * scale * m
        ds = torch.matmul(gb, vb.transpose(1, 2)) * scale * m * sg * (1 + x * (1 - sg)) * alpha
        dq[oq[b]: oq[b] + lq] = torch.matmul(ds, kb).permute(1, 0, 2)
        dkb = torch.matmul(ds.transpose(1, 2), qb)                                          # [Nq, lk, D]
        dvb = torch.matmul(p.transpose(1, 2), gb)
        dk[okk[b]: okk[b] + lk] = dkb.reshape(nk, ratio, lk, -1).sum(1).permute(1, 0, 2)
        dv[okk[b]: okk[b] + lk] = dvb.reshape(nk, ratio, lk, -1).sum(1).permute(1, 0, 2)
        if dbias is not None:
            dbias[b, :, :lq, :lk] = ds
    return dq, dk, dv, dbias


def hstu_dense_forward(q, k, v, *, max_seq_len: int, mask_type: int = MASK_TRIL, mask=None, attn_bias=None,
                       silu_scale: float = 0.0, **kw) -> torch.Tensor:
    """``[B, S, N, D]`` layout sibling (hstu_dense.cpp:20-41; alpha fixed at 1)."""
    b, s, n, d = q.shape
    off = torch.arange(b + 1, dtype=torch.int64) * s
    o = hstu_jagged_forward(q.reshape(b * s, n, d), k.reshape(b * s, k.shape[2], d),
                            v.reshape(b * s, v.shape[2], v.shape[3]), off, max_seq_len_q=max_seq_len,
                            mask_type=mask_type, mask=mask, attn_bias=attn_bias, silu_scale=silu_scale,
                            alpha=1.0, **kw)
    return o.reshape(b, s, n, -1)


def hstu_dense_backward(grad, q, k, v, *, max_seq_len: int, mask_type: int = MASK_TRIL, mask=None, attn_bias=None,
                        silu_scale: float = 0.0):
    """Backward of the ``[B, S, N, D]`` layout (hstu_dense.cpp:43-153: the jagged backward's kernel with layout
    "normal", alpha fixed at 1).  Returns ``(dq, dk, dv, dbias)`` shaped like q, k, v, attn_bias.
    PINNED by autograd through hstu_dense_forward (tests/test_oracle_backward.py)."""
    b, s, n, d = q.shape
    off = torch.arange(b + 1, dtype=torch.int64) * s
    dq, dk, dv, db = hstu_jagged_backward(grad.reshape(b * s, n, -1), q.reshape(b * s, n, d), k.reshape(b * s, n, d),
                                          v.reshape(b * s, n, -1), off, off, max_seq_len_q=max_seq_len,
                                          max_seq_len_k=max_seq_len, mask_type=mask_type, mask=mask, attn_bias=attn_bias,
                                          silu_scale=silu_scale, alpha=1.0)
    return dq.reshape(q.shape), dk.reshape(k.shape), dv.reshape(v.shape), db


# --------------------------------------------------------------------------
# paged KV cache
# --------------------------------------------------------------------------
def depage_history(kv_cache: torch.Tensor, page_offsets, page_ids, last_page_len, b: int):
    """History K and V rows of user b from a ``[pages, 2, page_size, Nk, D]`` cache
    (test_hstu_paged_forward.py:236-266)."""
    po, pi, lp = page_offsets.tolist(), page_ids.tolist(), last_page_len.tolist()
    ks, vs = [], []
    for p in range(po[b], po[b + 1]):
        n = lp[b] if p == po[b + 1] - 1 else kv_cache.shape[2]
        ks.append(kv_cache[pi[p], 0, :n])
        vs.append(kv_cache[pi[p], 1, :n])
    if not ks:
        e = kv_cache.new_zeros((0,) + tuple(kv_cache.shape[3:]))
        return e, e
    return torch.cat(ks), torch.cat(vs)


def assemble_paged_kv(k, v, kv_cache, seq_offset_q, page_offsets, page_ids, last_page_len, num_target):
    """K/V timeline per user = de-paged history ++ the last ``num_target`` rows of the
    user's input k/v segment.  Returns (k_cat, v_cat, seq_offset_k)."""
    oq = seq_offset_q.tolist()
    nt = [int(x) for x in num_target]
    kc, vc, lens = [], [], []
    for b in range(len(oq) - 1):
        hk, hv = depage_history(kv_cache, page_offsets, page_ids, last_page_len, b)
        new_hist = oq[b + 1] - oq[b] - nt[b]
        kc += [hk.to(k.dtype), k[oq[b] + new_hist: oq[b + 1]]]
        vc += [hv.to(v.dtype), v[oq[b] + new_hist: oq[b + 1]]]
        lens.append(hk.shape[0] + nt[b])
    off = torch.zeros(len(lens) + 1, dtype=torch.int64)
    off[1:] = torch.cumsum(torch.tensor(lens, dtype=torch.int64), 0)
    return torch.cat(kc), torch.cat(vc), off


def hstu_paged_forward(q, k, v, kv_cache, seq_offset_q, page_offsets, page_ids, last_page_len, num_target, *,
                       max_seq_len_q: int, max_seq_len_k: int, target_group_size: int = 1, **kw) -> torch.Tensor:
    k_cat, v_cat, off_k = assemble_paged_kv(k, v, kv_cache, seq_offset_q, page_offsets, page_ids, last_page_len,
                                            num_target)
    return hstu_jagged_forward(q, k_cat, v_cat, seq_offset_q, off_k, max_seq_len_q=max_seq_len_q,
                               max_seq_len_k=max_seq_len_k, num_target=num_target,
                               target_group_size=target_group_size, **kw)


# --------------------------------------------------------------------------
# fp8-e4m3 KV cache (build-defined: PARITY UNPINNED, no reference counterpart)
# --------------------------------------------------------------------------
def quantize_kv_cache_fp8(kv_cache: torch.Tensor):
    """``[pages, 2, page_size, Nk, D]`` -> (uint8 bit patterns of e4m3fn, fp32 scales ``[pages, 2, Nk]``)
    with ``scale = absmax/448`` over (page, k|v, head) and ``q8 = rne_e4m3(x/scale)``."""
    x = kv_cache.float()
    amax = x.abs().amax(dim=(2, 4))
    scales = torch.where(amax > 0, amax / FP8_E4M3_MAX, torch.ones_like(amax))
    q8 = (x / scales[:, :, None, :, None]).clamp(-FP8_E4M3_MAX, FP8_E4M3_MAX).to(torch.float8_e4m3fn)
    return q8.view(torch.uint8), scales


def dequantize_kv_cache_fp8(cache_u8: torch.Tensor, scales: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
    x = cache_u8.view(torch.float8_e4m3fn).float() * scales[:, :, None, :, None]
    return x.to(dtype)


# --------------------------------------------------------------------------
# brute force (tiny inputs only) and comparators
# --------------------------------------------------------------------------
def hstu_bruteforce(q, k, v, off_q, off_k, *, max_seq_len_q, mask_type=MASK_TRIL, mask=None, attn_bias=None,
                    silu_scale=0.0, alpha=1.0, num_context=None, num_target=None, target_group_size=0):
    """Scalar float64 loops; uses ``mask_point`` (not ``builtin_mask``) so that the two mask
    formulations check each other."""
    nq, nk, dqk, dv = q.shape[1], k.shape[1], q.shape[2], v.shape[2]
    ratio = nq // nk
    scale = (1.0 / max_seq_len_q) if silu_scale == 0.0 else silu_scale
    oq, okk = off_q.tolist(), off_k.tolist()
    out = [[[0.0] * dv for _ in range(nq)] for _ in range(q.shape[0])]
    ql, kl, vl = q.double().tolist(), k.double().tolist(), v.double().tolist()
    for b in range(len(oq) - 1):
        lq, lk = oq[b + 1] - oq[b], okk[b + 1] - okk[b]
        c = 0 if num_context is None else int(num_context[b])
        t = 0 if num_target is None else int(num_target[b])
        for h in range(nq):
            hk = h // ratio
            for i in range(lq):
                for j in range(lk):
                    if mask_type == MASK_TRIL:
                        mv = mask_point(i, j, lq, lk, c, t, target_group_size)
                    elif mask_type == MASK_CUSTOM:
                        mv = float(mask[b, h, i, j])
                    else:
                        mv = 1.0
                    if mv == 0:
                        continue
                    s = sum(ql[oq[b] + i][h][d] * kl[okk[b] + j][hk][d] for d in range(dqk))
                    if attn_bias is not None:
                        s += float(attn_bias[b, h, i, j])
                    x = alpha * s
                    p = x / (1.0 + math.exp(-x)) * scale * mv
                    row = out[oq[b] + i][h]
                    vr = vl[okk[b] + j][hk]
                    for d in range(dv):
                        row[d] += p * vr[d]
    return torch.tensor(out, dtype=torch.float64).reshape(q.shape[0], nq, dv)


def mismatch_ratio_close(a: torch.Tensor, b: torch.Tensor, atol: float, ratio: float) -> bool:
    """The reference's comparator (test_common_utils.py:57-61): fraction of elements with
    |a-b| > atol must stay below ``ratio``."""
    bad = ((a.float() - b.float()).abs() > atol).sum().item()
    return bad / max(a.numel(), 1) < ratio


def double_benchmark_close(actual, ref_lowp, ref_fp32, multiplier: float = 5.0) -> bool:
    """pytorch_native_backend.py:199-229: max|actual-ref32| <= multiplier*max|ref_lowp-ref32|,
    or plain allclose against the low-precision golden."""
    a, r, f = actual.float().reshape(-1), ref_lowp.float().reshape(-1), ref_fp32.float().reshape(-1)
    return bool((a - f).abs().max() <= multiplier * (r - f).abs().max()) or bool(torch.allclose(a, r))
