"""CPU oracle for the standalone attention-bias producers.  TEST INFRASTRUCTURE ONLY.

Restates the reference's goldens for ``mxrec::relative_attn_bias_time`` (``_with_index``, ``_backward``) and
``mxrec::relative_attn_bias_pos``; used by ``tests/`` and the ``cpu_baseline`` leg of ``bench.py``.  Nothing in the
shipped package imports it.

Definition followed (reference file:line):

* ``rab_time``: cust_op/test/relative_attn_bias/torch/utils.py:99-129 -- every timestamp repeated twice,
  ``bucket = trunc(log(clamp(|t_i - t_j|, 1, e^(128*0.301))) / divisor)`` in fp32, ``out = weights[:, bucket]``;
  the op returns the un-repeated ids ``[b, s, s]`` (test_relative_attn_bias.py:86-89).  The number of buckets is the
  table width minus one, as the kernel's host code derives it (relative_attn_bias_time/v220/op_host/relative_attn_bias_time.cpp:54-56).
* ``rab_time_backward``: utils.py:132-145 -- ids repeated 2x2, gradient summed per (layer, bucket) in fp32 (here fp64:
  the reference compares with rtol = atol = 1e-5 for fp32 gradients, 1e-3 for fp16, test_relative_attn_bias.py:101-102).
* ``rab_pos``: utils.py:148-166 -- rows from ``past_valid_len`` on replaced by row ``past_valid_len``, then
  ``x * (1 - identity) + identity * x[0, 0, 0]`` in the tensors' dtype.

Pinning status (tests/test_oracle_bias.py): element-by-element Python loops written from the prose definition on small
inputs; closed forms (equal timestamps -> column 0 of the table, |dt| at and just below e^(k*divisor), all-ones identity ->
constant rel[0, 0]); the adjoint identity <rab_time(w), G> = <w, rab_time_backward(G)> which ties the gather of the
forward to the scatter of the backward.  PINNED
"""
from __future__ import annotations

import torch

NUM_BUCKETS = 128
BUCKET_DIVISOR = 0.301


def time_buckets(timestamps: torch.Tensor, num_buckets: int = NUM_BUCKETS, bucket_divisor: float = BUCKET_DIVISOR) -> torch.Tensor:
    """``[b, s]`` timestamps -> ``[b, s, s]`` int64 bucket ids."""
    d = (timestamps[:, :, None] - timestamps[:, None, :]).abs().to(torch.float32)
    clamp_max = torch.exp(torch.tensor(num_buckets * bucket_divisor))
    return (torch.log(d.clamp(1, clamp_max.item())) / bucket_divisor).long()


def rab_time(timestamps: torch.Tensor, weights: torch.Tensor, bucket_divisor: float = BUCKET_DIVISOR):
    """``weights`` ``[num_layers, W]`` -> (``[num_layers, b, 2s, 2s]`` in the dtype of weights, ``[b, s, s]`` ids in the
    dtype of timestamps)."""
    ids = time_buckets(timestamps, weights.shape[1] - 1, bucket_divisor)
    b, s, _ = ids.shape
    out = weights[:, ids.reshape(-1)].reshape(weights.shape[0], b, s, s)
    out = out.repeat_interleave(2, dim=2).repeat_interleave(2, dim=3)
    return out, ids.to(timestamps.dtype)


def rab_time_backward(grad: torch.Tensor, bucket_ts: torch.Tensor, num_buckets: int) -> torch.Tensor:
    """``grad`` ``[n, b, 2s, 2s]``, ``bucket_ts`` ``[b, s, s]`` -> float64 ``[n, num_buckets]``."""
    n, b, s2, _ = grad.shape
    s = s2 // 2
    g = grad.double().reshape(n, b, s, 2, s, 2).sum(dim=(3, 5)).reshape(n, -1)
    ids = bucket_ts.reshape(-1).long()
    ok = (ids >= 0) & (ids < num_buckets)
    out = torch.zeros(n, num_buckets, dtype=torch.float64)
    out.index_add_(1, ids[ok], g[:, ok])
    return out


def rab_pos(rel_pos_bias: torch.Tensor, identity: torch.Tensor, past_valid_lens) -> torch.Tensor:
    """``[S2, S2]`` tables -> ``[bs, S2, S2]``."""
    x = rel_pos_bias.unsqueeze(0).repeat(len(past_valid_lens), 1, 1)
    for i, v in enumerate(past_valid_lens):
        x[i, int(v):, :] = rel_pos_bias[int(v), :]
    return x * (1 - identity) + identity * x[0, 0, 0]
