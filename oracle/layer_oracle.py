"""CPU oracle for ``mxrec::norm_multiply_dropout`` and ``mxrec::distance_in_linear_silu``.  TEST INFRASTRUCTURE ONLY.

Restates the reference's goldens; used by ``tests/`` and by the ``cpu_baseline`` leg of ``bench.py``.  Nothing in the
shipped package imports it.

Definition followed (reference file:line):

* forward: cust_op/ascendc_op/ai_core_op/norm_multiply_dropout/v220/README.md:41-60 -- LayerNorm over the last axis
  (biased variance, affine), times u, dropout (kept elements scaled by 1/(1-p)), computed in a wider type and rounded
  once to the I/O dtype; mean and var as the explicit golden returns them
  (cust_op/test/norm_multiply_dropout/torch/test_norm_multiply_dropout.py:137-156).
* backward: test_norm_multiply_dropout.py:220-243 (``ln_mul_bwd``), with the upstream gradient passed through the
  dropout mask first.
* mask layout: bit (e % 8) of byte (e / 8) = element e kept.  WHICH elements a seed keeps is this build's own choice
  (the reference draws its mask from aclnnDropoutGenMaskV2 and its tests only check that the call runs,
  test_norm_multiply_dropout.py:336-342): parity with the reference's random stream is neither possible nor claimed;
  the tests check the op against this oracle under the mask the op itself returned, and the keep rate.

* in_linear_silu: cust_op/test/in_linear_silu_test/test_in_linear_silu.py:31-45 -- ``addmm(bias, x, W^T)`` rounded to the
  I/O dtype (= linear_output), SiLU of that rounded tensor, rounded again, split along the last axis.

* in_linear_silu_backward: cust_op/test/in_linear_silu_test_backward/test_in_linear_silu_backward.py:37-88 --
  ``dlin = grad * sigmoid(lin) * (1 + lin * (1 - sigmoid(lin)))`` with grad the four gradients side by side,
  ``bias_grad = dlin.sum(0)`` from the unrounded dlin, ``x_grad = dlin @ W``, ``weight_grad = dlin^T @ x``; the
  device-side golden (:37-66) rounds dlin to the I/O dtype before the two products, the CPU golden (:69-88) does not:
  ``round_dlin`` selects.

Everything here is fp64 so that it can serve as the exact value for every I/O dtype (``in_linear_silu`` applies the
golden's two roundings to the I/O dtype on top of fp64 arithmetic).

Pinning status (tests/test_oracle_layer.py): forward against ``torch.nn.functional.layer_norm`` (a library routine
that shares no code with the explicit mean / var formula here) and ``F.dropout`` semantics under a given mask; backward
against autograd through that library forward, including the mask.  ``in_linear_silu`` against ``torch.addmm``,
``F.silu`` and ``torch.split`` evaluated in fp32 on values where fp32 is exact; ``in_linear_silu_backward`` against
autograd through ``F.linear`` / ``F.silu`` in fp64 (which knows nothing of the closed-form derivative used here) and
against central differences.  PINNED
"""
from __future__ import annotations

import torch


def unpack_mask(mask_bytes: torch.Tensor, numel: int) -> torch.Tensor:
    """uint8 ``[ceil(numel/128)*16]`` -> bool ``[numel]`` (bit e % 8 of byte e / 8)."""
    bits = (mask_bytes.to(torch.int32)[:, None] >> torch.arange(8, dtype=torch.int32)[None, :]) & 1
    return bits.reshape(-1)[:numel].bool()


def nmd_forward(x, u, weight, bias, eps: float, dropout_ratio: float = 0.0, keep=None):
    """Returns (y, mean, var) in fp64; ``keep``: bool ``[rows, cols]`` when ``dropout_ratio`` > 1e-10."""
    x, u, weight, bias = (t.double() for t in (x, u, weight, bias))
    mean = x.mean(dim=1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=1, keepdim=True)
    y = ((x - mean) / torch.sqrt(var + eps) * weight + bias) * u
    if dropout_ratio > 1e-10:
        y = torch.where(keep, y / (1.0 - dropout_ratio), torch.zeros_like(y)) if dropout_ratio < 1 else torch.zeros_like(y)
    return y, mean[:, 0], var[:, 0]


def nmd_backward(d_out, x, u, weight, bias, mean, var, eps: float, dropout_ratio: float = 0.0, keep=None):
    """Returns (d_x, d_u, d_weight, d_bias) in fp64."""
    dy, x, u, weight, bias = (t.double() for t in (d_out, x, u, weight, bias))
    mean, var = mean.double()[:, None], var.double()[:, None]
    if dropout_ratio > 1e-10:
        dy = torch.where(keep, dy / (1.0 - dropout_ratio), torch.zeros_like(dy)) if dropout_ratio < 1 else torch.zeros_like(dy)
    rstd = 1.0 / torch.sqrt(var + eps)
    xh = (x - mean) * rstd
    g = dy * u
    a = g * weight
    c = x.shape[1]
    dx = (a - (a.sum(dim=1, keepdim=True) + xh * (a * xh).sum(dim=1, keepdim=True)) / c) * rstd
    du = dy * (weight * xh + bias)
    return dx, du, (xh * g).sum(dim=0), g.sum(dim=0)


def in_linear_silu(x, weight, bias, split):
    """Returns (user, value, query, key, linear_output) in the dtype of x."""
    lin = x.double() @ weight.double().t()
    if bias is not None:
        lin = lin + bias.double()
    lin = lin.to(x.dtype)
    act = (lin.double() * torch.sigmoid(lin.double())).to(x.dtype)
    u, v, q, k = torch.split(act, list(split), dim=-1)
    return u.contiguous(), v.contiguous(), q.contiguous(), k.contiguous(), lin


def in_linear_silu_backward(grads, x, weight, linear_output, with_bias=True, round_dlin=True):
    """Returns (x_grad, weight_grad, bias_grad or None) in fp64."""
    grad = torch.cat([g.double() for g in grads], dim=-1)
    lin = linear_output.double()
    sg = torch.sigmoid(lin)
    dlin = grad * (sg * (1 + lin * (1 - sg)))
    bias_grad = dlin.sum(dim=0) if with_bias else None
    if round_dlin:
        dlin = dlin.to(x.dtype).double()
    return dlin @ weight.double(), dlin.t() @ x.double(), bias_grad
