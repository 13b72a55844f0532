"""Shared helpers of the parity tests: run a workload through the HIP path (C ABI via ctypes, or the
torch op which calls the same C ABI) and through the CPU oracle, and compare."""
from __future__ import annotations

import torch

from oracle import hstu_oracle as O


def _dev(t):
    return None if t is None else (t.cuda() if isinstance(t, torch.Tensor) else t)


def run_capi(cfg, *, op="jagged", flags=0, reuse_from=None, **over):
    """Call hstu_hip_<op>_forward through ctypes.  Returns the output on the CPU.

    ``reuse_from``: a configuration with the same geometry; it is run first and its workspace (work list) is then
    handed to the call for ``cfg`` with HSTU_FLAG_REUSE_WORKSPACE set."""
    from recsdk_amd import _capi
    c = dict(cfg)
    c.update(over)
    q, k, v = _dev(c["q"]), _dev(c["k"]), _dev(c["v"])
    dense = op == "dense"
    odt = _capi.out_dtype(q.dtype)
    if dense:
        out = torch.full(q.shape, float("nan"), dtype=odt, device="cuda")
    else:
        out = torch.full((q.shape[0], q.shape[1], v.shape[2]), float("nan"), dtype=odt, device="cuda")
    kw = dict(max_seq_len_q=c["max_seq_len"], max_seq_len_k=c.get("max_seq_len_k"), mask_type=c.get("mask_type", 0),
              mask=_dev(c.get("mask")), attn_bias=_dev(c.get("attn_bias")), silu_scale=c.get("silu_scale", 0.0),
              alpha=c.get("alpha", 1.0), num_context=_dev(c.get("num_context")), num_target=_dev(c.get("num_target")),
              target_group_size=c.get("target_group_size", 0), pos_table=_dev(c.get("pos_table")),
              ts_table=_dev(c.get("ts_table")), timestamps=_dev(c.get("timestamps")), flags=flags, dense=dense)
    if c.get("ts_table") is not None:
        import recsdk_amd
        kw["ts_bounds"] = recsdk_amd.time_bucket_bounds(c["ts_table"].numel() - 1, c.get("bucket_divisor", 0.301)).cuda()
        kw["bucket_divisor"] = c.get("bucket_divisor", 0.301)
    if not dense:
        kw["seq_offset_q"] = _dev(c["seq_offset"])
        kw["seq_offset_k"] = _dev(c.get("seq_offset_k"))
    if op == "paged":
        cache = c["kv_cache_fp8"] if c.get("use_fp8") else c["kv_cache"]
        kw.update(kv_cache=_dev(cache), page_offsets=_dev(c["page_offsets"]), page_ids=_dev(c["page_ids"]),
                  last_page_len=_dev(c["last_page_len"]), kv_scales=_dev(c["kv_scales"]) if c.get("use_fp8") else None)
    p, keep = _capi.make_params(q, k, v, out, **kw)
    name = _capi.describe_kernel(p)
    if reuse_from is not None:
        import ctypes as C
        r = dict(reuse_from)
        p0, keep0 = _capi.make_params(_dev(r["q"]), _dev(r["k"]), _dev(r["v"]), torch.empty_like(out), **kw)
        ws = _capi.run(op, p0)
        torch.cuda.synchronize()
        p.flags |= _capi.FLAG_REUSE_WORKSPACE
        rc = getattr(_capi.lib(), f"hstu_hip_{op}_forward")(C.byref(p), ws.data_ptr(), ws.numel(), None)
        assert rc == 0, _capi.lib().hstu_hip_last_error().decode()
    else:
        _capi.run(op, p)
    torch.cuda.synchronize()
    return out.cpu(), name


def run_capi_backward(cfg, grad, flags=0, op="jagged", **over):
    """Call hstu_hip_<op>_backward (jagged or dense) through ctypes.  Returns (dq, dk, dv, dbias or None) on the CPU."""
    from recsdk_amd import _capi
    c = dict(cfg)
    c.update(over)
    q, k, v, g = _dev(c["q"]), _dev(c["k"]), _dev(c["v"]), _dev(grad)
    bias = _dev(c.get("attn_bias"))
    kw = dict(max_seq_len_q=c["max_seq_len"], max_seq_len_k=c.get("max_seq_len_k"), mask_type=c.get("mask_type", 0),
              mask=_dev(c.get("mask")), attn_bias=bias, silu_scale=c.get("silu_scale", 0.0), alpha=c.get("alpha", 1.0),
              num_context=_dev(c.get("num_context")), num_target=_dev(c.get("num_target")),
              target_group_size=c.get("target_group_size", 0), flags=flags, dense=op == "dense")
    if op != "dense":
        kw.update(seq_offset_q=_dev(c["seq_offset"]), seq_offset_k=_dev(c.get("seq_offset_k")))
    fwd, keep = _capi.make_params(q, k, v, q, **kw)     # the forward's `out` is not read by the backward
    fwd.out = None
    nan = float("nan")
    dq, dk, dv = torch.full_like(q, nan), torch.full_like(k, nan), torch.full_like(v, nan)
    db = None if bias is None else torch.full_like(bias, nan)
    p = _capi.make_backward_params(fwd, g, dq, dk, dv, db)
    global last_backward_kernel
    last_backward_kernel = _capi.describe_backward_kernel(p)
    _capi.run_backward(p, op=op)
    torch.cuda.synchronize()
    return dq.cpu(), dk.cpu(), dv.cpu(), None if db is None else db.cpu()


last_backward_kernel = None   # name of the kernel variant the last run_capi_backward call selected


def run_op(cfg, *, op="jagged", **over):
    """Call torch.ops.mxrec.* (the drop-in entry).  Returns the output on the CPU."""
    import recsdk_amd  # noqa: F401  (loads the op library)
    c = dict(cfg)
    c.update(over)
    q, k, v = _dev(c["q"]), _dev(c["k"]), _dev(c["v"])
    m = torch.ops.mxrec
    if op == "jagged":
        if c.get("seq_offset_k") is None:
            out = m.hstu_jagged(q, k, v, _dev(c.get("mask")), _dev(c.get("attn_bias")), c.get("mask_type", 0),
                                c["max_seq_len"], c.get("silu_scale", 0.0), _dev(c["seq_offset"]),
                                _dev(c.get("num_context")), _dev(c.get("num_target")), c.get("target_group_size", 0),
                                c.get("alpha", 1.0))
        else:
            out = m.hstu_jagged(q, k, v, _dev(c.get("mask")), _dev(c.get("attn_bias")), c.get("mask_type", 0),
                                c["max_seq_len"], c["max_seq_len_k"], c.get("silu_scale", 0.0), _dev(c["seq_offset"]),
                                _dev(c["seq_offset_k"]), _dev(c.get("num_context")), _dev(c.get("num_target")),
                                c.get("target_group_size", 0), c.get("alpha", 1.0))
    elif op == "table":
        ok = c.get("seq_offset_k")
        out = m.hstu_jagged_table_bias(q, k, v, _dev(c.get("pos_table")), _dev(c.get("ts_table")), _dev(c.get("timestamps")),
                                       _dev(c.get("attn_bias")), c.get("mask_type", 0), c["max_seq_len"],
                                       c.get("max_seq_len_k") or c["max_seq_len"], c.get("silu_scale", 0.0),
                                       _dev(c["seq_offset"]), _dev(ok if ok is not None else c["seq_offset"]),
                                       _dev(c.get("num_context")), _dev(c.get("num_target")),
                                       c.get("target_group_size", 0), c.get("alpha", 1.0))
    elif op in ("paged", "paged_fp8"):
        common = dict(mask=_dev(c.get("mask")), attn_bias=None, mask_type=c.get("mask_type", 0),
                      max_seq_len=c["max_seq_len"], max_seq_len_k=c["max_seq_len_k"], silu_scale=c.get("silu_scale", 0.0),
                      seq_offset=_dev(c["seq_offset"]), seq_offset_k=_dev(c["seq_offset_k"]),
                      seq_offset_t=_dev(c["seq_offset_t"]), page_offsets=_dev(c["page_offsets"]),
                      page_ids=_dev(c["page_ids"]), last_page_len=_dev(c["last_page_len"]),
                      num_target=_dev(c["num_target"]), target_group_size=c.get("target_group_size", 1),
                      alpha=c.get("alpha", 1.0))
        if op == "paged":
            out = m.hstu_paged(q=q, k=k, v=v, kv_cache=_dev(c["kv_cache"]), **common)
        else:
            out = m.hstu_paged_fp8(q=q, k=k, v=v, kv_cache=_dev(c["kv_cache_fp8"]), kv_scales=_dev(c["kv_scales"]), **common)
    elif op == "dense":
        out = m.hstu_dense(q, k, v, _dev(c.get("mask")), _dev(c.get("attn_bias")), c.get("mask_type", 0),
                           c["max_seq_len"], c.get("silu_scale", 0.0))
    else:
        raise ValueError(op)
    torch.cuda.synchronize()
    return out.cpu()


def oracle_jagged(cfg, *, mode="exact", compute_dtype=torch.float32, **over):
    c = dict(cfg)
    c.update(over)
    bias = c.get("attn_bias")
    ok = c.get("seq_offset_k") if c.get("seq_offset_k") is not None else c["seq_offset"]
    mk = c.get("max_seq_len_k") or c["max_seq_len"]
    if c.get("pos_table") is not None or c.get("ts_table") is not None:
        tb = O.dense_bias_from_tables(c["seq_offset"], ok, c["q"].shape[1], c["max_seq_len"], mk,
                                      pos_table=c.get("pos_table"), ts_table=c.get("ts_table"),
                                      timestamps=c.get("timestamps"),
                                      **({} if c.get("ts_table") is None else
                                         dict(num_buckets=c["ts_table"].numel() - 1, bucket_divisor=c.get("bucket_divisor", 0.301))))
        bias = tb if bias is None else bias.float() + tb
    return O.hstu_jagged_forward(c["q"], c["k"], c["v"], c["seq_offset"], ok, max_seq_len_q=c["max_seq_len"],
                                 max_seq_len_k=mk, mask_type=c.get("mask_type", 0), mask=c.get("mask"), attn_bias=bias,
                                 silu_scale=c.get("silu_scale", 0.0), alpha=c.get("alpha", 1.0),
                                 num_context=c.get("num_context"), num_target=c.get("num_target"),
                                 target_group_size=c.get("target_group_size", 0), mode=mode, compute_dtype=compute_dtype)


def oracle_paged(cfg, *, cache=None, **kw):
    c = cfg
    return O.hstu_paged_forward(c["q"], c["k"], c["v"], c["kv_cache"] if cache is None else cache, c["seq_offset"],
                                c["page_offsets"], c["page_ids"], c["last_page_len"], c["num_target"],
                                max_seq_len_q=c["max_seq_len"], max_seq_len_k=c["max_seq_len_k"],
                                target_group_size=c.get("target_group_size", 1), alpha=c.get("alpha", 1.0),
                                silu_scale=c.get("silu_scale", 0.0), mask_type=c.get("mask_type", 0), **kw)


# tolerances stated for the build: fp32 1e-5 relative; bf16/fp16 rtol = atol = 2e-2; fp8 KV path 5e-2
TOL = {torch.float32: 1e-5, torch.float16: 2e-2, torch.bfloat16: 2e-2}


def assert_parity(out, ref, dtype, *, tol=None, what=""):
    """``ref`` is the oracle in higher precision.  Checks the stated tolerance and, because outputs are
    small (silu_scale = 1/max_seq_len), also the error relative to the tensor's own scale."""
    assert out.shape == ref.shape, (out.shape, ref.shape)
    assert torch.isfinite(out.float()).all(), f"{what}: non-finite output"
    o, r = out.double(), ref.double()
    tol = TOL[dtype] if tol is None else tol
    scale = r.abs().max().item()
    err = (o - r).abs().max().item()
    if dtype == torch.float32 and tol <= 1e-4:
        assert err <= tol * max(scale, 1e-30), f"{what}: max err {err:.3e} vs scale {scale:.3e}"
        assert torch.allclose(o, r, rtol=10 * tol, atol=tol * max(scale, 1e-30)), what
    else:
        assert torch.allclose(o, r, rtol=tol, atol=tol), f"{what}: stated tolerance rtol=atol={tol} violated"
        # scale-relative: bf16 P and output rounding stay near 2^-8 of the tensor scale
        assert err <= tol * max(scale, 1e-30), f"{what}: max err {err:.3e} vs scale {scale:.3e} (tol {tol})"
    return err / max(scale, 1e-30)
