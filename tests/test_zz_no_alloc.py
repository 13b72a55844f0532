"""hstu_hip_jagged_forward_noalloc (work list in the library's fixed array) against hstu_hip_jagged_forward
(work list in a caller workspace): same bits, on two calls in a row of which the second is smaller, so that the
second call runs over what the first one left in the array."""
import pytest
import torch

from recsdk_amd import workloads as W

pytestmark = pytest.mark.gpu


def _both(cfg, fp8=False):
    """(output of the entry point with a workspace, output of the one without), both through the C ABI."""
    from recsdk_amd import _capi
    q, k, v = cfg["q"].cuda(), cfg["k"].cuda(), cfg["v"].cuda()
    if fp8:
        q, k, v = (x.to(torch.float8_e4m3fn) for x in (q, k, v))
    outs = []
    for noalloc in (False, True):
        out = torch.full(q.shape, float("nan"), dtype=_capi.out_dtype(q.dtype), device="cuda")
        p, keep = _capi.make_params(q, k, v, out, seq_offset_q=cfg["seq_offset"].cuda(), max_seq_len_q=cfg["max_seq_len"],
                                    alpha=cfg["alpha"], num_target=None if cfg.get("num_target") is None else cfg["num_target"].cuda(),
                                    target_group_size=cfg.get("target_group_size", 0))
        assert _capi.describe_kernel(p).startswith("mfma_")
        if noalloc:
            _capi.run_noalloc(p)                      # (first call on this device: the library looks up its array once)
            torch.cuda.synchronize()
            out.fill_(float("nan"))
            free_before = torch.cuda.mem_get_info()[0]
            _capi.run_noalloc(p)
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free_before, "the allocation-free entry point changed the free device memory"
        else:
            _capi.run("jagged", p)
        torch.cuda.synchronize()
        outs.append(out.cpu())
    return outs


def test_noalloc_matches_the_workspace_entry_on_two_calls_in_a_row():
    big = W.jagged_config(3, 24, 4, 128, 100, 900, torch.bfloat16, max_seq_len=900)
    small = W.jagged_config(4, 5, 4, 128, 30, 400, torch.bfloat16, max_seq_len=400)
    small["num_target"] = torch.full((5,), 8, dtype=torch.int64)
    small["target_group_size"] = 1
    for cfg in (big, small):
        want, got = _both(cfg)
        assert torch.isfinite(want.float()).all()
        assert torch.equal(want.view(torch.int16), got.view(torch.int16))


def test_noalloc_with_fp8_inputs():
    cfg = W.jagged_config(5, 6, 2, 128, 60, 500, torch.bfloat16, max_seq_len=500)
    cfg["silu_scale"] = 1.0 / 64
    want, got = _both(cfg, fp8=True)
    assert want.dtype == torch.float16 and torch.isfinite(want.float()).all()
    assert torch.equal(want.view(torch.int16), got.view(torch.int16))


def test_noalloc_on_the_plain_kernel():
    """HSTU_FLAG_FORCE_GENERIC (and everything else the matrix-core kernels do not take) runs the plain kernel, which uses no
    device memory beyond its arguments: same bits as through the entry point with a workspace."""
    from recsdk_amd import _capi
    cfg = W.jagged_config(6, 4, 2, 64, 20, 200, torch.bfloat16, max_seq_len=200)
    q, k, v = cfg["q"].cuda(), cfg["k"].cuda(), cfg["v"].cuda()
    outs = []
    for noalloc in (False, True):
        out = torch.full_like(q, float("nan"))
        p, keep = _capi.make_params(q, k, v, out, seq_offset_q=cfg["seq_offset"].cuda(), max_seq_len_q=cfg["max_seq_len"],
                                    alpha=cfg["alpha"], flags=_capi.FLAG_FORCE_GENERIC)
        assert _capi.describe_kernel(p) == "generic_bf16"
        if noalloc:
            free_before = torch.cuda.mem_get_info()[0]
            _capi.run_noalloc(p)
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free_before
        else:
            _capi.run("jagged", p)
        torch.cuda.synchronize()
        outs.append(out.cpu())
    assert torch.isfinite(outs[0].float()).all() and torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))


def test_noalloc_rejects_a_batch_beyond_its_array():
    """More (Q tile, head) items than the fixed array holds: HSTU_ERR_WORKSPACE and a message, nothing launched."""
    from recsdk_amd import _capi
    import ctypes as C
    lens = [8] * 2048
    q = torch.zeros(sum(lens), 16, 128, dtype=torch.bfloat16, device="cuda")
    out = torch.full_like(q, 7.0)
    p, keep = _capi.make_params(q, q, q, out, seq_offset_q=W.offsets(lens).cuda(), max_seq_len_q=8, alpha=0.1)
    rc = _capi.lib().hstu_hip_jagged_forward_noalloc(C.byref(p), None)
    torch.cuda.synchronize()
    assert rc == -3 and b"hstu_hip_jagged_forward_noalloc holds" in _capi.lib().hstu_hip_last_error()
    assert bool((out == 7.0).all())
