"""hstu_hip_jagged_forward_noalloc (work list in the library's fixed array) against hstu_hip_jagged_forward
(work list in a caller workspace): same bits, on two calls in a row of which the second is smaller, so that the
second call runs over what the first one left in the array."""
import pytest
import torch

from recsdk_amd import workloads as W

pytestmark = pytest.mark.gpu


def _both(cfg):
    """(output of the entry point with a workspace, output of the one without), both through the C ABI."""
    from recsdk_amd import _capi
    q, k, v = cfg["q"].cuda(), cfg["k"].cuda(), cfg["v"].cuda()
    outs = []
    for noalloc in (False, True):
        out = torch.full_like(q, float("nan"))
        p, keep = _capi.make_params(q, k, v, out, seq_offset_q=cfg["seq_offset"].cuda(), max_seq_len_q=cfg["max_seq_len"],
                                    alpha=cfg["alpha"], num_target=None if cfg.get("num_target") is None else cfg["num_target"].cuda(),
                                    target_group_size=cfg.get("target_group_size", 0))
        assert _capi.describe_kernel(p).startswith("mfma_")
        if noalloc:
            _capi.run_noalloc(p)
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
