"""The issue-rate diagnostics (include/hstu_diag.h) run, finish and report sane clocks."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("mode,waves", [(0, 4), (1, 3), (2, 2), (3, 2), (4, 4)])
def test_block_rate_kernels_run(mode, waves):
    from recsdk_amd import _capi
    print("[case] rates", mode, waves, flush=True)
    L = _capi.lib()
    ops = (torch.rand(65536 * 8, device="cuda") - 0.5).to(torch.bfloat16)
    sink = torch.empty(256 * 256 * 4, device="cuda")
    ticks = torch.zeros(2 * 1024, device="cuda", dtype=torch.int64)
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert L.hstu_hip_measure_block_rates(mode, waves, 50, ops.data_ptr(), sink.data_ptr(), ticks.data_ptr(), st) == 0
    torch.cuda.synchronize()
    t = ticks[: 2 * 256 * waves].view(-1, 2)
    assert (t > 0).all(), "every workgroup reports its duration"
    ghz = float(t[:, 0].double().sum() / t[:, 1].double().sum()) * 0.1
    assert 0.5 < ghz < 3.0, ghz
