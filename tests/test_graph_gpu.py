"""The entry points record nothing but kernel launches on the caller's stream (no allocation, no memset, no
synchronisation), so a layer's forward and backward can be captured in a HIP graph and replayed: every replay, with new
inputs in the same buffers and eager work between the replays, must equal the eager result bit for bit."""
import ctypes as C

import pytest
import torch

from recsdk_amd import _capi, workloads as W
from tests.test_parity_gpu import say

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("batch,heads,lo,hi", [(6, 4, 100, 700), (32, 8, 1200, 2048)])
def test_forward_and_backward_replayed_from_a_graph(batch, heads, lo, hi):
    """The second geometry has more than 3000 items per backward kernel: the library then launches its dQ and K-side kernels
    on three streams forked from and joined to the caller's by events, which the capture must turn into edges of the graph;
    that case is also compared with the plain kernels, which run on the caller's stream alone."""
    say("graph capture of forward + backward", batch, heads, lo, hi)
    cfg = W.jagged_config(3, batch, heads, 128, lo, hi, torch.bfloat16, max_seq_len=hi)
    dev = W.to_device(cfg)
    q, k, v = dev["q"], dev["k"], dev["v"]
    grad = torch.randn_like(q)
    out, dq, dk, dv = (torch.empty_like(q) for _ in range(4))
    L = _capi.lib()
    fwd, keep = _capi.make_params(q, k, v, out, seq_offset_q=dev["seq_offset"], max_seq_len_q=cfg["max_seq_len"], alpha=cfg["alpha"])
    bwd = _capi.make_backward_params(fwd, grad, dq, dk, dv, None)
    nf, nb = C.c_uint64(0), C.c_uint64(0)
    assert L.hstu_hip_jagged_forward_get_workspace_size(C.byref(fwd), C.byref(nf)) == 0
    assert L.hstu_hip_jagged_backward_get_workspace_size(C.byref(bwd), C.byref(nb)) == 0
    wsf = torch.empty(max(nf.value, 16), dtype=torch.uint8, device="cuda")
    wsb = torch.empty(max(nb.value, 16), dtype=torch.uint8, device="cuda")

    def step(stream):
        s = C.c_void_p(stream.cuda_stream)
        assert L.hstu_hip_jagged_forward(C.byref(fwd), wsf.data_ptr(), nf.value, s) == 0, L.hstu_hip_last_error()
        assert L.hstu_hip_jagged_backward(C.byref(bwd), wsb.data_ptr(), nb.value, s) == 0, L.hstu_hip_last_error()

    def eager():
        step(torch.cuda.current_stream())
        torch.cuda.synchronize()
        return [t.clone() for t in (out, dq, dk, dv)]

    first = eager()   # everything the first call sets up lazily happens outside the capture
    if batch * heads > 64:
        # the same gradients from the plain fp32-FMA kernels (one stream), to the tolerance of two 16-bit implementations
        bwd.fwd.flags |= _capi.FLAG_FORCE_GENERIC
        ng = C.c_uint64(0)
        assert L.hstu_hip_jagged_backward_get_workspace_size(C.byref(bwd), C.byref(ng)) == 0
        wsg = torch.empty(max(ng.value, 16), dtype=torch.uint8, device="cuda")
        s0 = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        assert L.hstu_hip_jagged_backward(C.byref(bwd), wsg.data_ptr(), ng.value, s0) == 0, L.hstu_hip_last_error()
        torch.cuda.synchronize()
        for name, got, ref in zip(("dq", "dk", "dv"), first[1:], (dq, dk, dv)):
            scale = float(ref.float().abs().max())
            assert float((got.float() - ref.float()).abs().max()) <= 2e-2 * scale, name
        bwd.fwd.flags &= ~_capi.FLAG_FORCE_GENERIC
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(torch.cuda.current_stream())
    gen = torch.Generator(device="cuda").manual_seed(5)
    for replay in range(4):
        for t in (q, k, v, grad):   # new inputs in the captured buffers
            t.copy_((torch.randn(t.shape, generator=gen, device="cuda") * 0.5).to(t.dtype))
        want = eager()
        for t in (out, dq, dk, dv):
            t.fill_(float("nan"))
        q.float().square().sum().item()   # unrelated eager work and a synchronisation between the replays
        graph.replay()
        torch.cuda.synchronize()
        for name, got, ref in zip(("out", "dq", "dk", "dv"), (out, dq, dk, dv), want):
            assert torch.equal(got, ref), f"replay {replay}: {name} differs from the eager call"


def test_large_backward_from_two_host_threads_on_two_streams():
    """The streams and events that a large backward forks onto are shared by all callers of a device: two host threads that
    call at the same time on streams of their own must each get what they get alone, bit for bit."""
    import threading
    say("large backward from two host threads")
    L = _capi.lib()
    jobs = []
    for seed in (11, 12):
        cfg = W.jagged_config(seed, 32, 8, 128, 1200, 2048, torch.bfloat16, max_seq_len=2048)
        dev = W.to_device(cfg)
        q, k, v = dev["q"], dev["k"], dev["v"]
        grad = torch.randn_like(q)
        out, dq, dk, dv = (torch.empty_like(q) for _ in range(4))
        fwd, keep = _capi.make_params(q, k, v, out, seq_offset_q=dev["seq_offset"], max_seq_len_q=cfg["max_seq_len"], alpha=cfg["alpha"])
        bwd = _capi.make_backward_params(fwd, grad, dq, dk, dv, None)
        nb = C.c_uint64(0)
        assert L.hstu_hip_jagged_backward_get_workspace_size(C.byref(bwd), C.byref(nb)) == 0
        ws = torch.empty(max(nb.value, 16), dtype=torch.uint8, device="cuda")
        jobs.append(dict(bwd=bwd, nb=nb.value, ws=ws, outs=(dq, dk, dv), keep=(dev, keep, grad, out), stream=torch.cuda.Stream()))
    torch.cuda.synchronize()

    def run(job, times):
        s = C.c_void_p(job["stream"].cuda_stream)
        for _ in range(times):
            assert L.hstu_hip_jagged_backward(C.byref(job["bwd"]), job["ws"].data_ptr(), job["nb"], s) == 0, L.hstu_hip_last_error()

    want = []
    for job in jobs:   # alone
        run(job, 1)
        torch.cuda.synchronize()
        want.append([t.clone() for t in job["outs"]])
        for t in job["outs"]:
            t.fill_(float("nan"))
    torch.cuda.synchronize()
    threads = [threading.Thread(target=run, args=(job, 6)) for job in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    for job, ref in zip(jobs, want):
        for name, got, r in zip(("dq", "dk", "dv"), job["outs"], ref):
            assert torch.equal(got, r), name
