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


def _torch_op(q, k, v, off, max_len, alpha):
    return torch.ops.mxrec.hstu_jagged(q, k, v, None, None, 0, max_len, 0.0, off, None, None, 0, alpha)


def _capi_forward(q, k, v, off, max_len, alpha):
    """The same call through the C ABI with a workspace of its own (no list reuse)."""
    out = torch.empty_like(q)
    L = _capi.lib()
    fwd, keep = _capi.make_params(q, k, v, out, seq_offset_q=off, max_seq_len_q=max_len, alpha=alpha)
    n = C.c_uint64(0)
    assert L.hstu_hip_jagged_forward_get_workspace_size(C.byref(fwd), C.byref(n)) == 0
    ws = torch.empty(max(n.value, 16), dtype=torch.uint8, device="cuda")
    s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert L.hstu_hip_jagged_forward(C.byref(fwd), ws.data_ptr(), n.value, s) == 0, L.hstu_hip_last_error()
    torch.cuda.synchronize()
    return out


def _two_geometries(total, batch, seed):
    """Two offset vectors of `batch` sequences over the same number of rows."""
    g = torch.Generator().manual_seed(seed)
    offs = []
    for _ in range(2):
        cuts = torch.sort(torch.randperm(total - 1, generator=g)[: batch - 1] + 1).values
        offs.append(torch.cat([torch.zeros(1, dtype=torch.int64), cuts, torch.tensor([total])]).to(torch.int32))
    return offs


def test_torch_op_work_list_cache_under_stream_capture():
    """mxrec::hstu_jagged keeps the work list of its last call per (device, stream).  A capture must not record a call that
    reuses a list built outside the capture: the replay after the offsets tensor was rewritten in place has to follow the
    new offsets.  Two layers inside one capture still share one list, and a second graph captured afterwards on the same
    stream replays correctly by itself."""
    say("torch op: work-list cache under stream capture")
    total, batch, heads, d, max_len = 3000, 7, 4, 128, 3000
    off_a, off_b = (o.cuda() for o in _two_geometries(total, batch, 11))
    gen = torch.Generator(device="cuda").manual_seed(3)
    q, k, v = ((torch.randn(total, heads, d, generator=gen, device="cuda") * 0.5).to(torch.bfloat16) for _ in range(3))
    off = off_a.clone()
    alpha = d ** -0.5
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):   # eager warm-up on the capture stream: the second call reuses the first one's list
            warm = _torch_op(q, k, v, off, max_len, alpha)
    side.synchronize()
    assert torch.equal(warm, _capi_forward(q, k, v, off_a, max_len, alpha))
    g1 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g1, stream=side):
        out1 = _torch_op(q, k, v, off, max_len, alpha)          # builds its list inside the capture
        out2 = _torch_op(out1, k, v, off, max_len, alpha)       # second layer: reuses it
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g2, stream=side):
        out3 = _torch_op(q, k, v, off, max_len, alpha)
    for name, geometry in (("first", off_a), ("second", off_b), ("first again", off_a)):
        off.copy_(geometry)
        want1 = _capi_forward(q, k, v, geometry, max_len, alpha)
        want2 = _capi_forward(want1, k, v, geometry, max_len, alpha)
        for t in (out1, out2, out3):
            t.fill_(float("nan"))
        g1.replay()
        torch.cuda.synchronize()
        assert torch.equal(out1, want1), f"{name} geometry: layer 1 of the replay differs from the eager call"
        assert torch.equal(out2, want2), f"{name} geometry: layer 2 of the replay differs from the eager call"
        # an eager call on the capture stream in between must neither use nor disturb the graphs' lists
        with torch.cuda.stream(side):
            eager = _torch_op(q, k, v, off, max_len, alpha)
        side.synchronize()
        assert torch.equal(eager, want1), f"{name} geometry: eager call after the capture"
        g2.replay()
        torch.cuda.synchronize()
        assert torch.equal(out3, want1), f"{name} geometry: the second graph alone"


def test_torch_op_under_inference_mode():
    """Tensors created under torch.inference_mode() have no version counter: the op must run (without list reuse) and
    follow an in-place change of the offsets."""
    say("torch op under inference_mode")
    total, batch, heads, d, max_len = 2500, 5, 2, 128, 2500
    with torch.inference_mode():
        off_a, off_b = (o.cuda() for o in _two_geometries(total, batch, 5))
        gen = torch.Generator(device="cuda").manual_seed(9)
        q, k, v = ((torch.randn(total, heads, d, generator=gen, device="cuda") * 0.5).to(torch.bfloat16) for _ in range(3))
        off = off_a.clone()
        assert off.is_inference()
        got = [_torch_op(q, k, v, off, max_len, d ** -0.5) for _ in range(2)]
        off.copy_(off_b)
        got.append(_torch_op(q, k, v, off, max_len, d ** -0.5))
        torch.cuda.synchronize()
        want_a = _capi_forward(q, k, v, off_a, max_len, d ** -0.5)
        want_b = _capi_forward(q, k, v, off_b, max_len, d ** -0.5)
    assert torch.equal(got[0], want_a) and torch.equal(got[1], want_a) and torch.equal(got[2], want_b)
