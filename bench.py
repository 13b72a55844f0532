#!/usr/bin/env python3
"""Benchmark of the HSTU jagged attention forward on one MI355X.

A step is one call of the hot path (``hstu_hip_jagged_forward`` / ``hstu_hip_paged_forward`` through
the C ABI, on torch's current stream) over one synthetic batch whose inputs are already resident in
HBM.  Default workload: the headline configuration (B=64, h=4, d=128, L~U[256,1024], bf16, causal,
no bias, seed 0).  Prints ONE JSON line.

FLOPs follow the metric's definition: sum over sequences of 2*L^2*h*d (both GEMMs, halved by the
causal mask); for the paged workload 4*Lq*Lk*h*d (no causal halving: candidates see all history).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_FP8_TFLOPS = 5000.0    # MI355X dense fp8 MFMA
PEAK_HBM_GBS = 8000.0
# HBM-side bytes per launch from rocprofv3 FETCH_SIZE/WRITE_SIZE, each scaled by what the same counter reads for the
# plain 256 MiB copy of `--workload copy` (factors 2.000 and 1.000); see profiles/*.md
TRAFFIC_SOURCE = {"config2": "profiles/hstu_mfma_kernel_configs2-5.md", "config3": "profiles/hstu_mfma_kernel_configs2-5.md",
                  "config4": "profiles/hstu_mfma_kernel_configs2-5.md", "config5": "profiles/hstu_mfma_kernel_configs2-5.md",
                  "config2_bwd": "profiles/hstu_mfma_kernel_configs2-5.md", "config2_fp8": "profiles/hstu_mfma_fp8_kernel.md",
                  "ref_bias": "profiles/hstu_mfma_kernel_reference_benchmark_shape.md", "kv_append": "profiles/hstu_kv_append_kernel.md",
                  "rab_time": "profiles/hstu_rab_kernels.md", "rab_time_bwd": "profiles/hstu_rab_kernels.md", "rab_pos": "profiles/hstu_rab_kernels.md",
                  "nmd_fwd": "profiles/hstu_nmd_kernels.md", "nmd_bwd": "profiles/hstu_nmd_kernels.md",
                  "in_linear_silu": "profiles/hstu_in_linear_silu_kernel.md", "in_linear_silu_bwd": "profiles/hstu_in_linear_silu_backward_kernels.md",
                  "kv_append_fp8": "profiles/hstu_kv_append_fp8_kernels.md"}
MEASURED_TRAFFIC_BYTES = {"config2": 189.9e6, "config3": 112.5e6, "config4": 142.2e6, "config5": 205.6e6, "config2_bwd": 662.8e6, "config2_fp8": 116.5e6, "ref_bias": 1553.7e6, "kv_append": 351.9e6, "rab_time": 1443.4e6, "rab_time_bwd": 1589.7e6, "rab_pos": 297.7e6,
                          "nmd_fwd": 826.4e6, "nmd_bwd": 1380.0e6, "in_linear_silu": 1092.8e6, "in_linear_silu_bwd": 1458.3e6, "kv_append_fp8": 268.4e6}


def build_workload(name, torch, W):
    if name.endswith("_fp8"):
        # the same geometry with float8_e4m3fn q / k / v drawn like the reference's fp8 tests (uniform(-1, 1) rounded to
        # e4m3, test_hstu_jagged_forward.py:61-86) and fp16 output: 3 one-byte rows in, 1 two-byte row out
        c, op, flops, b, desc = build_workload(name[:-4], torch, W)
        g = torch.Generator().manual_seed(11)
        for x in "qkv":
            c[x] = (torch.rand(c[x].shape, generator=g) * 2 - 1).to(torch.float8_e4m3fn)
        c.setdefault("silu_scale", 1.0 / 64)   # keeps P above the subnormals of e4m3
        return c, op, flops, b * 5 // 8, desc.replace("bf16", "float8_e4m3fn in / fp16 out") + ", uniform(-1,1) data, silu_scale=" + f"{c['silu_scale']:.6f}"
    if name == "config2":
        c = W.config2()
        flops = W.headline_flops(c["lens"], 4, 128)
        t = sum(c["lens"])
        desc = "config2 headline: B=64 h=4 d=128 L~U[256,1024] bf16 causal no-bias seed0"
        return c, "jagged", flops, 4 * t * 4 * 128 * 2, desc
    if name == "config3":
        c = W.config3()
        flops = W.headline_flops(c["lens"], 8, 128)
        t = sum(c["lens"])
        return c, "jagged", flops, 4 * t * 8 * 128 * 2 + 8191 * 4, "config3 skewed: B=16 h=8 d=128 Zipf(1.2) L in [64,4096] bf16 rel-pos table"
    if name == "config4":
        c = W.config4()
        flops = W.headline_flops(c["lens"], 4, 64)
        t = sum(c["lens"])
        return c, "jagged", flops, 4 * t * 4 * 64 * 2 + t * 8, "config4 target-aware: B=128 h=4 d=64 hist~U[128,768]+64 targets bf16 time+pos tables"
    if name == "config5":
        c = W.config5()
        c["use_fp8"] = True
        flops = float(sum(4.0 * 256 * (h + 1) * 4 * 128 for h in c["hist"]))
        kv = sum(c["hist"]) * 2 * 4 * 128
        qo = 2 * 32 * 256 * 4 * 128 * 2
        return c, "paged", flops, kv + 2 * qo, "config5 paged fp8-KV: 32 users x 256 candidates, hist~U[1024,4096], 64-token pages"
    if name in ("config5_d32", "config5_d256"):
        # config 5's users and pages at the ends of the reference's head-dim sweep (paged rows through registers)
        d = int(name.split("_d")[1])
        c = W.paged_config(0, 32, 4, d, 1024, 4096, 256, 64, torch.bfloat16)
        c["kv_cache_fp8"], c["kv_scales"] = W.quantize_pages_fp8(c["kv_cache"])
        c["use_fp8"] = True
        flops = float(sum(4.0 * 256 * (h + 1) * 4 * d for h in c["hist"]))
        return c, "paged", flops, sum(c["hist"]) * 2 * 4 * d + 2 * 2 * 32 * 256 * 4 * d * 2, f"config5's geometry at head dim {d}: 32 users x 256 candidates, hist~U[1024,4096], fp8 KV in 64-token pages"
    if name in ("ref_bias_unmasked", "ref_nobias_unmasked"):
        # The reference's benchmark calls its op with window_size = (-1, -1): no mask at all, every row of a sequence sees
        # every column (test_forward_op_benchmark.py:201-205, 251-255; golden backend/pytorch_native_backend.py:74-81).
        # Here that is mask_type NONE of the jagged op: twice the causal FLOPs, the whole bias plane of a sequence.
        c = W.reference_benchmark_config(has_rab=name == "ref_bias_unmasked")
        c["mask_type"] = 2
        flops = 2.0 * W.headline_flops(c["lens"], 8, 128)
        t = sum(c["lens"])
        b = 4 * t * 8 * 128 * 2 + (sum(8 * l * l * 2 for l in c["lens"]) if "attn_bias" in c else 0)
        return c, "jagged", flops, b, ("reference benchmark shape as the reference runs it (test_forward_op_benchmark.py:246-259, window_size (-1, -1)): B=32 h=8 d=128 "
                                      "S=2048, every length 0.9 S, alpha=0.5, silu_scale=1/1024, bf16, no mask, " + ("dense attn_bias [B,h,S,S]" if "attn_bias" in c else "no bias"))
    if name in ("ref_bias", "ref_nobias", "ref_nobias_d32", "ref_nobias_d64", "ref_nobias_d256", "ref_nobias_d64v32", "ref_nobias_d128v48"):
        dims = name.split("_d")[1] if "_d" in name else "128"     # the ends and the middle of the reference's head-dim sweep,
        dim = int(dims.split("v")[0])                             # and the (dim_qk, dim_v) pairs of its user cases
        dim_v = int(dims.split("v")[1]) if "v" in dims else dim   # (test_forward_op_benchmark.py:192-193)
        c = W.reference_benchmark_config(has_rab=name == "ref_bias", dim=dim, dim_v=dim_v)
        flops = W.headline_flops(c["lens"], 8, (dim + dim_v) / 2)
        t = sum(c["lens"])
        b = 2 * t * 8 * (dim + dim_v) * 2
        # of the dense bias only the causal half is needed: sum over sequences and heads of L (L + 1) / 2 two-byte values
        if name == "ref_bias":
            b += sum(8 * l * (l + 1) // 2 * 2 for l in c["lens"])
        return c, "jagged", flops, b, ("reference benchmark shape (test_forward_op_benchmark.py:246-259): B=32 h=8 d=" + (str(dim) if dim_v == dim else f"({dim}, {dim_v})") + " S=2048, every length "
                                      "0.9 S, alpha=0.5, silu_scale=1/1024, bf16, causal, " + ("dense attn_bias [B,h,S,S]" if name == "ref_bias" else "no bias"))
    raise SystemExit(f"unknown workload {name}")


def bench_kind(workload):
    """Which leg of this file measures a workload (the names of several legs end alike)."""
    if workload in ("copy", "kv_append", "kv_append_fp8", "in_linear_silu", "in_linear_silu_bwd", "ref_grid", "ref_grid_bwd"):
        return workload
    if workload in ("rab_time", "rab_time_bwd", "rab_pos"):
        return "bias"
    if workload in ("nmd_fwd", "nmd_bwd"):
        return "nmd"
    if workload == "config2_bwd" or (workload.startswith("ref_") and workload.endswith("_bwd")):
        return "attention_backward"
    return "attention_forward"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=1000)
    ap.add_argument("--workload", default="config2", choices=["config2", "config3", "config4", "config5", "config5_d32", "config5_d256", "ref_grid", "ref_grid_bwd", "ref_bias", "ref_nobias", "ref_bias_unmasked", "ref_nobias_unmasked", "ref_nobias_d32", "ref_nobias_d64", "ref_nobias_d256", "ref_nobias_d64v32", "ref_nobias_d128v48", "config2_fp8", "ref_nobias_fp8", "config2_bwd", "ref_bias_bwd", "ref_nobias_bwd", "ref_nobias_d32_bwd", "ref_nobias_d64_bwd", "ref_nobias_d256_bwd", "kv_append", "kv_append_fp8", "rab_time", "rab_time_bwd", "rab_pos", "nmd_fwd", "nmd_bwd", "in_linear_silu", "in_linear_silu_bwd", "copy"],
                    help="'copy' runs a plain 256 MiB device copy: the known-size kernel the FETCH_SIZE/WRITE_SIZE counters are scaled by")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--timeline", action="store_true",
                    help="forward workloads: instead of timing the call, run it on the diagnostics flavour of the library "
                         "(lib/libhstu_hip_timeline.so, built by recsdk_amd/_build.py) and print where the workgroups of the main "
                         "kernel spend their time, from the stamps they leave")
    ap.add_argument("--settle-ms", type=float, default=80.0,
                    help="untimed calls before the warm-up until the GPU has been busy this long: its clocks need about 50 ms of load to "
                         "settle (reported as clock_settle; 0 switches it off)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs on ONE GPU: (sequence, head) work units are independent, so several GPUs "
                         "would each take a share of the sequences with no exchange between them. Run with --gpus 1.")
    import torch
    import recsdk_amd  # noqa: F401  (fails loudly if the HIP libraries are missing)
    from recsdk_amd import _capi, workloads as W

    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    kind = bench_kind(args.workload)
    if kind == "copy":
        return copy_calibration(args, torch)
    if kind in ("ref_grid", "ref_grid_bwd"):
        return reference_grid(args, torch, _capi, backward=kind == "ref_grid_bwd")
    if kind == "attention_backward":
        return backward_bench(args, torch, W, _capi)
    if kind == "kv_append":
        return kv_append_bench(args, torch, W)
    if kind == "kv_append_fp8":
        return kv_append_fp8_bench(args, torch, W)
    if kind == "bias":
        return bias_bench(args, torch)
    if kind == "nmd":
        return nmd_bench(args, torch)
    if kind == "in_linear_silu":
        return in_linear_silu_bench(args, torch)
    if kind == "in_linear_silu_bwd":
        return in_linear_silu_bwd_bench(args, torch)
    cfg, op, flops, alg_bytes, desc = build_workload(args.workload, torch, W)
    dev = W.to_device(cfg)
    q, k, v = dev["q"], dev["k"], dev["v"]
    out = torch.empty(q.shape, dtype=_capi.out_dtype(q.dtype), device=q.device)
    fp8 = q.dtype == torch.float8_e4m3fn
    peak = PEAK_FP8_TFLOPS if fp8 else PEAK_BF16_TFLOPS
    kw = dict(seq_offset_q=dev["seq_offset"], seq_offset_k=dev.get("seq_offset_k"), max_seq_len_q=cfg["max_seq_len"],
              max_seq_len_k=cfg.get("max_seq_len_k"), mask_type=cfg.get("mask_type", 0), alpha=cfg["alpha"], num_target=dev.get("num_target"),
              attn_bias=dev.get("attn_bias"), silu_scale=cfg.get("silu_scale", 0.0),
              target_group_size=cfg.get("target_group_size", 0), pos_table=dev.get("pos_table"),
              ts_table=dev.get("ts_table"), timestamps=dev.get("timestamps"))
    if cfg.get("ts_table") is not None:
        kw["ts_bounds"] = recsdk_amd.time_bucket_bounds(128, 0.301).cuda()
    if op == "paged":
        kw.update(kv_cache=dev["kv_cache_fp8"], kv_scales=dev["kv_scales"], page_offsets=dev["page_offsets"],
                  page_ids=dev["page_ids"], last_page_len=dev["last_page_len"])
    params, keep = _capi.make_params(q, k, v, out, **kw)
    kernel = _capi.describe_kernel(params)
    import ctypes as C
    L = _capi.lib()
    fn = getattr(L, f"hstu_hip_{op}_forward")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    pref = C.byref(params)
    # two-phase call like the reference's aclnn entry points: size query once, workspace allocated outside the timed region
    nws = C.c_uint64(0)
    if getattr(L, f"hstu_hip_{op}_forward_get_workspace_size")(pref, C.byref(nws)) != 0:
        raise RuntimeError(L.hstu_hip_last_error().decode())
    ws = torch.empty(max(int(nws.value), 4), dtype=torch.uint8, device="cuda")
    ws_ptr = C.c_void_p(ws.data_ptr())

    def step():
        rc = fn(pref, ws_ptr, nws.value, stream)
        if rc != 0:
            raise RuntimeError(L.hstu_hip_last_error().decode())

    if args.timeline:
        return item_timeline(args, torch, _capi, op, params, ws, nws.value, desc, kernel)
    settle = settle_clocks(step, args.settle_ms, torch)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    kern_ms = e0.elapsed_time(e1) / args.steps        # HIP events on the launch stream: average launch duration
    tflops = flops / (ms_per_step * 1e-3) / 1e12
    kern_tflops = flops / (kern_ms * 1e-3) / 1e12

    result = {
        "metric": "hstu_jagged_attn_fwd_tflops", "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "fp8_e4m3" if fp8 else "bf16", "data": "synthetic",
        "us_per_call": round(ms_per_step * 1e3, 2), ("pct_fp8_mfma_peak" if fp8 else "pct_bf16_mfma_peak"): round(100 * tflops / peak, 2),
        "config": {"workload": desc, "kernel": kernel, "flops_per_call": flops, "algorithmic_bytes_per_call": alg_bytes,
                   "entry": f"hstu_hip_{op}_forward (C ABI)", "l2_flushed_between_calls": False},
        "roofline": {"bound": "mfma", "achieved": round(kern_tflops, 2), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(kern_tflops / peak, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
                     "traffic_source": TRAFFIC_SOURCE.get(args.workload),
                     "kernel_us": round(kern_ms * 1e3, 2),
                     "hbm_algorithmic_gbs": round(alg_bytes / (kern_ms * 1e-3) / 1e9, 1),
                     "hbm_frac": round(alg_bytes / (kern_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)},
    }
    # the other layers of a model run on the same batch geometry: calls that keep the work list of the first one
    # (HSTU_FLAG_REUSE_WORKSPACE) skip the schedule kernel.  Reported beside the headline, never as `value`.
    if kernel.startswith("mfma_"):
        params.flags |= _capi.FLAG_REUSE_WORKSPACE
        step()
        torch.cuda.synchronize()
        r0, r1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        r0.record()
        for _ in range(args.steps):
            step()
        r1.record()
        torch.cuda.synchronize()
        reuse_ms = r0.elapsed_time(r1) / args.steps
        result["reuse_work_list"] = {"kernel_us": round(reuse_ms * 1e3, 2), "tflops": round(flops / (reuse_ms * 1e-3) / 1e12, 2)}
        params.flags &= ~_capi.FLAG_REUSE_WORKSPACE
    result["clock_settle"] = settle
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(cfg, op, flops, torch, args.workload, W)
    print(json.dumps(result), flush=True)


def item_timeline(args, torch, _capi, op, params, ws, ws_bytes, desc, kernel):
    """Per-workgroup timeline of the main forward kernel.  The diagnostics library is the product's sources with the
    kernel compiled under -DHSTU_ITEM_TIMING: thread 0 of every workgroup stamps (constant 100 MHz clock) its start, the
    moment it knows its item, its first K/V tile in LDS, the end of its last K loop and its end.  One JSON line per
    flavour of the call: as the C ABI runs it, and with the work list reused (HSTU_FLAG_REUSE_WORKSPACE)."""
    import ctypes as C
    import numpy as np
    from recsdk_amd import _build
    path = _build.timeline_lib_path()
    if not os.path.exists(path):
        raise SystemExit(f"{path} is missing: build it with `python recsdk_amd/_build.py timeline`")
    # a second copy of the library in this process: its own symbols first, none of them exported to later loads
    TL = C.CDLL(path, mode=os.RTLD_LOCAL | os.RTLD_DEEPBIND)
    fn = getattr(TL, f"hstu_hip_{op}_forward")
    fn.argtypes = [C.POINTER(_capi.HstuFwdParams), C.c_void_p, C.c_uint64, C.c_void_p]
    TL.hstu_hip_timeline_read.argtypes = [C.c_void_p, C.c_size_t]
    TL.hstu_hip_last_error.restype = C.c_char_p
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    for reuse in (False, True):
        if reuse:
            params.flags |= _capi.FLAG_REUSE_WORKSPACE

        def step():
            if fn(C.byref(params), C.c_void_p(ws.data_ptr()), ws_bytes, stream) != 0:
                raise RuntimeError(TL.hstu_hip_last_error().decode())
        if not reuse:
            step()
        settle_clocks(step, args.settle_ms, torch)
        for _ in range(max(args.warmup, 50)):
            step()
        torch.cuda.synchronize()
        buf = np.zeros(8 * 32768, dtype=np.uint32)
        if TL.hstu_hip_timeline_read(buf.ctypes.data_as(C.c_void_p), C.c_size_t(buf.nbytes)) != 0:
            raise RuntimeError("reading the stamps failed")
        r = buf.reshape(-1, 8)
        r = r[r[:, 0] != 0]
        us = lambda ticks: ticks / 100.0
        t0 = r[:, 0].astype(np.int64)
        t0 -= t0.min()
        pro, dur, ntk = r[:, 1].astype(np.int64), r[:, 2].astype(np.int64), r[:, 4].astype(np.int64)
        rec, loop = r[:, 6].astype(np.int64), r[:, 7].astype(np.int64)
        act = r[:, 5] != 0xffffffff
        end = t0 + dur
        span = int(end.max())
        T = span + 1
        resident, inloop, rate = np.zeros(T + 1), np.zeros(T + 1), np.zeros(T + 1)
        for s_, p_, l_, n_, d_ in zip(t0[act], pro[act], loop[act], ntk[act], dur[act]):
            resident[s_:s_ + d_] += 1
            if l_ > p_:
                inloop[s_ + p_:s_ + l_] += 1
                rate[s_ + p_:s_ + l_] += n_ / (l_ - p_)
        slots = int(resident.max())
        total = slots * span
        first = act & (t0 < 100)          # resident from the start: the first round of workgroups
        later = act & ~first
        st, en = np.sort(t0[act]), np.sort(end[act])
        lag = st[slots:] - en[:len(st) - slots] if len(st) > slots else np.zeros(1)
        step_t = 400
        longest = np.argsort(-dur * act)[:20]
        last = np.argsort(-end * act)[:20]
        row = lambda i: {"start_us": us(t0[i]), "k_tiles": int(ntk[i]), "to_first_tile_us": us(pro[i]), "k_loops_us": us(loop[i] - pro[i]),
                         "after_loops_us": us(dur[i] - loop[i]), "end_us": us(end[i])}
        out = {
            "metric": "hstu_item_timeline", "workload": desc, "kernel": kernel, "work_list_reused": reuse, "n_gpus": 1,
            "unit": "us (10 ns ticks of the constant clock, thread 0 of every workgroup)",
            "kernel_span_us": us(span), "workgroups": int(len(r)), "items": int(act.sum()), "slots": slots, "k_tiles": int(ntk[act].sum()),
            "slot_time_share": {"to_record": round(float(rec[act].sum()) / total, 3), "record_to_first_tile": round(float((pro - rec)[act].sum()) / total, 3),
                                "k_loops": round(float((loop - pro)[act].sum()) / total, 3), "after_loops": round(float((dur - loop)[act].sum()) / total, 3),
                                "empty": round(float(total - dur[act].sum()) / total, 3)},
            "first_round": {"items": int(first.sum()), "to_record_us": round(us(rec[first].mean()), 2), "to_first_tile_us": round(us(pro[first].mean()), 2),
                            "end_us_min_median_max": [us(x) for x in (end[first].min(), int(np.median(end[first])), end[first].max())] if first.any() else None},
            "later_items": {"items": int(later.sum()), "to_record_us": round(us(rec[later].mean()), 2) if later.any() else None,
                            "to_first_tile_us": round(us(pro[later].mean()), 2) if later.any() else None,
                            "start_us_min_max": [us(t0[later].min()), us(t0[later].max())] if later.any() else None,
                            "k_tiles_mean": round(float(ntk[later].mean()), 1) if later.any() else None},
            "us_per_k_tile_in_loop": round(us(float((loop - pro)[act].sum())) / max(int(ntk[act].sum()), 1), 3),
            "after_loops_us_mean": round(us(float((dur - loop)[act].mean())), 2),
            "slot_refill_lag_us_mean_p90": [round(us(float(lag.mean())), 2), round(us(float(np.percentile(lag, 90))), 2)],
            "every_4us": [{"t_us": us(i), "resident": int(resident[i:i + step_t].mean()), "in_k_loop": int(inloop[i:i + step_t].mean()),
                           "k_tiles_per_us": int(rate[i:i + step_t].mean() * 100)} for i in range(0, T, step_t)],
            "longest_items": [row(i) for i in longest],
            "last_ending_items": [row(i) for i in last],
        }
        print(json.dumps(out), flush=True)
    params.flags &= ~_capi.FLAG_REUSE_WORKSPACE


def backward_bench(args, torch, W, _capi):
    """The jagged backward (dQ, dK, dV) on the headline configuration: five GEMM-shaped products of L^2 * h * d
    multiply-adds each under the causal mask (S, dO V^T, dV, dK, dQ) = 2.5 x the forward's FLOPs."""
    import ctypes as C
    with_bias = args.workload == "ref_bias_bwd"
    ref_shape = args.workload.startswith("ref_")
    dim = int(args.workload.split("_d")[1].split("_")[0]) if "_d" in args.workload else 128
    # ref_*_bwd: the reference's benchmark shape (test_backward_op_benchmark.py: B=32 h=8 S=2048, lengths 0.9 S, head dims
    # 32 .. 256); ref_bias_bwd with a dense attn_bias, whose gradient (the same 2.1 GB again) the call also produces
    cfg = W.reference_benchmark_config(has_rab=with_bias, dim=dim) if ref_shape else W.config2()
    heads = 8 if ref_shape else 4
    dev = W.to_device(cfg)
    q, k, v = dev["q"], dev["k"], dev["v"]
    bias = dev.get("attn_bias")
    g = torch.Generator(device="cuda").manual_seed(1)
    grad = torch.randn(q.shape, generator=g, device="cuda", dtype=torch.float32).to(q.dtype)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dbias = None if bias is None else torch.empty_like(bias)
    fwd, keep = _capi.make_params(q, k, v, q, seq_offset_q=dev["seq_offset"], max_seq_len_q=cfg["max_seq_len"], alpha=cfg["alpha"],
                                  attn_bias=bias, silu_scale=cfg.get("silu_scale", 0.0))
    fwd.out = None
    p = _capi.make_backward_params(fwd, grad, dq, dk, dv, dbias)
    kernel = _capi.describe_backward_kernel(p)
    L = _capi.lib()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    flops = 2.5 * W.headline_flops(cfg["lens"], heads, dim)

    nws = C.c_uint64(0)
    if L.hstu_hip_jagged_backward_get_workspace_size(C.byref(p), C.byref(nws)) != 0:
        raise RuntimeError(L.hstu_hip_last_error().decode())
    ws = torch.empty(max(int(nws.value), 16), dtype=torch.uint8, device="cuda")
    ws_ptr = C.c_void_p(ws.data_ptr())

    def step():
        if L.hstu_hip_jagged_backward(C.byref(p), ws_ptr, nws.value, stream) != 0:
            raise RuntimeError(L.hstu_hip_last_error().decode())

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms = wall * 1e3 / args.steps
    kern_ms = e0.elapsed_time(e1) / args.steps
    tflops = flops / (ms * 1e-3) / 1e12
    t = sum(cfg["lens"])
    alg_bytes = 7 * t * heads * dim * 2   # Q, K, V, dO read once; dQ, dK, dV written once
    if with_bias:
        # the causal half of the bias is read by each of the three kernels' producers once (counted once), the whole
        # gradient buffer is zero-filled and its causal half written again
        half = sum(heads * l * (l + 1) // 2 * 2 for l in cfg["lens"])
        alg_bytes += half + bias.numel() * 2 + half
    desc = ("reference benchmark shape, backward with dense attn_bias and its gradient: B=32 h=8 d=128 S=2048, every length 0.9 S, bf16, causal"
            if with_bias else (f"reference benchmark shape, backward: B=32 h=8 d={dim} S=2048, every length 0.9 S, bf16, causal, no bias" if ref_shape
                               else "config2 shapes, backward: B=64 h=4 d=128 L~U[256,1024] bf16 causal no-bias seed0"))
    print(json.dumps({
        "metric": "hstu_jagged_attn_bwd_tflops", "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", "us_per_call": round(ms * 1e3, 2),
        "pct_bf16_mfma_peak": round(100 * tflops / PEAK_BF16_TFLOPS, 2),
        "config": {"workload": desc, "kernel": kernel,
                   "flops_per_call": flops, "algorithmic_bytes_per_call": alg_bytes, "entry": "hstu_hip_jagged_backward (C ABI)"},
        "roofline": {"bound": "mfma", "achieved": round(flops / (kern_ms * 1e-3) / 1e12, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(flops / (kern_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
                     "traffic_source": TRAFFIC_SOURCE.get(args.workload),
                     "kernel_us": round(kern_ms * 1e3, 2)},
    }), flush=True)


def kv_append_bench(args, torch, W):
    """The write side of the paged cache at the shape of config 5's history: 32 users, 1024-4096 new tokens each, 4 heads
    x 128, bf16, 64-token pages in shuffled order.  Every K and V row is read once and written once."""
    from recsdk_amd import kvcache
    cfg = W.kv_append_config(0, users=32, heads=4, dim=128, prev_lo=0, prev_hi=0, new_lo=1024, new_hi=4096, page_size=64)
    dev = W.to_device(cfg)
    n = cfg["nnz"]
    bi = torch.empty(n, dtype=torch.int32, device="cuda")
    pos = torch.empty_like(bi)
    kc, vc = dev["kv_cache"].unbind(1)

    def step():
        kvcache.get_paged_batch_indices_positions(dev["append_indptr"], dev["seq_lens"], bi, pos)
        kvcache.append_kvcache(dev["append_key"], dev["append_value"], bi, pos, dev["offsets"], dev["nnz_dev"], n, kc, vc,
                               dev["kv_indices"], dev["kv_indptr"], dev["kv_last_page_len"], 0)

    def append_only():
        kvcache.append_kvcache(dev["append_key"], dev["append_value"], bi, pos, dev["offsets"], dev["nnz_dev"], n, kc, vc,
                               dev["kv_indices"], dev["kv_indptr"], dev["kv_last_page_len"], 0)

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / args.steps, e0.elapsed_time(e1) / args.steps

    ms, _ = timed(step)                 # the whole job: positions + append
    _, kern_ms = timed(append_only)     # the dominant kernel alone, for the roofline
    row_bytes = 4 * 128 * 2
    alg_bytes = n * row_bytes * 4 + n * 4 * 4      # K, V rows read and written; batch_indices / positions written and read
    kern_bytes = n * row_bytes * 4 + n * 2 * 4     # the append kernel: rows, and its two index arrays read
    out = {
        "metric": "paged_kv_append_gbps", "value": round(alg_bytes / (ms * 1e-3) / 1e9, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u16", "data": "synthetic", "us_per_call": round(ms * 1e3, 2),
        "config": {"workload": f"append of {n} new tokens (32 users x U[1024,4096]) x 4 heads x 128, bf16, 64-token pages, seed 0",
                   "algorithmic_bytes_per_call": alg_bytes, "entry": "hstu_hip_kv_token_positions + hstu_hip_kv_append (C ABI)"},
        "roofline": {"bound": "hbm", "kernel": "hstu_kv_append_kernel", "achieved": round(kern_bytes / (kern_ms * 1e-3) / 1e9, 1),
                     "peak": 8000.0, "unit": "GB/s", "frac": round(kern_bytes / (kern_ms * 1e-3) / 1e9 / 8000.0, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES["kv_append"], "kernel_us": round(kern_ms * 1e3, 2),
                     "algorithmic_bytes_per_launch": kern_bytes},
    }
    if not args.no_cpu_baseline:
        from oracle import kvcache_oracle as KO
        t = cfg["kv_cache"].view(torch.int16).numpy()
        k16, v16 = cfg["append_key"].view(torch.int16).numpy(), cfg["append_value"].view(torch.int16).numpy()
        t0 = time.perf_counter()
        b_, p_ = KO.paged_batch_indices_positions(cfg["append_indptr"].numpy(), cfg["seq_lens"].numpy())
        KO.append_paged_kvcache(t[:, 0], t[:, 1], k16, v16, b_, p_, cfg["offsets"].numpy(), n, cfg["kv_indices"].numpy(),
                                cfg["kv_indptr"].numpy())
        dt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": round(alg_bytes / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"the whole append once, token loop in numpy, {dt:.2f} s"}
    print(json.dumps(out), flush=True)


def kv_append_fp8_bench(args, torch, W):
    """The fp8 write side at the kv_append workload's shape: the prefill of config 5's history (32 users, 1024-4096 tokens,
    4 heads x 128, bf16 rows) into an e4m3 table with per-(page, K|V, head) scales.  Algorithmic bytes: every row read
    once (2 bytes per element) and written once (1 byte); the rows of a page stay in registers between absmax and quantisation."""
    from recsdk_amd import kvcache
    cfg = W.kv_append_config(0, users=32, heads=4, dim=128, prev_lo=0, prev_hi=0, new_lo=1024, new_hi=4096, page_size=64)
    dev = W.to_device(cfg)
    n = cfg["nnz"]
    bi = torch.empty(n, dtype=torch.int32, device="cuda")
    pos = torch.empty_like(bi)
    kvcache.get_paged_batch_indices_positions(dev["append_indptr"], dev["seq_lens"], bi, pos)
    pages = cfg["kv_cache"].shape[0]
    cache8 = torch.zeros(pages, 2, 64, 4, 128, dtype=torch.uint8, device="cuda")
    scales = torch.ones(pages, 2, 4, device="cuda")
    ws = torch.empty(pages * 9 * 4, dtype=torch.uint8, device="cuda")

    def fn():
        kvcache.append_kvcache_fp8(dev["append_key"], dev["append_value"], bi, pos, dev["offsets"], dev["nnz_dev"], n, cache8, scales,
                                   dev["kv_indices"], dev["kv_indptr"], workspace=ws)
    for _ in range(args.warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    kern_ms = e0.elapsed_time(e1) / args.steps
    elems = n * 2 * 4 * 128
    alg = elems * 3 + pages * 8 * 4 + n * 2 * 4
    out = {
        "metric": "paged_kv_append_fp8_gbps", "value": round(alg / (ms * 1e-3) / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic", "us_per_call": round(ms * 1e3, 2),
        "config": {"workload": f"fp8 append of {n} new tokens (32 users x U[1024,4096]) x 4 heads x 128 from bf16, 64-token pages, seed 0",
                   "algorithmic_bytes_per_call": alg, "entry": "hstu_hip_kv_append_fp8 (C ABI): reset, runs, page kernels (+ two kernels for scattered pages that find nothing here)"},
        "roofline": {"bound": "hbm", "kernel": "hstu_kv_fp8_page_kernel (+ 4 small kernels; all inside the events)",
                     "achieved": round(alg / (kern_ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(alg / (kern_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
                     "kernel_us": round(kern_ms * 1e3, 2)},
    }
    if not args.no_cpu_baseline:
        from oracle import kvcache_oracle as KO
        users = 2
        last = int(cfg["append_indptr"][users])
        c8, sc = torch.zeros(pages, 2, 64, 4, 128, dtype=torch.uint8), torch.ones(pages, 2, 4)
        b_, p_ = KO.paged_batch_indices_positions(cfg["append_indptr"][: users + 1].numpy(), cfg["seq_lens"][:users].numpy())
        t0 = time.perf_counter()
        KO.append_paged_kvcache_fp8(c8, sc, cfg["append_key"], cfg["append_value"], b_, p_, cfg["offsets"].numpy(), last, cfg["kv_indices"].numpy(),
                                    cfg["kv_indptr"].numpy())
        dt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": round(alg * last / n / dt / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"the first {users} users ({last} tokens) once, page loop in torch, {dt:.2f} s"}
    print(json.dumps(out), flush=True)


def bias_bench(args, torch):
    """The standalone bias producers at the reference's evaluation shape (test_relative_attn_bias.py:106-113): 8 layers,
    train_len 2000 + 600 candidates -> s = 2300, 4 users, fp16 tables, int32 timestamps.  HBM-bound: the (2s)^2 outputs
    (the gradient input for the backward) dominate the bytes."""
    n, bs, train, cand = 8, 4, 2000, 600
    s = train + cand // 2
    g = torch.Generator().manual_seed(0)
    lens = torch.randint(0, train, (bs,), generator=g).tolist()
    ts = torch.zeros(bs, s)
    for i, v in enumerate(lens):
        ts[i, :v] = torch.arange(1, v + 1)
    ts[:, -(cand // 2):] = train + 1
    ts = ts.to(torch.int32)
    w = (torch.arange(129, dtype=torch.float32).repeat(n).reshape(n, 129) + torch.randn(n, 129, generator=g)).half()
    m = torch.ops.mxrec
    esz = 2
    if args.workload == "rab_time":
        tsd, wd = ts.cuda(), w.cuda()
        fn = lambda: m.relative_attn_bias_time_with_index(tsd, wd, 0.301)
        alg = n * bs * 4 * s * s * esz + bs * s * s * 4 + bs * s * 4
        kernel, desc = "hstu_rab_time_lines_kernel", "rab_time_out [8,4,4600,4600] fp16 + bucket ids [4,2300,2300] int32 written"
        cpu = lambda: BO.rab_time(ts, w, 0.301)
        cpu_bytes = alg
        sample = "the whole call once (oracle in torch)"
    elif args.workload == "rab_time_bwd":
        grad = (torch.randn(n, bs, 2 * s, 2 * s, generator=g, dtype=torch.float16) * 1e-2).cuda()
        # the bucket ids the backward consumes come from this library's forward
        idd = m.relative_attn_bias_time_with_index(ts.cuda(), w.cuda(), 0.301)[1].to(torch.int32)
        ids = idd.cpu()
        fn = lambda: m.relative_attn_bias_time_backward(grad, idd, 129)
        alg = n * bs * 4 * s * s * esz + bs * s * s * 4
        kernel, desc = "hstu_rab_time_bwd_kernel", "grad [8,4,4600,4600] fp16 and ids [4,2300,2300] int32 read (algorithmic: once each)"
        gc = grad[:, :1].cpu()
        cpu = lambda: BO.rab_time_backward(gc, ids[:1], 129)
        cpu_bytes = alg // bs
        sample = "one of the four users once (oracle in torch, fp64 sums)"
    else:
        s2 = 2 * s
        rel = torch.randn(s2, s2, generator=g).half()
        idx = torch.arange(s).repeat(s).view(s, s).unsqueeze(-1).repeat(1, 2, 2).reshape(s2, s2)
        ident = (idx.t() == idx).half().contiguous()
        reld, identd = rel.cuda(), ident.cuda()
        fn = lambda: m.relative_attn_bias_pos(reld, identd, lens)
        alg = bs * s2 * s2 * esz + 2 * s2 * s2 * esz
        kernel, desc = "hstu_rab_pos_kernel", "out [4,4600,4600] fp16 written, the two [4600,4600] tables read"
        cpu = lambda: [BO.rab_pos(rel, ident, lens) for _ in range(20)]
        cpu_bytes = 20 * alg
        sample = "the whole call 20 times (oracle in torch)"

    for _ in range(args.warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    kern_ms = e0.elapsed_time(e1) / args.steps
    out = {
        "metric": f"{args.workload}_gbps", "value": round(alg / (ms * 1e-3) / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic", "us_per_call": round(ms * 1e3, 2),
        "config": {"workload": f"{args.workload}: 8 layers, 4 users, s = 2300 (train 2000 + 600 candidates), fp16, seed 0; {desc}",
                   "algorithmic_bytes_per_call": alg, "entry": f"torch.ops.mxrec.* -> {kernel} (C ABI in include/hstu_bias.h)"},
        "roofline": {"bound": "hbm", "kernel": kernel, "achieved": round(alg / (kern_ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(alg / (kern_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
                     "kernel_us": round(kern_ms * 1e3, 2)},
    }
    if not args.no_cpu_baseline:
        from oracle import bias_oracle as BO
        t0 = time.perf_counter()
        cpu()
        dt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": round(cpu_bytes / dt / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"{sample}, {dt:.2f} s"}
    print(json.dumps(out), flush=True)


def nmd_bench(args, torch):
    """norm_multiply_dropout at the shape of the reference's sample (README of the op: 262144 x 512, bf16, eps 1e-5), with
    dropout 0.3 so that the mask is written and read.  HBM-bound: forward reads x, u and writes y (+ mask, mean, var);
    backward reads d_out, x, u (+ mask, mean, var) and writes d_x, d_u."""
    rows, cols, ratio, eps = 262144, 512, 0.3, 1e-5
    g = torch.Generator().manual_seed(321)
    mk = lambda *s: (torch.rand(*s, generator=g) * 2 - 1).to(torch.bfloat16)
    x, u, w, b, dy = mk(rows, cols), mk(rows, cols), mk(cols), mk(cols), mk(rows, cols)
    xd, ud, wd, bd, dyd = (t.cuda() for t in (x, u, w, b, dy))
    m = torch.ops.mxrec
    small = rows * 8 + rows * cols // 8      # mean, var (fp32) and the mask bits
    if args.workload == "nmd_fwd":
        fn = lambda: m.norm_multiply_dropout_forward(xd, ud, wd, bd, eps, ratio)
        alg = 3 * rows * cols * 2 + small
        kernel = "hstu_nmd_fwd_kernel"
        n_cpu = rows
        cpu = lambda: LO.nmd_forward(x[:n_cpu], u[:n_cpu], w, b, eps, ratio, torch.ones(n_cpu, cols, dtype=torch.bool))
        cpu_bytes = alg * n_cpu // rows
    else:
        _, mean, var, mask = m.norm_multiply_dropout_forward(xd, ud, wd, bd, eps, ratio)
        fn = lambda: m.norm_multiply_dropout_backward(dyd, xd, ud, wd, bd, mean, var, mask, eps, ratio)
        alg = 5 * rows * cols * 2 + small
        kernel = "hstu_nmd_bwd_kernel"
        n_cpu = rows // 2
        mc, vc = mean[:n_cpu].cpu(), var[:n_cpu].cpu()
        cpu = lambda: LO.nmd_backward(dy[:n_cpu], x[:n_cpu], u[:n_cpu], w, b, mc, vc, eps, ratio, torch.ones(n_cpu, cols, dtype=torch.bool))
        cpu_bytes = alg * n_cpu // rows
    for _ in range(args.warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    kern_ms = e0.elapsed_time(e1) / args.steps
    out = {
        "metric": f"norm_multiply_dropout_{args.workload[4:]}_gbps", "value": round(alg / (ms * 1e-3) / 1e9, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", "us_per_call": round(ms * 1e3, 2),
        "config": {"workload": f"{args.workload}: x, u [262144, 512] bf16, eps 1e-5, dropout 0.3, seed 321", "algorithmic_bytes_per_call": alg,
                   "entry": f"torch.ops.mxrec.norm_multiply_dropout_{'forward' if args.workload == 'nmd_fwd' else 'backward'} -> {kernel} (C ABI in include/hstu_layer.h)"},
        "roofline": {"bound": "hbm", "kernel": kernel, "achieved": round(alg / (kern_ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(alg / (kern_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
                     "kernel_us": round(kern_ms * 1e3, 2)},
    }
    if not args.no_cpu_baseline:
        from oracle import layer_oracle as LO
        t0 = time.perf_counter()
        cpu()
        dt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": round(cpu_bytes / dt / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"the first {n_cpu} rows once (oracle in torch, fp64), {dt:.2f} s"}
    print(json.dumps(out), flush=True)


def in_linear_silu_bench(args, torch):
    """The input projection at the largest shape of the reference's tests (test_in_linear_silu.py:101-109): m = 16384,
    n = 16384, k = 64, bf16, equal splits.  4 bytes written per output element against 2 k = 128 FLOPs: bounded by the HBM
    writes of linear_output and the four split outputs."""
    m_, n, k = 16384, 16384, 64
    g = torch.Generator().manual_seed(13)
    x = torch.randint(-100, 101, (m_, k), generator=g).to(torch.bfloat16)
    w = ((torch.rand(n, k, generator=g) * 2 - 1) * (6.0 / (n + k)) ** 0.5).to(torch.bfloat16)
    bias = torch.ones(n)
    sp = [n // 4] * 4
    xd, wd, bd = x.cuda(), w.cuda(), bias.cuda()
    fn = lambda: torch.ops.mxrec.distance_in_linear_silu(xd, wd, bd, sp)
    for _ in range(args.warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    kern_ms = e0.elapsed_time(e1) / args.steps
    alg = 2 * m_ * n * 2 + m_ * k * 2 + n * k * 2 + n * 4
    flops = 2.0 * m_ * n * k
    out = {
        "metric": "in_linear_silu_gbps", "value": round(alg / (ms * 1e-3) / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", "us_per_call": round(ms * 1e3, 2), "tflops": round(flops / (ms * 1e-3) / 1e12, 1),
        "config": {"workload": "in_linear_silu: x [16384, 64], W [16384, 64] bf16, bias fp32, splits 4 x 4096, seed 13",
                   "algorithmic_bytes_per_call": alg, "flops_per_call": flops,
                   "entry": "torch.ops.mxrec.distance_in_linear_silu -> hstu_in_linear_silu_kernel (C ABI in include/hstu_layer.h)"},
        "roofline": {"bound": "hbm", "kernel": "hstu_in_linear_silu_kernel", "achieved": round(alg / (kern_ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(alg / (kern_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
                     "kernel_us": round(kern_ms * 1e3, 2)},
    }
    if not args.no_cpu_baseline:
        from oracle import layer_oracle as LO
        rows = 4096
        t0 = time.perf_counter()
        LO.in_linear_silu(x[:rows], w, bias, sp)
        dt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": round(alg * rows / m_ / dt / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"the first {rows} rows once (oracle in torch, fp64), {dt:.2f} s"}
    print(json.dumps(out), flush=True)


def in_linear_silu_bwd_bench(args, torch):
    """Backward of the input projection at the forward workload's shape: m = n = 16384, k = 64, bf16, equal widths, with
    bias.  Through the C ABI with the workspace allocated once.  Algorithmic bytes: the four gradients and linear_output
    read once (2 m n esize), x and W read, x_grad, weight_grad and bias_grad written."""
    import ctypes as C
    from recsdk_amd import _capi
    m_, n, k = 16384, 16384, 64
    g = torch.Generator().manual_seed(13)
    sp = [n // 4] * 4
    grads = [torch.rand(m_, s_, generator=g).to(torch.bfloat16) for s_ in sp]
    u = lambda *s: (torch.rand(*s, generator=g) * 2 - 1).to(torch.bfloat16)
    x, w, lin = u(m_, k), u(n, k), u(m_, n)
    dev = [t.cuda() for t in grads]
    xd, wd, ld = x.cuda(), w.cuda(), lin.cuda()
    xg, wg = torch.empty_like(xd), torch.empty_like(wd)
    bg = torch.empty(n, device="cuda")
    L = _capi.lib()
    p = _capi.HstuInLinearSiluBwdParams()
    p.struct_size = C.sizeof(p)
    p.dtype, p.grad_dtype, p.m, p.k, p.n = _capi.HSTU_BF16, _capi.HSTU_BF16, m_, k, n
    for i in range(4):
        p.split[i] = sp[i]
        p.grad[i] = dev[i].data_ptr()
    p.x, p.weight, p.linear_output = xd.data_ptr(), wd.data_ptr(), ld.data_ptr()
    p.x_grad, p.weight_grad, p.bias_grad = xg.data_ptr(), wg.data_ptr(), bg.data_ptr()
    need = C.c_uint64(0)
    assert L.hstu_hip_in_linear_silu_backward_get_workspace_size(C.byref(p), C.byref(need)) == 0
    ws = torch.empty(need.value, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream

    def fn():
        rc = L.hstu_hip_in_linear_silu_backward(C.byref(p), ws.data_ptr(), need.value, stream)
        assert rc == 0, L.hstu_hip_last_error().decode()
    for _ in range(args.warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    kern_ms = e0.elapsed_time(e1) / args.steps
    alg = 2 * m_ * n * 2 + 2 * (m_ * k * 2 + n * k * 2) + n * 4
    flops = 4.0 * m_ * n * k
    out = {
        "metric": "in_linear_silu_bwd_gbps", "value": round(alg / (ms * 1e-3) / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", "us_per_call": round(ms * 1e3, 2), "tflops": round(flops / (ms * 1e-3) / 1e12, 1),
        "config": {"workload": "in_linear_silu_bwd: x [16384, 64], W [16384, 64], gradients 4 x [16384, 4096], linear_output [16384, 16384] bf16, seed 13",
                   "algorithmic_bytes_per_call": alg, "flops_per_call": flops, "workspace_bytes": need.value,
                   "entry": "hstu_hip_in_linear_silu_backward (include/hstu_layer.h): two operand packs, hstu_ilb_wgrad_kernel (one pass: weight_grad, bias_grad and x_grad slabs), three reductions"},
        "roofline": {"bound": "hbm", "kernel": "hstu_ilb_wgrad_kernel, one pass (+ 5 small kernels; all inside the events)",
                     "achieved": round(alg / (kern_ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(alg / (kern_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
                     "kernel_us": round(kern_ms * 1e3, 2)},
    }
    if not args.no_cpu_baseline:
        from oracle import layer_oracle as LO
        rows = 2048
        t0 = time.perf_counter()
        LO.in_linear_silu_backward([t[:rows] for t in grads], x[:rows], w, lin[:rows])
        dt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": round(alg * rows / m_ / dt / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"the first {rows} rows once (oracle in torch, fp64), {dt:.2f} s"}
    print(json.dumps(out), flush=True)


def reference_grid(args, torch, _capi, backward=False):
    """The grid of the reference's own forward benchmark (cust_op/test/hstu_v2/test_forward_op_benchmark.py:246-259; with
    `backward` that of test_backward_op_benchmark.py:246-259, the gradients dQ, dK, dV and, with a bias, dBias: 2.5 x the FLOPs): B = 32,
    h = 8, every sequence int(0.9 S) rows, S in {512, 1024, 2048, 4096} x head dim in {32, 64, 128, 256} x with / without a
    dense bias [B, h, S, S], no mask (its window_size (-1, -1)), alpha 0.5, silu_scale 1/1024, inputs uniform in (-1, 1) -- in
    bf16 (the reference also runs fp16).  One JSON line per point; --steps / --warmup apply to every point (capped at 50 / 20)."""
    import ctypes as C
    L = _capi.lib()
    steps, warm = min(args.steps, 50), min(args.warmup, 20)
    g = torch.Generator(device="cuda").manual_seed(123)
    uni = lambda *shape: (torch.rand(shape, generator=g, device="cuda") * 2 - 1).to(torch.bfloat16)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    for S in (512, 1024, 2048, 4096):
        l = int(0.9 * S)
        off = torch.arange(33, dtype=torch.int64, device="cuda") * l
        for d in (32, 64, 128, 256):
            q, k, v = uni(32 * l, 8, d), uni(32 * l, 8, d), uni(32 * l, 8, d)
            out = torch.empty_like(q)
            for rab in (False, True):
                bias = uni(32, 8, S, S) if rab else None
                p, keep = _capi.make_params(q, k, v, out, seq_offset_q=off, max_seq_len_q=S, mask_type=_capi.MASK_NONE, alpha=0.5,
                                            silu_scale=1.0 / 1024, attn_bias=bias)
                n = C.c_uint64(0)
                if backward:
                    if rab and S == 4096:
                        continue          # bias and its gradient: 2 x 8.6 GB per point; left out
                    grad, dq, dk, dv = uni(32 * l, 8, d), torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
                    dbias = torch.empty_like(bias) if rab else None
                    p.out = None
                    fwd, p = p, _capi.make_backward_params(p, grad, dq, dk, dv, dbias)
                    size_fn, run_fn, name = L.hstu_hip_jagged_backward_get_workspace_size, L.hstu_hip_jagged_backward, _capi.describe_backward_kernel(p)
                else:
                    size_fn, run_fn, name = L.hstu_hip_jagged_forward_get_workspace_size, L.hstu_hip_jagged_forward, _capi.describe_kernel(p)
                if size_fn(C.byref(p), C.byref(n)) != 0:
                    raise RuntimeError(L.hstu_hip_last_error().decode())
                ws = torch.empty(max(int(n.value), 16), dtype=torch.uint8, device="cuda")

                def step():
                    if run_fn(C.byref(p), C.c_void_p(ws.data_ptr()), n.value, stream) != 0:
                        raise RuntimeError(L.hstu_hip_last_error().decode())
                settle_clocks(step, args.settle_ms, torch)
                for _ in range(warm):
                    step()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                torch.cuda.synchronize()
                e0.record()
                for _ in range(steps):
                    step()
                e1.record()
                torch.cuda.synchronize()
                us = e0.elapsed_time(e1) / steps * 1e3
                flops = 32 * 4.0 * l * l * 8 * d * (2.5 if backward else 1.0)
                print(json.dumps({"metric": "hstu_reference_benchmark_grid" + ("_backward" if backward else ""), "S": S, "head_dim": d, "dense_bias": rab, "mask": "none", "dtype": "bf16",
                                  "batch": 32, "heads": 8, "rows_per_sequence": l, "kernel": name, "us_per_call": round(us, 1),
                                  "tflops": round(flops / us * 1e-6, 1), "pct_bf16_mfma_peak": round(flops / us * 1e-6 / PEAK_BF16_TFLOPS * 100, 1),
                                  "steps": steps, "warmup": warm, "n_gpus": 1}), flush=True)
                del bias


def copy_calibration(args, torch):
    n = 256 << 20
    src = torch.randint(0, 255, (n,), dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    for _ in range(args.warmup):
        dst.copy_(src)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        dst.copy_(src)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / args.steps
    print(json.dumps({"metric": "device_copy", "value": round(2 * n / (ms * 1e-3) / 1e9, 1), "unit": "GB/s", "n_gpus": 1,
                      "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 5),
                      "config": {"workload": "plain copy of 256 MiB (reads 262144 KiB, writes 262144 KiB per launch)"}}))


def settle_clocks(step, ms, torch):
    """Untimed calls until the GPU has been busy for `ms`: after idling, its clocks take about 50 ms of load to reach the
    state a model's steady stream of kernels sees.  Not part of warmup / steps; reported in the result."""
    if ms <= 0:
        return {"calls": 0, "ms": 0.0}
    calls, busy = 0, 0.0
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    while busy < ms and calls < 100000:
        n = 50 if calls == 0 else max(50, int(50 * (ms - busy) / max(busy / (calls / 50), 1e-3)))
        n = min(n, 20000)
        e0.record()
        for _ in range(n):
            step()
        e1.record()
        torch.cuda.synchronize()
        busy += e0.elapsed_time(e1)
        calls += n
    return {"calls": calls, "ms": round(busy, 2)}


def _median_seconds(f, runs=5):
    f()
    ts = []
    for _ in range(runs):
        t0 = time.perf_counter()
        f()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2]


def cpu_baseline(cfg, op, flops, torch, workload, W):
    """The CPU oracle (a from-scratch port of the reference's PyTorch golden: per sequence matmul -> fp32 SiLU -> mask ->
    matmul) timed on this box's host cores, same seeded inputs: one warm-up + the median of 5 runs.  For the headline
    workload: configs 1 and 2, bf16 (the golden's rounding points) and fp32, on all of this process's threads and on one."""
    from tests import hstu_testlib as T
    n = torch.get_num_threads()
    if op == "jagged" and (cfg.get("pos_table") is not None or cfg.get("ts_table") is not None or cfg.get("attn_bias") is not None):
        return {"value": None, "unit": "TFLOP/s", "cores": n, "kind": "port",
                "sample": "not timed: the dense-bias oracle of this workload needs tens of GB or minutes"}
    if workload != "config2":
        f = (lambda: T.oracle_paged(cfg)) if op == "paged" else (lambda: T.oracle_jagged(cfg, mode="lowp"))
        sec = _median_seconds(f, runs=2 if op == "paged" else 5)
        return {"value": round(flops / sec / 1e12, 4), "unit": "TFLOP/s", "cores": n, "kind": "port",
                "sample": f"the whole batch of this workload once (its I/O dtype, the golden's rounding points), {sec:.2f} s on {n} threads",
                "seconds_per_call": round(sec, 3)}
    detail = {}
    c1 = W.config1()
    f1 = W.headline_flops(c1["lens"], 2, 32)
    cases = {"config2": (cfg, flops), "config1": (c1, f1)}
    for name, (c, fl) in cases.items():
        c32 = dict(c, q=c["q"].float(), k=c["k"].float(), v=c["v"].float())
        cbf = dict(c, q=c["q"].bfloat16(), k=c["k"].bfloat16(), v=c["v"].bfloat16())
        detail[name] = {}
        for threads in (n, 1):
            torch.set_num_threads(threads)
            try:
                s32 = _median_seconds(lambda: T.oracle_jagged(c32, mode="exact", compute_dtype=torch.float32))
                sbf = _median_seconds(lambda: T.oracle_jagged(cbf, mode="lowp"))
            finally:
                torch.set_num_threads(n)
            detail[name][f"threads_{threads}"] = {"fp32_tflops": round(fl / s32 / 1e12, 5), "fp32_s": round(s32, 4),
                                                  "bf16_tflops": round(fl / sbf / 1e12, 5), "bf16_s": round(sbf, 4)}
    head = detail["config2"][f"threads_{n}"]
    return {"value": head["bf16_tflops"], "unit": "TFLOP/s", "cores": n, "kind": "port",
            "sample": f"the whole headline batch once per run (bf16 I/O with the golden's rounding points), median of 5 after a warm-up: "
                      f"{head['bf16_s']:.3f} s on {n} threads; fp32, one thread and config 1 in `detail`",
            "seconds_per_call": head["bf16_s"], "detail": detail}


if __name__ == "__main__":
    main()
