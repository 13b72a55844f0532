"""ctypes binding of the C ABI declared in ``include/*.h``.

This is the thinnest possible host binding: raw device pointers and sizes in, status code out.
It exists so that callers (and the parity tests) can drive the library without the torch op
layer; torch tensors are only used here as owners of device memory (``data_ptr()``).
"""
from __future__ import annotations

import ctypes as C
import math
import os
from typing import Optional

import torch

from . import _build

HSTU_F32, HSTU_F16, HSTU_BF16, HSTU_FP8_E4M3 = 0, 1, 2, 3
HSTU_I32, HSTU_I64 = 0, 1
MASK_TRIL, MASK_TRIU, MASK_NONE, MASK_CUSTOM = 0, 1, 2, 3
FLAG_DETERMINISTIC, FLAG_FORCE_GENERIC, FLAG_REUSE_WORKSPACE, FLAG_SERIAL_BACKWARD = 1, 2, 4, 8

EXPORTS = [
    "hstu_hip_jagged_forward_get_workspace_size", "hstu_hip_jagged_forward", "hstu_hip_jagged_forward_noalloc",
    "hstu_hip_paged_forward_get_workspace_size", "hstu_hip_paged_forward",
    "hstu_hip_dense_forward_get_workspace_size", "hstu_hip_dense_forward",
    "hstu_hip_jagged_backward_get_workspace_size", "hstu_hip_jagged_backward",
    "hstu_hip_dense_backward_get_workspace_size", "hstu_hip_dense_backward",
    "hstu_hip_last_error", "hstu_hip_describe_kernel", "hstu_hip_describe_backward_kernel", "hstu_hip_abi_version",
    "hstu_hip_kv_append", "hstu_hip_kv_token_positions", "hstu_hip_kv_append_fp8", "hstu_hip_kv_append_fp8_get_workspace_size",
    "hstu_hip_rab_time", "hstu_hip_rab_time_backward", "hstu_hip_rab_pos",
    "hstu_hip_norm_multiply_dropout", "hstu_hip_norm_multiply_dropout_backward",
    "hstu_hip_norm_multiply_dropout_backward_get_workspace_size", "hstu_hip_in_linear_silu",
    "hstu_hip_in_linear_silu_backward", "hstu_hip_in_linear_silu_backward_get_workspace_size",
]


class HstuFwdParams(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("flags", C.c_uint32), ("dtype", C.c_int32), ("index_type", C.c_int32),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("out", C.c_void_p),
        ("mask", C.c_void_p), ("attn_bias", C.c_void_p),
        ("seq_offset_q", C.c_void_p), ("seq_offset_k", C.c_void_p),
        ("num_context", C.c_void_p), ("num_target", C.c_void_p),
        ("total_q", C.c_int64), ("total_k", C.c_int64),
        ("batch", C.c_int32), ("heads_q", C.c_int32), ("heads_k", C.c_int32), ("dim_qk", C.c_int32),
        ("dim_v", C.c_int32), ("mask_type", C.c_int32), ("max_seq_len_q", C.c_int32), ("max_seq_len_k", C.c_int32),
        ("target_group_size", C.c_int32), ("silu_scale", C.c_float), ("alpha", C.c_float),
        ("kv_cache", C.c_void_p), ("page_offsets", C.c_void_p), ("page_ids", C.c_void_p),
        ("last_page_len", C.c_void_p), ("kv_scales", C.c_void_p),
        ("num_pages", C.c_int64), ("page_size", C.c_int32), ("cache_dtype", C.c_int32),
        ("pos_table", C.c_void_p), ("ts_table", C.c_void_p), ("ts_bounds", C.c_void_p), ("timestamps", C.c_void_p),
        ("num_buckets", C.c_int32), ("ts_log2_scale", C.c_float),
    ]


class HstuBwdParams(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("reserved", C.c_uint32), ("fwd", HstuFwdParams),
        ("grad_out", C.c_void_p), ("grad_q", C.c_void_p), ("grad_k", C.c_void_p), ("grad_v", C.c_void_p),
        ("grad_bias", C.c_void_p),
    ]


class HstuKvAppendParams(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("elem_bytes", C.c_int32), ("k_cache", C.c_void_p), ("v_cache", C.c_void_p),
        ("stride_page", C.c_int64), ("stride_n", C.c_int64), ("stride_h", C.c_int64),
        ("num_pages", C.c_int32), ("page_size", C.c_int32), ("num_heads", C.c_int32), ("head_dim", C.c_int32),
        ("kv_indices", C.c_void_p), ("kv_indptr", C.c_void_p), ("num_indices", C.c_int32), ("batch", C.c_int32),
        ("append_key", C.c_void_p), ("append_value", C.c_void_p),
        ("append_k_stride_n", C.c_int64), ("append_k_stride_h", C.c_int64),
        ("append_v_stride_n", C.c_int64), ("append_v_stride_h", C.c_int64), ("append_rows", C.c_int64),
        ("batch_indices", C.c_void_p), ("positions", C.c_void_p), ("offsets", C.c_void_p), ("nnz_dev", C.c_void_p),
        ("nnz_max", C.c_int32), ("reserved", C.c_int32),
    ]


class HstuKvAppendFp8Params(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("src_dtype", C.c_int32), ("kv_cache", C.c_void_p), ("kv_scales", C.c_void_p),
        ("num_pages", C.c_int32), ("page_size", C.c_int32), ("num_heads", C.c_int32), ("head_dim", C.c_int32),
        ("kv_indices", C.c_void_p), ("kv_indptr", C.c_void_p), ("num_indices", C.c_int32), ("batch", C.c_int32),
        ("append_key", C.c_void_p), ("append_value", C.c_void_p),
        ("append_k_stride_n", C.c_int64), ("append_k_stride_h", C.c_int64),
        ("append_v_stride_n", C.c_int64), ("append_v_stride_h", C.c_int64), ("append_rows", C.c_int64),
        ("batch_indices", C.c_void_p), ("positions", C.c_void_p), ("offsets", C.c_void_p), ("nnz_dev", C.c_void_p),
        ("nnz_max", C.c_int32), ("reserved", C.c_int32),
    ]


class HstuRabTimeParams(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("dtype", C.c_int32), ("index_type", C.c_int32), ("num_layers", C.c_int32),
        ("batch", C.c_int32), ("seq_len", C.c_int32), ("weight_cols", C.c_int32), ("bucket_divisor", C.c_float),
        ("timestamps", C.c_void_p), ("weights", C.c_void_p), ("bucket_bounds", C.c_void_p),
        ("rab_time_out", C.c_void_p), ("bucket_ts_out", C.c_void_p),
    ]


class HstuRabTimeBwdParams(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("dtype", C.c_int32), ("index_type", C.c_int32), ("num_layers", C.c_int32),
        ("batch", C.c_int32), ("seq_len", C.c_int32), ("num_buckets", C.c_int32), ("reserved", C.c_int32),
        ("grad", C.c_void_p), ("bucket_ts", C.c_void_p), ("grad_weights", C.c_void_p),
    ]


class HstuNmdParams(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("dtype", C.c_int32), ("rows", C.c_int64), ("cols", C.c_int32), ("eps", C.c_float),
        ("dropout_ratio", C.c_float), ("reserved", C.c_uint32), ("seed", C.c_uint64),
        ("x", C.c_void_p), ("u", C.c_void_p), ("weight", C.c_void_p), ("bias", C.c_void_p), ("out", C.c_void_p),
        ("mean", C.c_void_p), ("var", C.c_void_p), ("drop_mask", C.c_void_p),
    ]


class HstuNmdBwdParams(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("dtype", C.c_int32), ("rows", C.c_int64), ("cols", C.c_int32), ("eps", C.c_float),
        ("dropout_ratio", C.c_float), ("reserved", C.c_uint32),
        ("d_out", C.c_void_p), ("x", C.c_void_p), ("u", C.c_void_p), ("weight", C.c_void_p), ("bias", C.c_void_p),
        ("mean", C.c_void_p), ("var", C.c_void_p), ("drop_mask", C.c_void_p), ("d_x", C.c_void_p), ("d_u", C.c_void_p),
        ("d_weight", C.c_void_p), ("d_bias", C.c_void_p),
    ]


class HstuInLinearSiluParams(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("dtype", C.c_int32), ("m", C.c_int64), ("k", C.c_int32), ("n", C.c_int32),
        ("split", C.c_int32 * 4), ("x", C.c_void_p), ("weight", C.c_void_p), ("bias", C.c_void_p),
        ("out", C.c_void_p * 4), ("linear_output", C.c_void_p),
    ]


class HstuInLinearSiluBwdParams(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("dtype", C.c_int32), ("m", C.c_int64), ("k", C.c_int32), ("n", C.c_int32),
        ("split", C.c_int32 * 4), ("grad_dtype", C.c_int32), ("algorithm", C.c_int32),
        ("x", C.c_void_p), ("weight", C.c_void_p), ("grad", C.c_void_p * 4), ("linear_output", C.c_void_p),
        ("x_grad", C.c_void_p), ("weight_grad", C.c_void_p), ("bias_grad", C.c_void_p),
    ]


_lib: Optional[C.CDLL] = None


class HstuError(RuntimeError):
    pass


def lib() -> C.CDLL:
    """Load ``libhstu_hip.so``; raises if it has not been built (there is no fallback path)."""
    global _lib
    if _lib is None:
        path = _build.hip_lib_path()
        if not os.path.exists(path):
            raise HstuError(f"{path} is missing: build it with `python -m recsdk_amd._build` (hipcc, gfx950)")
        _lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
        _lib.hstu_hip_last_error.restype = C.c_char_p
        for n in ("jagged", "paged", "dense"):
            getattr(_lib, f"hstu_hip_{n}_forward").argtypes = [C.POINTER(HstuFwdParams), C.c_void_p, C.c_uint64, C.c_void_p]
            getattr(_lib, f"hstu_hip_{n}_forward_get_workspace_size").argtypes = [C.POINTER(HstuFwdParams), C.POINTER(C.c_uint64)]
        _lib.hstu_hip_jagged_forward_noalloc.argtypes = [C.POINTER(HstuFwdParams), C.c_void_p]
        for n in ("jagged", "dense"):
            getattr(_lib, f"hstu_hip_{n}_backward").argtypes = [C.POINTER(HstuBwdParams), C.c_void_p, C.c_uint64, C.c_void_p]
            getattr(_lib, f"hstu_hip_{n}_backward_get_workspace_size").argtypes = [C.POINTER(HstuBwdParams), C.POINTER(C.c_uint64)]
        _lib.hstu_hip_describe_kernel.argtypes = [C.POINTER(HstuFwdParams), C.c_char_p, C.c_size_t]
        _lib.hstu_hip_describe_backward_kernel.argtypes = [C.POINTER(HstuBwdParams), C.c_char_p, C.c_size_t]
        _lib.hstu_hip_kv_append.argtypes = [C.POINTER(HstuKvAppendParams), C.c_void_p]
        _lib.hstu_hip_kv_append_fp8.argtypes = [C.POINTER(HstuKvAppendFp8Params), C.c_void_p, C.c_uint64, C.c_void_p]
        _lib.hstu_hip_kv_append_fp8_get_workspace_size.argtypes = [C.POINTER(HstuKvAppendFp8Params), C.POINTER(C.c_uint64)]
        _lib.hstu_hip_rab_time.argtypes = [C.POINTER(HstuRabTimeParams), C.c_void_p]
        _lib.hstu_hip_norm_multiply_dropout.argtypes = [C.POINTER(HstuNmdParams), C.c_void_p]
        _lib.hstu_hip_in_linear_silu.argtypes = [C.POINTER(HstuInLinearSiluParams), C.c_void_p]
        _lib.hstu_hip_in_linear_silu_backward.argtypes = [C.POINTER(HstuInLinearSiluBwdParams), C.c_void_p, C.c_uint64, C.c_void_p]
        _lib.hstu_hip_in_linear_silu_backward_get_workspace_size.argtypes = [C.POINTER(HstuInLinearSiluBwdParams), C.POINTER(C.c_uint64)]
        _lib.hstu_hip_norm_multiply_dropout_backward.argtypes = [C.POINTER(HstuNmdBwdParams), C.c_void_p, C.c_uint64, C.c_void_p]
        _lib.hstu_hip_norm_multiply_dropout_backward_get_workspace_size.argtypes = [C.POINTER(HstuNmdBwdParams), C.POINTER(C.c_uint64)]
        _lib.hstu_hip_rab_time_backward.argtypes = [C.POINTER(HstuRabTimeBwdParams), C.c_void_p]
        _lib.hstu_hip_rab_pos.argtypes = [C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.POINTER(C.c_int64), C.c_int32, C.c_void_p, C.c_void_p]
        _lib.hstu_hip_kv_token_positions.argtypes = [C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p]
    return _lib


_DT = {torch.float32: HSTU_F32, torch.float16: HSTU_F16, torch.bfloat16: HSTU_BF16, torch.float8_e4m3fn: HSTU_FP8_E4M3}


def out_dtype(in_dtype):
    """dtype of the forward's output for q/k/v of ``in_dtype`` (fp16 for float8_e4m3fn, reference hstu_jagged.cpp:53-54)."""
    return torch.float16 if in_dtype == torch.float8_e4m3fn else in_dtype


def _ptr(t):
    return None if t is None else t.data_ptr()


def make_params(q, k, v, out, *, seq_offset_q=None, seq_offset_k=None, max_seq_len_q, max_seq_len_k=None,
                mask_type=MASK_TRIL, mask=None, attn_bias=None, silu_scale=0.0, alpha=1.0, num_context=None,
                num_target=None, target_group_size=0, kv_cache=None, page_offsets=None, page_ids=None,
                last_page_len=None, kv_scales=None, pos_table=None, ts_table=None, ts_bounds=None,
                timestamps=None, bucket_divisor=0.301, flags=0, dense=False):
    """Fill an argument block from tensors.  Returns (params, keepalive list)."""
    p = HstuFwdParams()
    p.struct_size = C.sizeof(HstuFwdParams)
    p.flags = flags
    p.dtype = _DT.get(q.dtype, -1)
    keep = [q, k, v, out, mask, attn_bias, seq_offset_q, seq_offset_k, num_context, num_target, kv_cache,
            page_offsets, page_ids, last_page_len, kv_scales, pos_table, ts_table, ts_bounds, timestamps]
    idx_dtype = seq_offset_q.dtype if seq_offset_q is not None else torch.int64
    p.index_type = HSTU_I64 if idx_dtype == torch.int64 else HSTU_I32
    if seq_offset_k is None:
        seq_offset_k = seq_offset_q

    def idx(t):
        if t is None:
            return None
        if t.dtype != idx_dtype:
            t = t.to(idx_dtype)
            keep.append(t)
        return t

    seq_offset_k, num_context, num_target = idx(seq_offset_k), idx(num_context), idx(num_target)
    page_offsets, page_ids, last_page_len = idx(page_offsets), idx(page_ids), idx(last_page_len)
    p.q, p.k, p.v, p.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    p.mask, p.attn_bias = _ptr(mask), _ptr(attn_bias)
    p.seq_offset_q, p.seq_offset_k = _ptr(seq_offset_q), _ptr(seq_offset_k)
    p.num_context, p.num_target = _ptr(num_context), _ptr(num_target)
    if dense:
        b, s, n, d = q.shape
        p.batch, p.total_q, p.total_k = b, b * s, b * s
        p.heads_q, p.heads_k, p.dim_qk, p.dim_v = n, k.shape[2], d, v.shape[3]
    else:
        p.batch = seq_offset_q.numel() - 1
        p.total_q, p.total_k = q.shape[0], k.shape[0]
        p.heads_q, p.heads_k, p.dim_qk, p.dim_v = q.shape[1], k.shape[1], q.shape[2], v.shape[2]
    p.mask_type = mask_type
    p.max_seq_len_q = max_seq_len_q
    p.max_seq_len_k = max_seq_len_q if max_seq_len_k is None else max_seq_len_k
    p.target_group_size = target_group_size
    p.silu_scale = (1.0 / max_seq_len_q) if silu_scale == 0.0 else silu_scale
    p.alpha = alpha
    if kv_cache is not None:
        p.kv_cache = kv_cache.data_ptr()
        p.num_pages, p.page_size = kv_cache.shape[0], kv_cache.shape[2]
        p.cache_dtype = HSTU_FP8_E4M3 if kv_cache.dtype in (torch.uint8, torch.float8_e4m3fn) else _DT.get(kv_cache.dtype, -1)
        p.page_offsets, p.page_ids, p.last_page_len = _ptr(page_offsets), _ptr(page_ids), _ptr(last_page_len)
        p.kv_scales = _ptr(kv_scales)
    p.pos_table, p.ts_table, p.ts_bounds, p.timestamps = _ptr(pos_table), _ptr(ts_table), _ptr(ts_bounds), _ptr(timestamps)
    p.num_buckets = 0 if ts_table is None else ts_table.numel() - 1
    p.ts_log2_scale = 0.0 if ts_table is None or not bucket_divisor else math.log(2.0) / bucket_divisor
    return p, keep


def _check(rc):
    if rc != 0:
        raise HstuError(lib().hstu_hip_last_error().decode())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def run(op: str, params: HstuFwdParams, stream=None):
    """Two-phase call: query the workspace size, allocate it, launch on ``stream`` (default: torch's current)."""
    L = lib()
    n = C.c_uint64(0)
    _check(getattr(L, f"hstu_hip_{op}_forward_get_workspace_size")(C.byref(params), C.byref(n)))
    ws = torch.empty(n.value, dtype=torch.uint8, device="cuda") if n.value else None
    _check(getattr(L, f"hstu_hip_{op}_forward")(C.byref(params), _ptr(ws), n.value, stream if stream is not None else _stream()))
    return ws


def run_noalloc(params: HstuFwdParams, stream=None):
    """The jagged forward through the entry point that allocates nothing (work list in the library's fixed array)."""
    _check(lib().hstu_hip_jagged_forward_noalloc(C.byref(params), stream if stream is not None else _stream()))


NOALLOC_SCRATCH_BYTES = 2 << 20


def make_backward_params(fwd: HstuFwdParams, grad_out, grad_q, grad_k, grad_v, grad_bias=None) -> HstuBwdParams:
    """Argument block of the jagged backward around the forward call's block (whose ``out`` is not read)."""
    p = HstuBwdParams()
    p.struct_size = C.sizeof(HstuBwdParams)
    p.fwd = fwd
    p.grad_out, p.grad_q, p.grad_k, p.grad_v = grad_out.data_ptr(), grad_q.data_ptr(), grad_k.data_ptr(), grad_v.data_ptr()
    p.grad_bias = _ptr(grad_bias)
    return p


def run_backward(params: HstuBwdParams, stream=None, op: str = "jagged"):
    """Two-phase call of the jagged (or dense) backward."""
    L = lib()
    n = C.c_uint64(0)
    _check(getattr(L, f"hstu_hip_{op}_backward_get_workspace_size")(C.byref(params), C.byref(n)))
    ws = torch.empty(n.value, dtype=torch.uint8, device="cuda") if n.value else None
    _check(getattr(L, f"hstu_hip_{op}_backward")(C.byref(params), _ptr(ws), n.value, stream if stream is not None else _stream()))
    return ws


def describe_backward_kernel(params: HstuBwdParams) -> str:
    buf = C.create_string_buffer(64)
    _check(lib().hstu_hip_describe_backward_kernel(C.byref(params), buf, 64))
    return buf.value.decode()


def describe_kernel(params: HstuFwdParams) -> str:
    buf = C.create_string_buffer(64)
    _check(lib().hstu_hip_describe_kernel(C.byref(params), buf, 64))
    return buf.value.decode()
