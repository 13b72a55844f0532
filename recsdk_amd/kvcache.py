"""Write side of the paged K/V cache, under the names and argument order of the reference's binding.

``append_kvcache`` mirrors ``kvcache_npu_cpp.append_kvcache`` (inference/kvcache_manager/src/pybind.cpp:63-117: same
positional arguments, checks and messages) and ``get_paged_batch_indices_positions`` the launcher
``kvcache::GetPagedBatchIndicesPositions`` (src/gather_scatter.cpp:137-142).  Both are one call into
``libhstu_hip.so`` on the current stream; tensors are device ("cuda") tensors and nothing is read on the host.
There is no CPU implementation.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _capi


def _check_int32_1d(t: torch.Tensor, device, name: str) -> None:
    if t.device != device:
        raise RuntimeError(f"{name} must be on {device}")
    if t.dtype != torch.int32:
        raise RuntimeError(f"{name} must have dtype int32")
    if t.dim() != 1:
        raise RuntimeError(f"{name} must be one-dimensional")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _check_kv_2byte(t: torch.Tensor, device, dims: int, name: str) -> None:
    if t.device != device:
        raise RuntimeError(f"{name} must be on {device}")
    if t.element_size() != 2:
        raise RuntimeError(f"{name} must have a 2-byte dtype (float16 or bfloat16)")
    if t.dim() != dims:
        raise RuntimeError(f"{name} must have {dims} dimensions")


def _require_gpu(t: torch.Tensor, what: str) -> None:
    if t.device.type != "cuda":
        raise RuntimeError(f"{what} has no CPU implementation: move the tensors to the MI355X (device 'cuda')")


def append_kvcache(append_key, append_value, batch_indices, positions, seqlen_offsets, nnz_npu, nnz: int,
                   paged_k_cache, paged_v_cache, kv_indices, kv_indptr, kv_last_page_len, kv_layout: int) -> None:
    """Copy the K and V rows of the new tokens into their pages.

    Token ``i`` (``i < nnz_npu[0]``) of user ``b = batch_indices[i]`` goes to page
    ``kv_indices[kv_indptr[b] + positions[i] // page_size]``, slot ``positions[i] % page_size``; its source row is
    ``i + seqlen_offsets[b]``.  ``paged_k_cache`` / ``paged_v_cache`` are the ``unbind(1)`` views of a
    ``[pages, 2, page_size, heads, dim]`` table (``kv_layout`` 0, NHD) or ``[pages, heads, page_size, dim]`` views
    (``kv_layout`` 1, HND); strides are taken from the tensors.  ``nnz`` (host) is accepted and ignored like in the reference
    (pybind.cpp:57-61): the launch covers ``min(len(batch_indices), len(positions))`` tokens and ``nnz_npu[0]`` says how many of
    them exist.
    """
    device = append_key.device
    _check_kv_2byte(append_key, device, 3, "append_key")
    _check_kv_2byte(append_value, device, 3, "append_value")
    if append_key.shape != append_value.shape:
        raise RuntimeError("append_key and append_value must have the same shape")
    _check_kv_2byte(paged_k_cache, device, 4, "paged_k_cache")
    _check_kv_2byte(paged_v_cache, device, 4, "paged_v_cache")
    _check_int32_1d(batch_indices, device, "batch_indices")
    _check_int32_1d(positions, device, "positions")
    _check_int32_1d(seqlen_offsets, device, "seqlen_offsets")
    _check_int32_1d(nnz_npu, device, "nnz_npu")
    _check_int32_1d(kv_indices, device, "kv_indices")
    _check_int32_1d(kv_indptr, device, "kv_indptr")
    _check_int32_1d(kv_last_page_len, device, "kv_last_page_len")
    if kv_layout not in (0, 1):
        raise RuntimeError(f"kv_layout must be 0 (NHD) or 1 (HND), got {kv_layout}")
    if paged_k_cache.shape != paged_v_cache.shape or paged_k_cache.stride() != paged_v_cache.stride():
        raise RuntimeError("paged_k_cache and paged_v_cache must have the same shape and strides")
    head_dim = paged_k_cache.size(3)
    if kv_layout == 1:
        num_heads, page_size = paged_k_cache.size(1), paged_k_cache.size(2)
    else:
        page_size, num_heads = paged_k_cache.size(1), paged_k_cache.size(2)
    if paged_k_cache.stride(3) != 1 or append_key.stride(2) != 1 or append_value.stride(2) != 1:
        raise RuntimeError("the head_dim axis of the caches and of append_key / append_value must be contiguous")
    if tuple(append_key.shape[1:]) != (num_heads, head_dim):
        raise RuntimeError(f"append_key shape {tuple(append_key.shape)} mismatch with cache heads {num_heads}, head_dim {head_dim}")
    # the reference's binding takes the host `nnz` and ignores it (pybind.cpp:57-61; its kernel reads nnz_npu only): a stale
    # or zero value must not lose tokens, so the launch is sized by the index arrays and the device count does the rest
    n = min(batch_indices.numel(), positions.numel())
    p = _capi.HstuKvAppendParams()
    p.struct_size = C.sizeof(_capi.HstuKvAppendParams)
    p.elem_bytes = 2
    p.k_cache, p.v_cache = paged_k_cache.data_ptr(), paged_v_cache.data_ptr()
    p.stride_page = paged_k_cache.stride(0)
    p.stride_n = head_dim if kv_layout == 1 else num_heads * head_dim      # as pybind.cpp:97-98
    p.stride_h = page_size * head_dim if kv_layout == 1 else head_dim
    p.num_pages, p.page_size, p.num_heads, p.head_dim = paged_k_cache.size(0), page_size, num_heads, head_dim
    p.kv_indices, p.kv_indptr = kv_indices.data_ptr(), kv_indptr.data_ptr()
    p.num_indices, p.batch = kv_indices.numel(), kv_indptr.numel() - 1
    if seqlen_offsets.numel() < p.batch:
        raise RuntimeError("seqlen_offsets must have one entry per user of kv_indptr")
    p.append_key, p.append_value = append_key.data_ptr(), append_value.data_ptr()
    p.append_k_stride_n, p.append_k_stride_h = append_key.stride(0), append_key.stride(1)
    p.append_v_stride_n, p.append_v_stride_h = append_value.stride(0), append_value.stride(1)
    p.append_rows = append_key.size(0)
    p.batch_indices, p.positions, p.offsets = batch_indices.data_ptr(), positions.data_ptr(), seqlen_offsets.data_ptr()
    p.nnz_dev, p.nnz_max = nnz_npu.data_ptr(), n
    _require_gpu(append_key, "append_kvcache")
    with torch.cuda.device(device):
        _capi._check(_capi.lib().hstu_hip_kv_append(C.byref(p), _capi._stream()))


def append_kvcache_fp8(append_key, append_value, batch_indices, positions, seqlen_offsets, nnz_npu, nnz: int,
                       kv_cache_fp8, kv_scales, kv_indices, kv_indptr, workspace=None):
    """``append_kvcache`` for the fp8-e4m3 table that ``torch.ops.mxrec.hstu_paged_fp8`` reads (no counterpart in the
    reference): ``kv_cache_fp8`` is ``[pages, 2, page_size, heads, dim]`` (uint8 or float8_e4m3fn, contiguous),
    ``kv_scales`` ``[pages, 2, heads]`` fp32.  The new rows are quantised with one scale per (page, K|V, head); a page
    that already holds rows keeps its scale unless the new rows need a larger one, in which case its old rows are
    requantised.  ``workspace`` (uint8, size from ``hstu_hip_kv_append_fp8_get_workspace_size``) is allocated when not given;
    returns it for reuse."""
    device = append_key.device
    _check_kv_2byte(append_key, device, 3, "append_key")
    _check_kv_2byte(append_value, device, 3, "append_value")
    if append_key.shape != append_value.shape or append_key.dtype != append_value.dtype:
        raise RuntimeError("append_key and append_value must have the same shape and dtype")
    if append_key.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("append_key must be float16 or bfloat16")
    for t, name in ((batch_indices, "batch_indices"), (positions, "positions"), (seqlen_offsets, "seqlen_offsets"), (nnz_npu, "nnz_npu"),
                    (kv_indices, "kv_indices"), (kv_indptr, "kv_indptr")):
        _check_int32_1d(t, device, name)
    if kv_cache_fp8.device != device or kv_cache_fp8.element_size() != 1 or kv_cache_fp8.dim() != 5 or kv_cache_fp8.size(1) != 2 \
            or not kv_cache_fp8.is_contiguous():
        raise RuntimeError("kv_cache_fp8 must be a contiguous 1-byte [pages, 2, page_size, heads, dim] tensor on the device of append_key")
    pages, _, page_size, num_heads, head_dim = kv_cache_fp8.shape
    if kv_scales.device != device or kv_scales.dtype != torch.float32 or tuple(kv_scales.shape) != (pages, 2, num_heads) or not kv_scales.is_contiguous():
        raise RuntimeError(f"kv_scales must be a contiguous float32 [{pages}, 2, {num_heads}] tensor on the device of append_key")
    if append_key.stride(2) != 1 or append_value.stride(2) != 1:
        raise RuntimeError("the head_dim axis of append_key / append_value must be contiguous")
    if tuple(append_key.shape[1:]) != (num_heads, head_dim):
        raise RuntimeError(f"append_key shape {tuple(append_key.shape)} mismatch with cache heads {num_heads}, head_dim {head_dim}")
    p = _capi.HstuKvAppendFp8Params()
    p.struct_size = C.sizeof(_capi.HstuKvAppendFp8Params)
    p.src_dtype = _capi.HSTU_BF16 if append_key.dtype == torch.bfloat16 else _capi.HSTU_F16
    p.kv_cache, p.kv_scales = kv_cache_fp8.data_ptr(), kv_scales.data_ptr()
    p.num_pages, p.page_size, p.num_heads, p.head_dim = pages, page_size, num_heads, head_dim
    p.kv_indices, p.kv_indptr = kv_indices.data_ptr(), kv_indptr.data_ptr()
    p.num_indices, p.batch = kv_indices.numel(), kv_indptr.numel() - 1
    if seqlen_offsets.numel() < p.batch:
        raise RuntimeError("seqlen_offsets must have one entry per user of kv_indptr")
    p.append_key, p.append_value = append_key.data_ptr(), append_value.data_ptr()
    p.append_k_stride_n, p.append_k_stride_h = append_key.stride(0), append_key.stride(1)
    p.append_v_stride_n, p.append_v_stride_h = append_value.stride(0), append_value.stride(1)
    p.append_rows = append_key.size(0)
    p.batch_indices, p.positions, p.offsets = batch_indices.data_ptr(), positions.data_ptr(), seqlen_offsets.data_ptr()
    p.nnz_dev, p.nnz_max = nnz_npu.data_ptr(), min(batch_indices.numel(), positions.numel())   # host nnz: a hint only, as above
    need = C.c_uint64(0)
    _capi._check(_capi.lib().hstu_hip_kv_append_fp8_get_workspace_size(C.byref(p), C.byref(need)))
    _require_gpu(append_key, "append_kvcache_fp8")
    with torch.cuda.device(device):
        if workspace is None or workspace.numel() * workspace.element_size() < need.value:
            workspace = torch.empty(need.value, dtype=torch.uint8, device=device)
        _capi._check(_capi.lib().hstu_hip_kv_append_fp8(C.byref(p), workspace.data_ptr(), workspace.numel() * workspace.element_size(), _capi._stream()))
    return workspace


def get_paged_batch_indices_positions(append_indptr, seq_lens, batch_indices, positions) -> None:
    """Fill ``batch_indices`` / ``positions`` (int32, one entry per new token) from ``append_indptr`` (``[batch + 1]``
    offsets of the new tokens of every user) and ``seq_lens`` (``[batch]`` tokens of every user after the append)."""
    device = append_indptr.device
    for t, name in ((append_indptr, "append_indptr"), (seq_lens, "seq_lens"), (batch_indices, "batch_indices"),
                    (positions, "positions")):
        _check_int32_1d(t, device, name)
    batch = append_indptr.numel() - 1
    if seq_lens.numel() < batch:
        raise RuntimeError("seq_lens must have one entry per user of append_indptr")
    _require_gpu(append_indptr, "get_paged_batch_indices_positions")
    with torch.cuda.device(device):
        _capi._check(_capi.lib().hstu_hip_kv_token_positions(batch, append_indptr.data_ptr(), seq_lens.data_ptr(),
                                                             batch_indices.data_ptr(), positions.data_ptr(),
                                                             min(batch_indices.numel(), positions.numel()), _capi._stream()))
