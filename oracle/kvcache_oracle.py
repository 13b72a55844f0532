"""CPU oracle for the write side of the paged K/V cache.  TEST INFRASTRUCTURE ONLY.

Restates, token by token, the two kernels of the reference's cache manager that sit before ``hstu_paged``; used by
``tests/`` and by the ``cpu_baseline`` leg of ``bench.py``.  Nothing in the shipped package imports it.

Definition followed (reference file:line):

* ``append_paged_kvcache``: inference/kvcache_manager/src/kernels/append_paged_kvcache/append_paged_kvcache_kernel.h:42-76
  (token i of user b = batch_indices[i] -> page indices[indptr[b] + positions[i] // page_size], slot
  positions[i] % page_size; source row i + offsets[b]); strides as the binding derives them (src/pybind.cpp:84-105).
* ``paged_batch_indices_positions``:
  .../get_paged_batch_indices_positions/get_paged_batch_indices_positions_kernel.h:24-49.
* ``gather_pages`` (the read-back of the reference's round-trip tests, ``NPUKVCacheManager.get``):
  recsys_kvcache_manager/npu_kvcache_manager.py:200-215 -- the first rows of a user's pages, the last page cut at
  kv_last_page_len.

* ``append_paged_kvcache_fp8``: NO reference counterpart (the reference's manager stores 2-byte rows unscaled).
  Build-defined: routing as above; a touched (page, K|V, head) ends up as ``rne_e4m3(clamp(x / s, -448, 448))`` with
  ``s = max(s_before, absmax(new) / 448)`` if rows sit below the first new slot, else ``absmax(new) / 448`` (1 if 0);
  old rows are requantised from ``q * s_before`` when s grew.  PARITY UNPINNED against the reference by construction;
  pinned here against whole-page quantisation (a page filled by one append equals ``quantize_kv_cache_fp8`` of the
  2-byte page) and by the error bound of e4m3 (tests/test_kvcache_cpu.py).

Pinning status (tests/test_kvcache_cpu.py): the reference holds no golden vectors for these kernels; its own tests
are put -> get round trips (inference/kvcache_manager/test/test_npu_kvcache_manager.py:197-300: one user, several
users, a sequence extended by a second append).  The oracle is pinned by the same round trips (what was appended is
what the pages hold, in position order, and nothing else in the table changes), by a vectorised second derivation
that shares no loop with it, and by the closed form of the positions (arange per user ending at seq_len).  PINNED
"""
from __future__ import annotations

import numpy as np


def paged_batch_indices_positions(append_indptr, seq_lens):
    """(batch_indices, positions), int32, one entry per new token."""
    append_indptr = np.asarray(append_indptr, dtype=np.int64)
    seq_lens = np.asarray(seq_lens, dtype=np.int64)
    n = int(append_indptr[-1])
    bi = np.zeros(n, dtype=np.int32)
    pos = np.zeros(n, dtype=np.int32)
    for b in range(len(append_indptr) - 1):
        first, count = int(append_indptr[b]), int(append_indptr[b + 1] - append_indptr[b])
        for i in range(count):
            bi[first + i] = b
            pos[first + i] = seq_lens[b] - count + i
    return bi, pos


def append_paged_kvcache(k_cache, v_cache, append_key, append_value, batch_indices, positions, offsets, nnz,
                         kv_indices, kv_indptr, kv_layout=0):
    """In-place append into ``k_cache`` / ``v_cache`` (numpy views ``[pages, page_size, heads, dim]`` for layout 0,
    ``[pages, heads, page_size, dim]`` for layout 1).  Returns nothing."""
    page_size = k_cache.shape[2] if kv_layout == 1 else k_cache.shape[1]
    for i in range(int(nnz)):
        b = int(batch_indices[i])
        page_iter, entry = divmod(int(positions[i]), page_size)
        page = int(kv_indices[int(kv_indptr[b]) + page_iter])
        row = i + int(offsets[b])
        if kv_layout == 1:
            k_cache[page, :, entry, :] = append_key[row]
            v_cache[page, :, entry, :] = append_value[row]
        else:
            k_cache[page, entry] = append_key[row]
            v_cache[page, entry] = append_value[row]


def gather_pages(cache, page_ids, last_page_len, kv_layout=0):
    """Rows of one user: its pages in order, the last one cut at ``last_page_len``."""
    rows = []
    for n, page in enumerate(page_ids):
        blk = cache[int(page)]
        if kv_layout == 1:
            blk = blk.transpose(1, 0, 2)
        rows.append(blk[: int(last_page_len)] if n == len(page_ids) - 1 else blk)
    return np.concatenate(rows) if rows else cache[:0].reshape((0,) + cache.shape[2:])


def append_paged_kvcache_fp8(cache_u8, scales, append_key, append_value, batch_indices, positions, offsets, nnz,
                             kv_indices, kv_indptr):
    """In-place append into ``cache_u8`` (torch uint8 ``[pages, 2, page_size, heads, dim]``) and ``scales`` (torch
    float32 ``[pages, 2, heads]``); ``append_key`` / ``append_value`` torch ``[rows, heads, dim]`` (fp16 / bf16)."""
    import torch
    page_size = cache_u8.shape[2]
    new = {}   # page -> list of (slot, source row)
    for i in range(int(nnz)):
        b = int(batch_indices[i])
        page_iter, slot = divmod(int(positions[i]), page_size)
        page = int(kv_indices[int(kv_indptr[b]) + page_iter])
        new.setdefault(page, []).append((slot, i + int(offsets[b])))
    f8 = cache_u8.view(torch.float8_e4m3fn)
    for page, items in new.items():
        first = min(s_ for s_, _ in items)
        for kv, src in ((0, append_key), (1, append_value)):
            rows = torch.stack([src[r].float() for _, r in items])            # [t, heads, dim]
            cand = rows.abs().amax(dim=(0, 2)) / 448.0                          # [heads]
            s_old = scales[page, kv].clone()
            if first > 0:
                s_new = torch.maximum(s_old, cand)
                grew = s_new != s_old
                old = f8[page, kv, :first].float() * s_old[None, :, None]
                req = (old / s_new[None, :, None]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
                keep = f8[page, kv, :first].clone()
                f8[page, kv, :first] = torch.where(grew[None, :, None], req.view(torch.uint8), keep.view(torch.uint8)).view(torch.float8_e4m3fn)
            else:
                s_new = torch.where(cand > 0, cand, torch.ones_like(cand))
            scales[page, kv] = s_new
            for (slot, r) in items:
                f8[page, kv, slot] = (src[r].float() / s_new[:, None]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
