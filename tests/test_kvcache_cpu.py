"""Pins of the paged K/V append oracle and host-side checks of its C ABI (no GPU needed).

The reference's own tests of these kernels are put -> get round trips
(inference/kvcache_manager/test/test_npu_kvcache_manager.py:197-300); the same three cases are restated here."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import kvcache_oracle as KO
from recsdk_amd import _capi, workloads as W

PAGE, HEADS, DIM = 32, 2, 64


def _table(pages):
    return np.zeros((pages, 2, PAGE, HEADS, DIM), dtype=np.float32)


def _put(table, k, v, append_indptr, seq_lens, kv_indices, kv_indptr, offsets=None):
    bi, pos = KO.paged_batch_indices_positions(append_indptr, seq_lens)
    off = np.zeros(len(seq_lens), dtype=np.int32) if offsets is None else offsets
    KO.append_paged_kvcache(table[:, 0], table[:, 1], k, v, bi, pos, off, len(bi), kv_indices, kv_indptr)
    return bi, pos


def test_roundtrip_single_user_two_full_pages():
    rng = np.random.default_rng(0)
    k, v = rng.normal(size=(64, HEADS, DIM)).astype(np.float32), rng.normal(size=(64, HEADS, DIM)).astype(np.float32)
    t = _table(4)
    _put(t, k, v, [0, 64], [64], [3, 1], [0, 2])
    assert np.array_equal(KO.gather_pages(t[:, 0], [3, 1], PAGE), k) and np.array_equal(KO.gather_pages(t[:, 1], [3, 1], PAGE), v)
    assert not t[[0, 2]].any()                                    # pages of nobody stay untouched


def test_roundtrip_several_users_and_ragged_last_page():
    rng = np.random.default_rng(1)
    lens = [64, 33, 0, 1]
    n = sum(lens)
    k, v = rng.normal(size=(n, HEADS, DIM)).astype(np.float32), rng.normal(size=(n, HEADS, DIM)).astype(np.float32)
    t = _table(8)
    indptr, ids = [0, 2, 4, 4, 5], [5, 0, 7, 2, 3]
    ap = np.concatenate([[0], np.cumsum(lens)])
    bi, pos = _put(t, k, v, ap, lens, ids, indptr)
    for u, l in enumerate(lens):
        got = KO.gather_pages(t[:, 0], ids[indptr[u]:indptr[u + 1]], l % PAGE or PAGE)
        assert np.array_equal(got[:l], k[ap[u]:ap[u + 1]])
        assert np.array_equal(pos[bi == u], np.arange(l))        # closed form: a user's positions end at seq_len - 1
    assert not t[[2, 3], :, 1:].any() and not t[[1, 4, 6]].any()   # slots past a sequence's end and free pages: untouched


def test_roundtrip_extended_sequence_keeps_the_old_rows():
    rng = np.random.default_rng(2)
    k1, k2 = rng.normal(size=(32, HEADS, DIM)).astype(np.float32), rng.normal(size=(40, HEADS, DIM)).astype(np.float32)
    t = _table(4)
    _put(t, k1, k1 + 1, [0, 32], [32], [2], [0, 1])
    bi, pos = _put(t, k2, k2 + 1, [0, 40], [72], [2, 0, 3], [0, 3])
    assert np.array_equal(pos, np.arange(32, 72))
    got = KO.gather_pages(t[:, 0], [2, 0, 3], 8)
    assert np.array_equal(got[:32], k1) and np.array_equal(got[32:], k2)
    assert np.array_equal(KO.gather_pages(t[:, 1], [2, 0, 3], 8)[32:], k2 + 1)


def test_append_matches_a_vectorised_derivation_with_offsets_and_hnd_layout():
    """Second derivation without a token loop: fancy-indexed scatter; also the per-user source offsets and layout 1."""
    c = W.kv_append_config(3, users=5, heads=HEADS, dim=DIM, prev_lo=0, prev_hi=70, new_lo=0, new_hi=90, page_size=PAGE, dtype=torch.float32)
    bi, pos = KO.paged_batch_indices_positions(c["append_indptr"].numpy(), c["seq_lens"].numpy())
    # source rows shifted per user: user u's rows sit u*3 rows further down in a longer buffer
    off = (np.arange(5) * 3).astype(np.int32)
    src_rows = np.arange(c["nnz"]) + off[bi]
    ak = np.zeros((c["nnz"] + 20, HEADS, DIM), dtype=np.float32)
    av = np.zeros_like(ak)
    ak[src_rows], av[src_rows] = c["append_key"].numpy(), c["append_value"].numpy()
    ids, indptr = c["kv_indices"].numpy(), c["kv_indptr"].numpy()
    for layout in (0, 1):
        t = c["kv_cache"].numpy().copy()
        want = t.copy()
        pages = ids[indptr[bi] + pos // PAGE]
        want[pages, 0, pos % PAGE], want[pages, 1, pos % PAGE] = ak[src_rows], av[src_rows]
        if layout == 1:
            t = np.ascontiguousarray(t.transpose(0, 1, 3, 2, 4))
        KO.append_paged_kvcache(t[:, 0], t[:, 1], ak, av, bi, pos, off, c["nnz"], ids, indptr, kv_layout=layout)
        assert np.array_equal(t.transpose(0, 1, 3, 2, 4) if layout == 1 else t, want)
    # the rows cached before the append are still there
    for u in range(5):
        got = KO.gather_pages(want[:, 0], ids[indptr[u]:indptr[u + 1]], int(c["kv_last_page_len"][u]))
        assert np.array_equal(got[:c["prev"][u]], c["history"][u][0].numpy())


# ---- C ABI, host side ---------------------------------------------------------------------------
def _kv_params(**over):
    p = _capi.HstuKvAppendParams()
    p.struct_size = C.sizeof(_capi.HstuKvAppendParams)
    p.elem_bytes = 2
    for f in ("k_cache", "v_cache", "append_key", "append_value", "kv_indices", "kv_indptr", "batch_indices", "positions", "offsets", "nnz_dev"):
        setattr(p, f, 0x1000)                # never dereferenced on the host
    p.stride_page, p.stride_n, p.stride_h = 2 * PAGE * HEADS * DIM, HEADS * DIM, DIM
    p.num_pages, p.page_size, p.num_heads, p.head_dim = 4, PAGE, HEADS, DIM
    p.num_indices, p.batch, p.append_rows = 4, 2, 10
    p.append_k_stride_n = p.append_v_stride_n = HEADS * DIM
    p.append_k_stride_h = p.append_v_stride_h = DIM
    p.nnz_max = 0                            # nothing to launch: validation only
    for k, v in over.items():
        setattr(p, k, v)
    return p


def _append(p):
    rc = _capi.lib().hstu_hip_kv_append(C.byref(p), None)
    return rc, _capi.lib().hstu_hip_last_error().decode()


def test_kv_append_validation():
    assert _append(_kv_params())[0] == 0
    rc, msg = _append(_kv_params(struct_size=8))
    assert rc == -1 and "size mismatch" in msg
    rc, msg = _append(_kv_params(elem_bytes=4))
    assert rc == -1 and "2-byte dtype" in msg                     # pybind.cpp:46-55
    rc, msg = _append(_kv_params(head_dim=80))
    assert rc == -1 and "head_dim expect 64, 128, 256 or 512" in msg   # dispatch_head_dim.h:22-48
    rc, msg = _append(_kv_params(positions=None))
    assert rc == -1 and "must not be NULL" in msg
    rc, msg = _append(_kv_params(stride_n=HEADS * DIM + 4))
    assert rc == -2 and "multiples of 8" in msg
    rc, msg = _append(_kv_params(v_cache=0x1008))
    assert rc == -2 and "16-byte aligned" in msg
    rc = _capi.lib().hstu_hip_kv_token_positions(0, 0x1000, 0x1000, 0x1000, 0x1000, 4, None)
    assert rc == -1 and "batch must be positive" in _capi.lib().hstu_hip_last_error().decode()
    rc = _capi.lib().hstu_hip_kv_token_positions(2, None, 0x1000, 0x1000, 0x1000, 4, None)
    assert rc == -1 and "must not be NULL" in _capi.lib().hstu_hip_last_error().decode()


def test_host_mirror_checks_like_the_reference_binding():
    """Messages of pybind.cpp:63-83, and no CPU path."""
    from recsdk_amd import kvcache
    i32 = lambda n: torch.zeros(n, dtype=torch.int32)
    k = torch.zeros(4, HEADS, DIM, dtype=torch.bfloat16)
    cache = torch.zeros(2, 2, PAGE, HEADS, DIM, dtype=torch.bfloat16)
    kc, vc = cache.unbind(1)
    args = lambda **o: [o.get("k", k), o.get("v", k), o.get("bi", i32(4)), i32(4), i32(1), i32(1), 4, kc, vc, i32(2), i32(2), i32(1), o.get("layout", 0)]
    with pytest.raises(RuntimeError, match="2-byte dtype"):
        kvcache.append_kvcache(*args(k=k.float()))
    with pytest.raises(RuntimeError, match="same shape"):
        kvcache.append_kvcache(*args(v=k[:2]))
    with pytest.raises(RuntimeError, match="batch_indices must have dtype int32"):
        kvcache.append_kvcache(*args(bi=torch.zeros(4, dtype=torch.int64)))
    with pytest.raises(RuntimeError, match=r"kv_layout must be 0 \(NHD\) or 1 \(HND\), got 2"):
        kvcache.append_kvcache(*args(layout=2))
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        kvcache.append_kvcache(*args())
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        kvcache.get_paged_batch_indices_positions(i32(2), i32(1), i32(4), i32(4))


def test_fp8_append_oracle_is_whole_page_quantisation_and_bounded():
    """The fp8 append has no reference counterpart; its oracle is pinned by what the definition implies: (1) pages filled
    by one append equal quantising the whole 2-byte page at once (``quantize_kv_cache_fp8``, scale = absmax / 448);
    (2) after a second append every stored value is within the e4m3 step (2^-4 relative to its own magnitude, or half the
    smallest subnormal step of the page's scale) -- twice that for rows that were requantised; (3) a second append that
    needs no larger scale leaves the old bytes alone."""
    import torch
    from oracle import hstu_oracle as O
    g = torch.Generator().manual_seed(3)
    page, heads, dim = 8, 2, 16
    kv_indices, kv_indptr = np.array([2, 0, 3, 1], dtype=np.int32), np.array([0, 2, 4], dtype=np.int32)
    cache = torch.zeros(5, 2, page, heads, dim, dtype=torch.uint8)
    scales = torch.ones(5, 2, heads)
    l1 = [11, 5]
    k1 = torch.randn(sum(l1), heads, dim, generator=g).to(torch.bfloat16)
    v1 = torch.randn(sum(l1), heads, dim, generator=g).to(torch.bfloat16)
    bi, pos = KO.paged_batch_indices_positions([0, 11, 16], l1)
    KO.append_paged_kvcache_fp8(cache, scales, k1, v1, bi, pos, [0, 0], 16, kv_indices, kv_indptr)
    # the same rows in a 2-byte table, quantised page by page
    table = torch.zeros(5, 2, page, heads, dim, dtype=torch.bfloat16)
    t16 = table.view(torch.int16).numpy()
    KO.append_paged_kvcache(t16[:, 0], t16[:, 1], k1.view(torch.int16).numpy(), v1.view(torch.int16).numpy(), bi, pos, [0, 0], 16, kv_indices, kv_indptr)
    want8, want_s = O.quantize_kv_cache_fp8(table)
    touched = [2, 0, 3]
    assert torch.equal(cache[touched], want8[touched]) and torch.equal(scales[touched], want_s[touched])
    assert torch.equal(scales[[1, 4]], torch.ones(2, 2, heads)) and int(cache[[1, 4]].abs().sum()) == 0
    # second append: user 0 gets larger rows (scale of page 0 grows), user 1 smaller ones (scale of page 3 stays)
    before = cache.clone()
    s_before = scales.clone()
    k2 = torch.cat([torch.randn(3, heads, dim, generator=g) * 8, torch.randn(2, heads, dim, generator=g) * 0.01]).to(torch.bfloat16)
    v2 = (k2.float() * 0.5).to(torch.bfloat16)
    bi2, pos2 = KO.paged_batch_indices_positions([0, 3, 5], [14, 7])
    KO.append_paged_kvcache_fp8(cache, scales, k2, v2, bi2, pos2, [0, 0], 5, kv_indices, kv_indptr)
    assert bool((scales[0] > s_before[0]).all()) and torch.equal(scales[3], s_before[3]) and torch.equal(scales[2], s_before[2])
    assert torch.equal(cache[3, :, :5], before[3, :, :5]) and torch.equal(cache[2], before[2])
    assert not torch.equal(cache[0, :, :3], before[0, :, :3])
    deq = O.dequantize_kv_cache_fp8(cache, scales)
    full_k = torch.cat([k1[:11], k2[:3]]).float()
    got_k = torch.cat([deq[2, 0], deq[0, 0, :6]])
    step = scales[[2] * 8 + [0] * 6, 0][:, :, None] * 2.0 ** -9          # half the subnormal spacing 2^-9 ... of e4m3 times the scale
    lim = full_k.abs() * 2.0 ** -4 + step
    lim[8:11] *= 2                                                         # requantised rows
    assert bool(((got_k - full_k).abs() <= lim * 1.001).all())


def test_fp8_append_abi_validation():
    L = _capi.lib()
    def call(ws=0x1000, ws_bytes=1 << 20, **over):
        p = _capi.HstuKvAppendFp8Params()
        p.struct_size = C.sizeof(_capi.HstuKvAppendFp8Params)
        p.src_dtype, p.num_pages, p.page_size, p.num_heads, p.head_dim = _capi.HSTU_BF16, 10, 16, 2, 64
        p.num_indices, p.batch, p.nnz_max, p.append_rows = 4, 2, 8, 8
        p.append_k_stride_n = p.append_v_stride_n = 128
        p.append_k_stride_h = p.append_v_stride_h = 64
        for f in ("kv_cache", "kv_scales", "kv_indices", "kv_indptr", "append_key", "append_value", "batch_indices", "positions", "offsets", "nnz_dev"):
            setattr(p, f, 0x1000)
        for k, v in over.items():
            setattr(p, k, v)
        return L.hstu_hip_kv_append_fp8(C.byref(p), ws, ws_bytes, None), L.hstu_hip_last_error().decode(), p
    for over, text in ((dict(src_dtype=_capi.HSTU_F32), "src_dtype expect float16 or bfloat16"), (dict(head_dim=96), "head_dim expect a power of two"),
                       (dict(num_pages=0), "must be positive"), (dict(kv_scales=None), "must not be NULL")):
        rc, msg, _ = call(**over)
        assert rc == -1 and text in msg, (over, msg)
    rc, msg, _ = call(append_k_stride_h=60)
    assert rc == -2 and "multiples of 8" in msg
    rc, msg, p = call(ws_bytes=16)
    assert rc == -3 and "workspace" in msg
    need = C.c_uint64(0)
    assert L.hstu_hip_kv_append_fp8_get_workspace_size(C.byref(p), C.byref(need)) == 0 and need.value == (72 + 8 * 8) * 4   # maxima, first slots and run counts of all pages (60 words), the count and list of (at most nnz_max) scattered pages (9), the count of runs, padding to 16 bytes (72), 8-word records of (at most nnz_max) runs
    rc, _, _ = call(nnz_max=0)
    assert rc == 0
