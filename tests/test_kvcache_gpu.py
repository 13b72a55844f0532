"""GPU parity of the paged K/V append (through the C ABI, via the host mirror of the reference's binding) against the
oracle: bit-exact, like every byte-moving path; plus the round trip append -> hstu_paged."""
import sys

import numpy as np
import pytest
import torch

from oracle import kvcache_oracle as KO
from recsdk_amd import kvcache, workloads as W
from tests import hstu_testlib as T

pytestmark = pytest.mark.gpu


def say(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def _positions(c):
    bi = torch.full((c["nnz"] + 3,), -7, dtype=torch.int32, device="cuda")   # slack entries must stay untouched
    pos = torch.full_like(bi, -7)
    kvcache.get_paged_batch_indices_positions(c["append_indptr"].cuda(), c["seq_lens"].cuda(), bi, pos)
    return bi, pos


def _append(c, bi, pos, table, layout=0, offsets=None, key=None, value=None, nnz=None):
    kc, vc = table.unbind(1)
    kvcache.append_kvcache(c["append_key"].cuda() if key is None else key, c["append_value"].cuda() if value is None else value, bi, pos,
                           (c["offsets"] if offsets is None else offsets).cuda(), c["nnz_dev"].cuda(), c["nnz"] if nnz is None else nnz,
                           kc, vc, c["kv_indices"].cuda(), c["kv_indptr"].cuda(), c["kv_last_page_len"].cuda(), layout)
    torch.cuda.synchronize()


def _oracle(c, layout=0, offsets=None, key=None, value=None):
    t = c["kv_cache"].view(torch.int16).numpy().copy()
    if layout == 1:
        t = np.ascontiguousarray(t.transpose(0, 1, 3, 2, 4))
    bi, pos = KO.paged_batch_indices_positions(c["append_indptr"].numpy(), c["seq_lens"].numpy())
    k = (c["append_key"] if key is None else key).view(torch.int16).numpy()
    v = (c["append_value"] if value is None else value).view(torch.int16).numpy()
    KO.append_paged_kvcache(t[:, 0], t[:, 1], k, v, bi, pos, (c["offsets"] if offsets is None else offsets).numpy(), c["nnz"],
                            c["kv_indices"].numpy(), c["kv_indptr"].numpy(), kv_layout=layout)
    return bi, pos, t


@pytest.mark.parametrize("dim,heads,page,dtype", [(64, 2, 32, torch.bfloat16), (128, 4, 64, torch.float16), (256, 1, 16, torch.bfloat16),
                                                  (512, 3, 8, torch.bfloat16)])
def test_append_matches_oracle_bit_for_bit(dim, heads, page, dtype):
    say("kv append", dim, heads, page, dtype)
    c = W.kv_append_config(40, users=7, heads=heads, dim=dim, prev_lo=0, prev_hi=100, new_lo=0, new_hi=150, page_size=page, dtype=dtype)
    wbi, wpos, want = _oracle(c)
    bi, pos = _positions(c)
    assert np.array_equal(bi[:c["nnz"]].cpu().numpy(), wbi) and np.array_equal(pos[:c["nnz"]].cpu().numpy(), wpos)
    assert bool((bi[c["nnz"]:] == -7).all()) and bool((pos[c["nnz"]:] == -7).all())
    table = c["kv_cache"].cuda()
    _append(c, bi, pos, table)
    assert np.array_equal(table.cpu().view(torch.int16).numpy(), want)


def test_append_hnd_layout_source_offsets_and_strided_source():
    """kv_layout 1 ([pages, heads, page_size, dim] views), per-user source offsets, append_key as a slice of a wider tensor."""
    say("kv append hnd/offsets/strides")
    c = W.kv_append_config(41, users=4, heads=2, dim=64, prev_lo=0, prev_hi=50, new_lo=1, new_hi=60, page_size=16)
    off = torch.tensor([0, 2, 5, 9], dtype=torch.int32)
    bi_np, _ = KO.paged_batch_indices_positions(c["append_indptr"].numpy(), c["seq_lens"].numpy())
    rows = torch.arange(c["nnz"]) + off[torch.from_numpy(bi_np).long()]
    wide = torch.zeros(c["nnz"] + 9, 2, 2, 64, dtype=torch.bfloat16)            # [rows, k|v, heads, dim]: row stride 2*heads*dim
    wide[rows, 0], wide[rows, 1] = c["append_key"], c["append_value"]
    _, _, want = _oracle(c, layout=1, offsets=off, key=wide[:, 0].contiguous(), value=wide[:, 1].contiguous())
    bi, pos = _positions(c)
    table = c["kv_cache"].transpose(2, 3).contiguous().cuda()                    # [pages, 2, heads, page_size, dim]
    wd = wide.cuda()
    _append(c, bi, pos, table, layout=1, offsets=off, key=wd[:, 0], value=wd[:, 1])
    assert np.array_equal(table.cpu().view(torch.int16).numpy(), want)


def test_append_skips_what_points_outside_and_honours_the_device_count():
    """nnz on the device smaller than the host bound: the tail is not written; a page id outside the table, a negative
    position or a user id outside the batch skip that token (no fault, nothing else disturbed)."""
    say("kv append guards")
    c = W.kv_append_config(42, users=3, heads=2, dim=64, prev_lo=0, prev_hi=0, new_lo=20, new_hi=40, page_size=16)
    bi, pos = _positions(c)
    n = c["nnz"]
    short = dict(c, nnz_dev=torch.tensor([n - 5], dtype=torch.int32))
    _, _, want = _oracle(dict(short, nnz=n - 5))
    table = c["kv_cache"].cuda()
    _append(short, bi, pos, table)
    assert np.array_equal(table.cpu().view(torch.int16).numpy(), want)
    # the host-side nnz is only a hint (the reference's binding ignores it, pybind.cpp:57-61): a stale 0 loses nothing
    table = c["kv_cache"].cuda()
    _append(c, bi, pos, table, nnz=0)
    assert np.array_equal(table.cpu().view(torch.int16).numpy(), _oracle(c)[2])
    # corrupt three tokens of a fresh append
    bad = dict(c, kv_indices=c["kv_indices"].clone())
    first_page_u0 = int(bad["kv_indices"][0])
    bad["kv_indices"][0] = 10 ** 6                   # user 0's first page: its first 16 tokens are skipped
    bi2, pos2 = bi.clone(), pos.clone()
    bi2[n - 1] = 99
    pos2[n - 2] = -3
    table = c["kv_cache"].cuda()
    _append(bad, bi2, pos2, table)
    _, _, want = _oracle(c)
    want[first_page_u0] = 0
    wbi, wpos = KO.paged_batch_indices_positions(c["append_indptr"].numpy(), c["seq_lens"].numpy())
    for t in (n - 1, n - 2):
        u, p = int(wbi[t]), int(wpos[t])
        want[int(c["kv_indices"][int(c["kv_indptr"][u]) + p // 16]), :, p % 16] = 0
    assert np.array_equal(table.cpu().view(torch.int16).numpy(), want)


@pytest.mark.parametrize("dtype", [torch.bfloat16])
def test_roundtrip_append_then_hstu_paged(dtype):
    """The write side feeds the read side: a table filled by two appends (history, then its extension) gives the paged
    forward the bits it gets from the table the workload builder filled on the host."""
    say("kv append -> hstu_paged", dtype)
    cfg = W.paged_config(43, 5, 2, 128, 60, 400, 40, 64, dtype)
    users, ps = 5, 64
    hist = cfg["hist"]
    ref_table = cfg["kv_cache"]
    po, ids = cfg["page_offsets"], cfg["page_ids"]
    rows = [torch.cat([ref_table[int(ids[p])] for p in range(int(po[u]), int(po[u + 1]))], dim=1)[:, :hist[u]] for u in range(users)]
    table = torch.zeros_like(ref_table).cuda()
    done = [0] * users
    for frac in (0.4, 1.0):
        upto = [max(int(h * frac), 1) if frac < 1 else h for h in hist]
        new = [a - b for a, b in zip(upto, done)]
        k = torch.cat([rows[u][0, done[u]:upto[u]] for u in range(users)]).cuda()
        v = torch.cat([rows[u][1, done[u]:upto[u]] for u in range(users)]).cuda()
        n = sum(new)
        bi = torch.empty(n, dtype=torch.int32, device="cuda")
        pos = torch.empty_like(bi)
        kvcache.get_paged_batch_indices_positions(W.offsets(new, torch.int32).cuda(), torch.tensor(upto, dtype=torch.int32).cuda(), bi, pos)
        kc, vc = table.unbind(1)
        kvcache.append_kvcache(k, v, bi, pos, torch.zeros(users, dtype=torch.int32, device="cuda"), torch.tensor([n], dtype=torch.int32).cuda(), n,
                               kc, vc, ids.cuda(), po.cuda(), cfg["last_page_len"].cuda(), 0)
        done = upto
    torch.cuda.synchronize()
    assert torch.equal(table.cpu(), ref_table)
    out_ref, _ = T.run_capi(cfg, op="paged")
    out, _ = T.run_capi(dict(cfg, kv_cache=table.cpu()), op="paged")
    assert torch.equal(out, out_ref)
    T.assert_parity(out, T.oracle_paged(cfg), dtype, what="paged forward over the appended table")


def _fp8_scenario(seed, users, heads, dim, page, dtype):
    """Two appends per user: a prefill of L1 rows, then A more rows whose amplitude is larger for some users (their
    pages' scales grow and the old rows are requantised) and smaller for others (scales stay)."""
    g = torch.Generator().manual_seed(seed)
    l1 = torch.randint(0, 3 * page, (users,), generator=g)
    add = torch.randint(0, 2 * page + 5, (users,), generator=g)
    need = ((l1 + add + page - 1) // page).clamp(min=1)
    pages = int(need.sum()) + 3
    perm = torch.randperm(pages, generator=g)[: int(need.sum())].to(torch.int32)
    indptr = torch.cat([torch.zeros(1, dtype=torch.int64), need.cumsum(0)]).to(torch.int32)
    amp = torch.tensor([0.25, 1.0, 4.0])[torch.randint(0, 3, (users,), generator=g)]
    steps = []
    for n_new, seq, a in ((l1, l1, torch.ones(users)), (add, l1 + add, amp)):
        ip = torch.cat([torch.zeros(1, dtype=torch.int64), n_new.cumsum(0)]).to(torch.int32)
        rows = int(n_new.sum())
        scale = torch.repeat_interleave(a, n_new)[:, None, None]
        k = (torch.randn(rows, heads, dim, generator=g) * scale).to(dtype)
        v = (torch.randn(rows, heads, dim, generator=g) * scale * 0.5).to(dtype)
        steps.append(dict(append_indptr=ip, seq_lens=seq.to(torch.int32), key=k, value=v, nnz=rows))
    return dict(pages=pages, kv_indices=perm, kv_indptr=indptr, steps=steps, users=users)


def _token_order(bi, nnz, order, seed):
    """A permutation of the new tokens: 'runs' keeps them as they come; 'mixed' shuffles the tokens of every third user,
    reverses those of the next and keeps the rest (pages with one run and pages with many in one call)."""
    perm = np.arange(nnz)
    if order == "runs":
        return perm
    rng = np.random.default_rng(seed)
    for b in np.unique(bi[:nnz]):
        idx = np.nonzero(bi[:nnz] == b)[0]
        if b % 3 == 0:
            perm[idx] = rng.permutation(idx)
        elif b % 3 == 1:
            perm[idx] = idx[::-1]
    return perm


@pytest.mark.parametrize("dim,heads,page,dtype,order", [(128, 4, 64, torch.bfloat16, "runs"), (64, 2, 32, torch.float16, "runs"),
                                                        (256, 1, 16, torch.bfloat16, "runs"), (8, 3, 8, torch.bfloat16, "runs"),
                                                        (128, 4, 64, torch.bfloat16, "mixed"), (32, 2, 24, torch.float16, "mixed"),
                                                        (512, 1, 64, torch.bfloat16, "runs"), (512, 2, 48, torch.float16, "mixed"),
                                                        (256, 2, 64, torch.bfloat16, "mixed"), (16, 1, 200, torch.bfloat16, "runs")])
def test_fp8_append_matches_oracle_bit_for_bit(dim, heads, page, dtype, order):
    """Bytes and scales after a prefill and after an extension of partly filled pages, against the oracle's restatement
    of this library's own definition (no reference counterpart: parity with the reference unpinned by construction).
    'runs': tokens in the order of hstu_hip_kv_token_positions (every page finished by the one-pass kernel, or, for pages
    of more than 2048 cells of 8 elements, by the kernels for scattered pages); 'mixed': tokens of some users out of order."""
    say("kv append fp8", dim, heads, page, dtype, order)
    s = _fp8_scenario(5, 9, heads, dim, page, dtype)
    cache = torch.zeros(s["pages"], 2, page, heads, dim, dtype=torch.uint8)
    scales = torch.ones(s["pages"], 2, heads)
    dc, ds = cache.cuda(), scales.cuda()
    ws = None
    zeros = torch.zeros(s["users"], dtype=torch.int32)
    for n, st in enumerate(s["steps"]):
        bi, pos = KO.paged_batch_indices_positions(st["append_indptr"].numpy(), st["seq_lens"].numpy())
        perm = _token_order(bi, st["nnz"], order, 100 + n)
        bi, pos = bi.copy(), pos.copy()
        bi[: st["nnz"]], pos[: st["nnz"]] = bi[perm], pos[perm]
        key, value = st["key"][torch.from_numpy(perm)], st["value"][torch.from_numpy(perm)]     # row of token i = i (offsets are zero)
        KO.append_paged_kvcache_fp8(cache, scales, key, value, bi, pos, zeros.numpy(), st["nnz"], s["kv_indices"].numpy(),
                                    s["kv_indptr"].numpy())
        dbi = torch.empty(max(st["nnz"], 1), dtype=torch.int32, device="cuda")
        dpos = torch.empty_like(dbi)
        if order == "runs":
            kvcache.get_paged_batch_indices_positions(st["append_indptr"].cuda(), st["seq_lens"].cuda(), dbi, dpos)
        else:
            dbi[: st["nnz"]] = torch.from_numpy(bi[: st["nnz"]].astype(np.int32)).cuda()
            dpos[: st["nnz"]] = torch.from_numpy(pos[: st["nnz"]].astype(np.int32)).cuda()
        ws = kvcache.append_kvcache_fp8(key.cuda(), value.cuda(), dbi, dpos, zeros.cuda(),
                                        torch.tensor([st["nnz"]], dtype=torch.int32, device="cuda"), st["nnz"], dc, ds,
                                        s["kv_indices"].cuda(), s["kv_indptr"].cuda(), workspace=ws)
        torch.cuda.synchronize()
        assert torch.equal(ds.cpu(), scales), f"scales after step {n}"
        diff = (dc.cpu() != cache)
        assert not bool(diff.any()), f"bytes after step {n}: {int(diff.sum())} differ"
    assert int((cache != 0).sum()) > 0


def test_fp8_append_skips_invalid_tokens_and_tokens_past_the_device_count():
    """Tokens with a user index or a position outside what the host described are skipped (the reference's kernel checks
    nothing: append_paged_kvcache_kernel.h:42-76; this library does, so that a bad index cannot write outside the table),
    and so are the tokens behind the count in device memory.  A skipped token in the middle of a run cuts the run in two:
    its page then goes through the kernels for scattered pages.  Expected: the oracle on the valid tokens alone."""
    say("kv append fp8, invalid tokens")
    heads, dim, page, dtype = 2, 64, 32, torch.bfloat16
    s = _fp8_scenario(11, 7, heads, dim, page, dtype)
    cache = torch.zeros(s["pages"], 2, page, heads, dim, dtype=torch.uint8)
    scales = torch.ones(s["pages"], 2, heads)
    dc, ds = cache.cuda(), scales.cuda()
    zeros = torch.zeros(s["users"], dtype=torch.int32)
    g = torch.Generator().manual_seed(3)
    for n, st in enumerate(s["steps"]):
        nnz = st["nnz"]
        bi, pos = KO.paged_batch_indices_positions(st["append_indptr"].numpy(), st["seq_lens"].numpy())
        bi, pos = bi.copy(), pos.copy()
        bad = torch.randperm(nnz, generator=g)[:9].numpy()
        bi[bad[:3]] = -1
        bi[bad[3:5]] = s["users"]
        pos[bad[5:7]] = -2
        pos[bad[7:9]] = 10 ** 6                       # far behind the user's pages
        count = nnz - 4                                 # the last four tokens are padding
        ok = np.ones(nnz, dtype=bool)
        ok[bad] = False
        ok[count:] = False
        keep = np.nonzero(ok)[0]
        KO.append_paged_kvcache_fp8(cache, scales, st["key"][torch.from_numpy(keep)], st["value"][torch.from_numpy(keep)], bi[keep], pos[keep],
                                    zeros.numpy(), len(keep), s["kv_indices"].numpy(), s["kv_indptr"].numpy())
        kvcache.append_kvcache_fp8(st["key"].cuda(), st["value"].cuda(), torch.from_numpy(bi.astype(np.int32)).cuda(),
                                   torch.from_numpy(pos.astype(np.int32)).cuda(), zeros.cuda(),
                                   torch.tensor([count], dtype=torch.int32, device="cuda"), nnz, dc, ds, s["kv_indices"].cuda(), s["kv_indptr"].cuda())
        torch.cuda.synchronize()
        assert torch.equal(ds.cpu(), scales), f"scales after step {n}"
        assert torch.equal(dc.cpu(), cache), f"bytes after step {n}"


def test_fp8_append_of_a_few_tokens_into_a_large_table_with_a_dirty_workspace():
    """The work of a call follows the new tokens: a 20000-page table, 11 new tokens of two users, a workspace full of
    arbitrary bytes.  Only the touched pages and their scales change."""
    say("kv append fp8, large table")
    pages, page, heads, dim = 20000, 8, 1, 8
    g = torch.Generator().manual_seed(77)
    kv_indices = torch.tensor([17, 19999, 4, 12345, 6], dtype=torch.int32)      # user 0: pages 17, 19999, 4; user 1: 12345, 6
    kv_indptr = torch.tensor([0, 3, 5], dtype=torch.int32)
    append_indptr = torch.tensor([0, 7, 11], dtype=torch.int32)                # 7 and 4 new tokens
    seq_lens = torch.tensor([19, 12], dtype=torch.int32)                       # lengths after the append: positions 12..18 and 8..11
    key = torch.randn(11, heads, dim, generator=g).to(torch.bfloat16)
    value = torch.randn(11, heads, dim, generator=g).to(torch.bfloat16)
    cache = torch.zeros(pages, 2, page, heads, dim, dtype=torch.uint8)
    scales = torch.ones(pages, 2, heads)
    bi, pos = KO.paged_batch_indices_positions(append_indptr.numpy(), seq_lens.numpy())
    zeros = torch.zeros(2, dtype=torch.int32)
    KO.append_paged_kvcache_fp8(cache, scales, key, value, bi, pos, zeros.numpy(), 11, kv_indices.numpy(), kv_indptr.numpy())
    dc, ds = torch.zeros_like(cache).cuda(), torch.ones_like(scales).cuda()
    dbi = torch.empty(11, dtype=torch.int32, device="cuda")
    dpos = torch.empty_like(dbi)
    kvcache.get_paged_batch_indices_positions(append_indptr.cuda(), seq_lens.cuda(), dbi, dpos)
    ws = torch.full((pages * (2 * heads + 2) * 4 + 4096,), 0xA5, dtype=torch.uint8, device="cuda")
    kvcache.append_kvcache_fp8(key.cuda(), value.cuda(), dbi, dpos, zeros.cuda(), torch.tensor([11], dtype=torch.int32, device="cuda"), 11,
                               dc, ds, kv_indices.cuda(), kv_indptr.cuda(), workspace=ws)
    torch.cuda.synchronize()
    assert torch.equal(ds.cpu(), scales) and torch.equal(dc.cpu(), cache)
    touched = sorted({int(kv_indices[int(kv_indptr[b]) + int(p) // page]) for b, p in zip(bi[:11], pos[:11])})
    assert touched == [4, 6, 19999], touched     # positions 12..18 of user 0 -> its second and third page; 8..11 of user 1 -> its second
    rest = torch.ones(pages, dtype=torch.bool)
    rest[touched] = False
    assert int((dc.cpu()[rest] != 0).sum()) == 0 and bool((ds.cpu()[rest] == 1).all())


def test_fp8_prefill_equals_whole_page_quantisation_and_feeds_paged_fp8():
    """One append into an empty table = quantising the 2-byte table (appended by the 2-byte kernel) page by page, which
    is what the hstu_paged_fp8 tests feed the attention with."""
    say("kv append fp8 prefill == quantize_pages_fp8")
    c = W.kv_append_config(41, users=6, heads=4, dim=128, prev_lo=0, prev_hi=0, new_lo=1, new_hi=200, page_size=64, dtype=torch.bfloat16)
    c["kv_cache"].zero_()
    # users start empty: every page is filled by this append alone
    assert int((c["seq_lens"] - (c["append_indptr"][1:] - c["append_indptr"][:-1])).abs().sum()) == 0
    bi, pos = _positions(c)
    table = c["kv_cache"].cuda()
    _append(c, bi, pos, table)
    want8, want_s = W.quantize_pages_fp8(table.cpu())
    cache8 = torch.zeros(table.shape, dtype=torch.uint8, device="cuda")
    sc = torch.ones(table.shape[0], 2, table.shape[3], device="cuda")
    kvcache.append_kvcache_fp8(c["append_key"].cuda(), c["append_value"].cuda(), bi, pos, c["offsets"].cuda(), c["nnz_dev"].cuda(), c["nnz"],
                               cache8, sc, c["kv_indices"].cuda(), c["kv_indptr"].cuda())
    torch.cuda.synchronize()
    touched = torch.zeros(table.shape[0], dtype=torch.bool)
    touched[c["kv_indices"].long()] = True
    assert torch.equal(sc.cpu()[touched], want_s[touched])
    assert torch.equal(cache8.cpu()[touched], want8.view(torch.uint8)[touched])


@pytest.mark.parametrize("dtype,spread", [(torch.bfloat16, False), (torch.float16, True), (torch.bfloat16, True)])
def test_fp8_prefill_at_the_bench_shape_against_torch_on_the_gpu(dtype, spread):
    """Config 5's history (32 users x U[1024, 4096] tokens, 4 heads x 128, 64-token pages) is too long for the token loop
    of the oracle; the prefill is checked through what it must equal: the 2-byte table written by the 2-byte append
    (bit-exact against the oracle at smaller sizes), quantised page by page with torch's own GPU routines (a true
    division per element: 87 million quotients against the kernel's shared-reciprocal division).  `spread`: every token's
    rows scaled by a power of two or a random factor over 18 octaves, so that the scales cover many binades and, for the
    powers of two, most quotients are exact and sit on e4m3 ties."""
    say("kv append fp8 at the bench shape", dtype, spread)
    c = W.kv_append_config(0, users=32, heads=4, dim=128, prev_lo=0, prev_hi=0, new_lo=1024, new_hi=4096, page_size=64, dtype=dtype)
    if spread:
        g = torch.Generator().manual_seed(9)
        rows = c["append_key"].shape[0]
        e = torch.randint(-12, 7, (rows, 1, 1), generator=g).float()
        amp = torch.where(torch.rand(rows, 1, 1, generator=g) < 0.5, torch.exp2(e), torch.exp2(e + torch.rand(rows, 1, 1, generator=g)))
        c["append_key"] = (c["append_key"].float() * amp).to(dtype)
        c["append_value"] = (c["append_value"].float() * amp * 0.75).to(dtype)
    d = W.to_device(c)
    n = c["nnz"]
    bi = torch.empty(n, dtype=torch.int32, device="cuda")
    pos = torch.empty_like(bi)
    kvcache.get_paged_batch_indices_positions(d["append_indptr"], d["seq_lens"], bi, pos)
    table = d["kv_cache"]
    kc, vc = table.unbind(1)
    kvcache.append_kvcache(d["append_key"], d["append_value"], bi, pos, d["offsets"], d["nnz_dev"], n, kc, vc, d["kv_indices"], d["kv_indptr"],
                           d["kv_last_page_len"], 0)
    cache8 = torch.zeros(table.shape, dtype=torch.uint8, device="cuda")
    sc = torch.ones(table.shape[0], 2, table.shape[3], device="cuda")
    kvcache.append_kvcache_fp8(d["append_key"], d["append_value"], bi, pos, d["offsets"], d["nnz_dev"], n, cache8, sc, d["kv_indices"], d["kv_indptr"])
    torch.cuda.synchronize()
    x = table.float()
    amax = x.abs().amax(dim=(2, 4))
    # tensor / tensor: torch divides for real there (a tensor over a Python number is multiplied by its rounded reciprocal)
    want_s = torch.where(amax > 0, amax / torch.full_like(amax, 448.0), torch.ones_like(amax))
    assert torch.equal(sc, want_s)
    want8 = (x / want_s[:, :, None, :, None]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
    diff = cache8 != want8
    assert not bool(diff.any()), f"{int(diff.sum())} of {diff.numel()} bytes differ"
    # and back: every stored value within the e4m3 step of the original
    deq = cache8.view(torch.float8_e4m3fn).float() * sc[:, :, None, :, None]
    lim = x.abs() * 2.0 ** -4 + sc[:, :, None, :, None] * 2.0 ** -10
    assert bool(((deq - x).abs() <= lim * 1.001).all())
