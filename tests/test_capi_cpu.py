"""CPU-side checks of the boundary: the C-ABI library loads and exports every symbol that
include/hstu_hip.h declares, the ctypes mirror of the argument block matches the C struct, argument
validation speaks the reference's messages, and the torch op layer rejects what the reference rejects
(test_hstu_jagged_forward.py:508-711).  No kernel is launched here."""
import ctypes as C
import os
import re

import pytest
import torch

import recsdk_amd
from recsdk_amd import _capi
from oracle import hstu_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    names = set()
    inc = os.path.join(ROOT, "include")
    for h in sorted(os.listdir(inc)):
        src = re.sub(r"/\*.*?\*/", "", open(os.path.join(inc, h)).read(), flags=re.S)
        names |= set(re.findall(r"\b(hstu_hip_\w+)\s*\(", src))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    names = _declared_functions()
    assert len(names) >= 9
    lib = _capi.lib()
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/*.h but not exported"
    assert sorted(names) == sorted(_capi.EXPORTS)
    assert lib.hstu_hip_abi_version() == 1


def _params(**over):
    p = _capi.HstuFwdParams()
    p.struct_size = C.sizeof(_capi.HstuFwdParams)
    p.dtype, p.index_type = _capi.HSTU_BF16, _capi.HSTU_I64
    for f in ("q", "k", "v", "out", "seq_offset_q", "seq_offset_k"):
        setattr(p, f, 0x1000)       # never dereferenced on the host
    p.total_q = p.total_k = 100
    p.batch, p.heads_q, p.heads_k, p.dim_qk, p.dim_v = 2, 4, 4, 128, 128
    p.max_seq_len_q = p.max_seq_len_k = 64
    p.silu_scale, p.alpha = 1 / 64, 0.1
    for k, v in over.items():
        setattr(p, k, v)
    return p


def _ws(p, op="jagged"):
    n = C.c_uint64(123)
    rc = getattr(_capi.lib(), f"hstu_hip_{op}_forward_get_workspace_size")(C.byref(p), C.byref(n))
    return rc, n.value, _capi.lib().hstu_hip_last_error().decode()


def test_noalloc_entry_rejects_a_work_list_beyond_its_fixed_array():
    # host checks only: nothing is launched and no device is touched before the size check
    p = _params(batch=2048, heads_q=16, heads_k=16, max_seq_len_q=20480, max_seq_len_k=20480, total_q=2048 * 20480, total_k=2048 * 20480)
    assert _capi.lib().hstu_hip_jagged_forward_noalloc(C.byref(p), None) == -3
    msg = _capi.lib().hstu_hip_last_error().decode()
    assert "hstu_hip_jagged_forward_noalloc holds %d" % _capi.NOALLOC_SCRATCH_BYTES in msg
    # and the ordinary validation comes first
    assert _capi.lib().hstu_hip_jagged_forward_noalloc(C.byref(_params(batch=0)), None) == -1


def test_struct_layout_matches_and_workspace_size():
    rc, n, msg = _ws(_params())
    # a size mismatch between ctypes and C would be rejected here.  MFMA kernels keep their work list in the
    # workspace: 16 header words + 8-word records: 8 XCD lists of cap records + an overflow list of `bound` records, with
    # bound = min(total_q // 128 + batch, batch * ceil(max_seq_len_q / 128)) * heads_q, cap = ceil(bound / 8) + tiles
    assert rc == 0 and n == 1024, msg                     # 4 * (16 + 8 * (8 * 2 + 8)) = 832, rounded up to 256
    rc, n, msg = _ws(_params(batch=257, total_q=25700))
    assert rc == 0 and n == 66304, msg                    # 4 * (16 + 8 * (8 * 130 + 1028)) = 66240, rounded up
    # few Q tiles, long K: the K range is split over 4 workgroups per tile and the fp32 partial sums follow the list
    rc, n, msg = _ws(_params(max_seq_len_k=4096))
    assert rc == 0 and n == 4 * (16 + 8 * (8 * (4 + 4) + 32)) // 256 * 256 + 256 + 4 * 100 * 4 * 128 * 4, msg
    rc, n, msg = _ws(_params(dtype=_capi.HSTU_F32))
    assert rc == 0 and n == 0, msg          # the generic kernel needs none
    rc, n, msg = _ws(_params(flags=_capi.FLAG_FORCE_GENERIC))
    assert rc == 0 and n == 0, msg
    # a call without the workspace is refused before anything is launched
    pp = _params()
    rc = _capi.lib().hstu_hip_jagged_forward(C.byref(pp), None, 0, None)
    assert rc == -3 and "workspace" in _capi.lib().hstu_hip_last_error().decode()
    rc, _, msg = _ws(_params(struct_size=8))
    assert rc == -1 and "size mismatch" in msg


@pytest.mark.parametrize("over,needle", [
    (dict(batch=0), "batchSize limit (0, 2048]"),
    (dict(batch=2049), "batchSize limit (0, 2048]"),
    (dict(max_seq_len_q=20481), "maxSeqLen expect in [1, 20480]"),
    (dict(max_seq_len_k=0), "maxSeqLenK expect in [1, 20480]"),
    (dict(heads_q=17, heads_k=17), "head num expect in [1, 16]"),
    (dict(heads_q=3, heads_k=2), "divisible"),
    (dict(dim_qk=513), "dim size expect in [1, 512]"),
    (dict(dim_v=24), "multiple of 16"),
    (dict(mask_type=1), "not support triu"),
    (dict(mask_type=3), "use custom mask must have valid mask tensor"),
    (dict(mask_type=4), "maskType expect in [0, 3]"),
    (dict(dtype=7), "dtype expect"),
    (dict(seq_offset_k=None), "seq_offset_q and seq_offset_k must not be NULL"),
    (dict(kv_cache=0x1000), "only taken by the paged op"),
])
def test_validation_messages(over, needle):
    rc, _, msg = _ws(_params(**over))
    assert rc == -1 and needle in msg, msg


def test_paged_and_dense_validation():
    rc, _, msg = _ws(_params(), op="paged")
    assert rc == -1 and "should not be nullptr" in msg
    ok = _params(kv_cache=0x1000, page_offsets=0x1000, page_ids=0x1000, last_page_len=0x1000, page_size=64,
                 cache_dtype=_capi.HSTU_BF16)
    assert _ws(ok, op="paged")[0] == 0
    rc, _, msg = _ws(_params(kv_cache=0x1000, page_offsets=0x1000, page_ids=0x1000, last_page_len=0x1000,
                             page_size=64, cache_dtype=_capi.HSTU_FP8_E4M3), op="paged")
    assert rc == -1 and "kv_scales" in msg
    rc, _, msg = _ws(_params(), op="dense")
    assert rc == -1 and "no sequence offsets" in msg
    d = _params(seq_offset_q=None, seq_offset_k=None, total_q=128, total_k=128)
    assert _ws(d, op="dense")[0] == 0


def test_describe_kernel_selection():
    buf = C.create_string_buffer(64)
    lib = _capi.lib()
    for over, want in [(dict(), "mfma_bf16_d128_selfsched"), (dict(flags=_capi.FLAG_REUSE_WORKSPACE), "mfma_bf16_d128"), (dict(batch=128), "mfma_bf16_d128_selfsched"), (dict(batch=129), "mfma_bf16_d128"),
                       (dict(num_target=0x2000), "mfma_bf16_d128_selfsched"), (dict(num_context=0x2000), "mfma_bf16_d128"),
                       (dict(mask_type=2), "mfma_bf16_d128_selfsched"),
                       (dict(dim_qk=64, dim_v=64, dtype=_capi.HSTU_F16), "mfma_f16_d64_selfsched"),
                       (dict(dtype=_capi.HSTU_F32), "generic_f32"), (dict(dim_v=64), "mfma_bf16_d128_padded"), (dict(dim_qk=64, dim_v=32), "mfma_bf16_d64_padded"),
                       (dict(dim_qk=72, dim_v=64), "generic_bf16"), (dict(dim_v=64, attn_bias=0x1000), "generic_bf16"),
                       (dict(dim_qk=32, dim_v=32), "mfma_bf16_d32_selfsched"), (dict(dim_qk=256, dim_v=256, dtype=_capi.HSTU_F16), "mfma_f16_d256"),
                       (dict(dim_qk=32, dim_v=32, attn_bias=0x1000), "mfma_bf16_d32_selfsched"), (dict(dim_qk=32, dim_v=32, attn_bias=0x1002), "mfma_bf16_d32"),
                       (dict(attn_bias=0x1000), "mfma_bf16_d128_selfsched"), (dict(attn_bias=0x1000, mask_type=3, mask=0x2000), "mfma_bf16_d128"),
                       (dict(dim_qk=96, dim_v=96), "mfma_bf16_d128_padded"),
                       (dict(q=0x1002), "generic_bf16"), (dict(out=0x1008), "generic_bf16"),   # not on a 16-byte boundary
                       (dict(flags=_capi.FLAG_FORCE_GENERIC), "generic_bf16")]:
        p = _params(**over)
        assert lib.hstu_hip_describe_kernel(C.byref(p), buf, 64) == 0
        assert buf.value.decode() == want
    # paged: the MFMA kernel keeps one user's page ids in LDS (640 entries; 320 in the head-dim-128 variant that takes its
    # tiles through registers: page sizes that are no multiple of 4); longer page lists take the generic kernel
    paged = dict(kv_cache=0x1000, page_offsets=0x1000, page_ids=0x1000, last_page_len=0x1000, cache_dtype=_capi.HSTU_BF16)
    for over, want in [(dict(page_size=64, max_seq_len_k=20480), "mfma_bf16_d128"),
                       (dict(page_size=32, max_seq_len_k=20480), "mfma_bf16_d128"),
                       (dict(page_size=8, max_seq_len_k=5120), "mfma_bf16_d128"),
                       (dict(page_size=8, max_seq_len_k=5121), "generic_bf16"),
                       (dict(page_size=10, max_seq_len_k=3200), "mfma_bf16_d128"),
                       (dict(page_size=10, max_seq_len_k=3201), "generic_bf16"),
                       (dict(page_size=64, dim_qk=256, dim_v=256), "mfma_bf16_d256"), (dict(page_size=16, dim_qk=32, dim_v=32), "mfma_bf16_d32")]:
        p = _params(**paged, **over)
        assert lib.hstu_hip_describe_kernel(C.byref(p), buf, 64) == 0
        assert buf.value.decode() == want, over


def test_fp8_inputs_selection_and_rejections():
    """float8_e4m3fn q / k / v: forward of the jagged and dense layouts only; matrix-core kernel for head dims 64 / 128 / 256
    without bias or custom mask, else the plain kernel; the work list is the only workspace."""
    buf = C.create_string_buffer(64)
    lib = _capi.lib()
    fp8 = dict(dtype=_capi.HSTU_FP8_E4M3)
    for over, want in [(dict(), "mfma_fp8_d128_selfsched"), (dict(dim_qk=64, dim_v=64), "mfma_fp8_d64_selfsched"), (dict(dim_qk=256, dim_v=256), "mfma_fp8_d256_selfsched"),
                       (dict(batch=129), "mfma_fp8_d128"), (dict(flags=_capi.FLAG_REUSE_WORKSPACE), "mfma_fp8_d128"),
                       (dict(dim_qk=32, dim_v=32), "mfma_fp8_d64_padded"), (dict(dim_qk=96, dim_v=80), "mfma_fp8_d128_padded"),
                       (dict(dim_qk=72, dim_v=32), "generic_fp8"), (dict(dim_qk=96, dim_v=80, attn_bias=0x1000), "generic_fp8"),
                       (dict(attn_bias=0x1000), "generic_fp8"), (dict(mask_type=3, mask=0x1000), "generic_fp8"),
                       (dict(mask_type=2), "mfma_fp8_d128_selfsched"), (dict(mask_type=2, num_context=0x2000), "mfma_fp8_d128"), (dict(k=0x1008), "generic_fp8"),
                       (dict(flags=_capi.FLAG_FORCE_GENERIC), "generic_fp8")]:
        p = _params(**fp8, **over)
        assert lib.hstu_hip_describe_kernel(C.byref(p), buf, 64) == 0, lib.hstu_hip_last_error()
        assert buf.value.decode() == want, over
    rc, n, _ = _ws(_params(**fp8))
    assert rc == 0 and n > 0 and n % 256 == 0
    rc, n, _ = _ws(_params(**fp8, attn_bias=0x1000))
    assert rc == 0 and n == 0
    paged = dict(kv_cache=0x1000, page_offsets=0x1000, page_ids=0x1000, last_page_len=0x1000, cache_dtype=_capi.HSTU_FP8_E4M3,
                 kv_scales=0x1000, page_size=64)
    rc, _, msg = _ws(_params(**fp8, **paged), op="paged")
    assert rc == -2 and "jagged and dense forward only" in msg, (rc, msg)
    b = _capi.HstuBwdParams()
    b.struct_size = C.sizeof(_capi.HstuBwdParams)
    b.fwd = _params(**fp8)
    b.grad_out = b.grad_q = b.grad_k = b.grad_v = 0x1000
    n = C.c_uint64(0)
    assert lib.hstu_hip_jagged_backward_get_workspace_size(C.byref(b), C.byref(n)) == -2
    assert "forward only" in lib.hstu_hip_last_error().decode()


# ---- torch op layer: same checks, same messages, on CPU tensors ------------------------------
def _call(q, off, mask_type=0, max_len=8, mask=None, **kw):
    return torch.ops.mxrec.hstu_jagged(q, q, q, mask, None, mask_type, max_len, 0.0, off, **kw)


def test_op_schemas_match_the_reference():
    s = {str(x) for o in ("hstu_jagged", "hstu_paged", "hstu_dense") for x in
         [torch._C._get_schema("mxrec::" + o, n) for n in (["equal", "delta"] if o == "hstu_jagged" else [""])]}
    eq = next(x for x in s if "hstu_jagged.equal" in x)
    assert "Tensor? mask=None, Tensor? attn_bias=None, int mask_type=0, int max_seq_len=0, float silu_scale=0." in eq
    assert "Tensor? num_context=None, Tensor? num_target=None, int? target_group_size=0, float? alpha=1." in eq
    assert "bool deterministic=False" in eq
    de = next(x for x in s if "hstu_jagged.delta" in x)
    assert "int max_seq_len=0, int max_seq_len_k=0, float silu_scale" in de and "Tensor seq_offset_k=None" in de
    pg = next(x for x in s if "hstu_paged" in x)
    for name in ("kv_cache", "seq_offset_t", "page_offsets", "page_ids", "last_page_len", "num_target"):
        assert name in pg


def test_op_error_messages():
    q = torch.randn(10, 2, 32)
    off = torch.tensor([0, 4, 10])
    with pytest.raises(RuntimeError, match="The q should be 3D in jagged layout"):
        _call(q[0], off)
    with pytest.raises(RuntimeError, match=r"maxSeqLen expect in \[1, 20480\], but value is 20481"):
        _call(q, off, max_len=20481)
    with pytest.raises(RuntimeError, match="maskType current not support triu now"):
        _call(q, off, mask_type=1)
    with pytest.raises(RuntimeError, match="use custom mask must have valid mask tensor"):
        _call(q, off, mask_type=3)
    with pytest.raises(RuntimeError, match=r"maskType expect in \[0, 3\]"):
        _call(q, off, mask_type=5)
    with pytest.raises(RuntimeError, match="acSeqOffset params error should have at least two element"):
        _call(q, off[:1])
    with pytest.raises(RuntimeError, match="The length of num_context expect 2"):
        _call(q, off, num_context=torch.tensor([1, 1, 1]))
    with pytest.raises(RuntimeError, match="V dim size"):
        x = torch.randn(10, 2, 24)
        _call(x, off)
    with pytest.raises(RuntimeError, match="head num expect"):
        x = torch.randn(10, 17, 32)
        _call(x, off)
    with pytest.raises(RuntimeError, match="The q should be 4D in dense layout"):
        torch.ops.mxrec.hstu_dense(q, q, q, None, None, 0, 8, 0.0)
    # the overload is chosen by the type of the 8th positional argument, as in the reference's tests
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        torch.ops.mxrec.hstu_jagged(q, q, q, None, None, 0, 8, 8, 0.0, off, off)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        _call(q, off)


def test_time_bucket_bounds_reproduce_the_reference_formula():
    """bucket(|dt|) from the bounds == trunc(log(clamp(|dt|,1,e^(128*0.301)))/0.301) in torch fp32
    (cust_op/test/relative_attn_bias/torch/utils.py:115-123), exactly, for every integer up to 3e6,
    powers of two and random 63-bit values."""
    b = recsdk_amd.time_bucket_bounds(128, 0.301)
    assert b.shape == (130,) and b[0] == 0 and torch.isinf(b[-1]) and torch.all(b[1:] >= b[:-1])
    g = torch.Generator().manual_seed(0)
    d = torch.cat([torch.arange(0, 3_000_000, dtype=torch.int64), 2 ** torch.arange(0, 63, dtype=torch.int64),
                   torch.randint(0, 2 ** 62, (200000,), generator=g)])
    want = O.time_bucket_ids(torch.zeros(1, dtype=torch.int64), d)[0]
    got = torch.bucketize(d.to(torch.float32), b[1:-1], right=True)
    assert torch.equal(want, got)
    assert want.max() == 128 and want.min() == 0


def test_header_is_plain_c_and_links(tmp_path):
    """The boundary header compiles as C99 (no C++-isms) and a C program can call the library through it."""
    import os
    import shutil
    import subprocess
    from recsdk_amd import _build
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "abi.c"
    src.write_text(r'''
#include <stdio.h>
#include <string.h>
#include <dlfcn.h>
#include "hstu_hip.h"
int main(int argc, char** argv) {
    void* h = dlopen(argv[1], RTLD_NOW | RTLD_GLOBAL);
    if (!h) { printf("dlopen: %s\n", dlerror()); return 2; }
    int (*ver)(void) = (int (*)(void))dlsym(h, "hstu_hip_abi_version");
    int (*wsz)(const hstu_fwd_params*, uint64_t*) = (int (*)(const hstu_fwd_params*, uint64_t*))dlsym(h, "hstu_hip_jagged_forward_get_workspace_size");
    const char* (*err)(void) = (const char* (*)(void))dlsym(h, "hstu_hip_last_error");
    if (!ver || !wsz || !err) return 3;
    hstu_fwd_params p;
    memset(&p, 0, sizeof p);
    p.struct_size = 8;                       /* wrong on purpose */
    uint64_t n = 0;
    int rc = wsz(&p, &n);
    printf("%d %d %d %s\n", ver(), (int)sizeof(hstu_fwd_params), rc, err());
    return 0;
}
''')
    exe = tmp_path / "abi"
    subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", "-I", os.path.join(root, "include"), str(src), "-o", str(exe), "-ldl"],
                   check=True)
    _capi.lib()   # make sure the library exists; its HIP runtime dependency resolves through torch's copy
    import torch
    env = dict(os.environ, LD_LIBRARY_PATH=os.path.join(os.path.dirname(torch.__file__), "lib") + ":/opt/rocm/lib:" + os.environ.get("LD_LIBRARY_PATH", ""))
    out = subprocess.run([str(exe), _build.hip_lib_path()], check=True, capture_output=True, text=True, env=env).stdout.split(None, 3)
    assert out[0] == "1" and int(out[1]) == C.sizeof(_capi.HstuFwdParams) and out[2] == "-1" and "size mismatch" in out[3]


def _bwd_params(**over):
    f = _params()
    f.out = None                       # the backward does not read the forward's output
    b = _capi.HstuBwdParams()
    b.struct_size = C.sizeof(_capi.HstuBwdParams)
    b.fwd = f
    for name in ("grad_out", "grad_q", "grad_k", "grad_v"):
        setattr(b, name, 0x1000)       # never dereferenced on the host
    for k, v in over.items():
        if hasattr(b, k):
            setattr(b, k, v)
        else:
            setattr(b.fwd, k, v)
    return b


def _bwd_ws(b, op="jagged"):
    n = C.c_uint64(123)
    rc = getattr(_capi.lib(), f"hstu_hip_{op}_backward_get_workspace_size")(C.byref(b), C.byref(n))
    return rc, n.value, _capi.lib().hstu_hip_last_error().decode()


def test_backward_validation_and_workspace():
    rc, n, msg = _bwd_ws(_bwd_params())
    # bf16, d=128, built-in mask, no bias: the MFMA kernels; self-attention without GQA -> one work list (as the forward's)
    assert rc == 0 and n == 1024, msg
    rc, n, msg = _bwd_ws(_bwd_params(heads_k=2))            # GQA: a second list for the K-side kernels (2 K/V heads:
    assert rc == 0 and n == 1024 + 768, msg                 # 4 tiles -> 4 * (16 + 8 * (8 * 2 + 4)) = 704 -> 768 bytes)
    rc, n, msg = _bwd_ws(_bwd_params(dtype=_capi.HSTU_F32))  # plain kernels: nothing to stage
    assert rc == 0 and n == 0, msg
    rc, n, msg = _bwd_ws(_bwd_params(attn_bias=0x1000, grad_bias=0x1000))
    assert rc == 0 and n == 1024, msg                        # dense bias whose rows are a multiple of 8 elements: MFMA kernels too
    rc, n, msg = _bwd_ws(_bwd_params(attn_bias=0x1000, grad_bias=0x1000, max_seq_len_q=60, max_seq_len_k=60))
    assert rc == 0 and n == 0, msg                           # rows of 60 elements -> plain kernels
    rc, n, msg = _bwd_ws(_bwd_params(mask=0x1000, mask_type=3))
    assert rc == 0 and n == 1024, msg                        # custom mask on aligned rows: MFMA kernels too
    rc, n, msg = _bwd_ws(_bwd_params(mask=0x1000, mask_type=3, attn_bias=0x1000, grad_bias=0x1000))
    assert rc == 0 and n == 0, msg                           # custom mask next to a bias -> plain kernels
    rc, n, msg = _bwd_ws(_bwd_params(mask=0x1000, mask_type=3, max_seq_len_q=60, max_seq_len_k=60))
    assert rc == 0 and n == 0, msg                           # rows of 60 elements -> plain kernels
    for d, want in ((32, True), (256, True), (96, False), (512, False)):
        rc, n, msg = _bwd_ws(_bwd_params(dim_qk=d, dim_v=d))
        assert rc == 0 and (n > 0) == want, (d, n, msg)      # head dims 32 / 64 / 128 / 256 have matrix-core kernels
    rc, _, msg = _bwd_ws(_bwd_params(attn_bias=0x1000))
    assert rc == -1 and "grad_bias must be given exactly when attn_bias is" in msg
    rc, _, msg = _bwd_ws(_bwd_params(grad_bias=0x1000))
    assert rc == -1 and "grad_bias" in msg
    rc, _, msg = _bwd_ws(_bwd_params(grad_k=None))
    assert rc == -1 and "must not be NULL" in msg
    rc, _, msg = _bwd_ws(_bwd_params(pos_table=0x1000))
    assert rc == -2 and "dense attn_bias only" in msg
    rc, _, msg = _bwd_ws(_bwd_params(struct_size=8))
    assert rc == -1 and "size mismatch" in msg
    rc, _, msg = _bwd_ws(_bwd_params(batch=0))               # the forward's checks apply
    assert rc == -1 and "batchSize" in msg
    # a call without the workspace is refused before anything is launched
    b = _bwd_params()
    rc = _capi.lib().hstu_hip_jagged_backward(C.byref(b), None, 0, None)
    assert rc == -3 and "workspace" in _capi.lib().hstu_hip_last_error().decode()


def test_dense_backward_validation():
    rc, _, msg = _bwd_ws(_bwd_params(), op="dense")
    assert rc == -1 and "no sequence offsets" in msg
    d = _bwd_params(seq_offset_q=None, seq_offset_k=None, total_q=128, total_k=128)
    rc, n, msg = _bwd_ws(d, op="dense")
    assert rc == 0 and n > 0 and n % 256 == 0, msg           # bf16 d=128: the MFMA kernels with one work list
    rc = _capi.lib().hstu_hip_dense_backward(C.byref(d), None, 0, None)
    assert rc == -3 and "workspace" in _capi.lib().hstu_hip_last_error().decode()


def test_bench_routes_every_workload_to_its_own_leg():
    """The workload names of several legs end alike (`*_bwd`): each must reach the leg that measures it."""
    import bench
    want = {"config2": "attention_forward", "config5": "attention_forward", "ref_bias": "attention_forward", "config2_fp8": "attention_forward",
            "config2_bwd": "attention_backward", "ref_bias_bwd": "attention_backward", "ref_nobias_d32_bwd": "attention_backward",
            "rab_time": "bias", "rab_time_bwd": "bias", "rab_pos": "bias", "nmd_fwd": "nmd", "nmd_bwd": "nmd",
            "in_linear_silu": "in_linear_silu", "in_linear_silu_bwd": "in_linear_silu_bwd", "kv_append": "kv_append",
            "kv_append_fp8": "kv_append_fp8", "copy": "copy"}
    for name, kind in want.items():
        assert bench.bench_kind(name) == kind, name
