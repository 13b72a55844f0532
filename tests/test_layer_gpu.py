"""GPU parity of norm_multiply_dropout (forward and backward, through the torch op and its autograd formula, which call
the C ABI) against the fp64 oracle on the reference's test inputs (uniform [-1, 1), seed 321;
test_norm_multiply_dropout.py:105-118).  Floating point: the tolerances of this build (fp32 1e-5 relative to the
tensor's scale, bf16 / fp16 rtol = atol = 2e-2); the column sums d_weight / d_bias are fp32 sums over all rows, compared
relative to their scale."""
import sys

import pytest
import torch

import recsdk_amd  # noqa: F401
from oracle import layer_oracle as LO
from tests import hstu_testlib as T

pytestmark = pytest.mark.gpu
EPS = 1e-5


def say(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def _inputs(dim0, dim1, dtype):
    g = torch.Generator().manual_seed(321)
    mk = lambda *s: (torch.rand(*s, generator=g) * 2 - 1).to(dtype)
    return mk(dim0, dim1), mk(dim0, dim1), mk(dim1), mk(dim1), mk(dim0, dim1)


def _close(got, want, dtype, what, colsum=False):
    got, want = got.double().cpu(), want.double()
    if dtype == torch.float32 or colsum:
        tol = 1e-5 if dtype == torch.float32 else 4e-3
        scale = float(want.abs().max()) or 1.0
        assert float((got - want).abs().max()) <= tol * scale, f"{what}: {float((got - want).abs().max()):.3e} vs scale {scale:.3e}"
    else:
        assert torch.allclose(got, want, rtol=2e-2, atol=2e-2), what


@pytest.mark.parametrize("dim0", [1, 1000, 2345, 16384])
@pytest.mark.parametrize("dim1", [512, 1024])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_forward_and_backward_without_dropout(dim0, dim1, dtype):
    say("nmd", dim0, dim1, dtype)
    x, u, w, b, dy = _inputs(dim0, dim1, dtype)
    y_want, mean_want, var_want = LO.nmd_forward(x, u, w, b, EPS)
    leaves = [t.cuda().requires_grad_(True) for t in (x, u, w, b)]
    outs = torch.ops.mxrec.norm_multiply_dropout(*leaves, EPS, 0.0)
    assert len(outs) == 1 and outs[0].dtype == dtype
    _close(outs[0].detach(), y_want, dtype, "y")
    outs[0].backward(dy.cuda())
    want = LO.nmd_backward(dy, x, u, w, b, mean_want, var_want, EPS)
    _close(leaves[0].grad, want[0], dtype, "d_x")
    _close(leaves[1].grad, want[1], dtype, "d_u")
    assert leaves[2].grad.dtype == dtype
    # the fp32 column sums before the cast to the parameter dtype
    raw = torch.ops.mxrec.norm_multiply_dropout_forward(x.cuda(), u.cuda(), w.cuda(), b.cuda(), EPS, 0.0)
    assert torch.allclose(raw[1].cpu().double(), mean_want, rtol=0, atol=2e-6) and torch.allclose(raw[2].cpu().double(), var_want, rtol=1e-5, atol=1e-6)
    g = torch.ops.mxrec.norm_multiply_dropout_backward(dy.cuda(), x.cuda(), u.cuda(), w.cuda(), b.cuda(), raw[1], raw[2], raw[3], EPS, 0.0)
    assert g[2].dtype == torch.float32 and g[3].dtype == torch.float32
    _close(g[2], want[2], dtype, "d_weight", colsum=True)
    _close(g[3], want[3], dtype, "d_bias", colsum=True)
    # reproducible: the column sums are formed in a fixed order
    g2 = torch.ops.mxrec.norm_multiply_dropout_backward(dy.cuda(), x.cuda(), u.cuda(), w.cuda(), b.cuda(), raw[1], raw[2], raw[3], EPS, 0.0)
    assert all(torch.equal(a, c) for a, c in zip(g, g2))


@pytest.mark.parametrize("dim1,dtype,ratio", [(512, torch.bfloat16, 0.3), (1024, torch.float32, 0.3), (512, torch.float16, 0.75)])
def test_dropout_under_the_mask_the_op_returns(dim1, dtype, ratio):
    say("nmd dropout", dim1, dtype, ratio)
    dim0 = 3000
    x, u, w, b, dy = _inputs(dim0, dim1, dtype)
    torch.manual_seed(5)
    y, mean, var, mask = torch.ops.mxrec.norm_multiply_dropout_forward(x.cuda(), u.cuda(), w.cuda(), b.cuda(), EPS, ratio)
    assert mask.dtype == torch.uint8 and mask.numel() == (dim0 * dim1 + 127) // 128 * 16
    keep = LO.unpack_mask(mask.cpu(), dim0 * dim1).reshape(dim0, dim1)
    rate = float(keep.double().mean())
    assert abs(rate - (1 - ratio)) < 4 * (ratio * (1 - ratio) / keep.numel()) ** 0.5 + 2e-5, rate     # 16-bit threshold: 1.5e-5 resolution
    # rows and columns are not correlated with the mask
    assert abs(float(keep[:, ::7].double().mean()) - rate) < 5e-3 and abs(float(keep[::5].double().mean()) - rate) < 5e-3
    y_want, mean_want, var_want = LO.nmd_forward(x, u, w, b, EPS, ratio, keep)
    _close(y, y_want, dtype, "y with dropout")
    assert torch.equal(y.cpu() == 0, ~keep | (y.cpu() == 0))
    g = torch.ops.mxrec.norm_multiply_dropout_backward(dy.cuda(), x.cuda(), u.cuda(), w.cuda(), b.cuda(), mean, var, mask, EPS, ratio)
    want = LO.nmd_backward(dy, x, u, w, b, mean_want, var_want, EPS, ratio, keep)
    _close(g[0], want[0], dtype, "d_x with dropout")
    _close(g[1], want[1], dtype, "d_u with dropout")
    _close(g[2], want[2], dtype, "d_weight with dropout", colsum=True)
    _close(g[3], want[3], dtype, "d_bias with dropout", colsum=True)
    # same seed, same mask; another seed, another mask
    torch.manual_seed(5)
    again = torch.ops.mxrec.norm_multiply_dropout_forward(x.cuda(), u.cuda(), w.cuda(), b.cuda(), EPS, ratio)[3]
    other = torch.ops.mxrec.norm_multiply_dropout_forward(x.cuda(), u.cuda(), w.cuda(), b.cuda(), EPS, ratio)[3]
    assert torch.equal(again, mask) and not torch.equal(other, mask)
    # through autograd (the reference's only route, test_norm_multiply_dropout.py:336-342)
    leaves = [t.cuda().requires_grad_(True) for t in (x, u, w, b)]
    out = torch.ops.mxrec.norm_multiply_dropout(*leaves, EPS, ratio)[0]
    out.backward(dy.cuda())
    assert all(l.grad is not None and bool(torch.isfinite(l.grad).all()) for l in leaves)
    # everything dropped
    y1 = torch.ops.mxrec.norm_multiply_dropout_forward(x.cuda(), u.cuda(), w.cuda(), b.cuda(), EPS, 1.0)[0]
    assert not bool(y1.any())


@pytest.mark.parametrize("m,n,k,split,dtype", [
    (2789, 9216, 64, None, torch.bfloat16), (256, 1024, 16, None, torch.float16), (2561, 1024, 128, "diff", torch.bfloat16),
    (512, 4096, 32, None, torch.float16), (1000, 9216, 48, "diff", torch.float16), (100, 64, 16, None, torch.bfloat16),
    (129, 2048, 256, "diff", torch.bfloat16), (33, 192, 48, None, torch.float16), (300, 3072, 768, None, torch.bfloat16),
    (65, 960, 240, "diff", torch.float16)])
def test_in_linear_silu_forward(m, n, k, split, dtype):
    """The reference's generators (test_in_linear_silu.py:70-99): integer x in [-100, 100], Xavier-uniform W, bias of ones;
    equal splits or (s - 16, s - 16, s + 16, s + 16).  Against the oracle's exactly rounded values the fp32 accumulation
    order can move a result by one unit in the last place of the I/O dtype; nothing more is allowed."""
    say("in_linear_silu", m, n, k, split, dtype)
    g = torch.Generator().manual_seed(13)
    x = torch.randint(-100, 101, (m, k), generator=g).to(dtype)
    bound = (6.0 / (n + k)) ** 0.5
    w = ((torch.rand(n, k, generator=g) * 2 - 1) * bound).to(dtype)
    bias = torch.ones(n)
    s = n // 4
    sp = [s, s, s, s] if split is None else [s - 16, s - 16, s + 16, s + 16]
    want = LO.in_linear_silu(x, w, bias, sp)
    got = torch.ops.mxrec.distance_in_linear_silu(x.cuda(), w.cuda(), bias.cuda(), sp)
    assert len(got) == 5
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10

    # fp32 accumulation of k products against the oracle's fp64: absolute error up to about 2^-20 of the largest sum of
    # absolute products, which matters where the result itself cancels to almost nothing
    acc_err = 2.0 ** -20 * float((x.double().abs() @ w.double().abs().t()).max())

    def within_one_ulp(a, wnt, name, extra=0.0):
        assert a.shape == wnt.shape and a.dtype == dtype, name
        d = (a.cpu().double() - wnt.double()).abs()
        lim = ulp * wnt.double().abs().clamp(min=2.0 ** -14) * 1.001 + extra
        assert bool((d <= lim).all()), f"{name}: more than one unit in the last place, max {float((d / lim).max()):.2f}"
        assert float((d > 0).double().mean()) < 0.02, f"{name}: {float((d > 0).double().mean()):.4f} of the elements differ"

    within_one_ulp(got[4], want[4], "linear_output", acc_err)
    # the four outputs are SiLU of the *rounded* linear output (a last-place difference there is magnified by up to
    # |1 + x (1 - sigmoid x)| in SiLU): checked against the oracle's SiLU of the linear output the kernel produced
    lin = got[4].cpu()
    act = (lin.double() * torch.sigmoid(lin.double())).to(dtype)
    for name, a, wnt in zip(("user", "value", "query", "key"), got[:4], torch.split(act, sp, dim=-1)):
        within_one_ulp(a, wnt, name)
    # no bias
    got0 = torch.ops.mxrec.distance_in_linear_silu(x.cuda(), w.cuda(), torch.zeros(n).cuda(), sp)
    want0 = LO.in_linear_silu(x, w, None, sp)
    within_one_ulp(got0[4], want0[4], "linear_output without bias", acc_err)


def _ilb_inputs(m, k, n, dtype, diff):
    """The reference's generators (test_in_linear_silu_backward.py:100-125): gradients uniform [0, 1), x, W and
    linear_output uniform [-1, 1); equal widths or (h - 32, h - 16, h + 16, h + 32)."""
    g = torch.Generator().manual_seed(0)
    h = n // 4
    sp = [h - 32, h - 16, h + 16, h + 32] if diff else [h] * 4
    grads = [torch.rand(m, s_, generator=g).to(dtype) for s_ in sp]
    u = lambda *s: (torch.rand(*s, generator=g) * 2 - 1).to(dtype)
    return grads, u(m, k), u(n, k), u(m, n), (torch.rand(n, generator=g) * 2 - 1), sp


def _ilb_close(got, want, dtype, what, f32=False):
    """fp32 sums of up to 32768 rounded products against the fp64 oracle, then (for the dtype outputs) one rounding to
    the I/O dtype: half a unit in the last place of the value plus the accumulation error relative to the tensor's scale."""
    got, want = got.double().cpu(), want.double()
    scale = float(want.abs().max()) or 1.0
    ulp = 0.0 if f32 else (2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11)
    lim = ulp * want.abs() * 1.001 + 1e-4 * scale
    d = (got - want).abs()
    assert bool((d <= lim).all()), f"{what}: worst {float((d / lim).max()):.2f} x the limit, scale {scale:.3e}"


@pytest.mark.parametrize("m", [1, 1123, 2048, 7687])
@pytest.mark.parametrize("kn", [(16, 128), (64, 512), (240, 960), (128, 2048), (768, 3072)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_in_linear_silu_backward(m, kn, dtype):
    """Shapes of the reference's test (test_in_linear_silu_backward.py:158-166), with and without bias, equal and unequal
    widths, against the oracle (dlin rounded to the I/O dtype before the products, as the reference's kernel does)."""
    k, n = kn
    for diff, with_bias in ((False, True), (True, False)):
        if diff and k <= 32:
            continue
        say("in_linear_silu_backward", m, k, n, dtype, "unequal" if diff else "equal", "bias" if with_bias else "no bias")
        grads, x, w, lin, bias, sp = _ilb_inputs(m, k, n, dtype, diff)
        want = LO.in_linear_silu_backward(grads, x, w, lin, with_bias=with_bias)
        got = torch.ops.mxrec.in_linear_silu_backward(x.cuda(), w.cuda(), bias.cuda() if with_bias else None, *[t.cuda() for t in grads], lin.cuda(), sp)
        assert len(got) == 4 and got[0].dtype == dtype and got[1].dtype == dtype and got[0].shape == x.shape and got[1].shape == w.shape
        _ilb_close(got[0], want[0], dtype, "x_grad")
        _ilb_close(got[1], want[1], dtype, "weight_grad")
        if with_bias:
            assert got[2].dtype == torch.float32
            _ilb_close(got[2], want[2], dtype, "bias_grad", f32=True)
        else:
            assert got[2] is None or got[2].numel() == 0


def test_in_linear_silu_backward_fp32_outputs_reproducible_and_large():
    """The C ABI's fp32 outputs (what the reference's kernel writes before its wrapper casts) on a shape whose k needs
    several column chunks (k = 512, n = 6144: test_in_linear_silu_backward.py:169-176); two runs give the same bits."""
    import ctypes as C
    from recsdk_amd import _capi
    m, k, n, dtype = 511, 512, 6144, torch.bfloat16
    say("in_linear_silu_backward C ABI fp32", m, k, n)
    grads, x, w, lin, bias, sp = _ilb_inputs(m, k, n, dtype, False)
    dev = [t.cuda() for t in grads]
    xd, wd, ld = x.cuda(), w.cuda(), lin.cuda()
    L = _capi.lib()
    outs = []
    for _ in range(2):
        xg = torch.full((m, k), float("nan"), device="cuda")
        wg = torch.full((n, k), float("nan"), device="cuda")
        bg = torch.full((n,), float("nan"), device="cuda")
        p = _capi.HstuInLinearSiluBwdParams()
        p.struct_size = C.sizeof(p)
        p.dtype, p.grad_dtype, p.m, p.k, p.n = _capi.HSTU_BF16, _capi.HSTU_F32, m, k, n
        for i in range(4):
            p.split[i] = sp[i]
            p.grad[i] = dev[i].data_ptr()
        p.x, p.weight, p.linear_output = xd.data_ptr(), wd.data_ptr(), ld.data_ptr()
        p.x_grad, p.weight_grad, p.bias_grad = xg.data_ptr(), wg.data_ptr(), bg.data_ptr()
        need = C.c_uint64(0)
        assert L.hstu_hip_in_linear_silu_backward_get_workspace_size(C.byref(p), C.byref(need)) == 0
        ws = torch.empty(need.value, dtype=torch.uint8, device="cuda")
        rc = L.hstu_hip_in_linear_silu_backward(C.byref(p), ws.data_ptr(), need.value, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, L.hstu_hip_last_error().decode()
        torch.cuda.synchronize()
        outs.append((xg.cpu(), wg.cpu(), bg.cpu()))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    want = LO.in_linear_silu_backward(grads, x, w, lin)
    for name, a, wnt in zip(("x_grad", "weight_grad", "bias_grad"), outs[0], want):
        _ilb_close(a, wnt, dtype, name, f32=True)


def test_in_linear_silu_autograd():
    """mxrec::in_linear_silu differentiates like the reference's (test_in_linear_silu_autograd.py): the gradients that
    reach x, W and the bias equal the backward op applied to the forward's own linear_output."""
    m, k, n, dtype = 777, 64, 512, torch.bfloat16
    say("in_linear_silu autograd", m, k, n)
    grads, x, w, _, bias, sp = _ilb_inputs(m, k, n, dtype, True)
    leaves = [t.cuda().requires_grad_(True) for t in (x, w, bias)]
    outs = torch.ops.mxrec.in_linear_silu(*leaves, sp)
    assert len(outs) == 5
    sum((o * g_.cuda()).sum() for o, g_ in zip(outs[:4], grads)).backward()
    direct = torch.ops.mxrec.in_linear_silu_backward(x.cuda(), w.cuda(), bias.cuda(), *[t.cuda() for t in grads], outs[4].detach(), sp)
    for leaf, d in zip(leaves, direct[:3]):
        assert leaf.grad is not None and leaf.grad.dtype == leaf.dtype and torch.equal(leaf.grad, d.to(leaf.dtype))
    want = LO.in_linear_silu_backward(grads, x, w, outs[4].detach().cpu())
    _ilb_close(leaves[0].grad, want[0], dtype, "x.grad")
    _ilb_close(leaves[1].grad, want[1], dtype, "weight.grad")


@pytest.mark.parametrize("m,k,n", [(511, 8160, 32640), (16384, 64, 16384), (20480, 48, 9216)])
def test_in_linear_silu_backward_largest_reference_shape(m, k, n):
    """k = 8160, n = 32640 at m = 511 (test_in_linear_silu_backward.py:169-176): 64 blocks of k per workgroup column, one
    range of m; the bench shape m = n = 16384, k = 64; the longest m of the reference's tests.  Too large for the fp64
    oracle in a test; checked against the same formula evaluated with torch's own GPU routines in fp32 (sigmoid, rounding
    of dlin to bf16, two matrix products) -- a checker, not a code path of the op."""
    dtype = torch.bfloat16
    say("in_linear_silu_backward largest", m, k, n)
    g = torch.Generator(device="cuda").manual_seed(0)
    sp = [n // 4] * 4
    grads = [torch.rand(m, s_, generator=g, device="cuda").to(dtype) for s_ in sp]
    u = lambda *s: (torch.rand(*s, generator=g, device="cuda") * 2 - 1).to(dtype)
    x, w, lin = u(m, k), u(n, k), u(m, n)
    bias = torch.zeros(n, device="cuda")
    got = torch.ops.mxrec.in_linear_silu_backward(x, w, bias, *grads, lin, sp)
    torch.cuda.synchronize()
    z = lin.float()
    sg = torch.sigmoid(z)
    dlin = torch.cat(grads, dim=-1).float() * (sg * (1 + z * (1 - sg)))
    want_b = dlin.sum(dim=0)
    dl = dlin.to(dtype).float()
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        want_x, want_w = dl @ w.float(), dl.t() @ x.float()
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev
    for name, a, wnt, f32 in (("x_grad", got[0], want_x, False), ("weight_grad", got[1], want_w, False), ("bias_grad", got[2], want_b, True)):
        a, wnt = a.double(), wnt.double()
        scale = float(wnt.abs().max())
        lim = (0.0 if f32 else 2.0 ** -8) * wnt.abs() * 1.001 + 2e-4 * scale
        d = (a - wnt).abs()
        assert bool((d <= lim).all()), f"{name}: worst {float((d / lim).max()):.2f} x the limit, scale {scale:.3e}"


def _ilb_capi(grads, x, w, lin, sp, algorithm, dtype_code):
    import ctypes as C
    from recsdk_amd import _capi
    m, k, n = x.shape[0], x.shape[1], w.shape[0]
    dev = [t.cuda() for t in grads]
    xd, wd, ld = x.cuda(), w.cuda(), lin.cuda()
    xg = torch.full((m, k), float("nan"), device="cuda")
    wg = torch.full((n, k), float("nan"), device="cuda")
    bg = torch.full((n,), float("nan"), device="cuda")
    L = _capi.lib()
    p = _capi.HstuInLinearSiluBwdParams()
    p.struct_size = C.sizeof(p)
    p.dtype, p.grad_dtype, p.m, p.k, p.n, p.algorithm = dtype_code, _capi.HSTU_F32, m, k, n, algorithm
    for i in range(4):
        p.split[i] = sp[i]
        p.grad[i] = dev[i].data_ptr()
    p.x, p.weight, p.linear_output = xd.data_ptr(), wd.data_ptr(), ld.data_ptr()
    p.x_grad, p.weight_grad, p.bias_grad = xg.data_ptr(), wg.data_ptr(), bg.data_ptr()
    need = C.c_uint64(0)
    assert L.hstu_hip_in_linear_silu_backward_get_workspace_size(C.byref(p), C.byref(need)) == 0
    ws = torch.empty(need.value, dtype=torch.uint8, device="cuda")
    rc = L.hstu_hip_in_linear_silu_backward(C.byref(p), ws.data_ptr(), need.value, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, L.hstu_hip_last_error().decode()
    torch.cuda.synchronize()
    return xg.cpu(), wg.cpu(), bg.cpu()


@pytest.mark.parametrize("m,k,n,diff", [(1123, 64, 512, True), (2048, 32, 1152, False), (77, 16, 64, False), (4099, 64, 4096, True)])
def test_in_linear_silu_backward_one_pass_against_two_product_kernels(m, k, n, diff):
    """`algorithm` = 2 (the library's own choice at k <= 64) runs one pass over the inputs (x_grad as partial slabs per
    512 columns of n), `algorithm` = 1 the two product kernels.  Same roundings, different order of the fp32 sums: both against the oracle, and against each other
    to the accumulation error alone."""
    from recsdk_amd import _capi
    say("in_linear_silu_backward one pass vs two", m, k, n, diff)
    dtype = torch.bfloat16
    grads, x, w, lin, bias, sp = _ilb_inputs(m, k, n, dtype, diff)
    one = _ilb_capi(grads, x, w, lin, sp, 2, _capi.HSTU_BF16)
    two = _ilb_capi(grads, x, w, lin, sp, 1, _capi.HSTU_BF16)
    assert all(torch.equal(a, b) for a, b in zip(one, _ilb_capi(grads, x, w, lin, sp, 0, _capi.HSTU_BF16)))   # 0 = 2 at k <= 64
    want = LO.in_linear_silu_backward(grads, x, w, lin)
    for name, a, b, wnt in zip(("x_grad", "weight_grad", "bias_grad"), one, two, want):
        _ilb_close(a, wnt, dtype, name + " (one pass)", f32=True)
        _ilb_close(b, wnt, dtype, name + " (two kernels)", f32=True)
    # (the two plans cut m into different numbers of ranges, so the fp32 partial sums are grouped differently)
    for a, b, wnt in zip(one, two, want):
        assert float((a - b).abs().max()) <= 1e-5 * float(wnt.abs().max())


@pytest.mark.parametrize("m,n,k", [(16384, 16384, 64), (20480, 9216, 48)])
def test_in_linear_silu_forward_largest_reference_shapes(m, n, k):
    """The largest shapes of the reference's forward tests (test_in_linear_silu.py:110-127), too large for the fp64 oracle
    in a test: linear_output against torch's fp32 product on the GPU (one unit in the last place of bf16: the order of
    the fp32 sums differs), the four outputs against SiLU of the linear_output the kernel itself wrote."""
    dtype = torch.bfloat16
    say("in_linear_silu forward largest", m, n, k)
    g = torch.Generator(device="cuda").manual_seed(13)
    x = torch.randint(-100, 101, (m, k), generator=g, device="cuda").to(dtype)
    w = ((torch.rand(n, k, generator=g, device="cuda") * 2 - 1) * (6.0 / (n + k)) ** 0.5).to(dtype)
    bias = torch.ones(n, device="cuda")
    sp = [n // 4] * 4
    got = torch.ops.mxrec.distance_in_linear_silu(x, w, bias, sp)
    torch.cuda.synchronize()
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        want = x.float() @ w.float().t() + bias
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev
    lin = got[4].float()
    acc_err = 2.0 ** -20 * float((x.float().abs() @ w.float().abs().t()).max())
    d = (lin - want).abs()
    lim = 2.0 ** -7 * want.abs().clamp(min=2.0 ** -14) * 1.001 + acc_err
    assert bool((d <= lim).all()), f"linear_output: worst {float((d / lim).max()):.2f} x the limit"
    del d, lim, want
    act = torch.cat(got[:4], dim=-1).float()
    ref = lin * torch.sigmoid(lin)
    d = (act - ref).abs()
    assert bool((d <= 2.0 ** -7 * ref.abs().clamp(min=2.0 ** -14) * 1.001).all()), "outputs: more than one unit in the last place of silu(linear_output)"
    assert [t.shape[1] for t in got] == sp + [n]


def test_norm_multiply_dropout_at_the_bench_shape():
    """262144 x 512 bf16 (the shape of the reference's sample), without dropout: forward against torch's own layer_norm
    on the GPU in fp32, backward against autograd through it; with dropout 0.3: the kept fraction and that dropped
    positions (read from the mask bits) are exactly zero in y and in d_u."""
    import torch.nn.functional as F
    rows, cols, dtype = 262144, 512, torch.bfloat16
    say("nmd at the bench shape", rows, cols)
    g = torch.Generator(device="cuda").manual_seed(321)
    mk = lambda *s: (torch.rand(*s, generator=g, device="cuda") * 2 - 1).to(dtype)
    x, u, w, b, dy = mk(rows, cols), mk(rows, cols), mk(cols), mk(cols), mk(rows, cols)
    leaves = [t.clone().requires_grad_(True) for t in (x, u, w, b)]
    y = torch.ops.mxrec.norm_multiply_dropout(*leaves, EPS, 0.0)[0]
    y.backward(dy)
    ref = [t.float().requires_grad_(True) for t in (x, u, w, b)]
    yr = F.layer_norm(ref[0], (cols,), ref[2], ref[3], EPS) * ref[1]
    yr.backward(dy.float())
    assert torch.allclose(y.float(), yr, rtol=2e-2, atol=2e-2)
    assert torch.allclose(leaves[0].grad.float(), ref[0].grad, rtol=2e-2, atol=2e-2)
    assert torch.allclose(leaves[1].grad.float(), ref[1].grad, rtol=2e-2, atol=2e-2)
    for a, r in ((leaves[2].grad, ref[2].grad), (leaves[3].grad, ref[3].grad)):   # sums over 262144 rows, handed over in bf16
        assert float((a.float() - r).abs().max()) <= 1e-2 * float(r.abs().max())
    del ref, yr
    outs = torch.ops.mxrec.norm_multiply_dropout_forward(x, u, w, b, EPS, 0.3)
    # bit e % 8 of mask byte e / 8 = element e kept
    bits = (outs[3][: rows * cols // 8, None] >> torch.arange(8, device="cuda", dtype=torch.uint8)) & 1
    keep = bits.reshape(rows, cols).bool()
    assert abs(float(keep.float().mean()) - 0.7) < 2e-3
    assert not bool(outs[0][~keep].any())
    gr = torch.ops.mxrec.norm_multiply_dropout_backward(dy, x, u, w, b, outs[1], outs[2], outs[3], EPS, 0.3)
    assert not bool(gr[1][~keep].any())
    # kept elements are the undropped result scaled by 1 / (1 - p), up to the one rounding
    y0 = torch.ops.mxrec.norm_multiply_dropout_forward(x, u, w, b, EPS, 0.0)[0]
    assert torch.allclose(outs[0][keep].float(), y0[keep].float() / 0.7, rtol=2e-2, atol=2e-2)
