"""Host-side checks of norm_multiply_dropout (no GPU needed): the C ABI's validation and the torch op's schema, checks
and messages (the reference's own exception tests, test_norm_multiply_dropout.py:365-470, run on the CPU key here)."""
import ctypes as C

import pytest
import torch

import recsdk_amd  # noqa: F401
from recsdk_amd import _capi


def _params(cls=_capi.HstuNmdParams, **over):
    p = cls()
    p.struct_size = C.sizeof(cls)
    p.dtype, p.rows, p.cols, p.eps, p.dropout_ratio = _capi.HSTU_BF16, 100, 512, 1e-5, 0.0
    for name, _ in cls._fields_:
        if name in ("x", "u", "weight", "bias", "out", "mean", "var", "d_out", "d_x", "d_u", "d_weight", "d_bias"):
            setattr(p, name, 0x1000)
    for k, v in over.items():
        setattr(p, k, v)
    return p


def test_c_abi_validation():
    L = _capi.lib()
    err = lambda: L.hstu_hip_last_error().decode()
    for over, text in ((dict(struct_size=3), "size mismatch"), (dict(rows=0), "x dim0 must in range:[1,1000000]"),
                       (dict(rows=1000001), "x dim0 must in range"), (dict(cols=768), "x dim1 must equal with 512 or 1024"),
                       (dict(eps=1e-3), "eps must in range"), (dict(eps=1e-11), "eps must in range"), (dict(dropout_ratio=1.5), "dropout_ratio must in range"),
                       (dict(dropout_ratio=-0.1), "dropout_ratio must in range"), (dict(dtype=9), "dtype expect"), (dict(u=None), "must not be NULL"),
                       (dict(dropout_ratio=0.3), "drop_mask with dropout")):
        assert L.hstu_hip_norm_multiply_dropout(C.byref(_params(**over)), None) == -1 and text in err(), (over, err())
    assert L.hstu_hip_norm_multiply_dropout(C.byref(_params(x=0x1004)), None) == -2 and "16-byte aligned" in err()
    b = _params(_capi.HstuNmdBwdParams)
    n = C.c_uint64(0)
    assert L.hstu_hip_norm_multiply_dropout_backward_get_workspace_size(C.byref(b), C.byref(n)) == 0
    assert n.value == 25 * 2 * 512 * 4           # 100 rows -> 25 workgroups of 4 rows, one [2, cols] fp32 partial each
    big = _params(_capi.HstuNmdBwdParams, rows=1000000, cols=1024)
    assert L.hstu_hip_norm_multiply_dropout_backward_get_workspace_size(C.byref(big), C.byref(n)) == 0 and n.value == 1024 * 2 * 1024 * 4
    assert L.hstu_hip_norm_multiply_dropout_backward(C.byref(b), None, 0, None) == -3 and "workspace" in err()
    assert L.hstu_hip_norm_multiply_dropout_backward(C.byref(_params(_capi.HstuNmdBwdParams, d_x=None)), 0x1000, 1 << 20, None) == -1


def test_torch_op_schema_and_checks():
    m = torch.ops.mxrec
    assert str(m.norm_multiply_dropout.default._schema) == \
        "mxrec::norm_multiply_dropout(Tensor x, Tensor u, Tensor weight, Tensor bias, float eps, float dropout_ratio) -> Tensor[]"
    x, w = torch.zeros(8, 512, dtype=torch.float16), torch.zeros(512, dtype=torch.float16)
    run = lambda x_=x, u_=x, w_=w, b_=w, eps=1e-5, r=0.1: m.norm_multiply_dropout(x_, u_, w_, b_, eps, r)
    for kw, text in ((dict(x_=x[None]), "norm_multiply_dropout input x must be 2D"), (dict(u_=x[None]), "norm_multiply_dropout input u must be 2D"),
                     (dict(w_=w[None]), "norm_multiply_dropout input weight must be 1D"), (dict(b_=w[None]), "norm_multiply_dropout input bias must be 1D"),
                     (dict(u_=x[:4]), "is not equal to u dim0"), (dict(u_=torch.zeros(8, 1024, dtype=torch.float16)), "is not equal to u dim1"),
                     (dict(b_=w[:256]), "must be same but not equal"), (dict(x_=torch.zeros(8, 768, dtype=torch.float16), u_=torch.zeros(8, 768, dtype=torch.float16),
                                                                        w_=torch.zeros(768, dtype=torch.float16), b_=torch.zeros(768, dtype=torch.float16)), "x dim1 must equal with"),
                     (dict(eps=1e-11), "eps must in range"), (dict(eps=1e-3), "eps must in range"), (dict(r=-0.1), "dropout_ratio must in range"),
                     (dict(r=1.1), "dropout_ratio must in range"), (dict(), "no CPU implementation")):
        with pytest.raises(RuntimeError, match=text):
            run(**kw)


def test_in_linear_silu_validation():
    """C ABI and torch op reject what the reference rejects (in_linear_silu.cpp:34-66; its tests
    test_in_linear_silu.py:133-161), before any launch."""
    L = _capi.lib()
    def call(**over):
        p = _capi.HstuInLinearSiluParams()
        p.struct_size = C.sizeof(_capi.HstuInLinearSiluParams)
        p.dtype, p.m, p.k, p.n = _capi.HSTU_F16, 100, 16, 64
        for i in range(4):
            p.split[i] = 16
            p.out[i] = 0x1000
        p.x = p.weight = p.bias = p.linear_output = 0x1000
        for k, v in over.items():
            if k == "split":
                for i, s_ in enumerate(v):
                    p.split[i] = s_
            else:
                setattr(p, k, v)
        return L.hstu_hip_in_linear_silu(C.byref(p), None), L.hstu_hip_last_error().decode()
    for over, text in ((dict(split=[16, 17, 15, 16]), "uvqk dim must in range[16, 8192] and multiples of 16"),
                       (dict(split=[16, 16, 32, 32]), "weight_dim[0] must equal to sum(splitList)"), (dict(k=24), "x dim[1] must in range[16, 8192] and multiples of 16"),
                       (dict(n=48, split=[16, 16, 16, 0]), "uvqk dim"), (dict(k=32), "weight dim[0] must be a multiple of 4 x dim[1]"),
                       (dict(dtype=_capi.HSTU_F32), "dtype expect float16 or bfloat16"), (dict(m=0), "x dim[0] must in range"), (dict(x=None), "must not be NULL")):
        rc, msg = call(**over)
        assert rc == -1 and text in msg, (over, msg)
    rc, msg = call(bias=0x1004)
    assert rc == -2 and "16-byte aligned" in msg
    m = torch.ops.mxrec
    assert str(m.distance_in_linear_silu.default._schema) == "mxrec::distance_in_linear_silu(Tensor x, Tensor weight, Tensor bias, int[] attr_dict) -> Tensor[]"
    x, w, b = torch.zeros(100, 16, dtype=torch.float16), torch.zeros(64, 16, dtype=torch.float16), torch.ones(64)
    for args, text in (((x, w, b, [16, 17, 15, 16]), "uvqk dim must in range"), ((x, w, b, [16, 16, 32, 32]), "must equal to sum"),
                       ((x, w, b, [16, 16, 32]), "splitList must have 4 elements"), ((x, w, x.clone(), [16] * 4), "bias must be 1D"),
                       ((x, w[None], b, [16] * 4), "weight must be 2D"), ((x, w[:, :8], b, [16] * 4), "weight dim\\[1\\] must equal to x dim\\[1\\]"),
                       ((x, w, b, [16] * 4), "no CPU implementation")):
        with pytest.raises(RuntimeError, match=text):
            m.distance_in_linear_silu(*args)


def test_in_linear_silu_backward_validation_and_workspace():
    """The backward's C ABI rejects what the reference's checks reject (in_linear_silu.cpp:34-66), sizes its workspace
    without a GPU, and the torch ops carry the reference's schemas (in_linear_silu.cpp:202-210)."""
    L = _capi.lib()
    def mk(**over):
        p = _capi.HstuInLinearSiluBwdParams()
        p.struct_size = C.sizeof(_capi.HstuInLinearSiluBwdParams)
        p.dtype, p.grad_dtype, p.m, p.k, p.n = _capi.HSTU_BF16, _capi.HSTU_BF16, 100, 16, 64
        for i in range(4):
            p.split[i] = 16
            p.grad[i] = 0x1000
        p.x = p.weight = p.linear_output = p.x_grad = p.weight_grad = p.bias_grad = 0x1000
        for k, v in over.items():
            if k == "split":
                for i, s_ in enumerate(v):
                    p.split[i] = s_
            else:
                setattr(p, k, v)
        return p
    def call(**over):
        p = mk(**over)
        return L.hstu_hip_in_linear_silu_backward(C.byref(p), 0x1000, 1 << 40, None), L.hstu_hip_last_error().decode()
    for over, text in ((dict(split=[16, 17, 15, 16]), "uvqk dim must in range[16, 8192] and multiples of 16"),
                       (dict(split=[16, 16, 32, 32]), "weight_dim[0] must equal to sum(splitList)"), (dict(k=24), "x dim[1] must in range"),
                       (dict(k=32), "weight dim[0] must be a multiple of 4 x dim[1]"), (dict(dtype=_capi.HSTU_F32), "dtype expect float16 or bfloat16"),
                       (dict(grad_dtype=_capi.HSTU_F16), "grad_dtype expect float32 or the dtype of x"), (dict(m=0), "x dim[0] must in range"),
                       (dict(algorithm=3), "algorithm expect 0, 1 or 2"), (dict(algorithm=2, k=128, n=512, split=[128] * 4), "needs x dim[1] <= 64"), (dict(x_grad=None), "must not be NULL")):
        rc, msg = call(**over)
        assert rc == -1 and text in msg, (over, msg)
    rc, msg = call(bias_grad=0x1004)
    assert rc == -2 and "16-byte aligned" in msg
    p = mk()
    rc = L.hstu_hip_in_linear_silu_backward(C.byref(p), 0x1000, 16, None)
    assert rc == -3 and "workspace" in L.hstu_hip_last_error().decode()
    need = C.c_uint64(0)
    # m = 100 -> x^T padded to 128 rows; operand fragments of 1 KiB (32 columns k x 16 rows, k padded to 32); one range
    # of rows per 32-row tile at most
    assert L.hstu_hip_in_linear_silu_backward_get_workspace_size(C.byref(p), C.byref(need)) == 0
    parts = 4
    al = lambda v: (v + 255) // 256 * 256
    # (the library's choice at k <= 64 is the one-pass kernel: its x_grad leaves as one partial slab per 512 columns of n)
    assert need.value == al(128 // 16 * 1024) + al(64 // 16 * 1024) + al(parts * 64 * 16 * 4) + al(parts * 64 * 4) + al(1 * 100 * 16 * 4)
    p.algorithm = 1
    assert L.hstu_hip_in_linear_silu_backward_get_workspace_size(C.byref(p), C.byref(need)) == 0
    assert need.value == al(128 // 16 * 1024) + al(64 // 16 * 1024) + al(parts * 64 * 16 * 4) + al(parts * 64 * 4)
    big = mk(m=16384, k=64, n=16384, split=[4096] * 4, algorithm=1)
    assert L.hstu_hip_in_linear_silu_backward_get_workspace_size(C.byref(big), C.byref(need)) == 0
    # the two product kernels: 16 ranges of m for weight_grad, 2 ranges of n for x_grad
    assert need.value == al(64 * 16384 * 2) * 2 + al(16 * 16384 * 64 * 4) + al(16 * 16384 * 4) + al(2 * 16384 * 64 * 4)
    for algorithm in (0, 2):
        # one pass: 8 ranges of m (one workgroup per CU), 32 slabs of x_grad
        big.algorithm = algorithm
        assert L.hstu_hip_in_linear_silu_backward_get_workspace_size(C.byref(big), C.byref(need)) == 0
        assert need.value == al(64 * 16384 * 2) * 2 + al(8 * 16384 * 64 * 4) + al(8 * 16384 * 4) + al(32 * 16384 * 64 * 4)
    m = torch.ops.mxrec
    assert str(m.in_linear_silu.default._schema) == "mxrec::in_linear_silu(Tensor x, Tensor weight, Tensor bias, int[] attr_dict) -> Tensor[]"
    assert str(m.in_linear_silu_backward.default._schema) == ("mxrec::in_linear_silu_backward(Tensor x, Tensor weight, Tensor? bias, Tensor user_grad, "
        "Tensor value_grad, Tensor query_grad, Tensor key_grad, Tensor linear_output, int[] attr_dict) -> Tensor[]")
    x, w = torch.zeros(100, 16, dtype=torch.float16), torch.zeros(64, 16, dtype=torch.float16)
    gs = [torch.zeros(100, 16, dtype=torch.float16) for _ in range(4)]
    lin = torch.zeros(100, 64, dtype=torch.float16)
    for args, text in (((x, w, None, *gs, lin, [16, 17, 15, 16]), "uvqk dim must in range"),
                       ((x, w, None, gs[0][:, :8], *gs[1:], lin, [16] * 4), "must be equal to splitList"),
                       ((x, w, None, gs[0][:50], *gs[1:], lin, [16] * 4), "dim\\[0\\] must equal to x dim\\[0\\]"),
                       ((x, w, None, *gs, lin[:, :32], [16] * 4), "linear_output dim\\[1\\] must equal to weight dim\\[0\\]"),
                       ((x, w, None, *gs, lin, [16] * 4), "no CPU implementation")):
        with pytest.raises(RuntimeError, match=text):
            m.in_linear_silu_backward(*args)
