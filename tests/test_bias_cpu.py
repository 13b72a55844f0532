"""Host-side checks of the bias-producer C ABI and torch ops (no GPU needed)."""
import ctypes as C

import pytest
import torch

import recsdk_amd  # noqa: F401  (registers torch.ops.mxrec.*)
from recsdk_amd import _capi


def _time_params(**over):
    p = _capi.HstuRabTimeParams()
    p.struct_size = C.sizeof(_capi.HstuRabTimeParams)
    p.dtype, p.index_type = _capi.HSTU_F16, _capi.HSTU_I32
    p.num_layers, p.batch, p.seq_len, p.weight_cols = 2, 3, 40, 129
    for f in ("timestamps", "weights", "bucket_bounds", "rab_time_out", "bucket_ts_out"):
        setattr(p, f, 0x1000)
    for k, v in over.items():
        setattr(p, k, v)
    return p


def _call(fn, p):
    rc = getattr(_capi.lib(), fn)(C.byref(p), None)
    return rc, _capi.lib().hstu_hip_last_error().decode()


def test_rab_time_validation():
    """Every case is rejected before a launch (the limits are the reference's, relative_attn_bias_time.cpp op_host:40-43)."""
    for over, text in ((dict(struct_size=4), "size mismatch"), (dict(seq_len=4301), "between 1 and 4300"), (dict(seq_len=0), "between 1 and 4300"),
                       (dict(num_layers=21), "num_layer expects a value in the range [1, 20]"), (dict(weight_cols=130), "num_buckets expects a value in the range [1, 129]"),
                       (dict(dtype=7), "Invalid data type of timestamps_weights"), (dict(index_type=5), "Invalid data type of timestamps"),
                       (dict(batch=0), "batchsize"), (dict(weights=None), "must not be NULL")):
        rc, msg = _call("hstu_hip_rab_time", _time_params(**over))
        assert rc == -1 and text in msg, (over, msg)
    rc, msg = _call("hstu_hip_rab_time", _time_params(rab_time_out=0x1004))
    assert rc == -2 and "16-byte aligned" in msg


def test_rab_time_backward_and_pos_validation():
    p = _capi.HstuRabTimeBwdParams()
    p.struct_size = C.sizeof(_capi.HstuRabTimeBwdParams)
    p.dtype, p.index_type, p.num_layers, p.batch, p.seq_len, p.num_buckets = _capi.HSTU_F32, _capi.HSTU_I32, 2, 2, 8, 130
    p.grad = p.bucket_ts = p.grad_weights = 0x1000
    rc, msg = _call("hstu_hip_rab_time_backward", p)
    assert rc == -1 and "num_buckets expects a value in the range [1, 129]" in msg
    p.num_buckets, p.seq_len = 128, 5000
    rc, msg = _call("hstu_hip_rab_time_backward", p)
    assert rc == -1 and "Sequence len expects a value in the range [1, 8600]" in msg
    L = _capi.lib()
    lens = (C.c_int64 * 2)(1, 9)
    rc = L.hstu_hip_rab_pos(_capi.HSTU_F32, 8, 0x1000, 0x1000, lens, 2, 0x1000, None)
    assert rc == -1 and "past_valid_lens[1] expected in [0, 8), but got 9" in L.hstu_hip_last_error().decode()
    rc = L.hstu_hip_rab_pos(_capi.HSTU_F32, 0, 0x1000, 0x1000, lens, 2, 0x1000, None)
    assert rc == -1 and "Invalid sequence len of rel_pos_bias" in L.hstu_hip_last_error().decode()


def test_torch_ops_have_the_reference_schemas_and_checks():
    m = torch.ops.mxrec
    assert str(m.relative_attn_bias_time.default._schema) == \
        "mxrec::relative_attn_bias_time(Tensor timestamps, Tensor timestamps_weights, float bucket_divisor) -> Tensor"
    assert str(m.relative_attn_bias_time_with_index.default._schema).endswith("-> Tensor[]")
    assert str(m.relative_attn_bias_time_backward.default._schema) == \
        "mxrec::relative_attn_bias_time_backward(Tensor rab_time_grad, Tensor bucket_timestamps, int num_buckets) -> Tensor"
    assert str(m.relative_attn_bias_pos.default._schema) == \
        "mxrec::relative_attn_bias_pos(Tensor rel_pos_bias, Tensor identity, int[] past_valid_lens) -> Tensor"
    ts, w = torch.zeros(2, 8, dtype=torch.int32), torch.zeros(2, 129)
    with pytest.raises(RuntimeError, match="timestampsWeightsConti must be 2D"):
        m.relative_attn_bias_time(ts, w[0], 0.301)
    with pytest.raises(RuntimeError, match="timestamps size must be between 1 and 4300"):
        m.relative_attn_bias_time(torch.zeros(1, 4301, dtype=torch.int32), w, 0.301)
    with pytest.raises(RuntimeError, match="tensor must be non-empty"):
        m.relative_attn_bias_time(ts[:0], w, 0.301)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        m.relative_attn_bias_time(ts, w, 0.301)
    with pytest.raises(RuntimeError, match="rabTimeGrad must be 4D"):
        m.relative_attn_bias_time_backward(torch.zeros(2, 4, 4), torch.zeros(1, 2, 2, dtype=torch.int32), 128)
    with pytest.raises(RuntimeError, match="Mismatch sequence len of rel_pos_bias and identity"):
        m.relative_attn_bias_pos(torch.zeros(4, 4), torch.zeros(4, 6), [1])
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        m.relative_attn_bias_pos(torch.zeros(4, 4), torch.zeros(4, 4), [1])
