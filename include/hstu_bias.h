/*
 * hstu_bias.h -- C ABI of the standalone producers of the dense attention-bias tensors (relative position, time
 * buckets) that models hand to the attention ops as attn_bias, and of the gradient of the time-bucket weights.
 *
 * Same conventions as hstu_hip.h: device pointers unless stated, asynchronous on `stream`, nothing read on the host,
 * 0 or a negative hstu_status with the message in hstu_hip_last_error().  dtype: HSTU_F32 / HSTU_F16 / HSTU_BF16.
 */
#ifndef HSTU_BIAS_H
#define HSTU_BIAS_H

#include "hstu_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* limits of the reference's host checks (relative_attn_bias_time/v220/op_host/relative_attn_bias_time.cpp:40-43) */
#define HSTU_RAB_MAX_LAYERS 20
#define HSTU_RAB_MAX_BUCKETS 129 /* columns of timestamps_weights */
#define HSTU_RAB_MAX_SEQ_LEN 4300

/* Time-bucket bias.  Replaces aclnnRelativeAttnBiasTime and the repeat the reference's wrapper applies to its output
 * (cust_op/framework/torch_plugin/torch_library/relative_attn_bias/relative_attn_bias_time.cpp:29-62):
 *   bucket[b,i,j] = trunc(log(clamp(|t[b,i] - t[b,j]|, 1, e^((W-1)*divisor))) / divisor)      W = weight_cols
 *   rab_time_out[n, b, 2i+a, 2j+c] = weights[n, bucket[b,i,j]]        a, c in {0, 1}
 *   bucket_ts_out[b, i, j] = bucket[b,i,j]                            (optional)
 * The bucket is found by comparing |dt| (as fp32) with bucket_bounds: [W + 1] floats, bounds[0] = 0, bounds[k] = the
 * smallest fp32 |dt| of bucket k (k = 1..W-1), bounds[W] = +inf -- the table hstu_fwd_params.ts_bounds takes. */
typedef struct hstu_rab_time_params {
    uint32_t struct_size;
    int32_t dtype;              /* of weights and rab_time_out */
    int32_t index_type;         /* of timestamps and bucket_ts_out: HSTU_I32 / HSTU_I64 */
    int32_t num_layers;
    int32_t batch;
    int32_t seq_len;            /* s */
    int32_t weight_cols;        /* W */
    float bucket_divisor;       /* the divisor the bounds were made for: a first guess only, the ids are decided by
                                   bucket_bounds; <= 0: not known */
    const void* timestamps;     /* [batch, s] */
    const void* weights;        /* [num_layers, W] */
    const float* bucket_bounds; /* [W + 1] */
    void* rab_time_out;         /* [num_layers, batch, 2s, 2s] */
    void* bucket_ts_out;        /* [batch, s, s] or NULL */
} hstu_rab_time_params;
int hstu_hip_rab_time(const hstu_rab_time_params* p, void* stream);

/* Gradient of the weights.  Replaces aclnnRelativeAttnBiasBackward and the repeat its wrapper applies to the bucket
 * ids (relative_attn_bias_time.cpp:64-85):
 *   grad_weights[n, k] = sum over b, i, j with bucket_ts[b,i,j] == k, a, c of grad[n, b, 2i+a, 2j+c]     (fp32)
 * Ids outside [0, num_buckets) contribute nothing.  The sums are formed with floating-point atomics: their order, and
 * with it the last bits of the result, can differ from run to run. */
typedef struct hstu_rab_time_bwd_params {
    uint32_t struct_size;
    int32_t dtype;              /* of grad */
    int32_t index_type;         /* of bucket_ts */
    int32_t num_layers;
    int32_t batch;
    int32_t seq_len;            /* s: grad is [num_layers, batch, 2s, 2s], bucket_ts [batch, s, s] */
    int32_t num_buckets;        /* columns of grad_weights */
    int32_t reserved;
    const void* grad;
    const void* bucket_ts;
    float* grad_weights;        /* [num_layers, num_buckets] fp32, overwritten */
} hstu_rab_time_bwd_params;
int hstu_hip_rab_time_backward(const hstu_rab_time_bwd_params* p, void* stream);

/* Relative-position bias per user.  Replaces aclnnRelativeAttnBiasPos (relative_attn_bias_pos.cpp:22-43; golden
 * cust_op/test/relative_attn_bias/torch/utils.py:143-163):
 *   r[b,i,j]   = rel_pos_bias[min(i, past_valid_lens[b]), j]
 *   out[b,i,j] = r[b,i,j] * (1 - identity[i,j]) + identity[i,j] * rel_pos_bias[0,0]
 * every operation rounded to the tensors' dtype.  With the 0/1 identity the reference builds this selects
 * rel_pos_bias[0,0] on the marked entries and copies r elsewhere, exactly.
 * past_valid_lens is a HOST array (the reference passes it as an attribute); entries must lie in [0, seq2). */
int hstu_hip_rab_pos(int32_t dtype, int32_t seq2, const void* rel_pos_bias, const void* identity,
                     const int64_t* past_valid_lens_host, int32_t batch, void* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HSTU_BIAS_H */
