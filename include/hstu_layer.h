/*
 * hstu_layer.h -- C ABI of the steps either side of the attention in an HSTU layer: the input projection
 * SiLU(x W^T + b) split into U, V, Q, K before it (mxrec::in_linear_silu, forward and backward), and LayerNorm(x) * u with
 * dropout after it, forward and backward (mxrec::norm_multiply_dropout).
 *
 * Same conventions as hstu_hip.h: device pointers, asynchronous on `stream`, nothing read on the host, 0 or a negative
 * hstu_status with the message in hstu_hip_last_error().  dtype: HSTU_F32 / HSTU_F16 / HSTU_BF16 for x, u, weight,
 * bias and the outputs shaped like them.
 *
 *   x_hat = (x - mean) / sqrt(var + eps)              mean, var over the columns of a row (var biased), fp32
 *   y     = dropout((x_hat * weight + bias) * u, p)   dropout: kept elements scaled by 1 / (1 - p)
 * (cust_op/ascendc_op/ai_core_op/norm_multiply_dropout/v220/README.md:41-60).
 *
 * Dropout mask: bit (e % 8) of byte (e / 8) is 1 where flat element e = row * cols + col is kept; the buffer holds
 * ceil(rows * cols / 128) * 16 bytes like the reference's (norm_multiply_dropout.cpp:38-45).  The forward fills it
 * from (seed, element index) with a counter-based generator of this library; which elements are dropped therefore
 * differs from the reference's generator (aclnnDropoutGenMaskV2), as it differs between any two seeds.
 */
#ifndef HSTU_LAYER_H
#define HSTU_LAYER_H

#include "hstu_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

#define HSTU_NMD_MAX_ROWS 1000000 /* norm_multiply_dropout.cpp:28-31: rows in [1, 1e6], cols 512 or 1024 */

/* Replaces aclnnNormMultiplyDropout (norm_multiply_dropout.cpp:69-94). */
typedef struct hstu_nmd_params {
    uint32_t struct_size;
    int32_t dtype;
    int64_t rows;
    int32_t cols;
    float eps;             /* [1e-10, 1e-4] */
    float dropout_ratio;   /* [0, 1]; <= 1e-10: no dropout, drop_mask is neither written nor read */
    uint32_t reserved;
    uint64_t seed;
    const void* x;         /* [rows, cols] */
    const void* u;         /* [rows, cols] */
    const void* weight;    /* [cols] */
    const void* bias;      /* [cols] */
    void* out;             /* [rows, cols] */
    float* mean;           /* [rows] */
    float* var;            /* [rows] */
    uint8_t* drop_mask;    /* see above; may be NULL without dropout */
} hstu_nmd_params;
int hstu_hip_norm_multiply_dropout(const hstu_nmd_params* p, void* stream);

/* Replaces aclnnNormMultiplyDropoutBackward (norm_multiply_dropout.cpp:97-111; formulas of the golden
 * cust_op/test/norm_multiply_dropout/torch/test_norm_multiply_dropout.py:220-243):
 *   g = dropout'(d_out) * u          d_weight = sum over rows of x_hat * g        d_bias = sum over rows of g
 *   a = g * weight                   d_x = (a - (sum_c a + x_hat * sum_c a * x_hat) / cols) / sqrt(var + eps)
 *   d_u = dropout'(d_out) * (weight * x_hat + bias)
 * The column sums are formed in a fixed order (per-workgroup partial sums in the workspace, then one pass over them):
 * results are reproducible. */
typedef struct hstu_nmd_bwd_params {
    uint32_t struct_size;
    int32_t dtype;
    int64_t rows;
    int32_t cols;
    float eps;
    float dropout_ratio;
    uint32_t reserved;
    const void* d_out;
    const void* x;
    const void* u;
    const void* weight;
    const void* bias;
    const float* mean;         /* from the forward */
    const float* var;
    const uint8_t* drop_mask;  /* from the forward; may be NULL without dropout */
    void* d_x;
    void* d_u;
    float* d_weight;           /* [cols] fp32, overwritten */
    float* d_bias;             /* [cols] fp32, overwritten */
} hstu_nmd_bwd_params;
int hstu_hip_norm_multiply_dropout_backward_get_workspace_size(const hstu_nmd_bwd_params* p, uint64_t* workspace_bytes);
int hstu_hip_norm_multiply_dropout_backward(const hstu_nmd_bwd_params* p, void* workspace, uint64_t workspace_bytes, void* stream);

/* Input projection.  Replaces aclnnInLinearSilu (cust_op/framework/torch_plugin/torch_library/in_linear_silu/
 * in_linear_silu.cpp:96-117; golden cust_op/test/in_linear_silu_test/test_in_linear_silu.py:31-45):
 *   linear_output = round(x W^T + bias)               [m, n], fp32 accumulation, rounded to the I/O dtype
 *   (user | value | query | key) = round(silu(linear_output)) split along n into widths split[0..3]
 * dtype: HSTU_F16 / HSTU_BF16 for x, weight and the outputs; bias is fp32 and may be NULL (no bias).
 * Limits of the reference's checks (in_linear_silu.cpp:34-66): k in [16, 8192], n in [64, 32768], every split width in
 * [16, 8192], all multiples of 16; sum(split) == n; n a multiple of 4 k. */
typedef struct hstu_in_linear_silu_params {
    uint32_t struct_size;
    int32_t dtype;
    int64_t m;
    int32_t k;
    int32_t n;
    int32_t split[4];         /* widths of user, value, query, key */
    const void* x;            /* [m, k] */
    const void* weight;       /* [n, k] */
    const float* bias;        /* [n] or NULL */
    void* out[4];             /* user [m, split[0]], value [m, split[1]], query [m, split[2]], key [m, split[3]] */
    void* linear_output;      /* [m, n] */
} hstu_in_linear_silu_params;
int hstu_hip_in_linear_silu(const hstu_in_linear_silu_params* p, void* stream);

/* Backward of the input projection.  Replaces aclnnInLinearSiluBackward (in_linear_silu.cpp:121-163; golden
 * cust_op/test/in_linear_silu_test_backward/test_in_linear_silu_backward.py:37-66):
 *   dlin = round(grad * silu'(linear_output))   grad = (grad[0] | grad[1] | grad[2] | grad[3]) along n,
 *                                               silu'(z) = s (1 + z (1 - s)), s = sigmoid(z)
 *   x_grad = dlin W  [m, k]     weight_grad = dlin^T x  [n, k]     bias_grad = column sums of the unrounded dlin  [n]
 * The four gradients are read where they are (the reference concatenates them first when the widths differ, :143-146).
 * x_grad and weight_grad are written in grad_dtype: HSTU_F32 (what the reference's kernel produces, :139-140) or the
 * dtype of x (what its wrapper hands back after a cast, :158); nothing needs zeroing.  Sums over m are formed in a fixed
 * order: results are reproducible.  The workspace needs no initialisation and must be 16-byte aligned. */
typedef struct hstu_in_linear_silu_bwd_params {
    uint32_t struct_size;
    int32_t dtype;            /* HSTU_F16 / HSTU_BF16: x, weight, grad[], linear_output */
    int64_t m;
    int32_t k;
    int32_t n;
    int32_t split[4];
    int32_t grad_dtype;       /* HSTU_F32 or dtype */
    int32_t algorithm;        /* 0: the library chooses (today: 2 for k <= 64, else 1); 1: two product kernels that each
                                 stream the inputs; 2: one pass over the inputs, k <= 64 only: x_grad as fp32 partial slabs
                                 per 512 columns of n in the workspace (ceil(n / 512) * m * k * 4 bytes); half the HBM
                                 traffic, a third less time at m = n = 16384 */
    const void* x;            /* [m, k] */
    const void* weight;       /* [n, k] */
    const void* grad[4];      /* user_grad [m, split[0]], value_grad, query_grad, key_grad */
    const void* linear_output;/* [m, n], from the forward */
    void* x_grad;             /* [m, k] */
    void* weight_grad;        /* [n, k] */
    float* bias_grad;         /* [n] fp32, or NULL */
} hstu_in_linear_silu_bwd_params;
int hstu_hip_in_linear_silu_backward_get_workspace_size(const hstu_in_linear_silu_bwd_params* p, uint64_t* workspace_bytes);
int hstu_hip_in_linear_silu_backward(const hstu_in_linear_silu_bwd_params* p, void* workspace, uint64_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HSTU_LAYER_H */
