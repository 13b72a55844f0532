/*
 * hstu_hip.h -- C ABI of the MI355X (gfx950) HSTU fused attention forward (and the jagged backward).
 *
 * out = (SiLU(alpha * (Q K^T + bias)) * silu_scale * mask) V   over packed ("jagged") sequences,
 * no softmax, no materialised score matrix.
 *
 * This is the boundary a host framework binds to.  It plays the role of the two-phase aclnn C entry
 * points the reference's torch plugin resolves with dlsym and calls through EXEC_NPU_CMD
 * (cust_op/framework/torch_plugin/torch_library/common/pytorch_npu_helper.hpp:508-558):
 *     aclnnXGetWorkspaceSize(args..., &ws_bytes, &executor);  aclnnX(ws, ws_bytes, executor, stream);
 * Here the argument list is a POD struct of raw device pointers and sizes; there are no torch types.
 * Every call is asynchronous on `stream` (a hipStream_t passed as void*; NULL = the null stream),
 * never synchronises the device and never reads a device buffer on the host.
 * All functions return 0 on success and a negative hstu_status otherwise; the message for the
 * calling thread is available from hstu_hip_last_error() (the role of aclGetRecentErrMsg()).
 */
#ifndef HSTU_HIP_H
#define HSTU_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HSTU_HIP_ABI_VERSION 1

typedef enum hstu_status {
    HSTU_OK = 0,
    HSTU_ERR_INVALID_ARGUMENT = -1, /* shape / attribute rejected (reference: op_host tiling checks) */
    HSTU_ERR_UNSUPPORTED = -2,      /* valid in the reference, not built here */
    HSTU_ERR_WORKSPACE = -3,        /* workspace pointer missing or too small */
    HSTU_ERR_LAUNCH = -4            /* HIP runtime refused the launch */
} hstu_status;

typedef enum hstu_dtype { HSTU_F32 = 0, HSTU_F16 = 1, HSTU_BF16 = 2, HSTU_FP8_E4M3 = 3 } hstu_dtype;
typedef enum hstu_index_type { HSTU_I32 = 0, HSTU_I64 = 1 } hstu_index_type;

/* mask_type values of the reference (hstu_common.h:47-50). 1 (triu) is rejected like there. */
enum { HSTU_MASK_TRIL = 0, HSTU_MASK_TRIU = 1, HSTU_MASK_NONE = 2, HSTU_MASK_CUSTOM = 3 };

/* limits of the reference's host checks (hstu_common.h:30-45, tiling_policy.cpp:69-94) */
#define HSTU_MAX_BATCH 2048
#define HSTU_MAX_SEQ_LEN 20480
#define HSTU_MAX_HEADS 16
#define HSTU_MAX_HEAD_DIM 512

/* flags */
#define HSTU_FLAG_DETERMINISTIC 1u /* accepted; every output row has one producer, so results never depend on it */
#define HSTU_FLAG_FORCE_GENERIC 2u /* run the plain fp32-FMA kernel even where an MFMA kernel exists (testing) */
/* The workspace still holds the work list an earlier call built for the same sequence offsets, num_context,
 * num_target, page offsets, shapes and attributes (e.g. the other layers of one model on one batch): do not
 * rebuild it.  Only q/k/v/out/bias/table contents may differ between such calls.  (Every call without the flag leaves
 * the list in the workspace, also the calls that need no schedule kernel of their own: self-attention under the causal
 * mask or none on at most 128 sequences at head dims 32, 64 and 128, whose workgroups derive their items from the offsets and write them down as
 * they go.) */
#define HSTU_FLAG_REUSE_WORKSPACE 4u
/* backward only: run all kernels of this call on `stream` itself (see hstu_hip_jagged_backward) */
#define HSTU_FLAG_SERIAL_BACKWARD 8u

/*
 * One argument block for the three forward ops.  Pointers are device pointers unless stated.
 * Layouts (row-major, innermost last):
 *   q   [total_q, heads_q, dim_qk]     k [total_k, heads_k, dim_qk]     v [total_k, heads_k, dim_v]
 *   out [total_q, heads_q, dim_v]      same dtype as q; fp16 when q / k / v are FP8_E4M3 (reference: hstu_jagged.cpp:53-54)
 *   seq_offset_q / seq_offset_k  [batch+1] of index_type; sequence b owns rows off[b]..off[b+1]-1.
 *     Q row i of a sequence sits at position i + (Lk - Lq) of its K timeline ("delta-q").
 *     Both NULL = dense layout: every sequence has max_seq_len_q (= max_seq_len_k) rows.
 *   mask, attn_bias  [batch, heads_q, max_seq_len_q, max_seq_len_k] in `dtype`, or NULL
 *   num_context, num_target  [batch] of index_type, or NULL (= zeros)
 * (reference: hstu_jagged.cpp:22-67, hstu_jagged_forward_kernel.h:457-459,507-510)
 */
typedef struct hstu_fwd_params {
    uint32_t struct_size; /* sizeof(hstu_fwd_params) of the caller, for ABI checking */
    uint32_t flags;
    int32_t dtype;      /* hstu_dtype of q/k/v/out/mask/attn_bias: F32, F16 or BF16; FP8_E4M3 (float8_e4m3fn q/k/v/mask/attn_bias,
                           fp16 out, scores and sums in fp32, P rounded to e4m3 before P*V) in the jagged and dense forward only */
    int32_t index_type; /* hstu_index_type of every integer tensor */

    const void* q;
    const void* k;
    const void* v;
    void* out;
    const void* mask;
    const void* attn_bias;
    const void* seq_offset_q;
    const void* seq_offset_k;
    const void* num_context;
    const void* num_target;

    int64_t total_q;
    int64_t total_k;
    int32_t batch;
    int32_t heads_q;
    int32_t heads_k;
    int32_t dim_qk;
    int32_t dim_v;
    int32_t mask_type;
    int32_t max_seq_len_q;
    int32_t max_seq_len_k;
    int32_t target_group_size;
    float silu_scale; /* already resolved: the caller applies "0 means 1/max_seq_len_q" */
    float alpha;

    /*
     * Paged history (hstu_paged only; reference hstu_paged_forward_kernel.h:469-532).
     * K/V column j of user b:  j < hist_b  ->  kv_cache[page_ids[page_offsets[b] + j / page_size]][0|1][j % page_size][kv head][:]
     *                          else        ->  input k/v row seq_offset_q[b] + (Lq_b - num_target_b) + (j - hist_b)
     * with hist_b = Lk_b - num_target_b.
     *   kv_cache [num_pages, 2, page_size, heads_k, dim] in cache_dtype (== dtype, or FP8_E4M3)
     *   kv_scales [num_pages, 2, heads_k] float, dequantised value = fp8 * scale (FP8_E4M3 caches only;
     *   this cache format has no counterpart in the reference)
     */
    const void* kv_cache;
    const void* page_offsets;  /* [batch+1] */
    const void* page_ids;      /* [page_offsets[batch]] */
    const void* last_page_len; /* [batch]; implied by seq_offset_k, accepted for signature parity */
    const float* kv_scales;
    int64_t num_pages;
    int32_t page_size;
    int32_t cache_dtype;

    /*
     * Fused bias tables (no counterpart in the reference op, which takes the dense attn_bias that
     * relative_attn_bias_pos/_time produce: cust_op/test/relative_attn_bias/torch/utils.py:38-51,99-129).
     *   pos_table [2*max_seq_len_k - 1] float:  bias += pos_table[(max_seq_len_k-1) + j - (i + Lk - Lq)]
     *   timestamps [total_k] int64 on the K timeline; ts_table [num_buckets+1] float;
     *   ts_bounds [num_buckets+2] float, ascending, bounds[0] = 0, bounds[num_buckets+1] = +inf:
     *     bucket(i,j) = the b with bounds[b] <= (float)|t_i - t_j| < bounds[b+1];  bias += ts_table[bucket]
     *   ts_log2_scale: optional search hint.  If non-zero, bounds[b] must sit near 2^(b / ts_log2_scale), within half
     *     a bucket (for the reference's log buckets the scale is ln(2)/bucket_divisor).  The matrix-core kernels then
     *     keep a table in LDS that is indexed by the exponent and top three mantissa bits of (float)|dt|: a cell spans at
     *     most a factor 1.125, so (for ts_log2_scale <= 5, buckets at least 2^(1/5) apart) at most one bound falls into
     *     it and one comparison with that exact bound picks the bucket; the hint is only used to build the table.
     *     0, a larger scale, or num_buckets > 62 * ts_log2_scale = binary search over ts_bounds.  With the table the
     *     kernel takes |dt| from timestamps held as doubles relative to the sequence's first one: exact while one
     *     sequence spans < 2^53 ticks.
     * Added to attn_bias when both are given.
     */
    const float* pos_table;
    const float* ts_table;
    const float* ts_bounds;
    const int64_t* timestamps;
    int32_t num_buckets;
    float ts_log2_scale;
} hstu_fwd_params;

/* replaces aclnnHstuJaggedForwardGetWorkspaceSize / aclnnHstuJaggedForward (hstu_jagged.cpp:63-65).
 * The workspace needs no initialisation; the MFMA kernels keep their work list (tiles sorted by length, grouped
 * per XCD) in it, the plain kernel needs none.  It must be 16-byte aligned. */
int hstu_hip_jagged_forward_get_workspace_size(const hstu_fwd_params* p, uint64_t* workspace_bytes);
int hstu_hip_jagged_forward(const hstu_fwd_params* p, void* workspace, uint64_t workspace_bytes, void* stream);

/*
 * hstu_hip_jagged_forward for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as
 * hstu_hip_jagged_forward without a workspace: the work list lives in a fixed array of HSTU_NOALLOC_SCRATCH_BYTES
 * that the library holds in the memory of every GPU it runs on until the process ends.  The call allocates nothing
 * (the first call on a GPU looks the array's address up once; make that call outside a capture).
 *   - a batch whose work list does not fit is rejected with HSTU_ERR_WORKSPACE (the list takes about 64 bytes per
 *     128-row Q tile and head: the array holds about 30 000 of them);
 *   - every Q tile stays one work item (hstu_hip_jagged_forward splits the K range of serving-shaped batches and adds
 *     the parts through its workspace), and HSTU_FLAG_REUSE_WORKSPACE is ignored: the list is rebuilt by every call;
 *   - all calls on one GPU share the array: calls that overlap on one GPU (two streams, two threads) race.
 *     Calls on one stream are ordered and safe.
 */
#define HSTU_NOALLOC_SCRATCH_BYTES (2u << 20)
int hstu_hip_jagged_forward_noalloc(const hstu_fwd_params* p, void* stream);

/* replaces aclnnHstuPagedForwardGetWorkspaceSize / aclnnHstuPagedForward (hstu_paged.cpp:67-69) */
int hstu_hip_paged_forward_get_workspace_size(const hstu_fwd_params* p, uint64_t* workspace_bytes);
int hstu_hip_paged_forward(const hstu_fwd_params* p, void* workspace, uint64_t workspace_bytes, void* stream);

/* replaces aclnnHstuDenseForwardGetWorkspaceSize / aclnnHstuDenseForward (hstu_dense.cpp:37-39);
 * q/k/v are [batch, max_seq_len_q, heads, dim]; seq_offset_* must be NULL */
int hstu_hip_dense_forward_get_workspace_size(const hstu_fwd_params* p, uint64_t* workspace_bytes);
int hstu_hip_dense_forward(const hstu_fwd_params* p, void* workspace, uint64_t workspace_bytes, void* stream);

/*
 * Backward of the jagged op (the .equal and .delta overloads; seq_offset_k == seq_offset_q for .equal).
 * replaces aclnnHstuJaggedBackwardGetWorkspaceSize / aclnnHstuJaggedBackward (hstu_jagged.cpp:69-138):
 *     x  = alpha * (Q K^T + bias)        P  = silu(x) * silu_scale * mask
 *     dS = (dO V^T) * silu_scale * mask * sigmoid(x) * (1 + x * (1 - sigmoid(x))) * alpha
 *     dQ = dS K     dK = dS^T Q     dV = P^T dO     dBias = dS
 * (golden: build/presmoke/hstu/hstu_common.py:387-476).  `fwd` holds the arguments of the forward call; its `out`
 * is not read and may be NULL.  Only what the reference's backward takes is accepted: dense attn_bias (no bias
 * tables), built-in or custom mask, no paged cache.  P and dS are rounded to the I/O dtype before the second
 * GEMMs like P in the forward; every gradient element has one producing workgroup and a fixed summation order
 * (deterministic, no atomics).  With GQA, grad_k / grad_v sum over the query heads of a K/V head.
 */
typedef struct hstu_bwd_params {
    uint32_t struct_size;   /* sizeof(hstu_bwd_params) */
    uint32_t reserved;
    hstu_fwd_params fwd;
    const void* grad_out;   /* [total_q, heads_q, dim_v]   upstream gradient, I/O dtype */
    void* grad_q;           /* [total_q, heads_q, dim_qk]  every row is written (rows past the last offset: zeros) */
    void* grad_k;           /* [total_k, heads_k, dim_qk] */
    void* grad_v;           /* [total_k, heads_k, dim_v] */
    void* grad_bias;        /* [batch, heads_q, max_seq_len_q, max_seq_len_k] or NULL; required iff fwd.attn_bias;
                             * written completely (zeros outside the sequences and where the mask is 0) */
} hstu_bwd_params;

/* To the caller the backward is one piece of work on `stream`, also under stream capture.  Large calls (3000 and more
 * (Q tile, head) items) run their dQ and K-side kernels side by side on two streams of the library's own, forked from and
 * joined to `stream` by events (default priority; one pair per caller stream, up to 8 per device, created at that stream's
 * first such call outside a capture -- a capture that comes first runs on `stream` alone).  While such a call is being
 * captured its side streams capture too: another host thread's large backward on the same caller stream must not overlap
 * the capture.  HSTU_FLAG_SERIAL_BACKWARD in fwd.flags keeps the call on `stream`; HSTU_HIP_SERIAL_BACKWARD=1 in the
 * environment (read once) does so for every call. */
int hstu_hip_jagged_backward_get_workspace_size(const hstu_bwd_params* p, uint64_t* workspace_bytes);
int hstu_hip_jagged_backward(const hstu_bwd_params* p, void* workspace, uint64_t workspace_bytes, void* stream);

/* Backward of the dense op: replaces aclnnHstuDenseBackwardGetWorkspaceSize / aclnnHstuDenseBackward
 * (hstu_dense.cpp:43-153).  Same argument block; fwd as for hstu_hip_dense_forward (seq_offset_* NULL, q/k/v and the
 * gradients [batch, max_seq_len_q, heads, dim]). */
int hstu_hip_dense_backward_get_workspace_size(const hstu_bwd_params* p, uint64_t* workspace_bytes);
int hstu_hip_dense_backward(const hstu_bwd_params* p, void* workspace, uint64_t workspace_bytes, void* stream);

/* replaces aclGetRecentErrMsg() (pytorch_npu_helper.hpp:510-543): message of the last failing call on this thread */
const char* hstu_hip_last_error(void);

/* Name of the kernel variant the given arguments select ("mfma_bf16_d128", "generic_f32", ...);
 * written NUL-terminated into buf.  Diagnostic: lets a caller assert that the MFMA path is the one in use.  The
 * matrix-core kernels take bf16 / fp16 with dim_qk == dim_v in {32, 64, 128, 256} (paged too, with at most 640 pages per
 * user, 320 at head dim 128 when the page size is no multiple of 4) and buffers on 16-byte boundaries; other multiples of
 * 16 up to 256 and dim_qk != dim_v under the built-in mask or none without a bias ("mfma_bf16_d128_padded"); FP8_E4M3
 * with the built-in mask or none and no bias ("mfma_fp8_d128"); everything else (fp32, unaligned buffers, other head dims
 * with a bias or pages, fp8 with a bias or a custom mask) runs the plain fp32-FMA kernel, which is an order of magnitude
 * slower. */
int hstu_hip_describe_kernel(const hstu_fwd_params* p, char* buf, size_t buf_bytes);

/* The same for the backward: "mfma_bwd_bf16_d128", "mfma_bwd_f16_d64_bias", "generic_bwd_f32", ...  The matrix-core
 * kernels take bf16 / fp16, head dim 32, 64, 128 or 256 (dim_qk == dim_v), the built-in mask or none, an optional dense attn_bias
 * whose rows hold a multiple of 8 elements, and buffers on 16-byte boundaries; everything else (fp32, other head dims, a
 * custom mask) runs the plain fp32-FMA kernels, which are an order of magnitude slower. */
int hstu_hip_describe_backward_kernel(const hstu_bwd_params* p, char* buf, size_t buf_bytes);

int hstu_hip_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* HSTU_HIP_H */
