/*
 * hstu_kvcache.h -- C ABI of the write side of the paged K/V cache that hstu_hip_paged_forward reads.
 *
 * The cache is the reference's per-layer table [pages, 2, page_size, heads, dim] (K plane, then V plane, of every
 * page; inference/kvcache_manager/test/test_npu_kvcache_manager.py:322-327), handed over as its two unbind(1) views.
 * Appending the new tokens of a batch is byte work: each token's K and V row is copied to
 * page kv_indices[kv_indptr[user] + position / page_size], slot position % page_size.
 *
 * Same conventions as hstu_hip.h: device pointers, asynchronous on `stream`, nothing read on the host, 0 or a negative
 * hstu_status with the message in hstu_hip_last_error().
 */
#ifndef HSTU_KVCACHE_H
#define HSTU_KVCACHE_H

#include "hstu_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Argument block of hstu_hip_kv_append: the argument list of the reference's launcher
 * kvcache::AppendPagedKVCache (inference/kvcache_manager/src/gather_scatter.cpp:144-160) with the sizes the kernel
 * checks its indices against.  Strides are in elements. */
typedef struct hstu_kv_append_params {
    uint32_t struct_size;     /* sizeof(hstu_kv_append_params) */
    int32_t elem_bytes;       /* 2: fp16 / bf16 payload, as the reference (pybind.cpp:46-55) */
    void* k_cache;            /* paged_k_cache: element (page, slot, head, d) at page*stride_page + slot*stride_n + head*stride_h + d */
    void* v_cache;            /* paged_v_cache, same strides */
    int64_t stride_page;
    int64_t stride_n;
    int64_t stride_h;
    int32_t num_pages;        /* pages of the table: tokens whose page id is outside [0, num_pages) are skipped */
    int32_t page_size;
    int32_t num_heads;
    int32_t head_dim;         /* 64, 128, 256 or 512 (dispatch_head_dim.h:22-48) */
    const int32_t* kv_indices;   /* [num_indices] page ids, users back to back */
    const int32_t* kv_indptr;    /* [batch + 1] first entry of every user in kv_indices */
    int32_t num_indices;
    int32_t batch;
    const void* append_key;   /* [append_rows, heads, dim] with the strides below */
    const void* append_value;
    int64_t append_k_stride_n, append_k_stride_h;
    int64_t append_v_stride_n, append_v_stride_h;
    int64_t append_rows;      /* rows of append_key / append_value: a token whose source row is outside is skipped */
    const int32_t* batch_indices; /* [nnz] user of new token i */
    const int32_t* positions;     /* [nnz] position of new token i in its user's sequence */
    const int32_t* offsets;       /* [batch] source row of token i is i + offsets[user] */
    const int32_t* nnz_dev;       /* device scalar: number of new tokens */
    int32_t nnz_max;          /* host-side bound of *nnz_dev (length of batch_indices / positions) */
    int32_t reserved;
} hstu_kv_append_params;

/* Replaces kvcache::AppendPagedKVCache (gather_scatter.cpp:144-160; kernel append_paged_kvcache_kernel.h:42-76). */
int hstu_hip_kv_append(const hstu_kv_append_params* p, void* stream);

/* Replaces kvcache::GetPagedBatchIndicesPositions (gather_scatter.cpp:137-142; kernel
 * get_paged_batch_indices_positions_kernel.h): for user b with new tokens [append_indptr[b], append_indptr[b+1]) and
 * seq_lens[b] tokens after the append, batch_indices[t] = b and positions[t] = seq_lens[b] - count + (t - first).
 * nnz_max bounds the writes. */
int hstu_hip_kv_token_positions(int32_t batch, const int32_t* append_indptr, const int32_t* seq_lens,
                                int32_t* batch_indices, int32_t* positions, int32_t nnz_max, void* stream);

/* Append to an fp8-e4m3 table with one fp32 scale per (page, K|V, head): the write side of what
 * hstu_hip_paged_forward reads with cache_dtype = HSTU_FP8_E4M3 and kv_scales.  No counterpart in the reference (its
 * cache manager stores 2-byte rows unscaled); for the callers that keep the history in fp8.  Tokens are routed like
 * hstu_hip_kv_append.  After the call a touched (page, K|V, head) holds q = rne_e4m3(clamp(x / s, -448, 448)) with
 *   s = max(s before, absmax(new rows) / 448)   if the page already held rows below its first new slot,
 *   s = absmax(new rows) / 448 (1 if that is 0)  otherwise;
 * rows already there are requantised from q * (s before) when s grew, and untouched when it did not.  Pages fill from
 * slot 0 upwards (what the reference's manager does).  The workspace (16-byte aligned) needs no initialisation; the
 * work of a call grows with the new tokens, not with the size of the table.  Tokens may come in any order; in the order
 * of hstu_hip_kv_token_positions (consecutive positions of a user side by side) every source row is read once. */
typedef struct hstu_kv_append_fp8_params {
    uint32_t struct_size;
    int32_t src_dtype;        /* HSTU_F16 / HSTU_BF16: append_key, append_value */
    uint8_t* kv_cache;        /* [num_pages, 2, page_size, num_heads, head_dim] e4m3 bytes, contiguous */
    float* kv_scales;         /* [num_pages, 2, num_heads] */
    int32_t num_pages;
    int32_t page_size;
    int32_t num_heads;
    int32_t head_dim;         /* a power of two in [8, 512] */
    const int32_t* kv_indices;
    const int32_t* kv_indptr;
    int32_t num_indices;
    int32_t batch;
    const void* append_key;   /* [append_rows, heads, dim] with the strides below (elements) */
    const void* append_value;
    int64_t append_k_stride_n, append_k_stride_h;
    int64_t append_v_stride_n, append_v_stride_h;
    int64_t append_rows;
    const int32_t* batch_indices;
    const int32_t* positions;
    const int32_t* offsets;
    const int32_t* nnz_dev;
    int32_t nnz_max;
    int32_t reserved;
} hstu_kv_append_fp8_params;
int hstu_hip_kv_append_fp8_get_workspace_size(const hstu_kv_append_fp8_params* p, uint64_t* workspace_bytes);
int hstu_hip_kv_append_fp8(const hstu_kv_append_fp8_params* p, void* workspace, uint64_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HSTU_KVCACHE_H */
