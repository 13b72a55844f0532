// C-ABI entry points: argument validation (the role of the reference's op_host tiling checks,
// tiling_policy.cpp:69-94, tiling_policy_jagged.cpp:63-205, tiling_policy_paged.cpp:120-222),
// kernel selection and launch.  No device synchronisation, no host reads of device memory.
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>

#include "hstu_internal.h"

namespace hstu {

static thread_local std::string g_last_error;

int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

static bool in_range(int64_t v, int64_t lo, int64_t hi) { return v >= lo && v <= hi; }

// Work list of hstu_hip_jagged_forward_noalloc: a fixed array in every GPU's memory instead of a caller workspace.
// Host code never uses the array's name as an address: scratch_of_current_device() asks the runtime for the
// device address once per GPU and every launch gets that pointer.
static __device__ __align__(256) unsigned char scratch[HSTU_NOALLOC_SCRATCH_BYTES];
constexpr int MAX_DEVICES = 64;
static void* g_scratch_ptr[MAX_DEVICES];
static std::mutex g_scratch_mutex;

static int scratch_of_current_device(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "hipGetDevice failed: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= MAX_DEVICES) return fail(HSTU_ERR_UNSUPPORTED, "device index %d outside [0, %d)", dev, MAX_DEVICES);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            return fail(HSTU_ERR_LAUNCH, "hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return HSTU_OK;
}

static int validate(const hstu_fwd_params* p, int op, KArgs* out, bool need_out = true) {
    if (!p) return fail(HSTU_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(hstu_fwd_params))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "hstu_fwd_params size mismatch: caller %u, library %zu (ABI version %d)",
                    p->struct_size, sizeof(hstu_fwd_params), HSTU_HIP_ABI_VERSION);
    if (p->dtype != HSTU_F32 && p->dtype != HSTU_F16 && p->dtype != HSTU_BF16 && p->dtype != HSTU_FP8_E4M3)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "dtype expect float32, float16, bfloat16 or float8_e4m3fn, but value is %d", p->dtype);
    if (p->dtype == HSTU_FP8_E4M3 && op == OP_PAGED)
        return fail(HSTU_ERR_UNSUPPORTED, "float8_e4m3fn q/k/v are taken by the jagged and dense forward only (the paged op takes an fp8 cache)");
    if (p->index_type != HSTU_I32 && p->index_type != HSTU_I64)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "index_type expect int32 or int64, but value is %d", p->index_type);
    if (!p->q || !p->k || !p->v || (need_out && !p->out)) return fail(HSTU_ERR_INVALID_ARGUMENT, "q, k, v and out must not be NULL");
    if (p->batch == 0 || p->batch > HSTU_MAX_BATCH || p->batch < 0)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "batchSize limit (0, %d], but get %d", HSTU_MAX_BATCH, p->batch);
    if (!in_range(p->max_seq_len_q, 1, HSTU_MAX_SEQ_LEN))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "maxSeqLen expect in [1, %d], but value is %d", HSTU_MAX_SEQ_LEN, p->max_seq_len_q);
    if (!in_range(p->max_seq_len_k, 1, HSTU_MAX_SEQ_LEN))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "maxSeqLenK expect in [1, %d], but value is %d", HSTU_MAX_SEQ_LEN, p->max_seq_len_k);
    if (!in_range(p->heads_q, 1, HSTU_MAX_HEADS) || !in_range(p->heads_k, 1, HSTU_MAX_HEADS))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "head num expect in [1, %d], but get q %d, k %d", HSTU_MAX_HEADS, p->heads_q, p->heads_k);
    if (p->heads_q % p->heads_k != 0)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "For GQA, headNumQ must be divisible by headNumK (%d, %d)", p->heads_q, p->heads_k);
    if (!in_range(p->dim_qk, 1, HSTU_MAX_HEAD_DIM))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "Q/K dim size expect in [1, %d], but get %d", HSTU_MAX_HEAD_DIM, p->dim_qk);
    if (!in_range(p->dim_v, 16, HSTU_MAX_HEAD_DIM) || p->dim_v % 16 != 0)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "V dim size expect a multiple of 16 in [16, %d], but get %d", HSTU_MAX_HEAD_DIM, p->dim_v);
    if (p->mask_type < HSTU_MASK_TRIL || p->mask_type > HSTU_MASK_CUSTOM)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "maskType expect in [0, 3], but value is %d", p->mask_type);
    if (p->mask_type == HSTU_MASK_TRIU)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "maskType current not support triu now, pls use custom mask");
    if (p->mask_type == HSTU_MASK_CUSTOM && !p->mask)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "use custom mask must have valid mask tensor");
    if (p->target_group_size < 0) return fail(HSTU_ERR_INVALID_ARGUMENT, "targetGroupSize must not be negative");
    if (p->total_q < 0 || p->total_k < 0) return fail(HSTU_ERR_INVALID_ARGUMENT, "negative row count");
    if (!std::isfinite(p->silu_scale) || !std::isfinite(p->alpha))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "silu_scale and alpha must be finite");

    if (op == OP_DENSE) {
        if (p->seq_offset_q || p->seq_offset_k)
            return fail(HSTU_ERR_INVALID_ARGUMENT, "dense layout takes no sequence offsets");
        if (p->heads_q != p->heads_k || p->dim_qk != p->dim_v || p->max_seq_len_q != p->max_seq_len_k)
            return fail(HSTU_ERR_INVALID_ARGUMENT, "dense layout needs q, k and v of one shape");
        if (p->dim_qk % 16 != 0) return fail(HSTU_ERR_INVALID_ARGUMENT, "dense layout needs dim %% 16 == 0, but get %d", p->dim_qk);
        if (p->total_q != (int64_t)p->batch * p->max_seq_len_q || p->total_k != p->total_q)
            return fail(HSTU_ERR_INVALID_ARGUMENT, "dense layout: total rows must equal batch * seq_len");
        if (p->num_context || p->num_target) return fail(HSTU_ERR_INVALID_ARGUMENT, "dense layout takes no num_context/num_target");
    } else {
        if (!p->seq_offset_q || !p->seq_offset_k)
            return fail(HSTU_ERR_INVALID_ARGUMENT, "seq_offset_q and seq_offset_k must not be NULL in jagged layout");
    }
    if (op == OP_PAGED) {
        if (!p->kv_cache || !p->page_offsets || !p->page_ids || !p->last_page_len)
            return fail(HSTU_ERR_INVALID_ARGUMENT, "pagedIds, pagedOffset, lastPageLen and kvCache should not be nullptr.");
        if (p->page_size < 1) return fail(HSTU_ERR_INVALID_ARGUMENT, "PageSize must be positive, but get %d", p->page_size);
        if (p->dim_qk != p->dim_v) return fail(HSTU_ERR_INVALID_ARGUMENT, "K, V shape mismatch");
        if (p->total_q != p->total_k) return fail(HSTU_ERR_INVALID_ARGUMENT, "Q, K, V seqlen mismatch");
        if (p->cache_dtype == HSTU_FP8_E4M3) {
            if (!p->kv_scales) return fail(HSTU_ERR_INVALID_ARGUMENT, "fp8 kv_cache needs kv_scales");
        } else if (p->cache_dtype != p->dtype) {
            return fail(HSTU_ERR_INVALID_ARGUMENT, "kv_cache dtype must equal the q dtype or be fp8-e4m3");
        }
    } else if (p->kv_cache) {
        return fail(HSTU_ERR_INVALID_ARGUMENT, "kv_cache is only taken by the paged op");
    }
    if (p->ts_table) {
        if (!p->timestamps || !p->ts_bounds || p->num_buckets < 1)
            return fail(HSTU_ERR_INVALID_ARGUMENT, "ts_table needs timestamps, ts_bounds and num_buckets >= 1");
        if (!std::isfinite(p->ts_log2_scale) || p->ts_log2_scale < 0)
            return fail(HSTU_ERR_INVALID_ARGUMENT, "ts_log2_scale must be finite and non-negative");
    }

    out->p = *p;
    out->p.flags &= HSTU_FLAG_DETERMINISTIC | HSTU_FLAG_FORCE_GENERIC | HSTU_FLAG_REUSE_WORKSPACE | HSTU_FLAG_SERIAL_BACKWARD;   // the rest is the library's own
    out->op = op;
    out->head_ratio = p->heads_q / p->heads_k;
    out->out_scale = p->alpha * p->silu_scale;
    out->exp_scale = -p->alpha * 1.4426950408889634f;
    return HSTU_OK;
}

static int run(const hstu_fwd_params* p, int op, void* workspace, uint64_t workspace_bytes, void* stream) {
    KArgs a;
    int rc = validate(p, op, &a);
    if (rc != HSTU_OK) return rc;
    if (p->total_q == 0) return HSTU_OK;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const char* name = nullptr;
    hipError_t e;
    if (!(p->flags & HSTU_FLAG_FORCE_GENERIC) && mfma_supported(a, &name)) {
        const uint64_t need = mfma_workspace_bytes(a);
        if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15))
            return fail(HSTU_ERR_WORKSPACE, "workspace of %llu bytes (16-byte aligned) needed, got %llu at %p",
                        (unsigned long long)need, (unsigned long long)workspace_bytes, workspace);
        e = launch_mfma(a, workspace, st);
    } else {
        e = launch_generic(a, st);
    }
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    return HSTU_OK;
}

static int ws_size(const hstu_fwd_params* p, int op, uint64_t* bytes) {
    if (!bytes) return fail(HSTU_ERR_INVALID_ARGUMENT, "workspace_bytes is NULL");
    KArgs a;
    int rc = validate(p, op, &a);
    if (rc != HSTU_OK) return rc;
    // every output row has exactly one producing workgroup: no partials, no flags; the MFMA kernels keep
    // their work list here
    const char* name = nullptr;
    *bytes = (!(p->flags & HSTU_FLAG_FORCE_GENERIC) && mfma_supported(a, &name)) ? mfma_workspace_bytes(a) : 0;
    return HSTU_OK;
}

// the jagged backward: the forward's checks plus what the reference's backward does not take
static int validate_backward(const hstu_bwd_params* p, int op, BArgs* out) {
    if (!p) return fail(HSTU_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(hstu_bwd_params))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "hstu_bwd_params size mismatch: caller %u, library %zu (ABI version %d)",
                    p->struct_size, sizeof(hstu_bwd_params), HSTU_HIP_ABI_VERSION);
    int rc = validate(&p->fwd, op, &out->f, false);
    if (rc != HSTU_OK) return rc;
    if (p->fwd.dtype == HSTU_FP8_E4M3) return fail(HSTU_ERR_UNSUPPORTED, "the backward takes float32, float16 or bfloat16 (float8_e4m3fn is forward only)");
    if (p->fwd.pos_table || p->fwd.ts_table)
        return fail(HSTU_ERR_UNSUPPORTED, "the backward takes a dense attn_bias only (no bias tables)");
    if (!p->grad_out || !p->grad_q || !p->grad_k || !p->grad_v)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "grad_out, grad_q, grad_k and grad_v must not be NULL");
    if ((p->fwd.attn_bias != nullptr) != (p->grad_bias != nullptr))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "grad_bias must be given exactly when attn_bias is");
    out->grad_out = p->grad_out;
    out->grad_q = p->grad_q;
    out->grad_k = p->grad_k;
    out->grad_v = p->grad_v;
    out->grad_bias = p->grad_bias;
    return HSTU_OK;
}

}  // namespace hstu

using namespace hstu;

extern "C" {

int hstu_hip_jagged_forward_get_workspace_size(const hstu_fwd_params* p, uint64_t* b) { return ws_size(p, OP_JAGGED, b); }
int hstu_hip_jagged_forward(const hstu_fwd_params* p, void* ws, uint64_t n, void* s) { return run(p, OP_JAGGED, ws, n, s); }

int hstu_hip_jagged_forward_noalloc(const hstu_fwd_params* p, void* stream) {
    KArgs a;
    int rc = validate(p, OP_JAGGED, &a);
    if (rc != HSTU_OK) return rc;
    if (p->total_q == 0) return HSTU_OK;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const char* name = nullptr;
    hipError_t e;
    if (!(a.p.flags & HSTU_FLAG_FORCE_GENERIC) && mfma_supported(a, &name)) {
        // whole Q tiles only (no partial sums of split K ranges, which would need a buffer that grows with the batch); the
        // list is rebuilt by every call because the array is shared by all callers of this GPU
        a.p.flags = (a.p.flags & ~HSTU_FLAG_REUSE_WORKSPACE) | FLAG_WHOLE_TILES;
        const uint64_t need = mfma_workspace_bytes(a);
        if (need > HSTU_NOALLOC_SCRATCH_BYTES)
            return fail(HSTU_ERR_WORKSPACE, "the work list of this batch needs %llu bytes, hstu_hip_jagged_forward_noalloc holds %u: "
                        "use hstu_hip_jagged_forward with a caller workspace", (unsigned long long)need, (unsigned)HSTU_NOALLOC_SCRATCH_BYTES);
        void* ptr = nullptr;
        rc = scratch_of_current_device(&ptr);
        if (rc != HSTU_OK) return rc;
        e = launch_mfma(a, ptr, st);
    } else {
        e = launch_generic(a, st);   // uses no device memory beyond its arguments
    }
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    return HSTU_OK;
}

int hstu_hip_paged_forward_get_workspace_size(const hstu_fwd_params* p, uint64_t* b) { return ws_size(p, OP_PAGED, b); }
int hstu_hip_paged_forward(const hstu_fwd_params* p, void* ws, uint64_t n, void* s) { return run(p, OP_PAGED, ws, n, s); }
int hstu_hip_dense_forward_get_workspace_size(const hstu_fwd_params* p, uint64_t* b) { return ws_size(p, OP_DENSE, b); }
int hstu_hip_dense_forward(const hstu_fwd_params* p, void* ws, uint64_t n, void* s) { return run(p, OP_DENSE, ws, n, s); }

static int backward_ws_size(const hstu_bwd_params* p, int op, uint64_t* bytes) {
    if (!bytes) return fail(HSTU_ERR_INVALID_ARGUMENT, "workspace_bytes is NULL");
    BArgs a;
    int rc = validate_backward(p, op, &a);
    if (rc != HSTU_OK) return rc;
    // every gradient element has one producing workgroup: no partial sums; the MFMA kernels keep their work lists here
    const bool mfma = !(p->fwd.flags & HSTU_FLAG_FORCE_GENERIC) && mfma_backward_supported(a);
    *bytes = mfma ? mfma_backward_workspace_bytes(a) : 0;
    return HSTU_OK;
}

static int backward_run(const hstu_bwd_params* p, int op, void* workspace, uint64_t workspace_bytes, void* stream) {
    BArgs a;
    int rc = validate_backward(p, op, &a);
    if (rc != HSTU_OK) return rc;
    if (p->fwd.total_q == 0 && p->fwd.total_k == 0) return HSTU_OK;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const bool mfma = !(p->fwd.flags & HSTU_FLAG_FORCE_GENERIC) && mfma_backward_supported(a);
    if (mfma) {
        const uint64_t need = mfma_backward_workspace_bytes(a);
        if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15))
            return fail(HSTU_ERR_WORKSPACE, "workspace of %llu bytes (16-byte aligned) needed, got %llu at %p",
                        (unsigned long long)need, (unsigned long long)workspace_bytes, workspace);
    }
    hipError_t e = mfma ? launch_backward_mfma(a, workspace, st) : launch_backward_generic(a, st);
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    return HSTU_OK;
}

int hstu_hip_jagged_backward_get_workspace_size(const hstu_bwd_params* p, uint64_t* b) { return backward_ws_size(p, OP_JAGGED, b); }
int hstu_hip_jagged_backward(const hstu_bwd_params* p, void* ws, uint64_t n, void* s) { return backward_run(p, OP_JAGGED, ws, n, s); }
int hstu_hip_dense_backward_get_workspace_size(const hstu_bwd_params* p, uint64_t* b) { return backward_ws_size(p, OP_DENSE, b); }
int hstu_hip_dense_backward(const hstu_bwd_params* p, void* ws, uint64_t n, void* s) { return backward_run(p, OP_DENSE, ws, n, s); }

const char* hstu_hip_last_error(void) { return g_last_error.c_str(); }

int hstu_hip_describe_kernel(const hstu_fwd_params* p, char* buf, size_t n) {
    if (!buf || n == 0) return fail(HSTU_ERR_INVALID_ARGUMENT, "buf is NULL");
    KArgs a;
    int op = (p && p->kv_cache) ? OP_PAGED : ((p && !p->seq_offset_q) ? OP_DENSE : OP_JAGGED);
    int rc = validate(p, op, &a);
    if (rc != HSTU_OK) return rc;
    const char* name = nullptr;
    const bool mfma = !(p->flags & HSTU_FLAG_FORCE_GENERIC) && mfma_supported(a, &name);
    if (!mfma) name = p->dtype == HSTU_F32 ? "generic_f32" : (p->dtype == HSTU_F16 ? "generic_f16" : (p->dtype == HSTU_BF16 ? "generic_bf16" : "generic_fp8"));
    snprintf(buf, n, "%s%s", name, mfma && mfma_self_scheduled(a) ? "_selfsched" : "");
    return HSTU_OK;
}

int hstu_hip_describe_backward_kernel(const hstu_bwd_params* p, char* buf, size_t n) {
    if (!buf || n == 0) return fail(HSTU_ERR_INVALID_ARGUMENT, "buf is NULL");
    BArgs a;
    int rc = validate_backward(p, (p && !p->fwd.seq_offset_q) ? OP_DENSE : OP_JAGGED, &a);
    if (rc != HSTU_OK) return rc;
    const bool mfma = !(p->fwd.flags & HSTU_FLAG_FORCE_GENERIC) && mfma_backward_supported(a);
    const char* dt = p->fwd.dtype == HSTU_F32 ? "f32" : (p->fwd.dtype == HSTU_F16 ? "f16" : "bf16");
    if (mfma) snprintf(buf, n, "mfma_bwd_%s_d%d%s", dt, p->fwd.dim_qk, p->fwd.attn_bias ? "_bias" : (p->fwd.mask_type == HSTU_MASK_CUSTOM ? "_mask" : ""));
    else snprintf(buf, n, "generic_bwd_%s", dt);
    return HSTU_OK;
}

int hstu_hip_abi_version(void) { return HSTU_HIP_ABI_VERSION; }

}  // extern "C"
