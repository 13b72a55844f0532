// Write side of the paged K/V cache: append the new tokens of a batch to their pages, and the per-token
// (user, position) pairs the append consumes.  Byte work bounded by HBM: every K and V row is read once and written
// once, 16 bytes per lane, a row's heads*dim elements by consecutive lanes (with the reference's NHD layout the
// destination row is one contiguous run).
// Semantics: inference/kvcache_manager/src/kernels/append_paged_kvcache/append_paged_kvcache_kernel.h:42-76 and
// .../get_paged_batch_indices_positions/get_paged_batch_indices_positions_kernel.h.
#include "hstu_internal.h"
#include "../../include/hstu_kvcache.h"

namespace hstu {

typedef __attribute__((ext_vector_type(4))) unsigned int kv_u32x4;

// one lane moves the K and the V chunk (8 elements) of one (token, head); indices that point outside the buffers the
// host described skip the token instead of faulting.  IDX: type of the flat chunk index (32 bits whenever
// nnz_max * chunks per token fits).  KV_UNROLL chunks per lane and pass, all loads before the first store: 1 runs at
// the rate of a plain device copy (5.3 of 5.4 TB/s measured); 4 spreads a workgroup's accesses too far apart (3.9 TB/s).
// The rows are touched once: loads and stores carry the nontemporal hint (5.7 TB/s on the kernel).
constexpr int KV_UNROLL = 1;

template <typename IDX>
__global__ __launch_bounds__(256) void hstu_kv_append_kernel(const hstu_kv_append_params p) {
    const unsigned cph = (unsigned)p.head_dim / 8;       // 16-byte chunks per head
    const unsigned cpt = cph * (unsigned)p.num_heads;    // per token
    const int nnz = min(max(*p.nnz_dev, 0), p.nnz_max);
    const IDX total = (IDX)nnz * cpt;
    const IDX stride = (IDX)gridDim.x * blockDim.x;
    const unsigned short* ak = reinterpret_cast<const unsigned short*>(p.append_key);
    const unsigned short* av = reinterpret_cast<const unsigned short*>(p.append_value);
    unsigned short* kc = reinterpret_cast<unsigned short*>(p.k_cache);
    unsigned short* vc = reinterpret_cast<unsigned short*>(p.v_cache);
    for (IDX g0 = (IDX)blockIdx.x * blockDim.x + threadIdx.x; g0 < total; g0 += stride * KV_UNROLL) {
        kv_u32x4 kx[KV_UNROLL], vx[KV_UNROLL];
        int64_t dst[KV_UNROLL];
        bool ok[KV_UNROLL];
#pragma unroll
        for (int u = 0; u < KV_UNROLL; u++) {
            const IDX g = g0 + (IDX)u * stride;
            ok[u] = false;
            if (g >= total) continue;
            const unsigned i = (unsigned)(g / cpt), rem = (unsigned)(g % cpt);
            const unsigned head = rem / cph, c = rem % cph;
            const int b = p.batch_indices[i];
            const int pos = p.positions[i];
            if (b < 0 || b >= p.batch || pos < 0) continue;
            const unsigned page_iter = (unsigned)pos / (unsigned)p.page_size, entry = (unsigned)pos % (unsigned)p.page_size;
            const int first = p.kv_indptr[b], last = p.kv_indptr[b + 1];
            if (first < 0 || last > p.num_indices || (int64_t)page_iter >= (int64_t)last - first) continue;
            const int page = p.kv_indices[first + (int)page_iter];
            const int64_t row = (int64_t)i + p.offsets[b];
            if (page < 0 || page >= p.num_pages || row < 0 || row >= p.append_rows) continue;
            ok[u] = true;
            dst[u] = (int64_t)page * p.stride_page + (int64_t)head * p.stride_h + (int64_t)entry * p.stride_n + 8 * c;
            kx[u] = __builtin_nontemporal_load(reinterpret_cast<const kv_u32x4*>(ak + row * p.append_k_stride_n + head * p.append_k_stride_h + 8 * c));
            vx[u] = __builtin_nontemporal_load(reinterpret_cast<const kv_u32x4*>(av + row * p.append_v_stride_n + head * p.append_v_stride_h + 8 * c));
        }
#pragma unroll
        for (int u = 0; u < KV_UNROLL; u++) {
            if (!ok[u]) continue;
            __builtin_nontemporal_store(kx[u], reinterpret_cast<kv_u32x4*>(kc + dst[u]));
            __builtin_nontemporal_store(vx[u], reinterpret_cast<kv_u32x4*>(vc + dst[u]));
        }
    }
}

// blockIdx.x = user, blockIdx.y strides over its new tokens
__global__ __launch_bounds__(256) void hstu_kv_token_positions_kernel(int batch, const int* append_indptr, const int* seq_lens,
                                                                      int* batch_indices, int* positions, int nnz_max) {
    const int b = blockIdx.x;
    if (b >= batch) return;
    const int first = append_indptr[b], count = append_indptr[b + 1] - first;
    const int pos0 = seq_lens[b] - count;
    for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < count; i += gridDim.y * blockDim.x) {
        const int t = first + i;
        if (t < 0 || t >= nnz_max) continue;
        batch_indices[t] = b;
        positions[t] = pos0 + i;
    }
}

}  // namespace hstu

using namespace hstu;

extern "C" int hstu_hip_kv_append(const hstu_kv_append_params* p, void* stream) {
    if (!p) return fail(HSTU_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(hstu_kv_append_params))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "hstu_kv_append_params size mismatch: caller %u, library %zu", p->struct_size,
                    sizeof(hstu_kv_append_params));
    if (p->elem_bytes != 2) return fail(HSTU_ERR_INVALID_ARGUMENT, "k/v must have a 2-byte dtype (float16 or bfloat16), but elem_bytes is %d", p->elem_bytes);
    if (!p->k_cache || !p->v_cache || !p->append_key || !p->append_value || !p->kv_indices || !p->kv_indptr || !p->batch_indices ||
        !p->positions || !p->offsets || !p->nnz_dev)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "k_cache, v_cache, append_key, append_value, kv_indices, kv_indptr, batch_indices, positions, offsets and nnz_dev must not be NULL");
    if (p->head_dim != 64 && p->head_dim != 128 && p->head_dim != 256 && p->head_dim != 512)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "head_dim expect 64, 128, 256 or 512, but value is %d", p->head_dim);
    if (p->num_heads < 1 || p->page_size < 1 || p->num_pages < 1 || p->batch < 1 || p->num_indices < 0 || p->nnz_max < 0 || p->append_rows < 0)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "num_heads, page_size, num_pages, batch must be positive and num_indices, nnz_max, append_rows non-negative");
    // 16-byte lanes: every row and head starts on a 16-byte boundary
    const int64_t strides[] = {p->stride_page, p->stride_n, p->stride_h, p->append_k_stride_n, p->append_k_stride_h,
                               p->append_v_stride_n, p->append_v_stride_h};
    for (int64_t s : strides)
        if (s < 0 || s % 8) return fail(HSTU_ERR_UNSUPPORTED, "strides must be non-negative multiples of 8 elements, but one is %lld", (long long)s);
    const void* bases[] = {p->k_cache, p->v_cache, p->append_key, p->append_value};
    for (const void* q : bases)
        if (reinterpret_cast<uintptr_t>(q) & 15) return fail(HSTU_ERR_UNSUPPORTED, "k_cache, v_cache, append_key and append_value must be 16-byte aligned");
    if (p->nnz_max == 0) return HSTU_OK;
    const int64_t lanes = (int64_t)p->nnz_max * p->num_heads * (p->head_dim / 8);
    const int64_t want = (lanes + 256 * KV_UNROLL - 1) / (256 * KV_UNROLL);
    const unsigned grid = (unsigned)(want < 1 ? 1 : (want > 65536 ? 65536 : want));
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (lanes + (int64_t)grid * 256 * KV_UNROLL < (int64_t)1 << 32)
        hipLaunchKernelGGL(hstu_kv_append_kernel<unsigned>, dim3(grid), dim3(256), 0, st, *p);
    else
        hipLaunchKernelGGL(hstu_kv_append_kernel<unsigned long long>, dim3(grid), dim3(256), 0, st, *p);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    return HSTU_OK;
}

extern "C" int hstu_hip_kv_token_positions(int32_t batch, const int32_t* append_indptr, const int32_t* seq_lens, int32_t* batch_indices,
                                           int32_t* positions, int32_t nnz_max, void* stream) {
    if (batch < 1) return fail(HSTU_ERR_INVALID_ARGUMENT, "batch must be positive, but value is %d", batch);
    if (nnz_max < 0) return fail(HSTU_ERR_INVALID_ARGUMENT, "nnz_max must be non-negative, but value is %d", nnz_max);
    if (!append_indptr || !seq_lens || !batch_indices || !positions)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "append_indptr, seq_lens, batch_indices and positions must not be NULL");
    // workgroups per user: enough for the average user's tokens at 256 per workgroup, at most 64
    const int64_t avg = ((int64_t)nnz_max / batch + 255) / 256;
    const unsigned per_user = (unsigned)(avg < 1 ? 1 : (avg > 64 ? 64 : avg));
    hipLaunchKernelGGL(hstu_kv_token_positions_kernel, dim3((unsigned)batch, per_user), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), batch,
                       append_indptr, seq_lens, batch_indices, positions, nnz_max);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    return HSTU_OK;
}
