// Append to an fp8-e4m3 paged K/V cache with one fp32 scale per (page, K|V, head): the write side of the table that
// hstu_hip_paged_forward reads with cache_dtype = HSTU_FP8_E4M3.  No counterpart in the reference (its cache manager
// stores 2-byte rows unscaled, append_paged_kvcache_kernel.h:42-76); the routing of a token to its page and slot is the
// reference's, the quantisation is this library's:
//   after an append, a touched (page, K|V, head) holds  q = rne_e4m3(clamp(x / s, -448, 448))  with
//   s = max(s_before, absmax(new rows) / 448)  if the page already held rows below the first new slot,
//   s = absmax(new rows) / 448 (1 if that is 0) otherwise;  rows already there are requantised from q * s_before
//   when s grew and are left untouched bit for bit when it did not.
// A page filled by one append therefore equals quantising the whole page at once.
// Four small kernels on the stream, nothing read on the host, all of them sized by the new tokens and not by the cache
// (a table of a million pages costs an append of one token no more than a table of ten):
//   reset  clears the per-unit maxima and the first slot of the pages the new tokens go to, and the list of touched pages
//   scan   absmax of every new (token, K|V, head) row -> atomic max per unit, atomic min of the slot per page; the token
//          that finds a page untouched enters it in the list
//   scale  per unit of a listed page: new scale, requantise the rows below the first new slot if the scale grew
//   write  quantise the new rows with the unit's scale
// Byte work bounded by HBM: the new rows are read twice (2 bytes per element) and written once (1 byte).
#include "hstu_device.h"
#include "../../include/hstu_kvcache.h"

namespace hstu {

typedef __attribute__((ext_vector_type(4))) unsigned int kf_u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int kf_u32x2;
constexpr float KF_MAX = 448.0f;
constexpr int KF_NOSLOT = 0x7fffffff;

__device__ __forceinline__ float kf_elem(unsigned word, int hi, int bf16) {
    const unsigned short h = (unsigned short)(hi ? word >> 16 : word & 0xffffu);
    return bf16 ? __builtin_bit_cast(float, (unsigned)h << 16) : (float)__builtin_bit_cast(_Float16, h);
}

// two values -> two e4m3 bytes in the low half of the result
__device__ __forceinline__ unsigned kf_quant2(float a, float b, float s) {
    a = fminf(fmaxf(a / s, -KF_MAX), KF_MAX);
    b = fminf(fmaxf(b / s, -KF_MAX), KF_MAX);
    return (unsigned)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xffffu;
}

// where a new token goes: page and slot, or false if any index points outside what the host described
__device__ __forceinline__ bool kf_route(const hstu_kv_append_fp8_params& p, unsigned i, int& page, int& slot, int64_t& row) {
    const int b = p.batch_indices[i];
    const int pos = p.positions[i];
    if (b < 0 || b >= p.batch || pos < 0) return false;
    const unsigned page_iter = (unsigned)pos / (unsigned)p.page_size;
    slot = (int)((unsigned)pos % (unsigned)p.page_size);
    const int first = p.kv_indptr[b], last = p.kv_indptr[b + 1];
    if (first < 0 || last > p.num_indices || (int64_t)page_iter >= (int64_t)last - first) return false;
    page = p.kv_indices[first + (int)page_iter];
    row = (int64_t)i + p.offsets[b];
    return page >= 0 && page < p.num_pages && row >= 0 && row < p.append_rows;
}

// one thread per new token: the workspace entries of its page start from scratch (several tokens of a page write the same values)
__global__ __launch_bounds__(256) void hstu_kv_fp8_reset_kernel(const hstu_kv_append_fp8_params p, unsigned* unit_max, int* first_slot, int* touched) {
    const int nnz = min(max(*p.nnz_dev, 0), p.nnz_max);
    if (blockIdx.x == 0 && threadIdx.x == 0) touched[0] = 0;
    for (unsigned i = blockIdx.x * 256 + threadIdx.x; i < (unsigned)nnz; i += gridDim.x * 256) {
        int page, slot;
        int64_t row;
        if (!kf_route(p, i, page, slot, row)) continue;
        for (int u = 0; u < 2 * p.num_heads; u++) unit_max[(int64_t)page * 2 * p.num_heads + u] = 0u;
        first_slot[page] = KF_NOSLOT;
    }
}

// one lane = the same 8 elements of the K row and of the V row of one (token, head); the dim / 8 lanes of a row sit
// side by side in a wave.  IDX: type of the flat lane index, 32 bits whenever nnz_max * lanes per token fits
template <typename IDX>
__global__ __launch_bounds__(256) void hstu_kv_fp8_scan_kernel(const hstu_kv_append_fp8_params p, unsigned* unit_max, int* first_slot, int* touched, int touched_cap) {
    const unsigned cph = (unsigned)p.head_dim / 8;
    const unsigned cpt = cph * (unsigned)p.num_heads;
    const int nnz = min(max(*p.nnz_dev, 0), p.nnz_max);
    const IDX total = (IDX)nnz * cpt;
    const IDX stride = (IDX)gridDim.x * 256;
    const int bf16 = p.src_dtype == HSTU_BF16;
    // every lane of a wave runs the same number of rounds: the shuffles below need all lanes of a row present
    const IDX rounds = (total + stride - 1) / stride;
    for (IDX r = 0; r < rounds; r++) {
        const IDX gidx = r * stride + (IDX)blockIdx.x * 256 + threadIdx.x;
        float kmax = 0.f, vmax = 0.f;
        bool ok = false;
        int page = 0, slot = 0;
        unsigned head = 0, c = 0;
        if (gidx < total) {
            const unsigned i = (unsigned)(gidx / cpt), rem = (unsigned)(gidx % cpt);
            head = rem / cph;
            c = rem % cph;
            int64_t row;
            ok = kf_route(p, i, page, slot, row);
            if (ok) {
                const kf_u32x4 kx = *reinterpret_cast<const kf_u32x4*>(reinterpret_cast<const unsigned short*>(p.append_key) +
                                                                       row * p.append_k_stride_n + head * p.append_k_stride_h + 8 * c);
                const kf_u32x4 vx = *reinterpret_cast<const kf_u32x4*>(reinterpret_cast<const unsigned short*>(p.append_value) +
                                                                       row * p.append_v_stride_n + head * p.append_v_stride_h + 8 * c);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    kmax = fmaxf(kmax, fmaxf(fabsf(kf_elem(kx[e], 0, bf16)), fabsf(kf_elem(kx[e], 1, bf16))));
                    vmax = fmaxf(vmax, fmaxf(fabsf(kf_elem(vx[e], 0, bf16)), fabsf(kf_elem(vx[e], 1, bf16))));
                }
            }
        }
        for (unsigned o = 1; o < cph; o <<= 1) {
            kmax = fmaxf(kmax, __shfl_xor(kmax, (int)o));
            vmax = fmaxf(vmax, __shfl_xor(vmax, (int)o));
        }
        if (ok && c == 0) {
            // non-negative floats order like their bit patterns
            atomicMax(unit_max + ((int64_t)page * 2 + 0) * p.num_heads + head, __builtin_bit_cast(unsigned, kmax));
            atomicMax(unit_max + ((int64_t)page * 2 + 1) * p.num_heads + head, __builtin_bit_cast(unsigned, vmax));
            // whoever finds the page untouched lists it: touched[0] = count, then the pages
            if (head == 0 && atomicMin(first_slot + page, slot) == KF_NOSLOT) {
                const int at = atomicAdd(touched, 1);
                if (at < touched_cap) touched[1 + at] = page;
            }
        }
    }
}

// blockIdx.x = (entry of the list of touched pages, K|V, head)
__global__ __launch_bounds__(256) void hstu_kv_fp8_scale_kernel(const hstu_kv_append_fp8_params p, const unsigned* unit_max, const int* first_slot, const int* touched, int touched_cap) {
    const int entry = blockIdx.x / (2 * p.num_heads);
    if (entry >= min(touched[0], touched_cap)) return;
    const int page = touched[1 + entry], kv = blockIdx.x / p.num_heads % 2, head = blockIdx.x % p.num_heads;
    const int unit = (page * 2 + kv) * p.num_heads + head;
    const int first = first_slot[page];
    if (first == KF_NOSLOT) return;   // (cannot happen for a listed page)
    const float cand = __builtin_bit_cast(float, unit_max[unit]) / KF_MAX;
    const float s_old = p.kv_scales[unit];
    const float s = first > 0 ? fmaxf(s_old, cand) : (cand > 0.f ? cand : 1.0f);
    if (first > 0 && s != s_old) {
        uint8_t* base = p.kv_cache + (((int64_t)page * 2 + kv) * p.page_size * p.num_heads + head) * p.head_dim;
        const int pairs = first * p.head_dim / 2;
        for (int i = threadIdx.x; i < pairs; i += 256) {
            const int slot = 2 * i / p.head_dim, d = 2 * i % p.head_dim;
            unsigned short* q = reinterpret_cast<unsigned short*>(base + (int64_t)slot * p.num_heads * p.head_dim + d);
            const unsigned short old = *q;
            *q = (unsigned short)kf_quant2(fp8_e4m3_to_float((uint8_t)(old & 0xff)) * s_old, fp8_e4m3_to_float((uint8_t)(old >> 8)) * s_old, s);
        }
    }
    __syncthreads();   // every thread has read s_old
    if (threadIdx.x == 0) p.kv_scales[unit] = s;
}

template <typename IDX>
__global__ __launch_bounds__(256) void hstu_kv_fp8_write_kernel(const hstu_kv_append_fp8_params p) {
    const unsigned cph = (unsigned)p.head_dim / 8;
    const unsigned cpt = cph * (unsigned)p.num_heads;
    const int nnz = min(max(*p.nnz_dev, 0), p.nnz_max);
    const IDX total = (IDX)nnz * cpt;
    const IDX stride = (IDX)gridDim.x * 256;
    const int bf16 = p.src_dtype == HSTU_BF16;
    for (IDX gidx = (IDX)blockIdx.x * 256 + threadIdx.x; gidx < total; gidx += stride) {
        const unsigned i = (unsigned)(gidx / cpt), rem = (unsigned)(gidx % cpt);
        const unsigned head = rem / cph, c = rem % cph;
        int page, slot;
        int64_t row;
        if (!kf_route(p, i, page, slot, row)) continue;
        const kf_u32x4 kx = *reinterpret_cast<const kf_u32x4*>(reinterpret_cast<const unsigned short*>(p.append_key) + row * p.append_k_stride_n +
                                                               head * p.append_k_stride_h + 8 * c);
        const kf_u32x4 vx = *reinterpret_cast<const kf_u32x4*>(reinterpret_cast<const unsigned short*>(p.append_value) + row * p.append_v_stride_n +
                                                               head * p.append_v_stride_h + 8 * c);
        const float sk = p.kv_scales[((int64_t)page * 2 + 0) * p.num_heads + head], sv = p.kv_scales[((int64_t)page * 2 + 1) * p.num_heads + head];
        unsigned qk[4], qv[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            qk[e] = kf_quant2(kf_elem(kx[e], 0, bf16), kf_elem(kx[e], 1, bf16), sk);
            qv[e] = kf_quant2(kf_elem(vx[e], 0, bf16), kf_elem(vx[e], 1, bf16), sv);
        }
        uint8_t* dst = p.kv_cache + ((((int64_t)page * 2) * p.page_size + slot) * p.num_heads + head) * p.head_dim + 8 * c;
        *reinterpret_cast<kf_u32x2*>(dst) = kf_u32x2{qk[0] | (qk[1] << 16), qk[2] | (qk[3] << 16)};
        *reinterpret_cast<kf_u32x2*>(dst + (int64_t)p.page_size * p.num_heads * p.head_dim) = kf_u32x2{qv[0] | (qv[1] << 16), qv[2] | (qv[3] << 16)};
    }
}

// pages one call can touch: every new token goes to one page
static int64_t kf_touched_cap(const hstu_kv_append_fp8_params* p) { return p->nnz_max < p->num_pages ? p->nnz_max : p->num_pages; }
// per unit a maximum, per page a first slot, then the count and the list of touched pages
static uint64_t kf_workspace_bytes(const hstu_kv_append_fp8_params* p) {
    return ((uint64_t)p->num_pages * (2 * p->num_heads + 1) + 1 + (uint64_t)kf_touched_cap(p)) * 4;
}

static int kf_check(const hstu_kv_append_fp8_params* p) {
    if (!p) return fail(HSTU_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(hstu_kv_append_fp8_params))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "hstu_kv_append_fp8_params size mismatch: caller %u, library %zu", p->struct_size,
                    sizeof(hstu_kv_append_fp8_params));
    if (p->src_dtype != HSTU_F16 && p->src_dtype != HSTU_BF16)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "src_dtype expect float16 or bfloat16, but value is %d", p->src_dtype);
    if (p->head_dim < 8 || p->head_dim > 512 || (p->head_dim & (p->head_dim - 1)))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "head_dim expect a power of two in [8, 512], but value is %d", p->head_dim);
    if (p->num_heads < 1 || p->page_size < 1 || p->num_pages < 1 || p->batch < 1 || p->num_indices < 0 || p->nnz_max < 0 || p->append_rows < 0)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "num_heads, page_size, num_pages, batch must be positive and num_indices, nnz_max, append_rows non-negative");
    if ((int64_t)p->num_pages * 2 * p->num_heads > 0x7fffffffLL) return fail(HSTU_ERR_UNSUPPORTED, "num_pages * 2 * num_heads too large for one launch");
    return HSTU_OK;
}

}  // namespace hstu

using namespace hstu;

extern "C" int hstu_hip_kv_append_fp8_get_workspace_size(const hstu_kv_append_fp8_params* p, uint64_t* workspace_bytes) {
    const int rc = kf_check(p);
    if (rc != HSTU_OK) return rc;
    if (!workspace_bytes) return fail(HSTU_ERR_INVALID_ARGUMENT, "workspace_bytes is NULL");
    *workspace_bytes = kf_workspace_bytes(p);
    return HSTU_OK;
}

extern "C" int hstu_hip_kv_append_fp8(const hstu_kv_append_fp8_params* p, void* workspace, uint64_t workspace_bytes, void* stream) {
    const int rc = kf_check(p);
    if (rc != HSTU_OK) return rc;
    if (!p->kv_cache || !p->kv_scales || !p->append_key || !p->append_value || !p->kv_indices || !p->kv_indptr || !p->batch_indices ||
        !p->positions || !p->offsets || !p->nnz_dev)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "kv_cache, kv_scales, append_key, append_value, kv_indices, kv_indptr, batch_indices, positions, offsets and nnz_dev must not be NULL");
    const int64_t strides[] = {p->append_k_stride_n, p->append_k_stride_h, p->append_v_stride_n, p->append_v_stride_h};
    for (int64_t s : strides)
        if (s < 0 || s % 8) return fail(HSTU_ERR_UNSUPPORTED, "strides must be non-negative multiples of 8 elements, but one is %lld", (long long)s);
    if ((reinterpret_cast<uintptr_t>(p->append_key) | reinterpret_cast<uintptr_t>(p->append_value)) & 15)
        return fail(HSTU_ERR_UNSUPPORTED, "append_key and append_value must be 16-byte aligned");
    if ((reinterpret_cast<uintptr_t>(p->kv_cache) & 7) || (reinterpret_cast<uintptr_t>(p->kv_scales) & 3) || (reinterpret_cast<uintptr_t>(workspace) & 3))
        return fail(HSTU_ERR_UNSUPPORTED, "kv_cache must be 8-byte aligned, kv_scales and the workspace 4-byte aligned");
    const uint64_t need = kf_workspace_bytes(p);
    if (!workspace || workspace_bytes < need)
        return fail(HSTU_ERR_WORKSPACE, "workspace of %llu bytes needed, %llu given", (unsigned long long)need, (unsigned long long)workspace_bytes);
    if (p->nnz_max == 0) return HSTU_OK;
    const int units = p->num_pages * 2 * p->num_heads;
    unsigned* unit_max = reinterpret_cast<unsigned*>(workspace);
    int* first_slot = reinterpret_cast<int*>(unit_max + units);
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    int* touched = first_slot + p->num_pages;
    const int touched_cap = (int)kf_touched_cap(p);
    const unsigned reset_grid = (unsigned)(((int64_t)p->nnz_max + 255) / 256 > 4096 ? 4096 : ((int64_t)p->nnz_max + 255) / 256);
    hipLaunchKernelGGL(hstu_kv_fp8_reset_kernel, dim3(reset_grid), dim3(256), 0, st, *p, unit_max, first_slot, touched);
    const int64_t lanes = (int64_t)p->nnz_max * p->num_heads * (p->head_dim / 8);
    const int64_t want = (lanes + 255) / 256;
    const unsigned grid = (unsigned)(want < 1 ? 1 : (want > 65536 ? 65536 : want));
    const bool small = lanes + 2 * (int64_t)grid * 256 < (int64_t)1 << 32;
    if (small) hipLaunchKernelGGL(hstu_kv_fp8_scan_kernel<unsigned>, dim3(grid), dim3(256), 0, st, *p, unit_max, first_slot, touched, touched_cap);
    else hipLaunchKernelGGL(hstu_kv_fp8_scan_kernel<unsigned long long>, dim3(grid), dim3(256), 0, st, *p, unit_max, first_slot, touched, touched_cap);
    hipLaunchKernelGGL(hstu_kv_fp8_scale_kernel, dim3((unsigned)(touched_cap * 2 * p->num_heads)), dim3(256), 0, st, *p, unit_max, first_slot, touched, touched_cap);
    if (small) hipLaunchKernelGGL(hstu_kv_fp8_write_kernel<unsigned>, dim3(grid), dim3(256), 0, st, *p);
    else hipLaunchKernelGGL(hstu_kv_fp8_write_kernel<unsigned long long>, dim3(grid), dim3(256), 0, st, *p);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    return HSTU_OK;
}
