// Append to an fp8-e4m3 paged K/V cache with one fp32 scale per (page, K|V, head): the write side of the table that
// hstu_hip_paged_forward reads with cache_dtype = HSTU_FP8_E4M3.  No counterpart in the reference (its cache manager
// stores 2-byte rows unscaled, append_paged_kvcache_kernel.h:42-76); the routing of a token to its page and slot is the
// reference's, the quantisation is this library's:
//   after an append, a touched (page, K|V, head) holds  q = rne_e4m3(clamp(x / s, -448, 448))  with
//   s = max(s_before, absmax(new rows) / 448)  if the page already held rows below the first new slot,
//   s = absmax(new rows) / 448 (1 if that is 0) otherwise;  rows already there are requantised from q * s_before
//   when s grew and are left untouched bit for bit when it did not.
// A page filled by one append therefore equals quantising the whole page at once.
// Nothing is read on the host and every kernel is sized by the new tokens, not by the cache (a table of a million pages
// costs an append of one token no more than a table of ten).  New tokens normally arrive as runs: consecutive tokens of
// one user at consecutive positions inside one page (what hstu_hip_kv_token_positions produces).  A page whose new
// tokens form ONE run is finished by one workgroup per head that holds the run's rows in registers between the absmax
// and the quantisation, so the rows are read once.  Pages whose new tokens are scattered over several runs (any order
// of (user, position) pairs is allowed) get their scale and their bytes from two more kernels that read the rows a
// second time; these find nothing to do otherwise.
//   reset  clears the per-unit maxima, the first slot and the run count of the pages the new tokens go to, and the lists
//   runs   one thread per token: the first token of a run enters the run in the run list, counts it for its page and
//          lowers the page's first slot; the second run of a page enters the page in the list of scattered pages
//   page   one workgroup per (run, head) of a page with one run: absmax, new scale, requantisation of the rows below
//          the first new slot if the scale grew, quantisation of the run
//          (a run of a scattered page only adds its absmax to the page's: atomic max per unit)
//   scan   (only when pages are too large for the kernel above) absmax of every new (token, K|V, head) row -> atomic max per unit
//   scale  (scattered pages) per unit: new scale, requantise the rows below the first new slot if the scale grew
//   write  (scattered pages) quantise the new rows with the unit's scale
// Byte work bounded by HBM: the new rows are read once (2 bytes per element) and written once (1 byte).
#include "hstu_device.h"
#include "../../include/hstu_kvcache.h"

namespace hstu {

typedef __attribute__((ext_vector_type(4))) unsigned int kf_u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int kf_u32x2;
typedef __attribute__((ext_vector_type(4))) int kf_i32x4;
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

// x / s for a divisor shared by many elements: r = 1.0f / s (rounded to nearest), the product x * r is corrected twice by
// its remainder (each fma is exact in the remainder).  The result is the IEEE quotient unless x / s lies within 2^-48
// (relative) of an fp32 rounding boundary, and the e4m3 byte differs only if that boundary is also next to an e4m3 tie.
// For s in [2^-100, 2^100] only (r and the remainders stay normal numbers); quotients below the fp32 normal range are far
// below half of the smallest e4m3 number and round to the same zero either way.
__device__ __forceinline__ float kf_div_by(float x, float s, float r) {
    float q = x * r;
    q = __builtin_fmaf(__builtin_fmaf(-s, q, x), r, q);
    return __builtin_copysignf(__builtin_fmaf(__builtin_fmaf(-s, q, x), r, q), x);   // (-0 stays -0: its remainder is +0)
}
__device__ __forceinline__ unsigned kf_quant2_by(float a, float b, float s, float r) {
    a = fminf(fmaxf(kf_div_by(a, s, r), -KF_MAX), KF_MAX);
    b = fminf(fmaxf(kf_div_by(b, s, r), -KF_MAX), KF_MAX);
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
__global__ __launch_bounds__(256) void hstu_kv_fp8_reset_kernel(const hstu_kv_append_fp8_params p, unsigned* unit_max, int* first_slot, int* run_count, int* touched, int* nruns) {
    const int nnz = min(max(*p.nnz_dev, 0), p.nnz_max);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        touched[0] = 0;
        nruns[0] = 0;
    }
    for (unsigned i = blockIdx.x * 256 + threadIdx.x; i < (unsigned)nnz; i += gridDim.x * 256) {
        int page, slot;
        int64_t row;
        if (!kf_route(p, i, page, slot, row)) continue;
        for (int u = 0; u < 2 * p.num_heads; u++) unit_max[(int64_t)page * 2 * p.num_heads + u] = 0u;
        first_slot[page] = KF_NOSLOT;
        run_count[page] = 0;
    }
}

// one thread per new token.  Token i continues the run of token i - 1 if both are valid, belong to the same user, sit at
// consecutive positions and i does not start a page; every other valid token starts a run and leaves a record of 8 words
// in the run list: token, page, slot, user, position, source row (2 words).  `force`: count every run twice, which sends
// all pages to the kernels for scattered pages (pages too large for the registers of a workgroup).
constexpr int KF_REC = 8;
__global__ __launch_bounds__(256) void hstu_kv_fp8_runs_kernel(const hstu_kv_append_fp8_params p, int* first_slot, int* run_count, int* touched, int touched_cap,
                                                               int* nruns, int* runs, int force) {
    __shared__ int s_n, s_base;
    const int nnz = min(max(*p.nnz_dev, 0), p.nnz_max);
    const unsigned stride = gridDim.x * 256;
    const unsigned rounds = ((unsigned)nnz + stride - 1) / stride;   // the same for every thread: barriers inside
    for (unsigned r = 0; r < rounds; r++) {
        const unsigned i = r * stride + blockIdx.x * 256 + threadIdx.x;
        if (threadIdx.x == 0) s_n = 0;
        __syncthreads();
        int page = 0, slot = 0, mine = -1;
        int64_t row = 0;
        int b = 0, pos = 0;
        if (i < (unsigned)nnz && kf_route(p, i, page, slot, row)) {
            b = p.batch_indices[i];
            pos = p.positions[i];
            // (a predecessor of the same user one position below, inside the same page, is valid if its source row is)
            const bool cont = i > 0 && slot != 0 && row > 0 && p.batch_indices[i - 1] == b && p.positions[i - 1] + 1 == pos;
            if (!cont) {
                atomicMin(first_slot + page, slot);
                const int inc = force ? 2 : 1;
                const int before = atomicAdd(run_count + page, inc);
                if (before < 2 && before + inc >= 2) {
                    const int at = atomicAdd(touched, 1);
                    if (at < touched_cap) touched[1 + at] = page;
                }
                mine = atomicAdd(&s_n, 1);
            }
        }
        __syncthreads();
        if (threadIdx.x == 0 && s_n) s_base = atomicAdd(nruns, s_n);   // one entry of the global count per workgroup
        __syncthreads();
        if (mine >= 0) {
            int* rec = runs + (int64_t)KF_REC * (s_base + mine);
            *reinterpret_cast<kf_i32x4*>(rec) = kf_i32x4{(int)i, page, slot, b};
            *reinterpret_cast<kf_i32x4*>(rec + 4) = kf_i32x4{pos, (int)(unsigned)(row & 0xffffffff), (int)(row >> 32), 0};
        }
    }
}

// one workgroup per (run, head) of a page that has this one run: thread t holds the same 8 elements of K and of V of
// ITEMS (token, 8-element column) cells, cell = t + 256 j -> token cell / (dim / 8) of the run
template <int ITEMS>
__global__ __launch_bounds__(256) void hstu_kv_fp8_page_kernel(const hstu_kv_append_fp8_params p, unsigned* unit_max, const int* run_count, const int* nruns, const int* runs) {
    __shared__ int s_len;
    __shared__ float s_red[2][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const unsigned cph = (unsigned)p.head_dim / 8;
    const int nnz = min(max(*p.nnz_dev, 0), p.nnz_max);
    const int bf16 = p.src_dtype == HSTU_BF16;
    const int total = min(nruns[0], p.nnz_max) * p.num_heads;
    for (int w = blockIdx.x; w < total; w += gridDim.x) {
        const int head = w % p.num_heads;
        const int* rec = runs + (int64_t)KF_REC * (w / p.num_heads);
        const kf_i32x4 r0 = *reinterpret_cast<const kf_i32x4*>(rec), r1 = *reinterpret_cast<const kf_i32x4*>(rec + 4);
        const int i0 = r0[0], page = r0[1], slot0 = r0[2], b = r0[3], pos0 = r1[0];
        const int64_t row0 = (int64_t)(((uint64_t)(unsigned)r1[2] << 32) | (unsigned)r1[1]);
        // the run ends before the page does, before the tokens do and before the source rows do
        const int maxlen = (int)min((int64_t)min(p.page_size - slot0, nnz - i0), p.append_rows - row0);
        // everything this workgroup needs is requested before the first wait: the rows of the longest run possible, the
        // tokens that may belong to it, the page's run count and the scales
        kf_u32x4 kx[ITEMS], vx[ITEMS];
#pragma unroll
        for (int j = 0; j < ITEMS; j++) {
            const unsigned cell = (unsigned)tid + 256u * j;
            const int t = min((int)(cell / cph), maxlen - 1);
            const unsigned c = cell % cph;
            kx[j] = __builtin_nontemporal_load(reinterpret_cast<const kf_u32x4*>(reinterpret_cast<const unsigned short*>(p.append_key) +
                                                                                 (row0 + t) * p.append_k_stride_n + head * p.append_k_stride_h + 8 * c));
            vx[j] = __builtin_nontemporal_load(reinterpret_cast<const kf_u32x4*>(reinterpret_cast<const unsigned short*>(p.append_value) +
                                                                                 (row0 + t) * p.append_v_stride_n + head * p.append_v_stride_h + 8 * c));
        }
        const int count = run_count[page];
        float sc_old[2];
        sc_old[0] = p.kv_scales[((int64_t)page * 2 + 0) * p.num_heads + head];
        sc_old[1] = p.kv_scales[((int64_t)page * 2 + 1) * p.num_heads + head];
        if (tid == 0) s_len = maxlen;
        __syncthreads();
        for (int t = tid + 1; t < maxlen; t += 256)
            if (p.batch_indices[i0 + t] != b || p.positions[i0 + t] != pos0 + t) atomicMin(&s_len, t);
        __syncthreads();
        const int len = s_len;
        float kmax = 0.f, vmax = 0.f;
#pragma unroll
        for (int j = 0; j < ITEMS; j++) {
            if ((int)(((unsigned)tid + 256u * j) / cph) >= len) continue;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                kmax = fmaxf(kmax, fmaxf(fabsf(kf_elem(kx[j][e], 0, bf16)), fabsf(kf_elem(kx[j][e], 1, bf16))));
                vmax = fmaxf(vmax, fmaxf(fabsf(kf_elem(vx[j][e], 0, bf16)), fabsf(kf_elem(vx[j][e], 1, bf16))));
            }
        }
        for (int o = 1; o < 64; o <<= 1) {
            kmax = fmaxf(kmax, __shfl_xor(kmax, o));
            vmax = fmaxf(vmax, __shfl_xor(vmax, o));
        }
        if (lane == 0) {
            s_red[0][wave] = kmax;
            s_red[1][wave] = vmax;
        }
        __syncthreads();
        float sc[2], amax[2];
#pragma unroll
        for (int kv = 0; kv < 2; kv++) {
            amax[kv] = fmaxf(fmaxf(s_red[kv][0], s_red[kv][1]), fmaxf(s_red[kv][2], s_red[kv][3]));
            const float cand = amax[kv] / KF_MAX;
            sc[kv] = slot0 > 0 ? fmaxf(sc_old[kv], cand) : (cand > 0.f ? cand : 1.0f);
        }
        __syncthreads();   // s_len and s_red are free for the next run
        if (count != 1) {
            // a scattered page (the same for all threads): the run adds its maxima to the page's (non-negative floats
            // order like their bit patterns), the kernels below do the rest
            if (tid < 2) atomicMax(unit_max + ((int64_t)page * 2 + tid) * p.num_heads + head, __builtin_bit_cast(unsigned, tid ? amax[1] : amax[0]));
            continue;
        }
#pragma unroll
        for (int kv = 0; kv < 2; kv++) {
            if (slot0 > 0 && sc[kv] != sc_old[kv]) {
                uint8_t* base = p.kv_cache + (((int64_t)page * 2 + kv) * p.page_size * p.num_heads + head) * p.head_dim;
                const int pairs = slot0 * p.head_dim / 2;
                for (int i = tid; i < pairs; i += 256) {
                    const int slot = 2 * i / p.head_dim, d = 2 * i % p.head_dim;
                    unsigned short* q = reinterpret_cast<unsigned short*>(base + (int64_t)slot * p.num_heads * p.head_dim + d);
                    const unsigned short old = *q;
                    *q = (unsigned short)kf_quant2(fp8_e4m3_to_float((uint8_t)(old & 0xff)) * sc_old[kv], fp8_e4m3_to_float((uint8_t)(old >> 8)) * sc_old[kv], sc[kv]);
                }
            }
        }
        // (every thread holds the old scales in registers: no barrier before they are replaced)
        if (tid < 2) p.kv_scales[((int64_t)page * 2 + tid) * p.num_heads + head] = tid ? sc[1] : sc[0];
        const float rc[2] = {1.0f / sc[0], 1.0f / sc[1]};
        const bool fast = fminf(sc[0], sc[1]) >= 0x1p-100f && fmaxf(sc[0], sc[1]) <= 0x1p100f;   // (the same for all threads)
#pragma unroll
        for (int j = 0; j < ITEMS; j++) {
            const unsigned cell = (unsigned)tid + 256u * j;
            const int t = (int)(cell / cph);
            const unsigned c = cell % cph;
            if (t >= len) continue;
            unsigned qk[4], qv[4];
            if (fast) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    qk[e] = kf_quant2_by(kf_elem(kx[j][e], 0, bf16), kf_elem(kx[j][e], 1, bf16), sc[0], rc[0]);
                    qv[e] = kf_quant2_by(kf_elem(vx[j][e], 0, bf16), kf_elem(vx[j][e], 1, bf16), sc[1], rc[1]);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    qk[e] = kf_quant2(kf_elem(kx[j][e], 0, bf16), kf_elem(kx[j][e], 1, bf16), sc[0]);
                    qv[e] = kf_quant2(kf_elem(vx[j][e], 0, bf16), kf_elem(vx[j][e], 1, bf16), sc[1]);
                }
            }
            uint8_t* dst = p.kv_cache + ((((int64_t)page * 2) * p.page_size + slot0 + t) * p.num_heads + head) * p.head_dim + 8 * c;
            __builtin_nontemporal_store(kf_u32x2{qk[0] | (qk[1] << 16), qk[2] | (qk[3] << 16)}, reinterpret_cast<kf_u32x2*>(dst));
            __builtin_nontemporal_store(kf_u32x2{qv[0] | (qv[1] << 16), qv[2] | (qv[3] << 16)},
                                        reinterpret_cast<kf_u32x2*>(dst + (int64_t)p.page_size * p.num_heads * p.head_dim));
        }
    }
}

// one lane = the same 8 elements of the K row and of the V row of one (token, head); the dim / 8 lanes of a row sit
// side by side in a wave.  IDX: type of the flat lane index, 32 bits whenever nnz_max * lanes per token fits
template <typename IDX>
__global__ __launch_bounds__(256) void hstu_kv_fp8_scan_kernel(const hstu_kv_append_fp8_params p, unsigned* unit_max, const int* run_count, const int* touched) {
    if (touched[0] == 0) return;   // no scattered page
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
            ok = kf_route(p, i, page, slot, row) && run_count[page] > 1;
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
        }
    }
}

// one workgroup per (entry of the list of scattered pages, K|V, head)
__global__ __launch_bounds__(256) void hstu_kv_fp8_scale_kernel(const hstu_kv_append_fp8_params p, const unsigned* unit_max, const int* first_slot, const int* touched, int touched_cap) {
    const int total = min(touched[0], touched_cap) * 2 * p.num_heads;
    for (int w = blockIdx.x; w < total; w += gridDim.x) {
        const int page = touched[1 + w / (2 * p.num_heads)], kv = w / p.num_heads % 2, head = w % p.num_heads;
        const int unit = (page * 2 + kv) * p.num_heads + head;
        const int first = first_slot[page];
        if (first == KF_NOSLOT) continue;   // (cannot happen for a listed page)
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
}

template <typename IDX>
__global__ __launch_bounds__(256) void hstu_kv_fp8_write_kernel(const hstu_kv_append_fp8_params p, const int* run_count, const int* touched) {
    if (touched[0] == 0) return;   // no scattered page
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
        if (!kf_route(p, i, page, slot, row) || run_count[page] <= 1) continue;
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
// word of the workspace where the run list starts (16-byte aligned records); the count of runs sits in the word before
static uint64_t kf_runs_word(const hstu_kv_append_fp8_params* p) {
    const uint64_t w = (uint64_t)p->num_pages * (2 * p->num_heads + 2) + 1 + (uint64_t)kf_touched_cap(p) + 1;
    return (w + 3) / 4 * 4;
}
// per unit a maximum, per page a first slot and a run count, then the count and the list of scattered pages, the count
// and the list of runs
static uint64_t kf_workspace_bytes(const hstu_kv_append_fp8_params* p) {
    return (kf_runs_word(p) + (uint64_t)KF_REC * p->nnz_max) * 4;
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
    if ((reinterpret_cast<uintptr_t>(p->kv_cache) & 7) || (reinterpret_cast<uintptr_t>(p->kv_scales) & 3) || (reinterpret_cast<uintptr_t>(workspace) & 15))
        return fail(HSTU_ERR_UNSUPPORTED, "kv_cache must be 8-byte aligned, kv_scales 4-byte and the workspace 16-byte aligned");
    const uint64_t need = kf_workspace_bytes(p);
    if (!workspace || workspace_bytes < need)
        return fail(HSTU_ERR_WORKSPACE, "workspace of %llu bytes needed, %llu given", (unsigned long long)need, (unsigned long long)workspace_bytes);
    if (p->nnz_max == 0) return HSTU_OK;
    const int units = p->num_pages * 2 * p->num_heads;
    unsigned* unit_max = reinterpret_cast<unsigned*>(workspace);
    int* first_slot = reinterpret_cast<int*>(unit_max + units);
    int* run_count = first_slot + p->num_pages;
    int* touched = run_count + p->num_pages;
    const int touched_cap = (int)kf_touched_cap(p);
    int* runs = reinterpret_cast<int*>(workspace) + kf_runs_word(p);
    int* nruns = runs - 1;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const unsigned token_grid = (unsigned)(((int64_t)p->nnz_max + 255) / 256 > 4096 ? 4096 : ((int64_t)p->nnz_max + 255) / 256);
    // cells of 8 elements per (page, head) over the 256 threads of a workgroup: up to 8 per thread stay in registers
    const int64_t cells = (int64_t)p->page_size * (p->head_dim / 8);
    const int items = cells <= 256 ? 1 : (cells <= 512 ? 2 : (cells <= 1024 ? 4 : (cells <= 2048 ? 8 : 0)));
    hipLaunchKernelGGL(hstu_kv_fp8_reset_kernel, dim3(token_grid), dim3(256), 0, st, *p, unit_max, first_slot, run_count, touched, nruns);
    hipLaunchKernelGGL(hstu_kv_fp8_runs_kernel, dim3(token_grid), dim3(256), 0, st, *p, first_slot, run_count, touched, touched_cap, nruns, runs, items == 0 ? 1 : 0);
    if (items) {
        // runs of well-formed input: every user's new tokens are one stretch of positions, cut at page boundaries
        int64_t bound = (int64_t)p->nnz_max / p->page_size + 2 * (int64_t)p->batch + 1;
        if (bound > p->nnz_max) bound = p->nnz_max;
        bound *= p->num_heads;
        const unsigned pgrid = (unsigned)(bound > (1 << 20) ? (1 << 20) : bound);
        if (items == 1) hipLaunchKernelGGL(hstu_kv_fp8_page_kernel<1>, dim3(pgrid), dim3(256), 0, st, *p, unit_max, run_count, nruns, runs);
        else if (items == 2) hipLaunchKernelGGL(hstu_kv_fp8_page_kernel<2>, dim3(pgrid), dim3(256), 0, st, *p, unit_max, run_count, nruns, runs);
        else if (items == 4) hipLaunchKernelGGL(hstu_kv_fp8_page_kernel<4>, dim3(pgrid), dim3(256), 0, st, *p, unit_max, run_count, nruns, runs);
        else hipLaunchKernelGGL(hstu_kv_fp8_page_kernel<8>, dim3(pgrid), dim3(256), 0, st, *p, unit_max, run_count, nruns, runs);
    }
    // the kernels for scattered pages: grids that cost little when they find nothing to do
    const int64_t lanes = (int64_t)p->nnz_max * p->num_heads * (p->head_dim / 8);
    const int64_t want = (lanes + 255) / 256;
    const unsigned grid = (unsigned)(want < 1 ? 1 : (want > 1024 ? 1024 : want));
    const bool small = lanes + 2 * (int64_t)grid * 256 < (int64_t)1 << 32;
    if (!items) {   // (otherwise the kernel above has collected the maxima of the scattered pages)
        if (small) hipLaunchKernelGGL(hstu_kv_fp8_scan_kernel<unsigned>, dim3(grid), dim3(256), 0, st, *p, unit_max, run_count, touched);
        else hipLaunchKernelGGL(hstu_kv_fp8_scan_kernel<unsigned long long>, dim3(grid), dim3(256), 0, st, *p, unit_max, run_count, touched);
    }
    const int64_t swant = (int64_t)touched_cap * 2 * p->num_heads;
    hipLaunchKernelGGL(hstu_kv_fp8_scale_kernel, dim3((unsigned)(swant > 1024 ? 1024 : swant)), dim3(256), 0, st, *p, unit_max, first_slot, touched, touched_cap);
    if (small) hipLaunchKernelGGL(hstu_kv_fp8_write_kernel<unsigned>, dim3(grid), dim3(256), 0, st, *p, run_count, touched);
    else hipLaunchKernelGGL(hstu_kv_fp8_write_kernel<unsigned long long>, dim3(grid), dim3(256), 0, st, *p, run_count, touched);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    return HSTU_OK;
}
