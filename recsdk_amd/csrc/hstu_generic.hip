// Full-feature HSTU forward kernel in plain fp32 FMA arithmetic.
//
// Covers everything the op accepts (fp32/fp16/bf16 I/O, float8_e4m3fn inputs with fp16 output, any head dim <= 512,
// Dqk != Dv, GQA, delta-q, context/target masks, custom mask, dense bias, bias tables, paged and fp8 caches).  It is the path
// for fp32 I/O (where bf16 MFMA cannot meet 1e-5) and for shapes the MFMA kernels do not specialise.
// Element-wise order follows the reference's vector pass (vector_score_inter.h:299-323,186-212):
//   x = alpha*(S + bias);  p = x*sigmoid(x);  p *= silu_scale*mask;  P = round_to_io_dtype(p).
#include "hstu_device.h"

namespace hstu {

constexpr int GBM = 16;   // Q rows per workgroup
constexpr int GBN = 64;   // K columns per step
constexpr int GDC = 64;   // head-dim chunk staged in LDS
constexpr int GLD = 65;   // padded leading dimension of the LDS tiles

struct RowSrc {
    const void* ptr;
    float scale;
    int fp8;
};

template <typename T>
__device__ __forceinline__ RowSrc kv_row(const KArgs& a, const Seq& s, int which, int j, int hk, int dim) {
    const hstu_fwd_params& p = a.p;
    RowSrc r;
    r.scale = 1.0f;
    r.fp8 = 0;
    if (a.op == OP_PAGED && j < s.hist_k) {
        const int is64 = p.index_type == HSTU_I64;
        int64_t page = ld_idx(p.page_ids, s.page0 + j / p.page_size, is64);
        int slot = j % p.page_size;
        int64_t e = ((((page * 2 + which) * p.page_size) + slot) * p.heads_k + hk) * (int64_t)dim;
        if (p.cache_dtype == HSTU_FP8_E4M3) {
            r.ptr = reinterpret_cast<const uint8_t*>(p.kv_cache) + e;
            r.scale = p.kv_scales[(page * 2 + which) * p.heads_k + hk];
            r.fp8 = 1;
        } else {
            r.ptr = reinterpret_cast<const T*>(p.kv_cache) + e;
        }
    } else {
        int64_t row = (a.op == OP_PAGED) ? s.cand_row + (j - s.hist_k) : s.k_start + j;
        const T* base = reinterpret_cast<const T*>(which ? p.v : p.k);
        r.ptr = base + (row * p.heads_k + hk) * (int64_t)dim;
    }
    return r;
}

template <typename T>
__device__ __forceinline__ float row_elem(const RowSrc& r, int d) {
    if (r.fp8) {
        // dequantised values are rounded to the I/O dtype, as the MFMA path stores them
        float x = fp8_e4m3_to_float(reinterpret_cast<const uint8_t*>(r.ptr)[d]) * r.scale;
        return to_float(from_float<T>(x));
    }
    return to_float(reinterpret_cast<const T*>(r.ptr)[d]);
}

template <typename T>
__global__ __launch_bounds__(256) void hstu_generic_kernel(const KArgs a) {
    const hstu_fwd_params& p = a.p;
    extern __shared__ float smem[];
    const int dqk_pad = (p.dim_qk + GDC - 1) / GDC * GDC;
    float* Qs = smem;                   // [GBM][dqk_pad]
    float* KVs = Qs + GBM * dqk_pad;    // [GBN][GLD]
    float* Ps = KVs + GBN * GLD;        // [GBM][GLD]

    const int tid = threadIdx.x;
    const int b = blockIdx.z, h = blockIdx.y;
    const int hk = h / a.head_ratio;
    const Seq s = load_seq(a, b);
    const T* q = reinterpret_cast<const T*>(p.q);
    typedef typename OutOf<T>::type OT;
    OT* out = reinterpret_cast<OT*>(p.out);
    const int r = tid / 16, cb = tid % 16;
    const int is_tril = p.mask_type == HSTU_MASK_TRIL;
    const int64_t bh = (int64_t)b * p.heads_q + h;

    for (int tile = blockIdx.x; tile * GBM < s.lq; tile += gridDim.x) {
        const int i0 = tile * GBM;
        const int i1 = min(i0 + GBM, s.lq);
        const int kend = (s.lk > 0) ? k_extent(a, s, i0, i1) : 0;
        // stage the Q rows (zero padded)
        for (int e = tid; e < GBM * dqk_pad; e += 256) {
            int rr = e / dqk_pad, d = e % dqk_pad;
            float x = 0.f;
            if (i0 + rr < s.lq && d < p.dim_qk) x = to_float(q[((s.q_start + i0 + rr) * p.heads_q + h) * (int64_t)p.dim_qk + d]);
            Qs[e] = x;
        }
        float oacc[32];
#pragma unroll
        for (int x = 0; x < 32; x++) oacc[x] = 0.f;
        const int i = i0 + r;
        const int64_t ti = (p.timestamps && i < s.lq && i + s.delta >= 0) ? p.timestamps[s.k_start + i + s.delta] : 0;

        for (int k0 = 0; k0 < kend; k0 += GBN) {
            float sacc[4] = {0.f, 0.f, 0.f, 0.f};
            for (int d0 = 0; d0 < p.dim_qk; d0 += GDC) {
                __syncthreads();
                {   // K chunk: 4 threads per key row, 16 elements each
                    int row = tid / 4, dseg = (tid % 4) * 16;
                    int j = k0 + row;
                    if (j < kend) {
                        RowSrc src = kv_row<T>(a, s, 0, j, hk, p.dim_qk);
                        for (int e = 0; e < 16; e++) {
                            int d = d0 + dseg + e;
                            KVs[row * GLD + dseg + e] = (d < p.dim_qk) ? row_elem<T>(src, d) : 0.f;
                        }
                    } else {
                        for (int e = 0; e < 16; e++) KVs[row * GLD + dseg + e] = 0.f;
                    }
                }
                __syncthreads();
                const float* qr = Qs + r * dqk_pad + d0;
#pragma unroll 8
                for (int d = 0; d < GDC; d++) {
                    float qv = qr[d];
#pragma unroll
                    for (int jj = 0; jj < 4; jj++) sacc[jj] = fmaf(qv, KVs[(cb + 16 * jj) * GLD + d], sacc[jj]);
                }
            }
            // score -> P
#pragma unroll
            for (int jj = 0; jj < 4; jj++) {
                const int c = cb + 16 * jj;
                const int j = k0 + c;
                float pv = 0.f;
                if (i < s.lq && j < kend) {
                    float bias = 0.f;
                    const bool in_attr = i < p.max_seq_len_q && j < p.max_seq_len_k;
                    const int64_t bm = (bh * p.max_seq_len_q + i) * (int64_t)p.max_seq_len_k + j;
                    if (p.attn_bias && in_attr) bias += to_float(reinterpret_cast<const T*>(p.attn_bias)[bm]);
                    if (p.pos_table) {
                        int idx = (p.max_seq_len_k - 1) + j - (i + s.delta);
                        if (idx >= 0 && idx < 2 * p.max_seq_len_k - 1) bias += p.pos_table[idx];
                    }
                    if (p.ts_table) {
                        float x = abs_dt_as_float(ti, p.timestamps[s.k_start + j]);
                        bias += p.ts_table[ts_bucket(p.ts_bounds, p.num_buckets, x)];
                    }
                    float m = 1.f;
                    if (is_tril) m = builtin_visible(s, p.target_group_size, i, j) ? 1.f : 0.f;
                    else if (p.mask_type == HSTU_MASK_CUSTOM) m = in_attr ? to_float(reinterpret_cast<const T*>(p.mask)[bm]) : 0.f;
                    float x = p.alpha * (sacc[jj] + bias);
                    float sg = 1.0f / (1.0f + expf(-x));
                    pv = x * sg;
                    pv *= p.silu_scale * m;
                    pv = to_float(from_float<T>(pv));
                }
                Ps[r * GLD + c] = pv;
            }
            // O += P V, one head-dim chunk at a time
#pragma unroll
            for (int ch = 0; ch < 8; ch++) {
                const int dv0 = ch * GDC;
                if (dv0 < p.dim_v) {
                    __syncthreads();
                    {
                        int row = tid / 4, dseg = (tid % 4) * 16;
                        int j = k0 + row;
                        if (j < kend) {
                            RowSrc src = kv_row<T>(a, s, 1, j, hk, p.dim_v);
                            for (int e = 0; e < 16; e++) {
                                int d = dv0 + dseg + e;
                                KVs[row * GLD + dseg + e] = (d < p.dim_v) ? row_elem<T>(src, d) : 0.f;
                            }
                        } else {
                            for (int e = 0; e < 16; e++) KVs[row * GLD + dseg + e] = 0.f;
                        }
                    }
                    __syncthreads();
                    const float* pr = Ps + r * GLD;
#pragma unroll 8
                    for (int kk = 0; kk < GBN; kk++) {
                        float pvv = pr[kk];
#pragma unroll
                        for (int jj = 0; jj < 4; jj++)
                            oacc[ch * 4 + jj] = fmaf(pvv, KVs[kk * GLD + cb + 16 * jj], oacc[ch * 4 + jj]);
                    }
                }
            }
        }
        if (i < s.lq) {
#pragma unroll
            for (int ch = 0; ch < 8; ch++) {
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    int d = ch * GDC + cb + 16 * jj;
                    if (d < p.dim_v) out[((s.q_start + i) * p.heads_q + h) * (int64_t)p.dim_v + d] = from_float<OT>(oacc[ch * 4 + jj]);
                }
            }
        }
        __syncthreads();
    }

    // rows past the last offset are defined to be zero (the reference zero-fills its output:
    // hstu_jagged.cpp:56-59); normally there are none
    if (p.seq_offset_q) {
        const int is64 = p.index_type == HSTU_I64;
        int64_t tail = ld_idx(p.seq_offset_q, p.batch, is64);
        if (tail < p.total_q) {
            int64_t n = (p.total_q - tail) * p.heads_q * (int64_t)p.dim_v;
            int64_t nblk = (int64_t)gridDim.x * gridDim.y * gridDim.z;
            int64_t blk = ((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
            OT* o = out + tail * p.heads_q * (int64_t)p.dim_v;
            for (int64_t e = blk * 256 + tid; e < n; e += nblk * 256) o[e] = from_float<OT>(0.f);
        }
    }
}

hipError_t launch_generic(const KArgs& a, hipStream_t stream) {
    const hstu_fwd_params& p = a.p;
    int tiles = (p.max_seq_len_q + GBM - 1) / GBM;
    dim3 grid(tiles, p.heads_q, p.batch);
    int dqk_pad = (p.dim_qk + GDC - 1) / GDC * GDC;
    size_t lds = sizeof(float) * (GBM * dqk_pad + GBN * GLD + GBM * GLD);
    switch (p.dtype) {
        case HSTU_F32: hipLaunchKernelGGL(hstu_generic_kernel<float>, grid, dim3(256), lds, stream, a); break;
        case HSTU_F16: hipLaunchKernelGGL(hstu_generic_kernel<_Float16>, grid, dim3(256), lds, stream, a); break;
        case HSTU_BF16: hipLaunchKernelGGL(hstu_generic_kernel<__bf16>, grid, dim3(256), lds, stream, a); break;
        case HSTU_FP8_E4M3: hipLaunchKernelGGL(hstu_generic_kernel<fp8e4>, grid, dim3(256), lds, stream, a); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace hstu
