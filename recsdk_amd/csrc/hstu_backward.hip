// Backward of the jagged HSTU attention in plain fp32 FMA arithmetic (every dtype, head dim, mask and dense bias the
// reference's backward takes).  Definition (golden: build/presmoke/hstu/hstu_common.py:387-476):
//     x  = alpha * (Q K^T + bias)        P  = silu(x) * silu_scale * mask
//     dS = (dO V^T) * silu_scale * mask * sigmoid(x) * (1 + x * (1 - sigmoid(x))) * alpha
//     dQ = dS K     dK = dS^T Q     dV = P^T dO     dBias = dS
// Two kernels, so that every gradient element has one producing workgroup (no atomics, fixed summation order):
//   hstu_bwd_dq_kernel   one workgroup per 16 Q rows of a (sequence, head): recomputes x and dO V^T over the K tiles,
//                        writes dBias and accumulates dQ
//   hstu_bwd_dkv_kernel  one workgroup per 16 K rows of a (sequence, K/V head): the same scores transposed, over the
//                        Q tiles of every query head that shares the K/V head; accumulates dK and dV
// P and dS are rounded to the I/O dtype before the second GEMMs, like P in the forward.
#include "hstu_device.h"

namespace hstu {

constexpr int BBM = 16;   // rows owned by a workgroup (Q rows or K rows)
constexpr int BBN = 64;   // rows of the other side per step
constexpr int BDC = 64;   // head-dim chunk staged in LDS
constexpr int BLD = 65;   // padded leading dimension of the LDS tiles

struct Score {
    float p;    // silu(x) * silu_scale * mask
    float ds;   // d loss / d (Q K^T + bias)
};

// score math of one (Q row i, K column j); s = Q K^T, g = dO V^T.  The caller has checked i < lq, j < lk.
template <typename T>
__device__ __forceinline__ Score score_grad(const KArgs& a, const Seq& sq, int b, int h, int i, int j, float s, float g) {
    const hstu_fwd_params& p = a.p;
    const bool in_attr = i < p.max_seq_len_q && j < p.max_seq_len_k;
    const int64_t bm = ((((int64_t)b * p.heads_q + h) * p.max_seq_len_q + i) * (int64_t)p.max_seq_len_k) + j;
    float bias = 0.f;
    if (p.attn_bias && in_attr) bias = to_float(reinterpret_cast<const T*>(p.attn_bias)[bm]);
    float m = 1.f;
    if (p.mask_type == HSTU_MASK_TRIL) m = builtin_visible(sq, p.target_group_size, i, j) ? 1.f : 0.f;
    else if (p.mask_type == HSTU_MASK_CUSTOM) m = in_attr ? to_float(reinterpret_cast<const T*>(p.mask)[bm]) : 0.f;
    const float x = p.alpha * (s + bias);
    const float sg = 1.0f / (1.0f + expf(-x));
    Score r;
    r.p = to_float(from_float<T>(x * sg * p.silu_scale * m));
    r.ds = to_float(from_float<T>(g * p.silu_scale * m * sg * (1.0f + x * (1.0f - sg)) * p.alpha));
    return r;
}

// rows [row0, row0 + nrows) x dims [d0, d0 + BDC) of a [rows, heads, dim] tensor into tile[nrows][BLD] (zero padded);
// 256 threads, 4 per row for 64 rows or 16 per row for 16 rows
template <typename T>
__device__ __forceinline__ void stage_chunk(float* tile, const T* base, int64_t first_row, int valid_rows, int heads, int head,
                                            int dim, int d0, int nrows, int tid) {
    const int per_row = 256 / nrows, span = BDC / per_row;
    const int row = tid / per_row, dseg = (tid % per_row) * span;
    const bool ok = row < valid_rows;
    const T* src = base + ((first_row + (ok ? row : 0)) * heads + head) * (int64_t)dim;
    for (int e = 0; e < span; e++) {
        const int d = d0 + dseg + e;
        tile[row * BLD + dseg + e] = (ok && d < dim) ? to_float(src[d]) : 0.f;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void hstu_bwd_dq_kernel(const BArgs a) {
    const hstu_fwd_params& p = a.f.p;
    extern __shared__ float smem[];
    const int dqk_pad = (p.dim_qk + BDC - 1) / BDC * BDC, dv_pad = (p.dim_v + BDC - 1) / BDC * BDC;
    float* Qs = smem;                    // [BBM][dqk_pad]
    float* Gs = Qs + BBM * dqk_pad;      // [BBM][dv_pad]   upstream gradient rows
    float* KVs = Gs + BBM * dv_pad;      // [BBN][BLD]
    float* Ds = KVs + BBN * BLD;         // [BBM][BLD]      dS

    const int tid = threadIdx.x;
    const int b = blockIdx.z, h = blockIdx.y, hk = h / a.f.head_ratio;
    const Seq s = load_seq(a.f, b);
    const T* q = reinterpret_cast<const T*>(p.q);
    const T* k = reinterpret_cast<const T*>(p.k);
    const T* v = reinterpret_cast<const T*>(p.v);
    const T* go = reinterpret_cast<const T*>(a.grad_out);
    T* dq = reinterpret_cast<T*>(a.grad_q);
    T* dbias = reinterpret_cast<T*>(a.grad_bias);
    const int r = tid / 16, cb = tid % 16;
    // with a bias gradient the whole [max_q, max_k] plane of this (sequence, head) is written, zeros included
    const int row_end = dbias ? max(s.lq, p.max_seq_len_q) : s.lq;

    for (int tile = blockIdx.x; tile * BBM < row_end; tile += gridDim.x) {
        const int i0 = tile * BBM;
        const int i1 = min(i0 + BBM, s.lq);
        const int kend = (i0 < s.lq && s.lk > 0) ? k_extent(a.f, s, i0, i1) : 0;
        const int col_end = dbias ? max(kend, p.max_seq_len_k) : kend;
        __syncthreads();
        for (int e = tid; e < BBM * dqk_pad; e += 256) {
            const int rr = e / dqk_pad, d = e % dqk_pad;
            Qs[e] = (i0 + rr < s.lq && d < p.dim_qk) ? to_float(q[((s.q_start + i0 + rr) * p.heads_q + h) * (int64_t)p.dim_qk + d]) : 0.f;
        }
        for (int e = tid; e < BBM * dv_pad; e += 256) {
            const int rr = e / dv_pad, d = e % dv_pad;
            Gs[e] = (i0 + rr < s.lq && d < p.dim_v) ? to_float(go[((s.q_start + i0 + rr) * p.heads_q + h) * (int64_t)p.dim_v + d]) : 0.f;
        }
        float acc[32];
#pragma unroll
        for (int x = 0; x < 32; x++) acc[x] = 0.f;
        const int i = i0 + r;

        for (int k0 = 0; k0 < col_end; k0 += BBN) {
            const bool work = k0 < kend;   // else: only zeros of the bias gradient
            float sacc[4] = {0.f, 0.f, 0.f, 0.f}, gacc[4] = {0.f, 0.f, 0.f, 0.f};
            if (work) {
                for (int d0 = 0; d0 < p.dim_qk; d0 += BDC) {
                    __syncthreads();
                    stage_chunk<T>(KVs, k, s.k_start + k0, kend - k0, p.heads_k, hk, p.dim_qk, d0, BBN, tid);
                    __syncthreads();
                    const float* qr = Qs + r * dqk_pad + d0;
#pragma unroll 8
                    for (int d = 0; d < BDC; d++) {
                        const float x = qr[d];
#pragma unroll
                        for (int jj = 0; jj < 4; jj++) sacc[jj] = fmaf(x, KVs[(cb + 16 * jj) * BLD + d], sacc[jj]);
                    }
                }
                for (int d0 = 0; d0 < p.dim_v; d0 += BDC) {
                    __syncthreads();
                    stage_chunk<T>(KVs, v, s.k_start + k0, kend - k0, p.heads_k, hk, p.dim_v, d0, BBN, tid);
                    __syncthreads();
                    const float* gr = Gs + r * dv_pad + d0;
#pragma unroll 8
                    for (int d = 0; d < BDC; d++) {
                        const float x = gr[d];
#pragma unroll
                        for (int jj = 0; jj < 4; jj++) gacc[jj] = fmaf(x, KVs[(cb + 16 * jj) * BLD + d], gacc[jj]);
                    }
                }
            }
#pragma unroll
            for (int jj = 0; jj < 4; jj++) {
                const int c = cb + 16 * jj, j = k0 + c;
                float ds = 0.f;
                if (work && i < s.lq && j < kend) ds = score_grad<T>(a.f, s, b, h, i, j, sacc[jj], gacc[jj]).ds;
                Ds[r * BLD + c] = ds;
                if (dbias && i < p.max_seq_len_q && j < p.max_seq_len_k)
                    dbias[((((int64_t)b * p.heads_q + h) * p.max_seq_len_q + i) * (int64_t)p.max_seq_len_k) + j] = from_float<T>(ds);
            }
            if (!work) continue;
            // dQ += dS K, one head-dim chunk at a time
#pragma unroll
            for (int ch = 0; ch < 8; ch++) {
                const int d0 = ch * BDC;
                if (d0 < p.dim_qk) {
                    __syncthreads();
                    stage_chunk<T>(KVs, k, s.k_start + k0, kend - k0, p.heads_k, hk, p.dim_qk, d0, BBN, tid);
                    __syncthreads();
                    const float* dr = Ds + r * BLD;
#pragma unroll 8
                    for (int kk = 0; kk < BBN; kk++) {
                        const float x = dr[kk];
#pragma unroll
                        for (int jj = 0; jj < 4; jj++) acc[ch * 4 + jj] = fmaf(x, KVs[kk * BLD + cb + 16 * jj], acc[ch * 4 + jj]);
                    }
                }
            }
        }
        if (i < s.lq) {
#pragma unroll
            for (int ch = 0; ch < 8; ch++) {
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    const int d = ch * BDC + cb + 16 * jj;
                    if (d < p.dim_qk) dq[((s.q_start + i) * p.heads_q + h) * (int64_t)p.dim_qk + d] = from_float<T>(acc[ch * 4 + jj]);
                }
            }
        }
    }

    // rows past the last offset carry no gradient
    const int is64 = p.index_type == HSTU_I64;
    const int64_t tail = p.seq_offset_q ? ld_idx(p.seq_offset_q, p.batch, is64) : p.total_q;
    if (tail < p.total_q) {
        const int64_t n = (p.total_q - tail) * p.heads_q * (int64_t)p.dim_qk;
        const int64_t nblk = (int64_t)gridDim.x * gridDim.y * gridDim.z;
        const int64_t blk = ((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
        T* o = dq + tail * p.heads_q * (int64_t)p.dim_qk;
        for (int64_t e = blk * 256 + tid; e < n; e += nblk * 256) o[e] = from_float<T>(0.f);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void hstu_bwd_dkv_kernel(const BArgs a) {
    const hstu_fwd_params& p = a.f.p;
    extern __shared__ float smem[];
    const int dqk_pad = (p.dim_qk + BDC - 1) / BDC * BDC, dv_pad = (p.dim_v + BDC - 1) / BDC * BDC;
    float* Ks = smem;                    // [BBM][dqk_pad]
    float* Vs = Ks + BBM * dqk_pad;      // [BBM][dv_pad]
    float* QGs = Vs + BBM * dv_pad;      // [BBN][BLD]   Q rows or upstream gradient rows
    float* Pt = QGs + BBN * BLD;         // [BBM][BLD]   P^T
    float* St = Pt + BBM * BLD;          // [BBM][BLD]   dS^T

    const int tid = threadIdx.x;
    const int b = blockIdx.z, hk = blockIdx.y;
    const Seq s = load_seq(a.f, b);
    const T* q = reinterpret_cast<const T*>(p.q);
    const T* k = reinterpret_cast<const T*>(p.k);
    const T* v = reinterpret_cast<const T*>(p.v);
    const T* go = reinterpret_cast<const T*>(a.grad_out);
    T* dk = reinterpret_cast<T*>(a.grad_k);
    T* dv = reinterpret_cast<T*>(a.grad_v);
    const int r = tid / 16, cb = tid % 16;

    for (int tile = blockIdx.x; tile * BBM < s.lk; tile += gridDim.x) {
        const int j0 = tile * BBM;
        __syncthreads();
        for (int e = tid; e < BBM * dqk_pad; e += 256) {
            const int rr = e / dqk_pad, d = e % dqk_pad;
            Ks[e] = (j0 + rr < s.lk && d < p.dim_qk) ? to_float(k[((s.k_start + j0 + rr) * p.heads_k + hk) * (int64_t)p.dim_qk + d]) : 0.f;
        }
        for (int e = tid; e < BBM * dv_pad; e += 256) {
            const int rr = e / dv_pad, d = e % dv_pad;
            Vs[e] = (j0 + rr < s.lk && d < p.dim_v) ? to_float(v[((s.k_start + j0 + rr) * p.heads_k + hk) * (int64_t)p.dim_v + d]) : 0.f;
        }
        float kacc[32], vacc[32];
#pragma unroll
        for (int x = 0; x < 32; x++) { kacc[x] = 0.f; vacc[x] = 0.f; }
        const int j = j0 + r;
        // first Q row that can see one of these K rows: causal -> j <= i + delta; context rows see the whole history
        int istart = 0;
        if (p.mask_type == HSTU_MASK_TRIL && s.ctx <= 0) istart = max(0, j0 - s.delta) / BBN * BBN;

        for (int hq = 0; hq < a.f.head_ratio; hq++) {
            const int h = hk * a.f.head_ratio + hq;
            for (int i0 = istart; i0 < s.lq; i0 += BBN) {
                float sacc[4] = {0.f, 0.f, 0.f, 0.f}, gacc[4] = {0.f, 0.f, 0.f, 0.f};
                for (int d0 = 0; d0 < p.dim_qk; d0 += BDC) {
                    __syncthreads();
                    stage_chunk<T>(QGs, q, s.q_start + i0, s.lq - i0, p.heads_q, h, p.dim_qk, d0, BBN, tid);
                    __syncthreads();
                    const float* kr = Ks + r * dqk_pad + d0;
#pragma unroll 8
                    for (int d = 0; d < BDC; d++) {
                        const float x = kr[d];
#pragma unroll
                        for (int jj = 0; jj < 4; jj++) sacc[jj] = fmaf(x, QGs[(cb + 16 * jj) * BLD + d], sacc[jj]);
                    }
                }
                for (int d0 = 0; d0 < p.dim_v; d0 += BDC) {
                    __syncthreads();
                    stage_chunk<T>(QGs, go, s.q_start + i0, s.lq - i0, p.heads_q, h, p.dim_v, d0, BBN, tid);
                    __syncthreads();
                    const float* vr = Vs + r * dv_pad + d0;
#pragma unroll 8
                    for (int d = 0; d < BDC; d++) {
                        const float x = vr[d];
#pragma unroll
                        for (int jj = 0; jj < 4; jj++) gacc[jj] = fmaf(x, QGs[(cb + 16 * jj) * BLD + d], gacc[jj]);
                    }
                }
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    const int c = cb + 16 * jj, i = i0 + c;
                    Score sc = {0.f, 0.f};
                    if (i < s.lq && j < s.lk) sc = score_grad<T>(a.f, s, b, h, i, j, sacc[jj], gacc[jj]);
                    Pt[r * BLD + c] = sc.p;
                    St[r * BLD + c] = sc.ds;
                }
                // dV += P^T dO and dK += dS^T Q, one head-dim chunk at a time
#pragma unroll
                for (int ch = 0; ch < 8; ch++) {
                    const int d0 = ch * BDC;
                    if (d0 < p.dim_v) {
                        __syncthreads();
                        stage_chunk<T>(QGs, go, s.q_start + i0, s.lq - i0, p.heads_q, h, p.dim_v, d0, BBN, tid);
                        __syncthreads();
                        const float* pr = Pt + r * BLD;
#pragma unroll 8
                        for (int kk = 0; kk < BBN; kk++) {
                            const float x = pr[kk];
#pragma unroll
                            for (int jj = 0; jj < 4; jj++) vacc[ch * 4 + jj] = fmaf(x, QGs[kk * BLD + cb + 16 * jj], vacc[ch * 4 + jj]);
                        }
                    }
                    if (d0 < p.dim_qk) {
                        __syncthreads();
                        stage_chunk<T>(QGs, q, s.q_start + i0, s.lq - i0, p.heads_q, h, p.dim_qk, d0, BBN, tid);
                        __syncthreads();
                        const float* sr = St + r * BLD;
#pragma unroll 8
                        for (int kk = 0; kk < BBN; kk++) {
                            const float x = sr[kk];
#pragma unroll
                            for (int jj = 0; jj < 4; jj++) kacc[ch * 4 + jj] = fmaf(x, QGs[kk * BLD + cb + 16 * jj], kacc[ch * 4 + jj]);
                        }
                    }
                }
            }
        }
        if (j < s.lk) {
#pragma unroll
            for (int ch = 0; ch < 8; ch++) {
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    const int d = ch * BDC + cb + 16 * jj;
                    if (d < p.dim_qk) dk[((s.k_start + j) * p.heads_k + hk) * (int64_t)p.dim_qk + d] = from_float<T>(kacc[ch * 4 + jj]);
                    if (d < p.dim_v) dv[((s.k_start + j) * p.heads_k + hk) * (int64_t)p.dim_v + d] = from_float<T>(vacc[ch * 4 + jj]);
                }
            }
        }
    }

    // rows past the last offset carry no gradient
    const int is64 = p.index_type == HSTU_I64;
    const int64_t tail = p.seq_offset_k ? ld_idx(p.seq_offset_k, p.batch, is64) : p.total_k;
    if (tail < p.total_k) {
        const int64_t nblk = (int64_t)gridDim.x * gridDim.y * gridDim.z;
        const int64_t blk = ((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
        const int64_t nk = (p.total_k - tail) * p.heads_k * (int64_t)p.dim_qk, nv = (p.total_k - tail) * p.heads_k * (int64_t)p.dim_v;
        T* ok = dk + tail * p.heads_k * (int64_t)p.dim_qk;
        T* ov = dv + tail * p.heads_k * (int64_t)p.dim_v;
        for (int64_t e = blk * 256 + tid; e < nk; e += nblk * 256) ok[e] = from_float<T>(0.f);
        for (int64_t e = blk * 256 + tid; e < nv; e += nblk * 256) ov[e] = from_float<T>(0.f);
    }
}

template <typename T>
static hipError_t launch_backward_t(const BArgs& a, hipStream_t stream) {
    const hstu_fwd_params& p = a.f.p;
    const int dqk_pad = (p.dim_qk + BDC - 1) / BDC * BDC, dv_pad = (p.dim_v + BDC - 1) / BDC * BDC;
    const size_t lds_q = sizeof(float) * (BBM * dqk_pad + BBM * dv_pad + BBN * BLD + BBM * BLD);
    const size_t lds_kv = sizeof(float) * (BBM * dqk_pad + BBM * dv_pad + BBN * BLD + 2 * BBM * BLD);
    hipError_t e;
    if (lds_kv > 64 * 1024) {   // the default limit of dynamic LDS
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(hstu_bwd_dq_kernel<T>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_q);
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(hstu_bwd_dkv_kernel<T>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_kv);
        if (e != hipSuccess) return e;
    }
    const int qtiles = (p.max_seq_len_q + BBM - 1) / BBM, ktiles = (p.max_seq_len_k + BBM - 1) / BBM;
    hipLaunchKernelGGL(hstu_bwd_dq_kernel<T>, dim3(qtiles, p.heads_q, p.batch), dim3(256), lds_q, stream, a);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(hstu_bwd_dkv_kernel<T>, dim3(ktiles, p.heads_k, p.batch), dim3(256), lds_kv, stream, a);
    return hipGetLastError();
}

hipError_t launch_backward_generic(const BArgs& a, hipStream_t stream) {
    switch (a.f.p.dtype) {
        case HSTU_F32: return launch_backward_t<float>(a, stream);
        case HSTU_F16: return launch_backward_t<_Float16>(a, stream);
        case HSTU_BF16: return launch_backward_t<__bf16>(a, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace hstu
