// Device-side helpers shared by every HSTU forward kernel: sequence geometry, the built-in mask
// predicate, bias gathers and the K/V row lookup (plain or paged, optionally fp8).
#pragma once
#include "hstu_internal.h"

namespace hstu {

typedef __attribute__((ext_vector_type(2))) float f32x2;

__device__ __forceinline__ int64_t ld_idx(const void* ptr, int64_t i, int is64) {
    return is64 ? reinterpret_cast<const int64_t*>(ptr)[i] : (int64_t) reinterpret_cast<const int32_t*>(ptr)[i];
}

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(_Float16 x) { return (float)x; }
__device__ __forceinline__ float to_float(__bf16 x) { return (float)x; }
template <typename T> __device__ __forceinline__ T from_float(float x) { return (T)x; }

// float8_e4m3fn element of q / k / v / mask / attn_bias (the reference's fp8 path: hstu_jagged.cpp:53-54): scores and
// sums stay in fp32, P is rounded to e4m3 (to nearest even) before P*V, the output is fp16.
struct fp8e4 { uint8_t v; };
__device__ __forceinline__ float to_float(fp8e4 x) {
    f32x2 r = __builtin_amdgcn_cvt_pk_f32_fp8((int)x.v, false);
    return r[0];
}
template <> __device__ __forceinline__ fp8e4 from_float<fp8e4>(float x) {
    fp8e4 r;
    r.v = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(x, 0.f, 0, false) & 0xff);
    return r;
}
// element type of `out` for inputs of type T
template <typename T> struct OutOf { typedef T type; };
template <> struct OutOf<fp8e4> { typedef _Float16 type; };

// Geometry of one sequence.  Q row i sits at K position i + delta.
struct Seq {
    int64_t q_start;   // first row of the sequence in q / out
    int64_t k_start;   // first row in k / v (jagged, dense) -- unused for paged history columns
    int64_t cand_row;  // paged: input k/v row holding K column hist_k
    int64_t page0;     // paged: first entry of this user in page_ids
    int32_t lq, lk, delta;
    int32_t ctx, tgt;
    int32_t hist_q, hist_k;  // lq - tgt, lk - tgt
};

__device__ __forceinline__ Seq load_seq(const KArgs& a, int b) {
    const hstu_fwd_params& p = a.p;
    Seq s;
    const int is64 = p.index_type == HSTU_I64;
    if (p.seq_offset_q) {
        int64_t q0 = ld_idx(p.seq_offset_q, b, is64), q1 = ld_idx(p.seq_offset_q, b + 1, is64);
        int64_t k0 = ld_idx(p.seq_offset_k, b, is64), k1 = ld_idx(p.seq_offset_k, b + 1, is64);
        s.q_start = q0; s.lq = (int32_t)(q1 - q0);
        s.k_start = k0; s.lk = (int32_t)(k1 - k0);
    } else {
        s.q_start = (int64_t)b * p.max_seq_len_q; s.lq = p.max_seq_len_q;
        s.k_start = (int64_t)b * p.max_seq_len_k; s.lk = p.max_seq_len_k;
    }
    s.delta = s.lk - s.lq;
    s.ctx = p.num_context ? (int32_t)ld_idx(p.num_context, b, is64) : 0;
    s.tgt = p.num_target ? (int32_t)ld_idx(p.num_target, b, is64) : 0;
    s.hist_q = s.lq - s.tgt;
    s.hist_k = s.lk - s.tgt;
    s.cand_row = s.q_start + s.hist_q;
    s.page0 = (a.op == OP_PAGED) ? ld_idx(p.page_offsets, b, is64) : 0;
    return s;
}

// Built-in mask (mask_type 0): causal with delta, context rows, target groups.
// Reference: hstu_dense_causal_mask.h:63-117,204-237; test_target_mask.py:272-288.
__device__ __forceinline__ bool builtin_visible(const Seq& s, int tgs, int i, int j) {
    if (s.ctx > 0 && i < s.ctx && j < s.hist_k) return true;
    if (j > i + s.delta) return false;
    if (tgs > 0 && s.tgt > 0 && i >= s.hist_q && j >= s.hist_k) {
        int left = s.hist_k + ((i - s.hist_q) / tgs) * tgs;
        if (j < left) return false;
    }
    return true;
}

// Exclusive upper bound of the K columns any row of [i0, i1) can see.
__device__ __forceinline__ int k_extent(const KArgs& a, const Seq& s, int i0, int i1) {
    if (a.p.mask_type != HSTU_MASK_TRIL) return s.lk;
    int e = i1 + s.delta;
    if (s.ctx > 0 && i0 < s.ctx && s.hist_k > e) e = s.hist_k;
    return e < 0 ? 0 : (e > s.lk ? s.lk : e);
}

// bucket with bounds[b] <= x < bounds[b+1]; bounds has nb+2 entries, bounds[0]=0, bounds[nb+1]=+inf
__device__ __forceinline__ int ts_bucket(const float* bounds, int nb, float x) {
    int lo = 0, hi = nb;  // answer in [lo, hi]
    while (lo < hi) {
        int mid = (lo + hi + 1) >> 1;
        if (x >= bounds[mid]) lo = mid; else hi = mid - 1;
    }
    return lo;
}

__device__ __forceinline__ float abs_dt_as_float(int64_t ti, int64_t tj) {
    int64_t d = ti - tj;
    if (d < 0) d = -d;
    return (float)d;
}

__device__ __forceinline__ float fp8_e4m3_to_float(uint8_t v) {
    f32x2 r = __builtin_amdgcn_cvt_pk_f32_fp8((int)v, false);
    return r[0];
}

}  // namespace hstu
