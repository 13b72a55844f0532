// Standalone producers of the dense attention-bias tensors and the gradient of the time-bucket weights.  All three are
// bounded by HBM: the outputs (or, for the gradient, the input) are (2s)^2 elements per (layer, user), everything else
// is tiny.
//   hstu_rab_time_kernel      one lane = 4 consecutive columns j of one (user, row i): 4 bucket searches, then per layer
//                             two 16-byte stores (rows 2i and 2i+1, columns 2j..2j+7), the 2x2 repeat of the reference's
//                             wrapper fused into the store
//   hstu_rab_time_bwd_kernel  the same mapping backwards: 2x2 gradient elements summed per (i, j), accumulated per bucket
//                             in an LDS table, one global atomic per bucket and workgroup
//   hstu_rab_pos_kernel       one lane = 8 consecutive columns of one (user, row)
// Definitions: cust_op/test/relative_attn_bias/torch/utils.py:99-163; wrappers
// cust_op/framework/torch_plugin/torch_library/relative_attn_bias/relative_attn_bias_{time,pos}.cpp.
#include "hstu_device.h"
#include "../../include/hstu_bias.h"

namespace hstu {

constexpr int RAB_NT = 256;
constexpr int RAB_JPT = 4;   // columns j per lane

template <typename I>
__device__ __forceinline__ float abs_diff_f32(I a, I b) {
    int64_t d = (int64_t)a - (int64_t)b;
    if (d < 0) d = -d;
    return (float)d;
}

// Bucket of x from the bounds table: a first guess from the hardware log2 (within one of the answer), settled by
// comparisons with the table, so the id is the table's whatever the guess was.  inv = ln 2 / divisor, or 0: search only.
__device__ __forceinline__ int bucket_of(const float* bounds, int nb, float x, float inv) {
    if (inv > 0.f) {
        int e = min((int)(__log2f(fmaxf(x, 1.0f)) * inv), nb);
        if (x < bounds[e]) e--;
        else if (x >= bounds[e + 1]) e++;
        if (e >= 0 && e <= nb && x >= bounds[e] && x < bounds[e + 1]) return e;
    }
    return ts_bucket(bounds, nb, x);
}

// grid: x = (b * s + i) * column groups + column group of RAB_NT * RAB_JPT.  The table sits in LDS transposed,
// [bucket][layer], so that one bucket's values for all layers are one or a few 16-byte reads.
template <typename T, typename I>
__global__ __launch_bounds__(RAB_NT) void hstu_rab_time_kernel(const hstu_rab_time_params p) {
    constexpr int LPV = 16 / sizeof(T);   // layers per 16-byte read
    constexpr int MAXL = (HSTU_RAB_MAX_LAYERS + LPV - 1) / LPV * LPV;
    typedef __attribute__((ext_vector_type(4))) unsigned int u4;
    __shared__ float bounds[HSTU_RAB_MAX_BUCKETS + 1];
    __shared__ __attribute__((aligned(16))) T wtab[HSTU_RAB_MAX_BUCKETS * MAXL];
    const int W = p.weight_cols, s = p.seq_len, nl = p.num_layers;
    const int lpad = (nl + LPV - 1) / LPV * LPV;
    for (int k = threadIdx.x; k <= W; k += RAB_NT) bounds[k] = p.bucket_bounds[k];
    for (int k = threadIdx.x; k < nl * W; k += RAB_NT) wtab[(k % W) * lpad + k / W] = reinterpret_cast<const T*>(p.weights)[k];
    __syncthreads();
    const unsigned groups = (unsigned)(s + RAB_NT * RAB_JPT - 1) / (RAB_NT * RAB_JPT);
    const unsigned row = blockIdx.x / groups;
    const int b = row / s, i = row % s;
    const int j0 = ((blockIdx.x % groups) * RAB_NT + threadIdx.x) * RAB_JPT;
    if (j0 >= s) return;
    const float inv = p.bucket_divisor > 0.f ? 0.69314718f / p.bucket_divisor : 0.f;
    const I* ts = reinterpret_cast<const I*>(p.timestamps) + (int64_t)b * s;
    const I ti = ts[i];
    int bucket[RAB_JPT];
    // a lane's four timestamps and ids as 16-byte accesses when the rows start on 16-byte boundaries (four accesses of one
    // element per lane would each ask for every cache line of the wave's stretch)
    constexpr int NI = RAB_JPT * sizeof(I) / 16;
    const bool whole = j0 + RAB_JPT <= s && ((int64_t)s * sizeof(I)) % 16 == 0;
    I tj[RAB_JPT];
    if (whole && (reinterpret_cast<uintptr_t>(p.timestamps) & 15) == 0) {
#pragma unroll
        for (int q = 0; q < NI; q++) reinterpret_cast<u4*>(tj)[q] = reinterpret_cast<const u4*>(ts + j0)[q];
    } else {
#pragma unroll
        for (int k = 0; k < RAB_JPT; k++) tj[k] = ts[min(j0 + k, s - 1)];
    }
#pragma unroll
    for (int k = 0; k < RAB_JPT; k++) bucket[k] = bucket_of(bounds, W - 1, abs_diff_f32<I>(ti, tj[k]), inv);
    if (p.bucket_ts_out) {
        I* bo = reinterpret_cast<I*>(p.bucket_ts_out) + ((int64_t)b * s + i) * s;
        if (whole && (reinterpret_cast<uintptr_t>(p.bucket_ts_out) & 15) == 0) {
            I bi[RAB_JPT];
#pragma unroll
            for (int k = 0; k < RAB_JPT; k++) bi[k] = (I)bucket[k];
#pragma unroll
            for (int q = 0; q < NI; q++) reinterpret_cast<u4*>(bo + j0)[q] = reinterpret_cast<const u4*>(bi)[q];
        } else {
#pragma unroll
            for (int k = 0; k < RAB_JPT; k++)
                if (j0 + k < s) bo[j0 + k] = (I)bucket[k];
        }
    }
    T* out = reinterpret_cast<T*>(p.rab_time_out);
    const int64_t s2 = 2 * (int64_t)s;
    const bool wide = j0 + RAB_JPT <= s && (s2 * sizeof(T)) % 16 == 0;   // whole group, rows start on 16-byte boundaries
    for (int n0 = 0; n0 < nl; n0 += LPV) {
        T v[RAB_JPT][LPV];
#pragma unroll
        for (int k = 0; k < RAB_JPT; k++) *reinterpret_cast<u4*>(v[k]) = *reinterpret_cast<const u4*>(wtab + bucket[k] * lpad + n0);
#pragma unroll
        for (int l = 0; l < LPV; l++) {
            const int n = n0 + l;
            if (n >= nl) break;
            T* orow = out + (((int64_t)n * p.batch + b) * s2 + 2 * i) * s2 + 2 * j0;
            if (wide) {
                T pk[2 * RAB_JPT];
#pragma unroll
                for (int k = 0; k < RAB_JPT; k++) pk[2 * k] = pk[2 * k + 1] = v[k][l];
                constexpr int NV = 2 * RAB_JPT * sizeof(T) / 16;
                const u4* src = reinterpret_cast<const u4*>(pk);
#pragma unroll
                for (int q = 0; q < NV; q++) {
                    __builtin_nontemporal_store(src[q], reinterpret_cast<u4*>(orow) + q);
                    __builtin_nontemporal_store(src[q], reinterpret_cast<u4*>(orow + s2) + q);
                }
            } else {
#pragma unroll
                for (int k = 0; k < RAB_JPT; k++) {
                    if (j0 + k >= s) break;
                    orow[2 * k] = orow[2 * k + 1] = v[k][l];
                    orow[s2 + 2 * k] = orow[s2 + 2 * k + 1] = v[k][l];
                }
            }
        }
    }
}

// The same for rows whose length is a multiple of 4 (rows of the outputs then start on 16-byte boundaries, but in general
// not on cache lines: 2s = 4600 two-byte columns are 71.9 lines).  A wave's store of 64 x 16 bytes that starts inside a
// line leaves two lines half written for the neighbouring wave to finish, and those partial writes cost the memory 40 %
// of its rate (s = 2304 ran at 5.6 TB/s where s = 2300 ran at 3.9).  So the lanes of a wave are made to cover whole lines
// of every row: a "unit" is what a lane stores (4 columns j = 8 output columns), a workgroup computes the buckets of 256
// units, parks them in LDS (4 ids of one byte), and stores 248 of them per output row, starting `a` units further right,
// where a < 8 is what brings lane 0 of each wave onto a line boundary of THAT row (rows 2i and 2i+1 differ); the
// first `a` units of a row go to the eight spare lanes of the row's first workgroup.
constexpr int RAB_UPW = 248;   // units a workgroup stores per row: a multiple of the units per line
template <typename T, typename I>
__global__ __launch_bounds__(RAB_NT) void hstu_rab_time_lines_kernel(const hstu_rab_time_params p) {
    constexpr int LPV = 16 / sizeof(T);
    constexpr int MAXL = (HSTU_RAB_MAX_LAYERS + LPV - 1) / LPV * LPV;
    typedef __attribute__((ext_vector_type(4))) unsigned int u4;
    __shared__ float bounds[HSTU_RAB_MAX_BUCKETS + 1];
    __shared__ __attribute__((aligned(16))) T wtab[HSTU_RAB_MAX_BUCKETS * MAXL];
    __shared__ unsigned ids[RAB_NT];
    const int W = p.weight_cols, s = p.seq_len, nl = p.num_layers;
    const int lpad = (nl + LPV - 1) / LPV * LPV;
    for (int k = threadIdx.x; k <= W; k += RAB_NT) bounds[k] = p.bucket_bounds[k];
    for (int k = threadIdx.x; k < nl * W; k += RAB_NT) wtab[(k % W) * lpad + k / W] = reinterpret_cast<const T*>(p.weights)[k];
    __syncthreads();
    const int units = s / RAB_JPT;
    const unsigned groups = (unsigned)(units + RAB_UPW - 1) / RAB_UPW;
    const unsigned row = blockIdx.x / groups, grp = blockIdx.x % groups;
    const int b = row / s, i = row % s, tid = threadIdx.x;
    const float inv = p.bucket_divisor > 0.f ? 0.69314718f / p.bucket_divisor : 0.f;
    const I* ts = reinterpret_cast<const I*>(p.timestamps) + (int64_t)b * s;
    {
        const int j0 = (RAB_UPW * (int)grp + tid) * RAB_JPT;
        unsigned packed = 0;
        if (j0 < s) {
            const I ti = ts[i];
#pragma unroll
            for (int k = 0; k < RAB_JPT; k++) packed |= (unsigned)bucket_of(bounds, W - 1, abs_diff_f32<I>(ti, ts[j0 + k]), inv) << (8 * k);
        }
        ids[tid] = packed;
    }
    __syncthreads();
    // which unit this lane stores for a row that starts at address `rowp`, chunks of CB bytes per lane; -1: none
    auto unit_of = [&](uintptr_t rowp, int cb, int& src) __attribute__((always_inline)) -> int {
        const int cpl = 128 / cb;
        const int a = (cpl - (int)((rowp / (unsigned)cb) % (unsigned)cpl)) % cpl;
        int v;
        if (tid < RAB_UPW) { src = tid + a; v = RAB_UPW * (int)grp + src; }
        else { src = tid - RAB_UPW; v = (grp == 0 && src < a) ? src : units; }
        return v < units ? v : -1;
    };
    if (p.bucket_ts_out) {
        I* bo = reinterpret_cast<I*>(p.bucket_ts_out) + ((int64_t)b * s + i) * s;
        int src;
        const int v = unit_of(reinterpret_cast<uintptr_t>(bo), RAB_JPT * sizeof(I), src);
        if (v >= 0) {
            const unsigned pk = ids[src];
            I bi[RAB_JPT];
#pragma unroll
            for (int k = 0; k < RAB_JPT; k++) bi[k] = (I)((pk >> (8 * k)) & 0xffu);
#pragma unroll
            for (int q = 0; q < (int)(RAB_JPT * sizeof(I) / 16); q++) reinterpret_cast<u4*>(bo + (int64_t)v * RAB_JPT)[q] = reinterpret_cast<const u4*>(bi)[q];
        }
    }
    T* out = reinterpret_cast<T*>(p.rab_time_out);
    const int64_t s2 = 2 * (int64_t)s;
#pragma unroll
    for (int rsel = 0; rsel < 2; rsel++) {
        // row 2i + rsel of layer 0; the planes of the other layers are a whole number of lines further on
        T* rowp = out + ((int64_t)b * s2 + 2 * i + rsel) * s2;
        int src;
        const int v = unit_of(reinterpret_cast<uintptr_t>(rowp), 2 * RAB_JPT * sizeof(T), src);
        if (v < 0) continue;
        const unsigned pk = ids[src];
        for (int n0 = 0; n0 < nl; n0 += LPV) {
            T val[RAB_JPT][LPV];
#pragma unroll
            for (int k = 0; k < RAB_JPT; k++) *reinterpret_cast<u4*>(val[k]) = *reinterpret_cast<const u4*>(wtab + ((pk >> (8 * k)) & 0xffu) * lpad + n0);
#pragma unroll
            for (int l = 0; l < LPV; l++) {
                const int n = n0 + l;
                if (n >= nl) break;
                T two[2 * RAB_JPT];
#pragma unroll
                for (int k = 0; k < RAB_JPT; k++) two[2 * k] = two[2 * k + 1] = val[k][l];
                T* dst = rowp + (int64_t)n * p.batch * s2 * s2 + (int64_t)v * (2 * RAB_JPT);
#pragma unroll
                for (int q = 0; q < (int)(2 * RAB_JPT * sizeof(T) / 16); q++) __builtin_nontemporal_store(reinterpret_cast<const u4*>(two)[q], reinterpret_cast<u4*>(dst) + q);
            }
        }
    }
}

// sum of x over the 64 lanes
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
    return x;
}

// A workgroup = one tile (64 * RAB_JPT columns x RAB_ROWS rows i) of one (layer, user); wave w takes rows w, w + 4, ...
// Neighbouring columns mostly share a bucket, so equal neighbours are first merged inside a lane and the lanes of a wave
// that hold one id are then summed across the wave (one LDS atomic per distinct id and wave instead of 64 colliding
// ones).  A workgroup per layer reads the ids again for every layer (a third of the gradient's bytes at fp16 with
// 4-byte ids), so the layers of one tile are numbered to run side by side on one XCD and all but the first find the ids
// in its L2 (484 -> 424 us at 8 layers); a lane's four ids are one 16-byte read (424 -> 337 us: four 4-byte reads
// per lane asked the memory pipeline for every cache line four times).  Several layers per workgroup measured slower
// (620-940 us): the reduction leaves a wave's loads idle, and more workgroups hide that better.  8 / 12 / 16 rows per
// workgroup measure the same, 32 and 64 are 8 % and 30 % slower.
constexpr int RAB_ROWS = 16;
template <typename T, typename I>
__global__ __launch_bounds__(RAB_NT) void hstu_rab_time_bwd_kernel(const hstu_rab_time_bwd_params p) {
    __shared__ float hist[HSTU_RAB_MAX_BUCKETS];
    const int nb = p.num_buckets, s = p.seq_len;
    for (int k = threadIdx.x; k < nb; k += RAB_NT) hist[k] = 0.f;
    __syncthreads();
    // workgroup L runs on XCD L % 8: the layers of one tile of ids are the workgroups L = (hi * layers + n) * 8 + lo of tile
    // hi * 8 + lo, so that they meet in one L2 within a few dispatches and the ids come from HBM once
    const unsigned L = blockIdx.x, nl = (unsigned)p.num_layers;
    const unsigned tile = (L / (8 * nl)) * 8 + L % 8;
    const int n = (int)((L / 8) % nl);
    const unsigned gx = (unsigned)(s + 64 * RAB_JPT - 1) / (64 * RAB_JPT), gy = (unsigned)(s + RAB_ROWS - 1) / RAB_ROWS;
    if (tile >= gx * gy * (unsigned)p.batch) return;   // (the whole workgroup: the padding of the last group of 8 tiles)
    const int b = (int)(tile / (gx * gy));
    const unsigned bx = tile % gx, by = tile / gx % gy;
    const int lane = threadIdx.x & 63;
    const int j0 = (bx * 64 + lane) * RAB_JPT;
    const int64_t s2 = 2 * (int64_t)s;
    const T* g = reinterpret_cast<const T*>(p.grad) + ((int64_t)n * p.batch + b) * s2 * s2;
    const I* bt = reinterpret_cast<const I*>(p.bucket_ts) + (int64_t)b * s * s;
    const bool wide = j0 + RAB_JPT <= s && (s2 * sizeof(T)) % 16 == 0;
    const bool wide_id = j0 + RAB_JPT <= s && ((int64_t)s * sizeof(I)) % 16 == 0 && (reinterpret_cast<uintptr_t>(p.bucket_ts) & 15) == 0;
    const int i_end = min((int)(by + 1) * RAB_ROWS, s);
    for (int i = by * RAB_ROWS + (threadIdx.x >> 6); i < i_end; i += RAB_NT / 64) {   // wave-uniform
        float sum[RAB_JPT];
        int id[RAB_JPT];
#pragma unroll
        for (int k = 0; k < RAB_JPT; k++) { sum[k] = 0.f; id[k] = -1; }
        if (j0 < s) {
            const T* row = g + (2 * (int64_t)i) * s2 + 2 * j0;
            if (wide) {
                typedef __attribute__((ext_vector_type(4))) unsigned int u4;
                constexpr int NV = 2 * RAB_JPT * sizeof(T) / 16;
                T r0[2 * RAB_JPT], r1[2 * RAB_JPT];
#pragma unroll
                for (int q = 0; q < NV; q++) {
                    reinterpret_cast<u4*>(r0)[q] = reinterpret_cast<const u4*>(row)[q];
                    reinterpret_cast<u4*>(r1)[q] = reinterpret_cast<const u4*>(row + s2)[q];
                }
#pragma unroll
                for (int k = 0; k < RAB_JPT; k++)
                    sum[k] = (to_float(r0[2 * k]) + to_float(r0[2 * k + 1])) + (to_float(r1[2 * k]) + to_float(r1[2 * k + 1]));
            } else {
#pragma unroll
                for (int k = 0; k < RAB_JPT; k++)
                    if (j0 + k < s)
                        sum[k] = (to_float(row[2 * k]) + to_float(row[2 * k + 1])) + (to_float(row[s2 + 2 * k]) + to_float(row[s2 + 2 * k + 1]));
            }
            if (wide_id) {
                // the lane's ids as 16-byte reads (rows of ids start on 16-byte boundaries)
                typedef __attribute__((ext_vector_type(4))) unsigned int u4;
                constexpr int NI = RAB_JPT * sizeof(I) / 16;
                I raw[RAB_JPT];
#pragma unroll
                for (int q = 0; q < NI; q++) reinterpret_cast<u4*>(raw)[q] = reinterpret_cast<const u4*>(bt + (int64_t)i * s + j0)[q];
#pragma unroll
                for (int k = 0; k < RAB_JPT; k++) {
                    const int64_t v = (int64_t)raw[k];
                    id[k] = (v >= 0 && v < nb) ? (int)v : -1;
                }
            } else {
#pragma unroll
                for (int k = 0; k < RAB_JPT; k++) {
                    if (j0 + k >= s) break;
                    const int64_t v = (int64_t)bt[(int64_t)i * s + j0 + k];
                    id[k] = (v >= 0 && v < nb) ? (int)v : -1;
                }
            }
            // equal neighbours inside the lane first
#pragma unroll
            for (int k = RAB_JPT - 1; k > 0; k--)
                if (id[k] == id[k - 1] && id[k] >= 0) { sum[k - 1] += sum[k]; id[k] = -1; }
        }
#pragma unroll
        for (int k = 0; k < RAB_JPT; k++) {
            bool todo = id[k] >= 0;
            unsigned long long m = __ballot(todo);
            while (m) {   // wave-uniform loop: one pass per distinct id still pending
                const int leader = __ffsll((long long)m) - 1;
                const int lid = __shfl(id[k], leader, 64);
                const bool mine = todo && id[k] == lid;
                const float tot = wave_sum(mine ? sum[k] : 0.f);
                if (lane == leader) atomicAdd(&hist[lid], tot);
                todo = todo && !mine;
                m = __ballot(todo);
            }
        }
    }
    __syncthreads();
    for (int k = threadIdx.x; k < nb; k += RAB_NT)
        if (hist[k] != 0.f) atomicAdd(p.grad_weights + (int64_t)n * nb + k, hist[k]);
}

__global__ void hstu_fill_zero_kernel(float* x, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = 0.f;
}

constexpr int RAB_POS_USERS = 64;   // users per launch: their lengths travel in the kernel arguments
struct RabPosLens {
    int v[RAB_POS_USERS];
};

template <typename T> __device__ __forceinline__ float rnd(float x) { return to_float(from_float<T>(x)); }
template <> __device__ __forceinline__ float rnd<float>(float x) { return x; }

// grid: x = column groups of RAB_NT * 8, y = row; the users of this launch one after the other, so that the identity
// row and rel row i (what every user with past_valid_len >= i takes) are read once.  A lane takes 8 consecutive columns
// with 16-byte (fp32: two) accesses when the rows start on 16-byte boundaries, else the 8 columns lane + 256 * k.
template <typename T>
__global__ __launch_bounds__(RAB_NT) void hstu_rab_pos_kernel(const T* rel, const T* identity, T* out, int seq2, int users, RabPosLens lens) {
    const int i = blockIdx.y;
    const float r00 = to_float(rel[0]);
    const T* irow = identity + (int64_t)i * seq2;
    auto blend = [&](T r_, T id_) __attribute__((always_inline)) -> T {
        const float id = to_float(id_), r = to_float(r_);
        // the golden's tensor expression, one rounding per operation (exact for a 0/1 identity)
        const float keep = rnd<T>(__fmul_rn(r, rnd<T>(__fsub_rn(1.0f, id))));
        const float fill = rnd<T>(__fmul_rn(id, r00));
        return from_float<T>(__fadd_rn(keep, fill));
    };
    const int base = blockIdx.x * RAB_NT * 8;
    if (seq2 % 8 == 0) {
        // rows of whole chunks of 8 columns: the lanes of a wave cover whole cache lines of output row i (the planes of the
        // users are a whole number of lines apart).  A workgroup takes RAB_UPW chunks, starting `a` chunks further right,
        // where a is what brings lane 0 of each wave onto a line boundary of this row; the first `a` chunks of the row go
        // to the spare lanes of its first workgroup.
        constexpr int cb = 8 * sizeof(T), cpl = 128 / cb;
        const int a = (cpl - (int)((reinterpret_cast<uintptr_t>(out + (int64_t)i * seq2) / cb) % cpl)) % cpl;
        const int tid = threadIdx.x;
        int chunk = tid < RAB_UPW ? RAB_UPW * (int)blockIdx.x + tid + a : ((blockIdx.x == 0 && tid - RAB_UPW < a) ? tid - RAB_UPW : seq2);
        const int j0 = chunk * 8;
        if (j0 >= seq2) return;
        typedef __attribute__((ext_vector_type(4))) unsigned int u4;
        constexpr int NV = 8 * sizeof(T) / 16;
        T own[8], d[8];
#pragma unroll
        for (int q = 0; q < NV; q++) {
            reinterpret_cast<u4*>(own)[q] = reinterpret_cast<const u4*>(rel + (int64_t)i * seq2 + j0)[q];
            reinterpret_cast<u4*>(d)[q] = reinterpret_cast<const u4*>(irow + j0)[q];
        }
        for (int u = 0; u < users; u++) {
            T r[8], o[8];
            const int v = lens.v[u];
#pragma unroll
            for (int q = 0; q < NV; q++)
                reinterpret_cast<u4*>(r)[q] = i <= v ? reinterpret_cast<const u4*>(own)[q] : reinterpret_cast<const u4*>(rel + (int64_t)v * seq2 + j0)[q];
#pragma unroll
            for (int k = 0; k < 8; k++) o[k] = blend(r[k], d[k]);
            T* orow = out + ((int64_t)u * seq2 + i) * seq2;
#pragma unroll
            for (int q = 0; q < NV; q++) __builtin_nontemporal_store(reinterpret_cast<const u4*>(o)[q], reinterpret_cast<u4*>(orow + j0) + q);
        }
    } else {
        for (int u = 0; u < users; u++) {
            const T* rrow = rel + (int64_t)min(i, lens.v[u]) * seq2;
            T* orow = out + ((int64_t)u * seq2 + i) * seq2;
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const int j = base + threadIdx.x + RAB_NT * k;
                if (j < seq2) orow[j] = blend(rrow[j], irow[j]);
            }
        }
    }
}

template <typename T, typename I>
static void launch_rab_time(const hstu_rab_time_params& p, hipStream_t st) {
    // rows of whole 16-byte chunks on chunk boundaries: the variant whose waves store whole cache lines
    const uintptr_t ob = reinterpret_cast<uintptr_t>(p.rab_time_out), ib = reinterpret_cast<uintptr_t>(p.bucket_ts_out);
    if (p.seq_len % RAB_JPT == 0 && ob % (2 * RAB_JPT * sizeof(T)) == 0 && ib % (RAB_JPT * sizeof(I)) == 0) {
        const unsigned groups = (unsigned)((p.seq_len / RAB_JPT + RAB_UPW - 1) / RAB_UPW);
        hipLaunchKernelGGL((hstu_rab_time_lines_kernel<T, I>), dim3(groups * (unsigned)(p.batch * p.seq_len)), dim3(RAB_NT), 0, st, p);
        return;
    }
    const unsigned gx = (unsigned)((p.seq_len + RAB_NT * RAB_JPT - 1) / (RAB_NT * RAB_JPT));
    hipLaunchKernelGGL((hstu_rab_time_kernel<T, I>), dim3(gx * (unsigned)(p.batch * p.seq_len)), dim3(RAB_NT), 0, st, p);
}

template <typename T, typename I>
static void launch_rab_time_bwd(const hstu_rab_time_bwd_params& p, hipStream_t st) {
    const unsigned gx = (unsigned)((p.seq_len + 64 * RAB_JPT - 1) / (64 * RAB_JPT));
    const unsigned gy = (unsigned)((p.seq_len + RAB_ROWS - 1) / RAB_ROWS);
    const unsigned tiles = gx * gy * (unsigned)p.batch;
    hipLaunchKernelGGL((hstu_rab_time_bwd_kernel<T, I>), dim3((tiles + 7) / 8 * 8 * (unsigned)p.num_layers), dim3(RAB_NT), 0, st, p);
}

template <typename T>
static void launch_rab_pos(int seq2, const void* rel, const void* identity, const int64_t* lens, int batch, void* out, hipStream_t st) {
    // (rows of whole 8-column chunks: RAB_UPW chunks per workgroup, see the kernel)
    const unsigned gx = seq2 % 8 == 0 ? (unsigned)((seq2 / 8 + RAB_UPW - 1) / RAB_UPW) : (unsigned)((seq2 + RAB_NT * 8 - 1) / (RAB_NT * 8));
    for (int u0 = 0; u0 < batch; u0 += RAB_POS_USERS) {
        RabPosLens l;
        const int nu = batch - u0 < RAB_POS_USERS ? batch - u0 : RAB_POS_USERS;
        for (int u = 0; u < RAB_POS_USERS; u++) l.v[u] = u < nu ? (int)lens[u0 + u] : 0;
        hipLaunchKernelGGL((hstu_rab_pos_kernel<T>), dim3(gx, (unsigned)seq2), dim3(RAB_NT), 0, st, reinterpret_cast<const T*>(rel),
                           reinterpret_cast<const T*>(identity), reinterpret_cast<T*>(out) + (int64_t)u0 * seq2 * seq2, seq2, nu, l);
    }
}

static int launched() {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    return HSTU_OK;
}

static bool io_dtype_ok(int d) { return d == HSTU_F32 || d == HSTU_F16 || d == HSTU_BF16; }

}  // namespace hstu

using namespace hstu;

#define RAB_DISPATCH(dtype, index_type, FN, ...)                                                    \
    do {                                                                                            \
        const bool i64 = (index_type) == HSTU_I64;                                                  \
        if ((dtype) == HSTU_F32) { if (i64) FN<float, int64_t>(__VA_ARGS__); else FN<float, int32_t>(__VA_ARGS__); }          \
        else if ((dtype) == HSTU_F16) { if (i64) FN<_Float16, int64_t>(__VA_ARGS__); else FN<_Float16, int32_t>(__VA_ARGS__); } \
        else { if (i64) FN<__bf16, int64_t>(__VA_ARGS__); else FN<__bf16, int32_t>(__VA_ARGS__); }  \
    } while (0)

extern "C" int hstu_hip_rab_time(const hstu_rab_time_params* p, void* stream) {
    if (!p) return fail(HSTU_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(hstu_rab_time_params))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "hstu_rab_time_params size mismatch: caller %u, library %zu", p->struct_size, sizeof(hstu_rab_time_params));
    if (!io_dtype_ok(p->dtype)) return fail(HSTU_ERR_INVALID_ARGUMENT, "Invalid data type of timestamps_weights.");
    if (p->index_type != HSTU_I32 && p->index_type != HSTU_I64) return fail(HSTU_ERR_INVALID_ARGUMENT, "Invalid data type of timestamps.");
    if (p->seq_len <= 0 || p->seq_len > HSTU_RAB_MAX_SEQ_LEN)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "timestamps size must be between 1 and %d, but got %d", HSTU_RAB_MAX_SEQ_LEN, p->seq_len);
    if (p->batch <= 0 || (int64_t)p->batch * p->seq_len > 0x7fffffffLL / 2)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "batchsize expects a positive value with batchsize * s < 2^30, but got %d", p->batch);
    if (p->num_layers <= 0 || p->num_layers > HSTU_RAB_MAX_LAYERS)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "num_layer expects a value in the range [1, %d], but the actual value is %d.", HSTU_RAB_MAX_LAYERS, p->num_layers);
    if (p->weight_cols <= 0 || p->weight_cols > HSTU_RAB_MAX_BUCKETS)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "num_buckets expects a value in the range [1, %d], but the actual value is %d.", HSTU_RAB_MAX_BUCKETS, p->weight_cols);
    if (!p->timestamps || !p->weights || !p->bucket_bounds || !p->rab_time_out)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "timestamps, weights, bucket_bounds and rab_time_out must not be NULL");
    if (reinterpret_cast<uintptr_t>(p->rab_time_out) & 15) return fail(HSTU_ERR_UNSUPPORTED, "rab_time_out must be 16-byte aligned");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    RAB_DISPATCH(p->dtype, p->index_type, launch_rab_time, *p, st);
    return launched();
}

extern "C" int hstu_hip_rab_time_backward(const hstu_rab_time_bwd_params* p, void* stream) {
    if (!p) return fail(HSTU_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(hstu_rab_time_bwd_params))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "hstu_rab_time_bwd_params size mismatch: caller %u, library %zu", p->struct_size, sizeof(hstu_rab_time_bwd_params));
    if (!io_dtype_ok(p->dtype) || (p->index_type != HSTU_I32 && p->index_type != HSTU_I64)) return fail(HSTU_ERR_INVALID_ARGUMENT, "Invalid data type.");
    if (p->num_layers <= 0 || p->num_layers > HSTU_RAB_MAX_LAYERS)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "num_layer expects a value in the range [1, %d], but the actual value is %d.", HSTU_RAB_MAX_LAYERS, p->num_layers);
    if (p->num_buckets <= 0 || p->num_buckets > HSTU_RAB_MAX_BUCKETS)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "num_buckets expects a value in the range [1, %d], but the actual value is %d.", HSTU_RAB_MAX_BUCKETS, p->num_buckets);
    if (p->seq_len <= 0 || p->seq_len > HSTU_RAB_MAX_SEQ_LEN)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "Sequence len expects a value in the range [1, %d], but the actual value is %d.", 2 * HSTU_RAB_MAX_SEQ_LEN, 2 * p->seq_len);
    if (p->batch <= 0 || p->batch > 65535 / HSTU_RAB_MAX_LAYERS)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "Batchsize expects a value in the range [1, %d], but the actual value is %d.", 65535 / HSTU_RAB_MAX_LAYERS, p->batch);
    if (!p->grad || !p->bucket_ts || !p->grad_weights) return fail(HSTU_ERR_INVALID_ARGUMENT, "grad, bucket_ts and grad_weights must not be NULL");
    if (reinterpret_cast<uintptr_t>(p->grad) & 15) return fail(HSTU_ERR_UNSUPPORTED, "grad must be 16-byte aligned");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const int n = p->num_layers * p->num_buckets;
    hipLaunchKernelGGL(hstu_fill_zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, p->grad_weights, n);
    RAB_DISPATCH(p->dtype, p->index_type, launch_rab_time_bwd, *p, st);
    return launched();
}

extern "C" int hstu_hip_rab_pos(int32_t dtype, int32_t seq2, const void* rel_pos_bias, const void* identity, const int64_t* lens,
                                int32_t batch, void* out, void* stream) {
    if (!io_dtype_ok(dtype)) return fail(HSTU_ERR_INVALID_ARGUMENT, "Invalid data type.");
    if (seq2 <= 0 || seq2 > 2 * HSTU_RAB_MAX_SEQ_LEN) return fail(HSTU_ERR_INVALID_ARGUMENT, "Invalid sequence len of rel_pos_bias.");
    if (batch <= 0 || batch > 65535) return fail(HSTU_ERR_INVALID_ARGUMENT, "batchsize of past_valid_lens is expected in [1, %d], but got %d", 65535, batch);
    if (!rel_pos_bias || !identity || !lens || !out) return fail(HSTU_ERR_INVALID_ARGUMENT, "rel_pos_bias, identity, past_valid_lens and out must not be NULL");
    for (int u = 0; u < batch; u++)
        if (lens[u] < 0 || lens[u] >= seq2)
            return fail(HSTU_ERR_INVALID_ARGUMENT, "past_valid_lens[%d] expected in [0, %d), but got %lld", u, seq2, (long long)lens[u]);
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (dtype == HSTU_F32) launch_rab_pos<float>(seq2, rel_pos_bias, identity, lens, batch, out, st);
    else if (dtype == HSTU_F16) launch_rab_pos<_Float16>(seq2, rel_pos_bias, identity, lens, batch, out, st);
    else launch_rab_pos<__bf16>(seq2, rel_pos_bias, identity, lens, batch, out, st);
    return launched();
}
