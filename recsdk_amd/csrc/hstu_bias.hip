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

// grid: x = column groups of RAB_NT * RAB_JPT, y = b * s + i
template <typename T, typename I>
__global__ __launch_bounds__(RAB_NT) void hstu_rab_time_kernel(const hstu_rab_time_params p) {
    __shared__ float bounds[HSTU_RAB_MAX_BUCKETS + 1];
    const int W = p.weight_cols, s = p.seq_len;
    for (int k = threadIdx.x; k <= W; k += RAB_NT) bounds[k] = p.bucket_bounds[k];
    __syncthreads();
    const int b = blockIdx.y / s, i = blockIdx.y % s;
    const int j0 = (blockIdx.x * RAB_NT + threadIdx.x) * RAB_JPT;
    if (j0 >= s) return;
    const I* ts = reinterpret_cast<const I*>(p.timestamps) + (int64_t)b * s;
    const I ti = ts[i];
    int bucket[RAB_JPT];
#pragma unroll
    for (int k = 0; k < RAB_JPT; k++) {
        const int j = min(j0 + k, s - 1);
        bucket[k] = ts_bucket(bounds, W - 1, abs_diff_f32<I>(ti, ts[j]));
    }
    if (p.bucket_ts_out) {
        I* bo = reinterpret_cast<I*>(p.bucket_ts_out) + ((int64_t)b * s + i) * s;
#pragma unroll
        for (int k = 0; k < RAB_JPT; k++)
            if (j0 + k < s) bo[j0 + k] = (I)bucket[k];
    }
    const T* w = reinterpret_cast<const T*>(p.weights);
    T* out = reinterpret_cast<T*>(p.rab_time_out);
    const int64_t s2 = 2 * (int64_t)s;
    const bool wide = j0 + RAB_JPT <= s && (s2 * sizeof(T)) % 16 == 0;   // whole group, rows start on 16-byte boundaries
    for (int n = 0; n < p.num_layers; n++) {
        T v[RAB_JPT];
#pragma unroll
        for (int k = 0; k < RAB_JPT; k++) v[k] = w[n * W + bucket[k]];
        T* row = out + (((int64_t)n * p.batch + b) * s2 + 2 * i) * s2 + 2 * j0;
        if (wide) {
            T pk[2 * RAB_JPT];
#pragma unroll
            for (int k = 0; k < RAB_JPT; k++) pk[2 * k] = pk[2 * k + 1] = v[k];
            typedef __attribute__((ext_vector_type(4))) unsigned int u4;
            constexpr int NV = 2 * RAB_JPT * sizeof(T) / 16;
            const u4* src = reinterpret_cast<const u4*>(pk);
#pragma unroll
            for (int q = 0; q < NV; q++) {
                reinterpret_cast<u4*>(row)[q] = src[q];
                reinterpret_cast<u4*>(row + s2)[q] = src[q];
            }
        } else {
#pragma unroll
            for (int k = 0; k < RAB_JPT; k++) {
                if (j0 + k >= s) break;
                row[2 * k] = row[2 * k + 1] = v[k];
                row[s2 + 2 * k] = row[s2 + 2 * k + 1] = v[k];
            }
        }
    }
}

// grid: x = column groups, y = row groups of RAB_ROWS rows i, z = n * batch + b
constexpr int RAB_ROWS = 16;
template <typename T, typename I>
__global__ __launch_bounds__(RAB_NT) void hstu_rab_time_bwd_kernel(const hstu_rab_time_bwd_params p) {
    __shared__ float hist[HSTU_RAB_MAX_BUCKETS];
    const int nb = p.num_buckets, s = p.seq_len;
    for (int k = threadIdx.x; k < nb; k += RAB_NT) hist[k] = 0.f;
    __syncthreads();
    const int n = blockIdx.z / p.batch, b = blockIdx.z % p.batch;
    const int j0 = (blockIdx.x * RAB_NT + threadIdx.x) * RAB_JPT;
    const int64_t s2 = 2 * (int64_t)s;
    const T* g = reinterpret_cast<const T*>(p.grad) + ((int64_t)n * p.batch + b) * s2 * s2;
    const I* bt = reinterpret_cast<const I*>(p.bucket_ts) + (int64_t)b * s * s;
    const bool wide = j0 + RAB_JPT <= s && (s2 * sizeof(T)) % 16 == 0;
    if (j0 < s) {
        for (int i = blockIdx.y * RAB_ROWS; i < min((int)(blockIdx.y + 1) * RAB_ROWS, s); i++) {
            const T* row = g + (2 * (int64_t)i) * s2 + 2 * j0;
            float sum[RAB_JPT];
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
                for (int k = 0; k < RAB_JPT; k++) {
                    sum[k] = 0.f;
                    if (j0 + k < s)
                        sum[k] = (to_float(row[2 * k]) + to_float(row[2 * k + 1])) + (to_float(row[s2 + 2 * k]) + to_float(row[s2 + 2 * k + 1]));
                }
            }
#pragma unroll
            for (int k = 0; k < RAB_JPT; k++) {
                if (j0 + k >= s) break;
                const int64_t id = (int64_t)bt[(int64_t)i * s + j0 + k];
                if (id >= 0 && id < nb) atomicAdd(&hist[id], sum[k]);
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

// grid: x = column groups of RAB_NT * 8, y = row, z = user within this launch
template <typename T>
__global__ __launch_bounds__(RAB_NT) void hstu_rab_pos_kernel(const T* rel, const T* identity, T* out, int seq2, RabPosLens lens) {
    const int i = blockIdx.y, u = blockIdx.z;
    const int src_row = min(i, lens.v[u]);
    const float r00 = to_float(rel[0]);
    const T* rrow = rel + (int64_t)src_row * seq2;
    const T* irow = identity + (int64_t)i * seq2;
    T* orow = out + ((int64_t)u * seq2 + i) * seq2;
    const int j0 = (blockIdx.x * RAB_NT + threadIdx.x) * 8;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const int j = j0 + k;
        if (j >= seq2) break;
        const float id = to_float(irow[j]), r = to_float(rrow[j]);
        // the golden's tensor expression, one rounding per operation (exact for a 0/1 identity)
        const float keep = rnd<T>(__fmul_rn(r, rnd<T>(__fsub_rn(1.0f, id))));
        const float fill = rnd<T>(__fmul_rn(id, r00));
        orow[j] = from_float<T>(__fadd_rn(keep, fill));
    }
}

template <typename T, typename I>
static void launch_rab_time(const hstu_rab_time_params& p, hipStream_t st) {
    const unsigned gx = (unsigned)((p.seq_len + RAB_NT * RAB_JPT - 1) / (RAB_NT * RAB_JPT));
    hipLaunchKernelGGL((hstu_rab_time_kernel<T, I>), dim3(gx, (unsigned)(p.batch * p.seq_len)), dim3(RAB_NT), 0, st, p);
}

template <typename T, typename I>
static void launch_rab_time_bwd(const hstu_rab_time_bwd_params& p, hipStream_t st) {
    const unsigned gx = (unsigned)((p.seq_len + RAB_NT * RAB_JPT - 1) / (RAB_NT * RAB_JPT));
    const unsigned gy = (unsigned)((p.seq_len + RAB_ROWS - 1) / RAB_ROWS);
    hipLaunchKernelGGL((hstu_rab_time_bwd_kernel<T, I>), dim3(gx, gy, (unsigned)(p.num_layers * p.batch)), dim3(RAB_NT), 0, st, p);
}

template <typename T>
static void launch_rab_pos(int seq2, const void* rel, const void* identity, const int64_t* lens, int batch, void* out, hipStream_t st) {
    const unsigned gx = (unsigned)((seq2 + RAB_NT * 8 - 1) / (RAB_NT * 8));
    for (int u0 = 0; u0 < batch; u0 += RAB_POS_USERS) {
        RabPosLens l;
        const int nu = batch - u0 < RAB_POS_USERS ? batch - u0 : RAB_POS_USERS;
        for (int u = 0; u < RAB_POS_USERS; u++) l.v[u] = u < nu ? (int)lens[u0 + u] : 0;
        hipLaunchKernelGGL((hstu_rab_pos_kernel<T>), dim3(gx, (unsigned)seq2, (unsigned)nu), dim3(RAB_NT), 0, st, reinterpret_cast<const T*>(rel),
                           reinterpret_cast<const T*>(identity), reinterpret_cast<T*>(out) + (int64_t)u0 * seq2 * seq2, seq2, l);
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
    if ((int64_t)p->batch * p->seq_len > 65535 * 32768LL) return fail(HSTU_ERR_UNSUPPORTED, "batch * s too large for one launch");
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
    if (p->batch <= 0 || (int64_t)p->batch * p->num_layers > 65535)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "Batchsize expects a positive value with num_layer * batchsize <= 65535, but the actual value is %d.", p->batch);
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
