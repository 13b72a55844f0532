// LayerNorm(x) * u with dropout, forward and backward (mxrec::norm_multiply_dropout).  HBM-bound row work: a wave
// owns a row (512 or 1024 columns = 8 or 16 per lane, read and written as 16-byte pieces of 8 consecutive columns so
// that one instruction of the wave covers 1 KiB at 2 bytes per element), the row statistics are wave reductions, and
// nothing but the inputs and outputs touches memory.  The backward's column sums (d_weight, d_bias) stay in registers
// across the rows a lane sees and leave through per-workgroup partial sums that a second kernel adds in a fixed order.
// Definitions: cust_op/ascendc_op/ai_core_op/norm_multiply_dropout/v220/README.md:41-60,
// cust_op/test/norm_multiply_dropout/torch/test_norm_multiply_dropout.py:220-243.
#include "hstu_device.h"
#include "../../include/hstu_layer.h"

namespace hstu {

constexpr int NMD_NT = 256;
constexpr int NMD_MAX_WGS = 1024;   // workgroups of the backward = rows of its partial-sum table

typedef __attribute__((ext_vector_type(4))) unsigned int nmd_u4;

__device__ __forceinline__ float nmd_wave_sum(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
    return x;
}

// 8 consecutive elements at p (16-byte aligned for 2-byte types, 32 for fp32).  Every row is touched once per call:
// loads and stores carry the nontemporal hint (worth 6-9 % on both directions)
template <typename T> __device__ __forceinline__ void load8(const T* p, float* v) {
    T t[8];
#pragma unroll
    for (int q = 0; q < (int)(8 * sizeof(T) / 16); q++) reinterpret_cast<nmd_u4*>(t)[q] = __builtin_nontemporal_load(reinterpret_cast<const nmd_u4*>(p) + q);
#pragma unroll
    for (int k = 0; k < 8; k++) v[k] = to_float(t[k]);
}
template <typename T> __device__ __forceinline__ void store8(T* p, const float* v) {
    T t[8];
#pragma unroll
    for (int k = 0; k < 8; k++) t[k] = from_float<T>(v[k]);
#pragma unroll
    for (int q = 0; q < (int)(8 * sizeof(T) / 16); q++) __builtin_nontemporal_store(reinterpret_cast<const nmd_u4*>(t)[q], reinterpret_cast<nmd_u4*>(p) + q);
}

__device__ __forceinline__ unsigned long long nmd_mix(unsigned long long z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

// keep bits of the 8 elements of mask byte `byte_index`: 16 random bits per element against the threshold
__device__ __forceinline__ unsigned nmd_keep_bits(unsigned long long seed, unsigned long long byte_index, unsigned threshold) {
    const unsigned long long r0 = nmd_mix(seed + (2 * byte_index + 1) * 0x9E3779B97F4A7C15ull);
    const unsigned long long r1 = nmd_mix(seed + (2 * byte_index + 2) * 0x9E3779B97F4A7C15ull);
    unsigned bits = 0;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        bits |= (((unsigned)(r0 >> (16 * k)) & 0xffffu) >= threshold ? 1u : 0u) << k;
        bits |= (((unsigned)(r1 >> (16 * k)) & 0xffffu) >= threshold ? 1u : 0u) << (4 + k);
    }
    return bits;
}

// column of element k of piece q of this lane: pieces of 512 columns, 8 per lane
#define NMD_COL(q, lane) ((q) * 512 + (lane) * 8)

template <typename T, int C>
__global__ __launch_bounds__(NMD_NT) void hstu_nmd_fwd_kernel(const hstu_nmd_params p, unsigned threshold, float keep_scale) {
    constexpr int NP = C / 512;
    const int lane = threadIdx.x & 63;
    const T* x = reinterpret_cast<const T*>(p.x);
    const T* u = reinterpret_cast<const T*>(p.u);
    T* out = reinterpret_cast<T*>(p.out);
    float w[NP][8], b[NP][8];
#pragma unroll
    for (int q = 0; q < NP; q++) {
        load8(reinterpret_cast<const T*>(p.weight) + NMD_COL(q, lane), w[q]);
        load8(reinterpret_cast<const T*>(p.bias) + NMD_COL(q, lane), b[q]);
    }
    const bool drop = p.dropout_ratio > 1e-10f;
    const int64_t wave = (int64_t)blockIdx.x * (NMD_NT / 64) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (NMD_NT / 64);
    for (int64_t row = wave; row < p.rows; row += nwaves) {
        float xv[NP][8], uv[NP][8];
#pragma unroll
        for (int q = 0; q < NP; q++) {
            load8(x + row * C + NMD_COL(q, lane), xv[q]);
            load8(u + row * C + NMD_COL(q, lane), uv[q]);
        }
        float s = 0.f;
#pragma unroll
        for (int q = 0; q < NP; q++)
#pragma unroll
            for (int k = 0; k < 8; k++) s += xv[q][k];
        const float mean = nmd_wave_sum(s) * (1.0f / C);
        float s2 = 0.f;
#pragma unroll
        for (int q = 0; q < NP; q++)
#pragma unroll
            for (int k = 0; k < 8; k++) { const float d = xv[q][k] - mean; s2 += d * d; }
        const float var = nmd_wave_sum(s2) * (1.0f / C);
        const float rstd = 1.0f / sqrtf(var + p.eps);
        if (lane == 0) { p.mean[row] = mean; p.var[row] = var; }
#pragma unroll
        for (int q = 0; q < NP; q++) {
            float y[8];
#pragma unroll
            for (int k = 0; k < 8; k++) y[k] = ((xv[q][k] - mean) * rstd * w[q][k] + b[q][k]) * uv[q][k];
            if (drop) {
                const unsigned long long byte_index = (unsigned long long)(row * C + NMD_COL(q, lane)) >> 3;
                const unsigned bits = nmd_keep_bits(p.seed, byte_index, threshold);
                p.drop_mask[byte_index] = (uint8_t)bits;
#pragma unroll
                for (int k = 0; k < 8; k++) y[k] = ((bits >> k) & 1u) ? y[k] * keep_scale : 0.f;
            }
            store8(out + row * C + NMD_COL(q, lane), y);
        }
    }
}

template <typename T, int C>
__global__ __launch_bounds__(NMD_NT) void hstu_nmd_bwd_kernel(const hstu_nmd_bwd_params p, float keep_scale, float* partial) {
    constexpr int NP = C / 512;
    __shared__ float red[2][NMD_NT / 64][C];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const T* x = reinterpret_cast<const T*>(p.x);
    const T* u = reinterpret_cast<const T*>(p.u);
    const T* dy = reinterpret_cast<const T*>(p.d_out);
    T* dx = reinterpret_cast<T*>(p.d_x);
    T* du = reinterpret_cast<T*>(p.d_u);
    float w[NP][8], b[NP][8], gw[NP][8], gb[NP][8];
#pragma unroll
    for (int q = 0; q < NP; q++) {
        load8(reinterpret_cast<const T*>(p.weight) + NMD_COL(q, lane), w[q]);
        load8(reinterpret_cast<const T*>(p.bias) + NMD_COL(q, lane), b[q]);
#pragma unroll
        for (int k = 0; k < 8; k++) gw[q][k] = gb[q][k] = 0.f;
    }
    const bool drop = p.dropout_ratio > 1e-10f;
    const int64_t wave = (int64_t)blockIdx.x * (NMD_NT / 64) + wv;
    const int64_t nwaves = (int64_t)gridDim.x * (NMD_NT / 64);
    for (int64_t row = wave; row < p.rows; row += nwaves) {
        float xh[NP][8], g[NP][8], dyv[NP][8];
        const float mean = p.mean[row];
        const float rstd = 1.0f / sqrtf(p.var[row] + p.eps);
        float r1 = 0.f, r2 = 0.f;
#pragma unroll
        for (int q = 0; q < NP; q++) {
            float uv[8];
            load8(x + row * C + NMD_COL(q, lane), xh[q]);
            load8(u + row * C + NMD_COL(q, lane), uv);
            load8(dy + row * C + NMD_COL(q, lane), dyv[q]);
            if (drop) {
                const unsigned bits = p.drop_mask[(unsigned long long)(row * C + NMD_COL(q, lane)) >> 3];
#pragma unroll
                for (int k = 0; k < 8; k++) dyv[q][k] = ((bits >> k) & 1u) ? dyv[q][k] * keep_scale : 0.f;
            }
#pragma unroll
            for (int k = 0; k < 8; k++) {
                xh[q][k] = (xh[q][k] - mean) * rstd;
                g[q][k] = dyv[q][k] * uv[k];
                gw[q][k] += xh[q][k] * g[q][k];
                gb[q][k] += g[q][k];
                const float a = g[q][k] * w[q][k];
                r1 += a;
                r2 += a * xh[q][k];
            }
        }
        r1 = nmd_wave_sum(r1) * (1.0f / C);
        r2 = nmd_wave_sum(r2) * (1.0f / C);
#pragma unroll
        for (int q = 0; q < NP; q++) {
            float ox[8], ou[8];
#pragma unroll
            for (int k = 0; k < 8; k++) {
                ox[k] = (g[q][k] * w[q][k] - (r1 + xh[q][k] * r2)) * rstd;
                ou[k] = dyv[q][k] * (w[q][k] * xh[q][k] + b[q][k]);
            }
            store8(dx + row * C + NMD_COL(q, lane), ox);
            store8(du + row * C + NMD_COL(q, lane), ou);
        }
    }
    // the workgroup's column sums: waves in order 0..3, then one row of the partial table
#pragma unroll
    for (int q = 0; q < NP; q++)
#pragma unroll
        for (int k = 0; k < 8; k++) {
            red[0][wv][NMD_COL(q, lane) + k] = gw[q][k];
            red[1][wv][NMD_COL(q, lane) + k] = gb[q][k];
        }
    __syncthreads();
    for (int c = threadIdx.x; c < 2 * C; c += NMD_NT) {
        const int which = c / C, col = c % C;
        float s = 0.f;
#pragma unroll
        for (int v = 0; v < NMD_NT / 64; v++) s += red[which][v][col];
        partial[((int64_t)blockIdx.x * 2 + which) * C + col] = s;
    }
}

// d_weight / d_bias = partial sums of the workgroups, added in a fixed order: 32 columns x 8 row slots per workgroup,
// slot r adds the rows r, r + 8, ... of the partial table, then the slots are added 0..7
__global__ __launch_bounds__(256) void hstu_nmd_colsum_kernel(const float* partial, int wgs, int cols, float* d_weight, float* d_bias) {
    __shared__ float part[8][32];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int c = blockIdx.x * 32 + tx;            // column of the [2 * cols] row: d_weight then d_bias
    const int which = c / cols, col = c % cols;
    float s = 0.f;
#pragma unroll 8
    for (int g = ty; g < wgs; g += 8) s += partial[((int64_t)g * 2 + which) * cols + col];
    part[ty][tx] = s;
    __syncthreads();
    if (ty == 0) {
        float t = 0.f;
#pragma unroll
        for (int r = 0; r < 8; r++) t += part[r][tx];
        (which ? d_bias : d_weight)[col] = t;
    }
}

static unsigned nmd_grid(int64_t rows) {
    const int64_t want = (rows + NMD_NT / 64 - 1) / (NMD_NT / 64);
    return (unsigned)(want < 1 ? 1 : (want > NMD_MAX_WGS ? NMD_MAX_WGS : want));
}

static int nmd_check(int32_t dtype, int64_t rows, int32_t cols, float eps, float ratio) {
    if (dtype != HSTU_F32 && dtype != HSTU_F16 && dtype != HSTU_BF16)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "dtype expect float32, float16 or bfloat16, but value is %d", dtype);
    if (rows < 1 || rows > HSTU_NMD_MAX_ROWS) return fail(HSTU_ERR_INVALID_ARGUMENT, "x dim0 must in range:[1,%d].", HSTU_NMD_MAX_ROWS);
    if (cols != 512 && cols != 1024) return fail(HSTU_ERR_INVALID_ARGUMENT, "x dim1 must equal with 512 or 1024");
    if (!(eps >= 1e-10f && eps <= 1e-4f)) return fail(HSTU_ERR_INVALID_ARGUMENT, "eps must in range:[1e-10,0.0001].");
    if (!(ratio >= 0.f && ratio <= 1.f)) return fail(HSTU_ERR_INVALID_ARGUMENT, "dropout_ratio must in range:[0,1].");
    return HSTU_OK;
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

static float nmd_keep_scale(float ratio) { return ratio < 1.f ? 1.0f / (1.0f - ratio) : 0.f; }

}  // namespace hstu

using namespace hstu;

#define NMD_DISPATCH(dtype, cols, KERNEL, grid, st, ...)                                                             \
    do {                                                                                                              \
        if ((dtype) == HSTU_F32) { if ((cols) == 512) hipLaunchKernelGGL((KERNEL<float, 512>), grid, dim3(NMD_NT), 0, st, __VA_ARGS__); else hipLaunchKernelGGL((KERNEL<float, 1024>), grid, dim3(NMD_NT), 0, st, __VA_ARGS__); } \
        else if ((dtype) == HSTU_F16) { if ((cols) == 512) hipLaunchKernelGGL((KERNEL<_Float16, 512>), grid, dim3(NMD_NT), 0, st, __VA_ARGS__); else hipLaunchKernelGGL((KERNEL<_Float16, 1024>), grid, dim3(NMD_NT), 0, st, __VA_ARGS__); } \
        else { if ((cols) == 512) hipLaunchKernelGGL((KERNEL<__bf16, 512>), grid, dim3(NMD_NT), 0, st, __VA_ARGS__); else hipLaunchKernelGGL((KERNEL<__bf16, 1024>), grid, dim3(NMD_NT), 0, st, __VA_ARGS__); } \
    } while (0)

extern "C" int hstu_hip_norm_multiply_dropout(const hstu_nmd_params* p, void* stream) {
    if (!p) return fail(HSTU_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(hstu_nmd_params))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "hstu_nmd_params size mismatch: caller %u, library %zu", p->struct_size, sizeof(hstu_nmd_params));
    const int rc = nmd_check(p->dtype, p->rows, p->cols, p->eps, p->dropout_ratio);
    if (rc != HSTU_OK) return rc;
    const bool drop = p->dropout_ratio > 1e-10f;
    if (!p->x || !p->u || !p->weight || !p->bias || !p->out || !p->mean || !p->var || (drop && !p->drop_mask))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "x, u, weight, bias, out, mean, var (and drop_mask with dropout) must not be NULL");
    if (!aligned16(p->x) || !aligned16(p->u) || !aligned16(p->weight) || !aligned16(p->bias) || !aligned16(p->out))
        return fail(HSTU_ERR_UNSUPPORTED, "x, u, weight, bias and out must be 16-byte aligned");
    const double t = (double)p->dropout_ratio * 65536.0 + 0.5;
    const unsigned threshold = drop ? (unsigned)(t > 65536.0 ? 65536.0 : t) : 0u;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    NMD_DISPATCH(p->dtype, p->cols, hstu_nmd_fwd_kernel, dim3(nmd_grid(p->rows) * 4 > 65536 ? 65536 : nmd_grid(p->rows) * 4), st, *p, threshold,
                 nmd_keep_scale(p->dropout_ratio));
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    return HSTU_OK;
}

static int nmd_bwd_validate(const hstu_nmd_bwd_params* p) {
    if (!p) return fail(HSTU_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(hstu_nmd_bwd_params))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "hstu_nmd_bwd_params size mismatch: caller %u, library %zu", p->struct_size, sizeof(hstu_nmd_bwd_params));
    const int rc = nmd_check(p->dtype, p->rows, p->cols, p->eps, p->dropout_ratio);
    if (rc != HSTU_OK) return rc;
    const bool drop = p->dropout_ratio > 1e-10f;
    if (!p->d_out || !p->x || !p->u || !p->weight || !p->bias || !p->mean || !p->var || !p->d_x || !p->d_u || !p->d_weight || !p->d_bias ||
        (drop && !p->drop_mask))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "d_out, x, u, weight, bias, mean, var, d_x, d_u, d_weight, d_bias (and drop_mask with dropout) must not be NULL");
    if (!aligned16(p->d_out) || !aligned16(p->x) || !aligned16(p->u) || !aligned16(p->weight) || !aligned16(p->bias) || !aligned16(p->d_x) || !aligned16(p->d_u))
        return fail(HSTU_ERR_UNSUPPORTED, "d_out, x, u, weight, bias, d_x and d_u must be 16-byte aligned");
    return HSTU_OK;
}

extern "C" int hstu_hip_norm_multiply_dropout_backward_get_workspace_size(const hstu_nmd_bwd_params* p, uint64_t* bytes) {
    if (!bytes) return fail(HSTU_ERR_INVALID_ARGUMENT, "workspace_bytes is NULL");
    const int rc = nmd_bwd_validate(p);
    if (rc != HSTU_OK) return rc;
    *bytes = (uint64_t)nmd_grid(p->rows) * 2 * p->cols * sizeof(float);
    return HSTU_OK;
}

extern "C" int hstu_hip_norm_multiply_dropout_backward(const hstu_nmd_bwd_params* p, void* workspace, uint64_t workspace_bytes, void* stream) {
    const int rc = nmd_bwd_validate(p);
    if (rc != HSTU_OK) return rc;
    const unsigned grid = nmd_grid(p->rows);
    const uint64_t need = (uint64_t)grid * 2 * p->cols * sizeof(float);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15))
        return fail(HSTU_ERR_WORKSPACE, "workspace of %llu bytes (16-byte aligned) needed, got %llu at %p", (unsigned long long)need,
                    (unsigned long long)workspace_bytes, workspace);
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    float* partial = reinterpret_cast<float*>(workspace);
    NMD_DISPATCH(p->dtype, p->cols, hstu_nmd_bwd_kernel, dim3(grid), st, *p, nmd_keep_scale(p->dropout_ratio), partial);
    hipLaunchKernelGGL(hstu_nmd_colsum_kernel, dim3((unsigned)(2 * p->cols / 32)), dim3(256), 0, st, partial, (int)grid, p->cols, p->d_weight,
                       p->d_bias);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    return HSTU_OK;
}
