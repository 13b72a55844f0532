// Backward of the input projection of an HSTU layer (mxrec::in_linear_silu_backward):
//   dlin        = round(grad * silu'(linear_output))      grad = (user_grad | value_grad | query_grad | key_grad) along n
//   x_grad      = dlin W            [m, k]   sum over n
//   weight_grad = dlin^T x          [n, k]   sum over m
//   bias_grad   = column sums of the unrounded dlin       [n], fp32
// (golden cust_op/test/in_linear_silu_test_backward/test_in_linear_silu_backward.py:37-66; the reference kernel also
// rounds dlin to the I/O dtype before its two matrix products and sums the bias gradient in fp32:
// cust_op/ascendc_op/ai_core_op/in_linear_silu_backward/v220/op_kernel/in_linear_silu_backward.h:267-332).
//
// n is at least 4 k, so both products are skinny: every element of dlin meets only k multiply-adds per product and the
// op is bounded by reading grad and linear_output from HBM.  dlin is therefore never written to memory: it is rebuilt in
// registers from grad and linear_output.
//   * k <= 64 (the library's choice there): ONE pass over the inputs.  hstu_ilb_wgrad_kernel<.., FUSED, 8 waves>: a wave
//     owns 64 columns n and walks down a range of m in tiles of 32 rows; dlin is built in the layout the loads arrive in
//     (a lane = 8 consecutive n of one row), parked in LDS and read back transposed (a lane = one column n, 8 consecutive
//     m) against rows of x^T for weight_grad, and row-wise against the wave's 64 rows of W (held in registers) for the
//     tile's x_grad; the eight waves' x_grad pieces meet in LDS and leave as the workgroup's partial slab (one slab per
//     512 columns of n).  The partial sums over the ranges of m (weight_grad, bias_grad) and over the slabs (x_grad) are
//     added in a fixed order by hstu_ilb_reduce_kernel, so the result is reproducible.
//   * k > 64, or on request: two product kernels that each stream the inputs once.
//     hstu_ilb_xgrad_kernel: a workgroup owns 32 rows m; its four waves take every fourth 64-column piece of n, build
//     dlin, park it in LDS, read it back as an MFMA operand (a lane = one row, 8 consecutive n: one 16-byte read) and
//     multiply by rows of W^T; the four partial results meet in LDS.
//     hstu_ilb_wgrad_kernel<.., not FUSED>: the weight_grad half of the one-pass kernel, four waves per workgroup.
// Both products want their small operand with the summed index contiguous per lane: W^T and x^T are written to the
// workspace first, already cut into MFMA operand fragments (hstu_ilb_pack_kernel: one fragment = 32 columns k x 16
// summed indices = 1 KiB that a wave loads with one fully contiguous instruction; together at most half of what grad
// alone takes, usually a few percent).
#include "hstu_device.h"
#include "../../include/hstu_layer.h"

namespace hstu {

typedef __attribute__((ext_vector_type(8))) __bf16 ilb_bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 ilb_f16x8;
typedef __attribute__((ext_vector_type(16))) float ilb_f32x16;
typedef __attribute__((ext_vector_type(4))) float ilb_f32x4;

template <typename T> struct IlbMM;
template <> struct IlbMM<__bf16> {
    typedef ilb_bf16x8 v8;
    static __device__ __forceinline__ ilb_f32x16 mfma(v8 a, v8 b, ilb_f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
template <> struct IlbMM<_Float16> {
    typedef ilb_f16x8 v8;
    static __device__ __forceinline__ ilb_f32x16 mfma(v8 a, v8 b, ilb_f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};

constexpr int ILB_NT = 256;
constexpr int ILB_FUSED_NW = 8, ILB_FUSED_COLS = 64 * ILB_FUSED_NW;   // the one-pass variant: waves per workgroup, columns of n per workgroup and slab
constexpr int ILB_PARK = 64 * 2 + 16;   // bytes of one parked row of 64 columns: 8 rows further down is 32 banks away

struct IlbArgs {
    hstu_in_linear_silu_bwd_params p;
    int base[5];          // first column of user, value, query, key, and n
    const void* xt;       // [mpad / 16, kbt] fragments of x^T, zero for rows >= m and columns >= k
    const void* wt;       // [n / 16, kbt]    fragments of W^T
    int kbt;              // ceil(k / 32)
    float* wpart;         // [S, n, k]
    float* bpart;         // [S, n]
    int64_t mpad;         // m rounded up to 32
    int64_t rows_per_part;
    int parts;            // S
    float* xpart;         // [ranges of n, m, k], only with more than one range
    int nparts;           // ranges of n of the x_grad kernel
    int cols_per_part;    // a multiple of 256
};

// grad * silu'(lin), unrounded
template <typename T>
__device__ __forceinline__ void ilb_dlin8(const typename IlbMM<T>::v8& g, const typename IlbMM<T>::v8& l, float* out) {
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const float x = to_float(l[e]);
        const float s = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504f * x));
        out[e] = to_float(g[e]) * (s * (1.0f + x * (1.0f - s)));
    }
}

// Fragments of in^T for in [rows, cols]: fragment (step, kb) holds columns 32 kb .. + 31 of the rows 16 step .. + 15 in
// the order an MFMA operand wants them: lane (l32, g) = column 32 kb + l32, rows 16 step + 8 g .. + 7 as 16 bytes at
// ((step * kbt + kb) * 64 + lane) * 16.  Zero outside in.  One thread per 16 bytes.
__global__ __launch_bounds__(256) void hstu_ilb_pack_kernel(const uint16_t* in, int64_t rows, int cols, int kbt, int64_t units, uint16_t* out) {
    typedef __attribute__((ext_vector_type(8))) uint16_t u16x8;
    const int64_t unit = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (unit >= units) return;
    const int lane = (int)(unit & 63);
    const int64_t blk = unit >> 6;
    const int kb = (int)(blk % kbt);
    const int64_t r0 = (blk / kbt) * 16 + 8 * (lane >> 5);
    const int c = 32 * kb + (lane & 31);
    u16x8 v;
#pragma unroll
    for (int e = 0; e < 8; e++) v[e] = (r0 + e < rows && c < cols) ? in[(r0 + e) * cols + c] : (uint16_t)0;
    *reinterpret_cast<u16x8*>(out + unit * 8) = v;
}

// pointer to 8 consecutive gradient columns starting at column n (a multiple of 8) of row `row`
template <typename T>
__device__ __forceinline__ const T* ilb_grad_ptr(const IlbArgs& a, int n, int64_t row) {
    int sel = 0;
#pragma unroll
    for (int i = 1; i < 4; i++) sel += n >= a.base[i] ? 1 : 0;
    const void* g = a.p.grad[0];
    int first = a.base[0], width = a.p.split[0];
#pragma unroll
    for (int i = 1; i < 4; i++)
        if (sel == i) { g = a.p.grad[i]; first = a.base[i]; width = a.p.split[i]; }
    return reinterpret_cast<const T*>(g) + row * width + (n - first);
}

template <typename T> __device__ __forceinline__ void ilb_store(void* out, int64_t idx, float v, int as_f32) {
    if (as_f32) reinterpret_cast<float*>(out)[idx] = v;
    else reinterpret_cast<T*>(out)[idx] = from_float<T>(v);
}

// x_grad.  grid = (ceil(m / 32), ceil(k / KC), ranges of n), 4 waves.
template <typename T, int KC>
__global__ __launch_bounds__(ILB_NT) void hstu_ilb_xgrad_kernel(const IlbArgs a) {
    typedef typename IlbMM<T>::v8 v8;
    constexpr int KB = KC / 32;
    constexpr int RED_BYTES = 3 * 32 * (KC + 1) * 4, PARK_BYTES = (ILB_NT / 64) * 32 * ILB_PARK;
    // the parked tiles of the loop and the sums of the epilogue share one buffer
    __shared__ __attribute__((aligned(16))) char lds[RED_BYTES > PARK_BYTES ? RED_BYTES : PARK_BYTES];
    float (*red)[32][KC + 1] = reinterpret_cast<float (*)[32][KC + 1]>(lds);
    const hstu_in_linear_silu_bwd_params& p = a.p;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int g = lane >> 5, l32 = lane & 31;
    const int N = p.n, K = p.k;
    const int64_t m0 = (int64_t)blockIdx.x * 32;
    const int k0 = blockIdx.y * KC;
    // load phase: lane = 8 consecutive columns (chunk) of the rows lrow, lrow + 8, lrow + 16, lrow + 24 of the tile, so that
    // eight lanes read 128 contiguous bytes; rows past the end repeat the last one and are not stored
    const int chunk = lane & 7, lrow = lane >> 3;
    int64_t rows[4];
#pragma unroll
    for (int i = 0; i < 4; i++) rows[i] = m0 + lrow + 8 * i < p.m ? m0 + lrow + 8 * i : p.m - 1;
    const T* lin = reinterpret_cast<const T*>(p.linear_output);
    const T* wfrag[KB];   // fragment column of this block of k (past the last one: repeats it, never stored), this lane
#pragma unroll
    for (int kb = 0; kb < KB; kb++) wfrag[kb] = reinterpret_cast<const T*>(a.wt) + ((int64_t)min(k0 / 32 + kb, a.kbt - 1) * 64 + lane) * 8;
    char* park = lds + w * (32 * ILB_PARK);
    ilb_f32x16 acc[KB];
#pragma unroll
    for (int kb = 0; kb < KB; kb++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[kb][r] = 0.f;
    const int cbeg = blockIdx.z * a.cols_per_part, cend = min(cbeg + a.cols_per_part, N);
    auto fetch = [&](int c, v8* gf, v8* lf) __attribute__((always_inline)) {
        const int ncol = c + 8 * chunk;
        const int ncl = ncol < N ? ncol : c;   // the last piece may be narrower than 64 columns
        const T* gp = ilb_grad_ptr<T>(a, ncl, 0);
        int gwidth = a.p.split[0];
#pragma unroll
        for (int i = 1; i < 4; i++)
            if (ncl >= a.base[i]) gwidth = a.p.split[i];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            gf[i] = __builtin_nontemporal_load(reinterpret_cast<const v8*>(gp + rows[i] * gwidth));
            lf[i] = __builtin_nontemporal_load(reinterpret_cast<const v8*>(lin + rows[i] * N + ncl));
        }
    };
    v8 gf[4], lf[4];
    int c = cbeg + 64 * w;
    if (c < cend) fetch(c, gf, lf);
    for (; c < cend; c += 256) {
        // the loads of the next piece are in flight while this one is worked on (the last piece asks for itself again)
        v8 gn[4], ln[4];
        fetch(c + 256 < cend ? c + 256 : c, gn, ln);
        const bool live = c + 8 * chunk < N;
        v8 wf[4][KB];   // W^T: columns c + 16 s + 8 g .. + 7 (a step past n re-reads the last one against zeros)
#pragma unroll
        for (int s = 0; s < 4; s++)
#pragma unroll
            for (int kb = 0; kb < KB; kb++) wf[s][kb] = *reinterpret_cast<const v8*>(wfrag[kb] + (int64_t)min(c / 16 + s, N / 16 - 1) * a.kbt * 512);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float d[8];
            ilb_dlin8<T>(gf[i], lf[i], d);
            v8 df;
#pragma unroll
            for (int e = 0; e < 8; e++) df[e] = from_float<T>(live ? d[e] : 0.f);
            *reinterpret_cast<v8*>(park + (lrow + 8 * i) * ILB_PARK + chunk * 16) = df;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int s = 0; s < 4; s++) {
            // row m0 + l32 of dlin, columns c + 16 s + 8 g .. + 7
            const v8 bf = *reinterpret_cast<const v8*>(park + l32 * ILB_PARK + (16 * s + 8 * g) * 2);
#pragma unroll
            for (int kb = 0; kb < KB; kb++) acc[kb] = IlbMM<T>::mfma(wf[s][kb], bf, acc[kb]);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int i = 0; i < 4; i++) { gf[i] = gn[i]; lf[i] = ln[i]; }
    }
    __syncthreads();   // every wave is done with its parked tile before the sums overwrite the buffer
    // accumulator register r of block kb: column k0 + 32 kb + 8 (r / 4) + 4 g + r % 4 of row m0 + l32.
    // Waves 1..3 park their sums, wave 0 adds them to its own in that order and parks the total in the first slot.
    if (w > 0) {
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) red[w - 1][l32][32 * kb + 8 * (r / 4) + 4 * g + (r % 4)] = acc[kb][r];
    }
    __syncthreads();
    if (w == 0) {
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int c = 32 * kb + 8 * (r / 4) + 4 * g + (r % 4);
                red[0][l32][c] = ((acc[kb][r] + red[0][l32][c]) + red[1][l32][c]) + red[2][l32][c];
            }
    }
    __syncthreads();
    // one range of n: the result; several: fp32 partial sums for hstu_ilb_reduce_kernel
    const int as_f32 = a.nparts > 1 || p.grad_dtype == HSTU_F32;
    void* dst = a.nparts > 1 ? (void*)(a.xpart + (int64_t)blockIdx.z * p.m * K) : p.x_grad;
    for (int i = threadIdx.x; i < 32 * KC; i += ILB_NT) {
        const int r = i / KC, cc = i % KC;
        if (m0 + r < p.m && k0 + cc < K) ilb_store<T>(dst, (m0 + r) * K + k0 + cc, red[0][r][cc], as_f32);
    }
}

// weight_grad and bias_grad partial sums.  grid = (ceil(n / (64 NW)), ceil(k / KC), S), NW waves of 64 columns n each.
// FUSED (k <= 64): the parked tile is also multiplied by the wave's 64 rows of W, which stay in registers; the waves'
// products meet in LDS and leave as this workgroup's partial x_grad of the tile (one slab per 64 NW columns of n, added up
// by hstu_ilb_reduce_kernel), so that the gradients and linear_output are streamed once instead of twice.  With four
// waves (64 slabs of 256 columns: as much partial-sum traffic again as half the inputs, two workgroup barriers per 16 KB
// of input) it measured no faster than the two product kernels (458 us at m = n = 16384); with eight waves (32 slabs,
// half the barriers per byte) and one workgroup per CU it takes 292 us.
template <typename T, int KC, bool FUSED, int NW = 4>
__global__ __launch_bounds__(64 * NW) void hstu_ilb_wgrad_kernel(const IlbArgs a) {
    typedef typename IlbMM<T>::v8 v8;
    constexpr int KB = KC / 32;
    constexpr int NT = 64 * NW;   // NW waves of 64 columns each
    __shared__ __attribute__((aligned(16))) char park_all[NW * 32 * ILB_PARK];
    __shared__ float red[FUSED ? NW : 1][FUSED ? 32 : 1][KC + 1];
    const hstu_in_linear_silu_bwd_params& p = a.p;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int g = lane >> 5, l32 = lane & 31;
    const int N = p.n, K = p.k;
    const int nw = blockIdx.x * NT + 64 * w;      // first column of this wave
    const bool wave_on = nw < N;
    if (!FUSED && !wave_on) return;               // whole wave; without FUSED nothing below synchronises across waves
    const int k0 = blockIdx.y * KC;
    const int64_t mbeg = (int64_t)blockIdx.z * a.rows_per_part;
    const int64_t mend = mbeg + a.rows_per_part < p.m ? mbeg + a.rows_per_part : p.m;
    // load phase: lane = 8 consecutive columns (chunk) of the rows lrow, lrow + 8, lrow + 16, lrow + 24 of a tile
    const int chunk = lane & 7, lrow = lane >> 3;
    const int ncol = nw + 8 * chunk;
    const bool live = wave_on && ncol < N;
    const int ncl = live ? ncol : 0;
    int sel = 0;
#pragma unroll
    for (int i = 1; i < 4; i++) sel += ncl >= a.base[i] ? 1 : 0;
    const void* gbase = p.grad[0];
    int gfirst = a.base[0], gwidth = p.split[0];
#pragma unroll
    for (int i = 1; i < 4; i++)
        if (sel == i) { gbase = p.grad[i]; gfirst = a.base[i]; gwidth = p.split[i]; }
    const T* gptr = reinterpret_cast<const T*>(gbase) + (ncl - gfirst);
    const T* lptr = reinterpret_cast<const T*>(p.linear_output) + ncl;
    const T* xfrag[KB];
#pragma unroll
    for (int kb = 0; kb < KB; kb++) xfrag[kb] = reinterpret_cast<const T*>(a.xt) + ((int64_t)min(k0 / 32 + kb, a.kbt - 1) * 64 + lane) * 8;
    char* park = park_all + w * (32 * ILB_PARK);
    ilb_f32x16 acc[2][KB];
#pragma unroll
    for (int nb = 0; nb < 2; nb++)
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[nb][kb][r] = 0.f;
    float bsum[8];
#pragma unroll
    for (int e = 0; e < 8; e++) bsum[e] = 0.f;
    auto fetch = [&](int64_t m0, v8* gf, v8* lf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int64_t r = m0 + lrow + 8 * i;
            const int64_t rc = r < mend ? r : mend - 1;
            gf[i] = __builtin_nontemporal_load(reinterpret_cast<const v8*>(gptr + rc * gwidth));
            lf[i] = __builtin_nontemporal_load(reinterpret_cast<const v8*>(lptr + rc * N));
        }
    };
    v8 wf[FUSED ? 4 : 1][KB];   // FUSED: W^T, columns nw + 16 s + 8 g .. + 7 (a step past n repeats the last one against zeros)
    if constexpr (FUSED) {
#pragma unroll
        for (int s = 0; s < 4; s++)
#pragma unroll
            for (int kb = 0; kb < KB; kb++)
                wf[s][kb] = *reinterpret_cast<const v8*>(reinterpret_cast<const T*>(a.wt) +
                                                         (((int64_t)min(nw / 16 + s, N / 16 - 1) * a.kbt + min(kb, a.kbt - 1)) * 64 + lane) * 8);
    }
    v8 gf[4], lf[4];
    fetch(mbeg, gf, lf);
    for (int64_t m0 = mbeg; m0 < mend; m0 += 32) {
        // the loads of the next tile are in flight while this one is worked on (the last tile asks for itself again)
        v8 gn[4], ln[4];
        fetch(m0 + 32 < mend ? m0 + 32 : m0, gn, ln);
        v8 xf[2][KB];   // x^T: columns m0 + 16 ks + 8 g .. + 7 (zero past m)
#pragma unroll
        for (int ks = 0; ks < 2; ks++)
#pragma unroll
            for (int kb = 0; kb < KB; kb++) xf[ks][kb] = *reinterpret_cast<const v8*>(xfrag[kb] + (m0 / 16 + ks) * a.kbt * 512);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float d[8];
            ilb_dlin8<T>(gf[i], lf[i], d);
            const bool in = live && m0 + lrow + 8 * i < mend;
            v8 df;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float v = in ? d[e] : 0.f;
                bsum[e] += v;
                df[e] = from_float<T>(v);
            }
            *reinterpret_cast<v8*>(park + (lrow + 8 * i) * ILB_PARK + chunk * 16) = df;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
#pragma unroll
            for (int nb = 0; nb < 2; nb++) {
                v8 af;   // column nw + 32 nb + l32 of dlin, rows m0 + 16 ks + 8 g .. + 7
#pragma unroll
                for (int j = 0; j < 8; j++) af[j] = *reinterpret_cast<const T*>(park + (16 * ks + 8 * g + j) * ILB_PARK + (32 * nb + l32) * 2);
#pragma unroll
                for (int kb = 0; kb < KB; kb++) acc[nb][kb] = IlbMM<T>::mfma(af, xf[ks][kb], acc[nb][kb]);
            }
        }
        if constexpr (FUSED) {
            ilb_f32x16 ax[KB];
#pragma unroll
            for (int kb = 0; kb < KB; kb++)
#pragma unroll
                for (int r = 0; r < 16; r++) ax[kb][r] = 0.f;
#pragma unroll
            for (int s = 0; s < 4; s++) {
                // row m0 + l32 of dlin, columns nw + 16 s + 8 g .. + 7
                const v8 bf = *reinterpret_cast<const v8*>(park + l32 * ILB_PARK + (16 * s + 8 * g) * 2);
#pragma unroll
                for (int kb = 0; kb < KB; kb++) ax[kb] = IlbMM<T>::mfma(wf[s][kb], bf, ax[kb]);
            }
            // register r of block kb: column 32 kb + 8 (r / 4) + 4 g + r % 4 of row m0 + l32
#pragma unroll
            for (int kb = 0; kb < KB; kb++)
#pragma unroll
                for (int r = 0; r < 16; r++) red[w][l32][32 * kb + 8 * (r / 4) + 4 * g + (r % 4)] = ax[kb][r];
            __syncthreads();
            float* xp = a.xpart + ((int64_t)blockIdx.x * p.m + m0) * K;
            for (int i = threadIdx.x; i < 32 * KC; i += NT) {
                const int r = i / KC, c = i % KC;
                float sum = red[0][r][c];
#pragma unroll
                for (int ww = 1; ww < NW; ww++) sum += red[ww][r][c];   // in the order of the waves: reproducible
                if (m0 + r < mend && c < K) xp[(int64_t)r * K + c] = sum;
            }
            __syncthreads();
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int i = 0; i < 4; i++) { gf[i] = gn[i]; lf[i] = ln[i]; }
    }
    // accumulator register r of block (nb, kb): row nw + 32 nb + 8 (r / 4) + 4 g + r % 4, column k0 + 32 kb + l32
    float* wp = a.wpart + (int64_t)blockIdx.z * N * K;
#pragma unroll
    for (int nb = 0; nb < 2; nb++)
#pragma unroll
        for (int kb = 0; kb < KB; kb++) {
            const int kc = k0 + 32 * kb + l32;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int nr = nw + 32 * nb + 8 * (r / 4) + 4 * g + (r % 4);
                if (nr < N && kc < K) wp[(int64_t)nr * K + kc] = acc[nb][kb][r];
            }
        }
    if (blockIdx.y == 0) {
        // the eight lanes of one chunk (one per row group) hold the sums of the same 8 columns
#pragma unroll
        for (int e = 0; e < 8; e++) {
            float s = bsum[e];
            s += __shfl_xor(s, 8);
            s += __shfl_xor(s, 16);
            s += __shfl_xor(s, 32);
            bsum[e] = s;
        }
        if (lrow == 0 && live) {
            float* bp = a.bpart + (int64_t)blockIdx.z * N + ncol;
            *reinterpret_cast<ilb_f32x4*>(bp) = ilb_f32x4{bsum[0], bsum[1], bsum[2], bsum[3]};
            *reinterpret_cast<ilb_f32x4*>(bp + 4) = ilb_f32x4{bsum[4], bsum[5], bsum[6], bsum[7]};
        }
    }
}

// out[i] = part[0][i] + part[1][i] + ... in that order, four elements per thread (count is a multiple of 4)
template <typename T>
__global__ __launch_bounds__(256) void hstu_ilb_reduce_kernel(const float* part, int parts, int64_t count, void* out, int as_f32) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= count) return;
    ilb_f32x4 s = *reinterpret_cast<const ilb_f32x4*>(part + i);
    for (int z = 1; z < parts; z++) {
        const ilb_f32x4 v = *reinterpret_cast<const ilb_f32x4*>(part + (int64_t)z * count + i);
#pragma unroll
        for (int e = 0; e < 4; e++) s[e] += v[e];
    }
#pragma unroll
    for (int e = 0; e < 4; e++) ilb_store<T>(out, i + e, s[e], as_f32);
}

struct IlbPlan {
    int kc;               // k columns per workgroup: 64 or 128
    int parts;
    int kbt, nparts, cols_per_part;
    bool fused;
    int64_t rows_per_part, mpad;
    uint64_t off_xt, off_wt, off_wpart, off_bpart, off_xpart, total;
};

static uint64_t ilb_align(uint64_t v) { return (v + 255) & ~(uint64_t)255; }

static IlbPlan ilb_plan(const hstu_in_linear_silu_bwd_params* p) {
    IlbPlan pl;
    pl.kc = p->k > 64 ? 128 : 64;
    const int64_t tiles = (p->m + 31) / 32;
    // one pass over the inputs (k <= 64): the library's choice unless the caller asks for the two product kernels
    pl.fused = p->algorithm == 2 || (p->algorithm == 0 && p->k <= 64);
    // ranges of m: about 1024 workgroups for the two product kernels; the one-pass kernel holds one workgroup of 8 waves per
    // CU, and one round of them (256) measured fastest: 292 us at m = n = 16384 against 310 / 353 us with 512 / 1024
    const int64_t blocks = pl.fused ? (int64_t)((p->n + ILB_FUSED_COLS - 1) / ILB_FUSED_COLS)
                                    : (int64_t)((p->n + 255) / 256) * ((p->k + pl.kc - 1) / pl.kc);
    int64_t parts = ((pl.fused ? 256 : 1024) + blocks - 1) / blocks;
    if (parts > tiles) parts = tiles;
    if (parts < 1) parts = 1;
    pl.rows_per_part = ((tiles + parts - 1) / parts) * 32;
    pl.parts = (int)((p->m + pl.rows_per_part - 1) / pl.rows_per_part);
    pl.mpad = tiles * 32;
    pl.kbt = (p->k + 31) / 32;
    uint64_t o = 0;
    pl.off_xt = o;
    o = ilb_align(o + (uint64_t)(pl.mpad / 16) * pl.kbt * 1024);
    pl.off_wt = o;
    o = ilb_align(o + (uint64_t)(p->n / 16) * pl.kbt * 1024);
    pl.off_wpart = o;
    o = ilb_align(o + (uint64_t)pl.parts * p->n * p->k * 4);
    pl.off_bpart = o;
    o = ilb_align(o + (uint64_t)pl.parts * p->n * 4);
    // x_grad: ranges of n (whole 256-column rounds of a workgroup) until about 1024 workgroups are there
    const int64_t xwgs = tiles * ((p->k + pl.kc - 1) / pl.kc);
    int64_t nparts = (1024 + xwgs / 2) / xwgs;
    const int64_t rounds = (p->n + 255) / 256;
    if (nparts > rounds / 4) nparts = rounds / 4;
    if (nparts < 1) nparts = 1;
    pl.cols_per_part = (int)((rounds + nparts - 1) / nparts) * 256;
    pl.nparts = (p->n + pl.cols_per_part - 1) / pl.cols_per_part;
    // one pass over the inputs: x_grad as one partial slab per 512 columns of n
    if (pl.fused) {
        pl.nparts = (int)((p->n + ILB_FUSED_COLS - 1) / ILB_FUSED_COLS);
        pl.cols_per_part = ILB_FUSED_COLS;
    }
    pl.off_xpart = o;
    if (pl.nparts > 1 || pl.fused) o = ilb_align(o + (uint64_t)pl.nparts * p->m * p->k * 4);
    pl.total = o;
    return pl;
}

static int ilb_check(const hstu_in_linear_silu_bwd_params* p) {
    if (!p) return fail(HSTU_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(hstu_in_linear_silu_bwd_params))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "hstu_in_linear_silu_bwd_params size mismatch: caller %u, library %zu", p->struct_size,
                    sizeof(hstu_in_linear_silu_bwd_params));
    if (p->dtype != HSTU_F16 && p->dtype != HSTU_BF16) return fail(HSTU_ERR_INVALID_ARGUMENT, "dtype expect float16 or bfloat16, but value is %d", p->dtype);
    if (p->grad_dtype != HSTU_F32 && p->grad_dtype != p->dtype)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "grad_dtype expect float32 or the dtype of x, but value is %d", p->grad_dtype);
    if (p->m < 1 || p->m > (1LL << 30)) return fail(HSTU_ERR_INVALID_ARGUMENT, "x dim[0] must in range[1, %lld], but got %lld", 1LL << 30, (long long)p->m);
    int total = 0;
    for (int i = 0; i < 4; i++) {
        if (p->split[i] < 16 || p->split[i] > 8192 || p->split[i] % 16) return fail(HSTU_ERR_INVALID_ARGUMENT, "uvqk dim must in range[16, 8192] and multiples of 16.");
        total += p->split[i];
    }
    if (p->k < 16 || p->k > 8192 || p->k % 16) return fail(HSTU_ERR_INVALID_ARGUMENT, "x dim[1] must in range[16, 8192] and multiples of 16.");
    if (p->n < 64 || p->n > 32768 || p->n % 16) return fail(HSTU_ERR_INVALID_ARGUMENT, "weight dim[0] must in range[64, 32768] and multiples of 16.");
    if (total != p->n) return fail(HSTU_ERR_INVALID_ARGUMENT, "weight_dim[0] must equal to sum(splitList).");
    if (p->n % (4 * p->k)) return fail(HSTU_ERR_INVALID_ARGUMENT, "weight dim[0] must be a multiple of 4 x dim[1]");
    if (p->algorithm < 0 || p->algorithm > 2) return fail(HSTU_ERR_INVALID_ARGUMENT, "algorithm expect 0, 1 or 2, but value is %d", p->algorithm);
    if (p->algorithm == 2 && p->k > 64) return fail(HSTU_ERR_INVALID_ARGUMENT, "algorithm 2 (one pass) needs x dim[1] <= 64, but got %d", p->k);
    return HSTU_OK;
}

}  // namespace hstu

using namespace hstu;

extern "C" int hstu_hip_in_linear_silu_backward_get_workspace_size(const hstu_in_linear_silu_bwd_params* p, uint64_t* workspace_bytes) {
    const int rc = ilb_check(p);
    if (rc != HSTU_OK) return rc;
    if (!workspace_bytes) return fail(HSTU_ERR_INVALID_ARGUMENT, "workspace_bytes is NULL");
    *workspace_bytes = ilb_plan(p).total;
    return HSTU_OK;
}

template <typename T>
static void ilb_launch(const IlbArgs& a, const IlbPlan& pl, hipStream_t st) {
    const hstu_in_linear_silu_bwd_params& p = a.p;
    const int64_t wunits = (int64_t)(p.n / 16) * pl.kbt * 64, xunits = (pl.mpad / 16) * pl.kbt * 64;
    hipLaunchKernelGGL(hstu_ilb_pack_kernel, dim3((unsigned)((wunits + 255) / 256)), dim3(256), 0, st, reinterpret_cast<const uint16_t*>(p.weight),
                       (int64_t)p.n, p.k, pl.kbt, wunits, reinterpret_cast<uint16_t*>(const_cast<void*>(a.wt)));
    hipLaunchKernelGGL(hstu_ilb_pack_kernel, dim3((unsigned)((xunits + 255) / 256)), dim3(256), 0, st, reinterpret_cast<const uint16_t*>(p.x), p.m,
                       p.k, pl.kbt, xunits, reinterpret_cast<uint16_t*>(const_cast<void*>(a.xt)));
    const unsigned kchunks = (unsigned)((p.k + pl.kc - 1) / pl.kc);
    const dim3 gx((unsigned)(pl.mpad / 32), kchunks, (unsigned)pl.nparts), gw((unsigned)((p.n + 255) / 256), kchunks, (unsigned)pl.parts);
    if (pl.fused) {
        const dim3 gf((unsigned)((p.n + ILB_FUSED_COLS - 1) / ILB_FUSED_COLS), kchunks, (unsigned)pl.parts);
        hipLaunchKernelGGL((hstu_ilb_wgrad_kernel<T, 64, true, ILB_FUSED_NW>), gf, dim3(64 * ILB_FUSED_NW), 0, st, a);
    } else if (pl.kc == 64) {
        hipLaunchKernelGGL((hstu_ilb_xgrad_kernel<T, 64>), gx, dim3(ILB_NT), 0, st, a);
        hipLaunchKernelGGL((hstu_ilb_wgrad_kernel<T, 64, false>), gw, dim3(ILB_NT), 0, st, a);
    } else {
        hipLaunchKernelGGL((hstu_ilb_xgrad_kernel<T, 128>), gx, dim3(ILB_NT), 0, st, a);
        hipLaunchKernelGGL((hstu_ilb_wgrad_kernel<T, 128, false>), gw, dim3(ILB_NT), 0, st, a);
    }
    if (pl.nparts > 1 || pl.fused) {
        const int64_t cx = p.m * p.k;
        hipLaunchKernelGGL(hstu_ilb_reduce_kernel<T>, dim3((unsigned)((cx / 4 + 255) / 256)), dim3(256), 0, st, a.xpart, pl.nparts, cx, p.x_grad,
                           (int)(p.grad_dtype == HSTU_F32));
    }
    const int64_t cw = (int64_t)p.n * p.k;
    hipLaunchKernelGGL(hstu_ilb_reduce_kernel<T>, dim3((unsigned)((cw / 4 + 255) / 256)), dim3(256), 0, st, a.wpart, pl.parts, cw, p.weight_grad,
                       (int)(p.grad_dtype == HSTU_F32));
    if (p.bias_grad)
        hipLaunchKernelGGL(hstu_ilb_reduce_kernel<T>, dim3((unsigned)((p.n / 4 + 255) / 256)), dim3(256), 0, st, a.bpart, pl.parts, (int64_t)p.n,
                           (void*)p.bias_grad, 1);
}

extern "C" int hstu_hip_in_linear_silu_backward(const hstu_in_linear_silu_bwd_params* p, void* workspace, uint64_t workspace_bytes, void* stream) {
    const int rc = ilb_check(p);
    if (rc != HSTU_OK) return rc;
    if (!p->x || !p->weight || !p->linear_output || !p->grad[0] || !p->grad[1] || !p->grad[2] || !p->grad[3] || !p->x_grad || !p->weight_grad)
        return fail(HSTU_ERR_INVALID_ARGUMENT, "x, weight, the four gradients, linear_output, x_grad and weight_grad must not be NULL");
    const void* ptrs[] = {p->x, p->weight, p->linear_output, p->grad[0], p->grad[1], p->grad[2], p->grad[3], p->x_grad, p->weight_grad, p->bias_grad, workspace};
    for (const void* q : ptrs)
        if (reinterpret_cast<uintptr_t>(q) & 15) return fail(HSTU_ERR_UNSUPPORTED, "every tensor and the workspace must be 16-byte aligned");
    const IlbPlan pl = ilb_plan(p);
    if (!workspace || workspace_bytes < pl.total)
        return fail(HSTU_ERR_WORKSPACE, "workspace of %llu bytes needed, %llu given", (unsigned long long)pl.total, (unsigned long long)workspace_bytes);
    if (pl.mpad / 32 > 0x7fffffffLL || pl.parts > 65535) return fail(HSTU_ERR_UNSUPPORTED, "m too large for one launch");
    IlbArgs a;
    a.p = *p;
    int total = 0;
    for (int i = 0; i < 4; i++) {
        a.base[i] = total;
        total += p->split[i];
    }
    a.base[4] = total;
    char* ws = reinterpret_cast<char*>(workspace);
    a.xt = ws + pl.off_xt;
    a.wt = ws + pl.off_wt;
    a.wpart = reinterpret_cast<float*>(ws + pl.off_wpart);
    a.bpart = reinterpret_cast<float*>(ws + pl.off_bpart);
    a.mpad = pl.mpad;
    a.kbt = pl.kbt;
    a.xpart = reinterpret_cast<float*>(ws + pl.off_xpart);
    a.nparts = pl.nparts;
    a.cols_per_part = pl.cols_per_part;
    a.rows_per_part = pl.rows_per_part;
    a.parts = pl.parts;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (p->dtype == HSTU_BF16) ilb_launch<__bf16>(a, pl, st);
    else ilb_launch<_Float16>(a, pl, st);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    return HSTU_OK;
}
