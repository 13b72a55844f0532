// Input projection of an HSTU layer: linear_output = x W^T + b, (U | V | Q | K) = silu(linear_output) split along n
// (mxrec::distance_in_linear_silu).  k is an embedding width (tens to a few hundred) and n four times a hidden width
// (thousands), so at 2 * k FLOPs per output element against 4 bytes written the op is bounded by the HBM writes of
// its two [m, n] results, not by the matrix cores: the kernel is an MFMA GEMM without any pipelining of the k loop,
// built around its stores.
//   workgroup = 64 rows m x 128 columns n as 2 x 2 waves; a wave = 32 rows x 64 columns (two 32 x 32 blocks: at 74
//   registers and 6.75 KiB of LDS per wave five waves share a SIMD, which is what keeps the stores flowing; four blocks
//   per wave measured 9 % slower, one block 23 % slower; 4 x 1 waves the same, 1 x 4 waves 8 % slower)
//   out^T block = W x^T: v_mfma_f32_32x32x16 with A = W fragment, B = x fragment; both operands are staged through LDS
//   64 columns of k at a time (loads of 128 contiguous bytes per row; a fragment is one 16-byte LDS read)
//   epilogue: + bias, round -> linear_output; silu of the rounded value, round -> the four outputs; both leave through
//   a per-wave LDS tile so that a lane stores 16 bytes of one output row and a wave instruction covers eight 128-byte runs
// Definition: cust_op/test/in_linear_silu_test/test_in_linear_silu.py:31-45.
#include "hstu_device.h"
#include "../../include/hstu_layer.h"

namespace hstu {

typedef __attribute__((ext_vector_type(8))) __bf16 ils_bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 ils_f16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 ils_bf16x2;
typedef __attribute__((ext_vector_type(2))) _Float16 ils_f16x2;
typedef __attribute__((ext_vector_type(16))) float ils_f32x16;
typedef __attribute__((ext_vector_type(4))) float ils_f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int ils_u4;
typedef __attribute__((ext_vector_type(2))) unsigned int ils_u2;

template <typename T> struct IlsMM;
template <> struct IlsMM<__bf16> {
    typedef ils_bf16x8 v8;
    static __device__ __forceinline__ ils_f32x16 mfma(v8 a, v8 b, ils_f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ unsigned pack2(__bf16 x, __bf16 y) { ils_bf16x2 r; r[0] = x; r[1] = y; return __builtin_bit_cast(unsigned, r); }
};
template <> struct IlsMM<_Float16> {
    typedef ils_f16x8 v8;
    static __device__ __forceinline__ ils_f32x16 mfma(v8 a, v8 b, ils_f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ unsigned pack2(_Float16 x, _Float16 y) { ils_f16x2 r; r[0] = x; r[1] = y; return __builtin_bit_cast(unsigned, r); }
};

constexpr int ILS_NB = 2;                                   // 32 x 32 blocks side by side per wave
constexpr int ILS_WCOLS = 32 * ILS_NB;                      // columns of a wave
constexpr int ILS_WN = 2, ILS_WM = 4 / ILS_WN;              // waves of a workgroup along n and along m
constexpr int ILS_BM = 32 * ILS_WM, ILS_BN = ILS_WCOLS * ILS_WN, ILS_NT = 256;
constexpr int ILS_LPR = ILS_WCOLS / 8, ILS_RPI = 64 / ILS_LPR;   // store phase: lanes per row, rows per instruction
constexpr int ILS_KC = 64, ILS_SROW = ILS_KC * 2 + 16;   // k columns per staging round; bytes of one staged operand row
constexpr int ILS_ROW = ILS_WCOLS * 2 + 16;   // bytes of one parked row: + 16 keeps the 8-byte column writes of 32 rows off one bank

struct IlsArgs {
    hstu_in_linear_silu_params p;
    int base[5];   // first column of user, value, query, key, and n
};

template <typename T>
__global__ __launch_bounds__(ILS_NT) void hstu_in_linear_silu_kernel(const IlsArgs a) {
    typedef typename IlsMM<T>::v8 v8;
    // operand staging of the k loop (x rows of the four waves, then the W rows they share) and, after it, the parked
    // output tiles of the epilogue share one buffer
    static_assert(4 * 32 * ILS_ROW <= (ILS_BM + ILS_BN) * ILS_SROW, "the four parked tiles fit into the staging buffer");
    __shared__ __attribute__((aligned(16))) char park_all[(ILS_BM + ILS_BN) * ILS_SROW];
    const hstu_in_linear_silu_params& p = a.p;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int g = lane >> 5, l32 = lane & 31;
    const int K = p.k, N = p.n;
    // Workgroup i of the 1-D grid runs on XCD i % 8 (each with its own L2).  Tiles are numbered so that one XCD sweeps
    // a contiguous eighth of the n range for a block of rows: what its L2 writes back to HBM is then runs of 32 tiles
    // (4 KiB) per row instead of 256-byte pieces interleaved with the other XCDs' at other times.
    const unsigned nt = (unsigned)(N + ILS_BN - 1) / ILS_BN;
    unsigned tn, tm;
    if (nt % 8 == 0) {
        const unsigned xcd = blockIdx.x & 7, j = blockIdx.x >> 3, per = nt / 8;
        tn = xcd * per + j % per;
        tm = j / per;
    } else {
        tn = blockIdx.x % nt;
        tm = blockIdx.x / nt;
    }
    const int wn = w % ILS_WN, wm = w / ILS_WN;
    const int n0 = tn * ILS_BN + ILS_WCOLS * wn;          // first column and row of this wave
    const int64_t m0 = (int64_t)tm * ILS_BM + 32 * wm;
    const T* x = reinterpret_cast<const T*>(p.x);
    const T* wt = reinterpret_cast<const T*>(p.weight);
    ils_f32x16 acc[ILS_NB];
#pragma unroll
    for (int nb = 0; nb < ILS_NB; nb++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[nb][r] = 0.f;
    // Operands come in through LDS: eight lanes read 128 contiguous bytes of a row (x and W are k-contiguous), each wave
    // a quarter of the workgroup's rows of x and of W; an MFMA fragment is then one
    // 16-byte LDS read (row stride 144 bytes: conflict-free).  Rows past the end repeat the last one (never stored),
    // columns past k are zero.
    {
        const int chunk = lane & 7, lrow = lane >> 3;
        constexpr int XR = ILS_BM / 4, WR = ILS_BN / 4;   // rows of x and of W that one wave brings in
        char* xsh = park_all;
        char* wsh = park_all + ILS_BM * ILS_SROW;
        const int64_t mt = (int64_t)tm * ILS_BM;
        const int ntile = tn * ILS_BN;
        const T* xsrc[XR / 8];
        const T* wsrc[WR / 8];
#pragma unroll
        for (int i = 0; i < XR / 8; i++) {
            const int64_t r = mt + XR * w + lrow + 8 * i;
            xsrc[i] = x + (r < p.m ? r : p.m - 1) * K + 8 * chunk;
        }
#pragma unroll
        for (int i = 0; i < WR / 8; i++) wsrc[i] = wt + (int64_t)min(ntile + WR * w + lrow + 8 * i, N - 1) * K + 8 * chunk;
        for (int k0 = 0; k0 < K; k0 += ILS_KC) {
            const bool in = k0 + 8 * chunk < K;
            v8 xv[XR / 8], wv[WR / 8];
#pragma unroll
            for (int i = 0; i < XR / 8; i++) xv[i] = in ? *reinterpret_cast<const v8*>(xsrc[i] + k0) : v8{};
#pragma unroll
            for (int i = 0; i < WR / 8; i++) wv[i] = in ? *reinterpret_cast<const v8*>(wsrc[i] + k0) : v8{};
#pragma unroll
            for (int i = 0; i < XR / 8; i++) *reinterpret_cast<v8*>(xsh + (XR * w + lrow + 8 * i) * ILS_SROW + chunk * 16) = xv[i];
#pragma unroll
            for (int i = 0; i < WR / 8; i++) *reinterpret_cast<v8*>(wsh + (WR * w + lrow + 8 * i) * ILS_SROW + chunk * 16) = wv[i];
            __syncthreads();
#pragma unroll
            for (int s = 0; s < ILS_KC / 16; s++) {
                const v8 xf = *reinterpret_cast<const v8*>(xsh + (32 * wm + l32) * ILS_SROW + (16 * s + 8 * g) * 2);
#pragma unroll
                for (int nb = 0; nb < ILS_NB; nb++) {
                    const v8 wf = *reinterpret_cast<const v8*>(wsh + (ILS_WCOLS * wn + 32 * nb + l32) * ILS_SROW + (16 * s + 8 * g) * 2);
                    acc[nb] = IlsMM<T>::mfma(wf, xf, acc[nb]);
                }
            }
            __syncthreads();
        }
    }
    // accumulator register r of block nb holds column n0 + 32 nb + 8 (r / 4) + 4 g + r % 4 of row m0 + l32
    char* park = park_all + w * (32 * ILS_ROW);
    T lin[ILS_NB][16];
#pragma unroll
    for (int nb = 0; nb < ILS_NB; nb++) {
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
            ils_f32x4 b = {0.f, 0.f, 0.f, 0.f};
            const int col = n0 + 32 * nb + 8 * rr + 4 * g;
            if (p.bias && col < N) b = *reinterpret_cast<const ils_f32x4*>(p.bias + col);
#pragma unroll
            for (int e = 0; e < 4; e++) lin[nb][4 * rr + e] = from_float<T>(acc[nb][4 * rr + e] + b[e]);
        }
    }
    const int orow = lane / ILS_LPR, ochunk = lane % ILS_LPR;   // store phase: a lane = 8 columns of a row
    const int col = n0 + 8 * ochunk;
    int which = 0;
#pragma unroll
    for (int sidx = 1; sidx < 4; sidx++) which += col >= a.base[sidx] ? 1 : 0;
#pragma unroll
    for (int phase = 0; phase < 2; phase++) {
#pragma unroll
        for (int nb = 0; nb < ILS_NB; nb++) {
#pragma unroll
            for (int rr = 0; rr < 4; rr++) {
                T v[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const T l = lin[nb][4 * rr + e];
                    if (phase == 0) v[e] = l;
                    else {
                        const float f = to_float(l);
                        v[e] = from_float<T>(f * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504f * f)));
                    }
                }
                ils_u2 o = {IlsMM<T>::pack2(v[0], v[1]), IlsMM<T>::pack2(v[2], v[3])};
                *reinterpret_cast<ils_u2*>(park + l32 * ILS_ROW + (32 * nb + 8 * rr + 4 * g) * 2) = o;
            }
        }
        __builtin_amdgcn_wave_barrier();
        if (col < N) {
            T* dst;
            int64_t stride;
            if (phase == 0) { dst = reinterpret_cast<T*>(p.linear_output) + col; stride = N; }
            else {
                void* o = p.out[0];
                int first = a.base[0], width = p.split[0];
#pragma unroll
                for (int sidx = 1; sidx < 4; sidx++)
                    if (which == sidx) { o = p.out[sidx]; first = a.base[sidx]; width = p.split[sidx]; }
                dst = reinterpret_cast<T*>(o) + (col - first);
                stride = width;
            }
#pragma unroll
            for (int i = 0; i < 32 / ILS_RPI; i++) {
                const int row = ILS_RPI * i + orow;
                const ils_u4 v = *reinterpret_cast<const ils_u4*>(park + row * ILS_ROW + ochunk * 16);
                if (m0 + row < p.m) __builtin_nontemporal_store(v, reinterpret_cast<ils_u4*>(dst + (m0 + row) * stride));
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
}

}  // namespace hstu

using namespace hstu;

extern "C" int hstu_hip_in_linear_silu(const hstu_in_linear_silu_params* p, void* stream) {
    if (!p) return fail(HSTU_ERR_INVALID_ARGUMENT, "params is NULL");
    if (p->struct_size != sizeof(hstu_in_linear_silu_params))
        return fail(HSTU_ERR_INVALID_ARGUMENT, "hstu_in_linear_silu_params size mismatch: caller %u, library %zu", p->struct_size,
                    sizeof(hstu_in_linear_silu_params));
    if (p->dtype != HSTU_F16 && p->dtype != HSTU_BF16) return fail(HSTU_ERR_INVALID_ARGUMENT, "dtype expect float16 or bfloat16, but value is %d", p->dtype);
    if (p->m < 1 || p->m > (1LL << 30)) return fail(HSTU_ERR_INVALID_ARGUMENT, "x dim[0] must in range[1, %lld], but got %lld", 1LL << 30, (long long)p->m);
    if (((p->n + ILS_BN - 1) / ILS_BN) * ((p->m + ILS_BM - 1) / ILS_BM) > 0x7fffffffLL) return fail(HSTU_ERR_UNSUPPORTED, "m * n too large for one launch");
    IlsArgs a;
    a.p = *p;
    int total = 0;
    for (int i = 0; i < 4; i++) {
        if (p->split[i] < 16 || p->split[i] > 8192 || p->split[i] % 16) return fail(HSTU_ERR_INVALID_ARGUMENT, "uvqk dim must in range[16, 8192] and multiples of 16.");
        a.base[i] = total;
        total += p->split[i];
    }
    a.base[4] = total;
    if (p->k < 16 || p->k > 8192 || p->k % 16) return fail(HSTU_ERR_INVALID_ARGUMENT, "x dim[1] must in range[16, 8192] and multiples of 16.");
    if (p->n < 64 || p->n > 32768 || p->n % 16) return fail(HSTU_ERR_INVALID_ARGUMENT, "weight dim[0] must in range[64, 32768] and multiples of 16.");
    if (total != p->n) return fail(HSTU_ERR_INVALID_ARGUMENT, "weight_dim[0] must equal to sum(splitList).");
    if (p->n % (4 * p->k)) return fail(HSTU_ERR_INVALID_ARGUMENT, "weight dim[0] must be a multiple of 4 x dim[1]");
    if (!p->x || !p->weight || !p->linear_output || !p->out[0] || !p->out[1] || !p->out[2] || !p->out[3])
        return fail(HSTU_ERR_INVALID_ARGUMENT, "x, weight, the four outputs and linear_output must not be NULL");
    const void* ptrs[] = {p->x, p->weight, p->bias, p->linear_output, p->out[0], p->out[1], p->out[2], p->out[3]};
    for (const void* q : ptrs)
        if (reinterpret_cast<uintptr_t>(q) & 15) return fail(HSTU_ERR_UNSUPPORTED, "x, weight, bias and the outputs must be 16-byte aligned");
    const dim3 grid((unsigned)((p->n + ILS_BN - 1) / ILS_BN) * (unsigned)((p->m + ILS_BM - 1) / ILS_BM));
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (p->dtype == HSTU_BF16) hipLaunchKernelGGL(hstu_in_linear_silu_kernel<__bf16>, grid, dim3(ILS_NT), 0, st, a);
    else hipLaunchKernelGGL(hstu_in_linear_silu_kernel<_Float16>, grid, dim3(ILS_NT), 0, st, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    return HSTU_OK;
}
