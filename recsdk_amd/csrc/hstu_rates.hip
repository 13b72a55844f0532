// Diagnostics: issue rates of the pieces of one 32 x 32 score block (SiLU, the two MFMA chains, both together) at 1..4
// waves per SIMD, with operands the caller chooses.  Declared in include/hstu_diag.h; used by `bench.py --workload rates`.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/hstu_diag.h"

namespace hstu_rates {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;

__device__ __forceinline__ unsigned pack2(float x, float y) {
    bf16x2 r; r[0] = (__bf16)x; r[1] = (__bf16)y;
    return __builtin_bit_cast(unsigned, r);
}

template <int MODE, int WAVES>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(WAVES, WAVES)))
rate_kernel(const u32x4* __restrict__ in, float* __restrict__ out, unsigned long long* __restrict__ ticks, int iters, float c) {
    const int tid = threadIdx.x + blockIdx.x * blockDim.x;
    // operands: 16 chunks of 16 bytes per thread out of the 65536 chunks of the buffer
    bf16x8 a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        a[i] = __builtin_bit_cast(bf16x8, in[(tid * 16 + i) & 65535]);
        b[i] = __builtin_bit_cast(bf16x8, in[(tid * 16 + 8 + i) & 65535]);
    }
    f32x16 o[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[j][r] = 0.f;
    float x[16];
#pragma unroll
    for (int r = 0; r < 16; r++) x[r] = 0.001f * (tid & 63) + 0.01f * r;
    f32x16 sc;
    u32x4 pp0 = in[tid & 1023], pp1 = in[(tid + 77) & 1023];
#pragma unroll
    for (int r = 0; r < 16; r++) sc[r] = x[r];
    __syncthreads();
    const unsigned long long t0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; it++) {
        if (MODE == HSTU_RATE_SILU) {
            u32x4 p0, p1;
            float pf[16];
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float e = __builtin_amdgcn_exp2f(x[r] * c);
                pf[r] = x[r] * __builtin_amdgcn_rcpf(1.0f + e);
            }
#pragma unroll
            for (int q = 0; q < 4; q++) { p0[q] = pack2(pf[2 * q], pf[2 * q + 1]); p1[q] = pack2(pf[8 + 2 * q], pf[9 + 2 * q]); }
            // feed the packed values back so that the next iteration depends on this one
#pragma unroll
            for (int q = 0; q < 4; q++) {
                x[q] += __builtin_bit_cast(float, p0[q] & 0x3fffffff);
                x[4 + q] += __builtin_bit_cast(float, p1[q] & 0x3fffffff);
            }
        } else if (MODE == HSTU_RATE_MFMA_FP8) {
            const i32x8 a8 = __builtin_bit_cast(i32x8, (u32x4[2]){__builtin_bit_cast(u32x4, a[0]), __builtin_bit_cast(u32x4, a[1])});
            const i32x8 b8 = __builtin_bit_cast(i32x8, (u32x4[2]){__builtin_bit_cast(u32x4, b[0]), __builtin_bit_cast(u32x4, b[1])});
#pragma unroll
            for (int j = 0; j < 4; j++) o[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, o[j], 0, 0, 0, 0, 0, 0);
        } else if (MODE == HSTU_RATE_PIPELINED) {
            f32x16 sn;
#pragma unroll
            for (int r = 0; r < 16; r++) sn[r] = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[i], sn, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; j++) o[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j], __builtin_bit_cast(bf16x8, pp0), o[j], 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; j++) o[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[4 + j], __builtin_bit_cast(bf16x8, pp1), o[j], 0, 0, 0);
            float pf[16];
            u32x4 q0, q1;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float e = __builtin_amdgcn_exp2f(sc[r] * c);
                pf[r] = sc[r] * __builtin_amdgcn_rcpf(1.0f + e);
            }
#pragma unroll
            for (int q = 0; q < 4; q++) { q0[q] = pack2(pf[2 * q], pf[2 * q + 1]); q1[q] = pack2(pf[8 + 2 * q], pf[9 + 2 * q]); }
            // one matrix instruction, then four vector and two transcendental ones, sixteen times
#pragma unroll
            for (int g = 0; g < 16; g++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
                __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);
            }
            pp0 = q0; pp1 = q1; sc = sn;
        } else {
            f32x16 s;
#pragma unroll
            for (int r = 0; r < 16; r++) s[r] = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[i], s, 0, 0, 0);
            u32x4 p0, p1;
            if (MODE == HSTU_RATE_BLOCK) {
                float pf[16];
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const float e = __builtin_amdgcn_exp2f(s[r] * c);
                    pf[r] = s[r] * __builtin_amdgcn_rcpf(1.0f + e);
                }
#pragma unroll
                for (int q = 0; q < 4; q++) { p0[q] = pack2(pf[2 * q], pf[2 * q + 1]); p1[q] = pack2(pf[8 + 2 * q], pf[9 + 2 * q]); }
            } else {
#pragma unroll
                for (int q = 0; q < 4; q++) { p0[q] = __builtin_bit_cast(unsigned, s[q]); p1[q] = __builtin_bit_cast(unsigned, s[4 + q]); }
            }
#pragma unroll
            for (int j = 0; j < 4; j++) o[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j], __builtin_bit_cast(bf16x8, p0), o[j], 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; j++) o[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[4 + j], __builtin_bit_cast(bf16x8, p1), o[j], 0, 0, 0);
        }
    }
    const unsigned long long t1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
    float s = 0;
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) s += o[j][r];
#pragma unroll
    for (int r = 0; r < 16; r++) s += x[r] + sc[r];
    s += __builtin_bit_cast(float, pp0[0] ^ pp1[3]);
    out[tid] = s;
    if (threadIdx.x == 0) {
        ticks[2 * blockIdx.x] = t1 - t0;
        ticks[2 * blockIdx.x + 1] = r1 - r0;
    }
}

template <int MODE>
static int launch_mode(int waves, int iters, const u32x4* in, float* out, unsigned long long* ticks, hipStream_t st) {
    const float c = -0.127f;
    switch (waves) {
        case 1: hipLaunchKernelGGL((rate_kernel<MODE, 1>), dim3(256), dim3(256), 0, st, in, out, ticks, iters, c); break;
        case 2: hipLaunchKernelGGL((rate_kernel<MODE, 2>), dim3(512), dim3(256), 0, st, in, out, ticks, iters, c); break;
        case 3: hipLaunchKernelGGL((rate_kernel<MODE, 3>), dim3(768), dim3(256), 0, st, in, out, ticks, iters, c); break;
        case 4: hipLaunchKernelGGL((rate_kernel<MODE, 4>), dim3(1024), dim3(256), 0, st, in, out, ticks, iters, c); break;
        default: return -1;
    }
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace hstu_rates

extern "C" int hstu_hip_measure_block_rates(int mode, int waves_per_simd, int iters, const void* operands, float* sink, uint64_t* ticks, void* stream) {
    using namespace hstu_rates;
    if (!operands || !sink || !ticks || iters < 1 || waves_per_simd < 1 || waves_per_simd > 4) return -1;
    // occupancies at which a mode's registers no longer fit (it would measure spills)
    if (((mode == HSTU_RATE_MFMA || mode == HSTU_RATE_BLOCK) && waves_per_simd > 3) || (mode == HSTU_RATE_PIPELINED && waves_per_simd > 2)) return -1;
    const u32x4* in = reinterpret_cast<const u32x4*>(operands);
    unsigned long long* tk = reinterpret_cast<unsigned long long*>(ticks);
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    switch (mode) {
        case HSTU_RATE_SILU: return launch_mode<HSTU_RATE_SILU>(waves_per_simd, iters, in, sink, tk, st);
        case HSTU_RATE_MFMA: return launch_mode<HSTU_RATE_MFMA>(waves_per_simd, iters, in, sink, tk, st);
        case HSTU_RATE_BLOCK: return launch_mode<HSTU_RATE_BLOCK>(waves_per_simd, iters, in, sink, tk, st);
        case HSTU_RATE_PIPELINED: return launch_mode<HSTU_RATE_PIPELINED>(waves_per_simd, iters, in, sink, tk, st);
        case HSTU_RATE_MFMA_FP8: return launch_mode<HSTU_RATE_MFMA_FP8>(waves_per_simd, iters, in, sink, tk, st);
        default: return -1;
    }
}
