// HSTU forward for float8_e4m3fn q / k / v on the gfx950 matrix cores (head dim 64, 128 or 256, built-in mask or none,
// GQA, delta-q; fp16 output).  The reference's fp8 path: hstu_jagged.cpp:53-54 (fp16 output for fp8 inputs), golden
// test_hstu_jagged_forward.py:150-189: operands up-cast exactly, scores and sums in fp32, P = silu(alpha * S) * silu_scale
// * mask rounded to e4m3 before P V.
//
// Same scheme as the 16-bit kernel, on v_mfma_f32_32x32x64_f8f6f4 (64 products per lane and instruction, twice the
// 16-bit rate): a workgroup (4 waves) owns a 128-row Q tile of one (sequence, head), wave w rows 32w..32w+31; K and V
// tiles of 64 keys stream through LDS (two stages, fetched into registers one tile ahead, one barrier per tile).
// Per tile and wave:
//     S^T = K Q^T      two 32-key blocks; A = K rows (32 bytes of the head dim per lane: 2 x ds_read_b128), B = Q rows
//                      (registers).  Lane half g of both operands holds head-dim bytes 64t + 32g .. + 31: the k index of a
//                      (lane half, byte) is the same for A and B, which is all a dot product needs.
//     P                s * sigmoid(alpha * s) * alpha * silu_scale in fp32, rounded to e4m3 (v_cvt_pk_fp8_f32), masked
//     O^T += V^T P^T   one instruction per 32 head-dim columns covers all 64 keys: B = the 32 P bytes of the lane, A = V^T
//                      from four transposing reads (ds_read_b64_tr_b8: 8 consecutive keys of one column per lane)
// A-row rho of an S^T block holds key (rho with bits 2 and 3 swapped): accumulator registers 8u..8u+7 of lane half g are
// then keys 16u + 8g .. + 7 of the block, 8 consecutive keys per transposing read.  alpha * silu_scale cannot move to the
// epilogue here: it decides where P falls on the e4m3 grid.
#include "hstu_device.h"
#include "hstu_self_sched.h"

namespace hstu {

typedef __attribute__((ext_vector_type(8))) int q_i32x8;
typedef __attribute__((ext_vector_type(2))) int q_i32x2;
typedef __attribute__((ext_vector_type(4))) unsigned int q_u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int q_u32x2;
typedef __attribute__((ext_vector_type(16))) float q_f32x16;
typedef __attribute__((ext_vector_type(2))) _Float16 q_f16x2;

#define FP8_LDS_PTR(type, p) ((__attribute__((address_space(3))) type*)(p))

constexpr int FBM = 128;   // Q rows per workgroup
constexpr int FBN = 64;    // keys per step

enum { FBLK_ALL = 0, FBLK_CAUSAL = 1, FBLK_PRED = 2, FBLK_SKIP = 3 };

// visibility class of Q rows r0..r0+31 against keys c0..c0+31 under the built-in mask
__device__ __forceinline__ int fp8_classify(const Seq& s, int tgs, int r0, int c0) {
    const bool has_ctx = s.ctx > 0 && r0 < s.ctx;
    const bool has_tgt = s.tgt > 0 && tgs > 0 && r0 + 31 >= s.hist_q && c0 + 31 >= s.hist_k;
    if (!has_ctx && c0 > r0 + 31 + s.delta) return FBLK_SKIP;
    if (has_ctx || has_tgt) return FBLK_PRED;
    if (c0 + 31 <= r0 + s.delta) return FBLK_ALL;
    return FBLK_CAUSAL;
}

// Waves per SIMD: as many as the registers allow (each more hides more of the LDS and matrix-core latency: measured 14 %
// from 2 to 3 at head dim 64 and 11 % at 128, 4 % from 3 to 4 at 64); head dim 256 needs a whole SIMD lane's registers.
template <int D> struct Fp8Shape { static constexpr int WAVES = D == 64 ? 4 : (D == 128 ? 3 : 1); };

// UNEVEN: head dims that are other multiples of 16 up to D, and dim_qk != dim_v (the reference's fp8 sweep draws dim_v from
// 16 .. 80, test_hstu_jagged_forward.py): rows have their real widths in memory, the chunks past them are zeros in the
// fragments and in LDS, the output keeps its dim_v columns.
// SELF: no schedule kernel; every wave derives the workgroup's record from the offsets (self_record) and wave 0 leaves it in
// the workspace, where the schedule kernel would have put it.
template <int D, bool UNEVEN = false, bool SELF = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(Fp8Shape<D>::WAVES, Fp8Shape<D>::WAVES)))
void hstu_mfma_fp8_kernel(const KArgs a, const unsigned* __restrict__ ws) {
    const hstu_fwd_params& p = a.p;
    const int dq_real = UNEVEN ? p.dim_qk : D, dv_real = UNEVEN ? p.dim_v : D;
    // row strides in bytes: +16 keeps the 16-byte row-wise reads of 16 K rows on distinct banks, +32 does the same for
    // the 8-row transposing reads of V
    constexpr int KS = D + 16, VS = D + 32;
    constexpr int NCH = D / 64;          // 16-byte chunks per thread, tile and tensor
    constexpr int CPR = D / 16;          // chunks per row
    __shared__ __attribute__((aligned(16))) unsigned char kst[2][FBN * KS];
    __shared__ __attribute__((aligned(16))) unsigned char vst[2][FBN * VS];

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 5, l32 = lane & 31;

    // workgroup -> record of the device-built work list
    unsigned rw[WORK_RECORD_WORDS];
    int64_t owned_rows;
    if constexpr (SELF) {
        __shared__ unsigned lds_hist[4 * 64];
        unsigned rv[WORK_RECORD_WORDS];
        if (p.seq_offset_k == p.seq_offset_q) self_record<true, false>(a, (p.max_seq_len_q + FBM - 1) / FBM, lane, lds_hist + 64 * w, rv, owned_rows);
        else self_record<true, true>(a, (p.max_seq_len_q + FBM - 1) / FBM, lane, lds_hist + 64 * w, rv, owned_rows);
#pragma unroll
        for (int i = 0; i < WORK_RECORD_WORDS; i++) rw[i] = __builtin_amdgcn_readfirstlane(rv[i]);
        if (tid < WORK_RECORD_WORDS) {
            const unsigned val = tid == 0 ? rw[0] : ((tid == 1 || tid == 3) ? rw[1] : ((tid == 2 || tid == 4) ? rw[2] : (tid == 6 ? rw[6] : 0u)));
            const_cast<unsigned*>(ws)[WORK_HEADER_WORDS + WORK_RECORD_WORDS * (size_t)blockIdx.x + tid] = val;
        }
        if (blockIdx.x == 0 && tid == 0) {
            const_cast<unsigned*>(ws)[0] = 0u;
            *reinterpret_cast<int64_t*>(const_cast<unsigned*>(ws) + 2) = owned_rows;
        }
    } else {
        const unsigned* rec = ws + WORK_HEADER_WORDS + WORK_RECORD_WORDS * (size_t)blockIdx.x;
#pragma unroll
        for (int i = 0; i < WORK_RECORD_WORDS; i++) rw[i] = rec[i];
        owned_rows = *reinterpret_cast<const int64_t*>(ws + 2);
    }
    const unsigned item = rw[0];
    const bool active = item != WORK_ITEM_EMPTY;
    const int b = active ? (int)(item & 0xfff) : 0, h = active ? (int)((item >> 12) & 0xf) : 0;
    const int tile0 = (int)((item >> 16) & 0xff);
    const int tile_last = ((item >> 24) & 1) ? 0x7fffff : tile0 + (int)((item >> 25) & 7);
    const int hk = h / a.head_ratio;
    Seq s;
    s.q_start = active ? (int)rw[1] : 0; s.lq = active ? (int)rw[2] : 0;
    s.k_start = active ? (int)rw[3] : 0; s.lk = active ? (int)rw[4] : 0;
    s.ctx = active ? (int)rw[5] : 0; s.tgt = active ? (int)rw[6] : 0; s.page0 = 0;
    s.delta = s.lk - s.lq; s.hist_q = s.lq - s.tgt; s.hist_k = s.lk - s.tgt; s.cand_row = s.q_start + s.hist_q;
    (void)b;
    const bool tril = p.mask_type == HSTU_MASK_TRIL;
    const int tgs = p.target_group_size;
    const float inv_scale = 1.0f / a.out_scale;   // +-inf when alpha is 0: P = x * rcp(inf) = 0, as x * sigmoid(0) * 0
    const unsigned char* qbase = reinterpret_cast<const unsigned char*>(p.q);
    const unsigned char* kbase = reinterpret_cast<const unsigned char*>(p.k);
    const unsigned char* vbase = reinterpret_cast<const unsigned char*>(p.v);
    _Float16* obase = reinterpret_cast<_Float16*>(p.out);

    // K fragment: A-row l32 holds key (l32 with bits 2 and 3 swapped) of the block
    const int krow = (l32 & 0x13) | ((l32 & 4) << 1) | ((l32 & 8) >> 1);
    const int kfrag_off = krow * KS + 32 * g;
    // V^T fragment: lane i of a 16-lane group addresses 8 bytes of key row i / 2; the group receives columns
    // 16 * (group % 2) .. + 15, keys 8 * g .. + 7 of the 16-key step
    const int vfrag_off = (8 * g + ((lane & 15) >> 1)) * VS + 16 * ((lane >> 4) & 1) + 8 * (lane & 1);

    for (int tile = tile0; active && tile <= tile_last && tile * FBM < s.lq; tile++) {
        const int i0 = tile * FBM;
        const int kend = (s.lk > 0) ? k_extent(a, s, i0, min(i0 + FBM, s.lq)) : 0;
        const int ntk = (kend + FBN - 1) / FBN;
        const int r0 = i0 + 32 * w;
        const int qi = r0 + l32;
        const bool qvalid = qi < s.lq;

        // Q fragments (B operand of S^T = K Q^T): column = Q row, lane half g holds head-dim bytes 64t + 32g .. + 31
        q_i32x8 qf[D / 64];
        {
            const unsigned char* qp = qbase + ((s.q_start + min(qi, s.lq - 1)) * p.heads_q + h) * (int64_t)dq_real + 32 * g;
#pragma unroll
            for (int t = 0; t < D / 64; t++) {
                const q_u32x4 z = {0, 0, 0, 0};
                const bool have0 = !UNEVEN || 64 * t + 32 * g < dq_real, have1 = !UNEVEN || 64 * t + 32 * g + 16 < dq_real;
                q_u32x4 x0 = *reinterpret_cast<const q_u32x4*>(have0 ? qp + 64 * t : qp - 32 * g);
                q_u32x4 x1 = *reinterpret_cast<const q_u32x4*>(have1 ? qp + 64 * t + 16 : qp - 32 * g);
                x0 = qvalid && have0 ? x0 : z;
                x1 = qvalid && have1 ? x1 : z;
                qf[t] = (q_i32x8){(int)x0[0], (int)x0[1], (int)x0[2], (int)x0[3], (int)x1[0], (int)x1[1], (int)x1[2], (int)x1[3]};
            }
        }
        q_f32x16 oacc[D / 32];
#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[db][r] = 0.f;

        // tile loader: thread t copies 16-byte chunk t % CPR of rows t / CPR (+ 256 / CPR per further chunk) of K and of V.
        // Offsets are 32-bit, relative to the first row of this sequence and kv head (a sequence spans at most
        // 20480 * 16 * 256 bytes)
        const unsigned rowstride = (unsigned)p.heads_k * dq_real, rowstride_v = (unsigned)p.heads_k * dv_real;
        const unsigned char* kseq = kbase + (s.k_start * p.heads_k + hk) * (int64_t)dq_real;
        const unsigned char* vseq = vbase + (s.k_start * p.heads_k + hk) * (int64_t)dv_real;
        const int lrow = tid / CPR, lcc = tid % CPR;
        // (uneven dims: a chunk past the real row width is read from chunk 0 and zeroed when written to LDS)
        const bool kchunk = !UNEVEN || 16 * lcc < dq_real, vchunk = !UNEVEN || 16 * lcc < dv_real;
        q_u32x4 nk[NCH], nv[NCH];
        auto fetch = [&](int kt) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                // nothing here waits for the data; rows past the end are read from the last row and zeroed in stash()
                const int row = min(kt * FBN + lrow + (256 / CPR) * i, kend - 1);
                nk[i] = *reinterpret_cast<const q_u32x4*>(kseq + __umul24((unsigned)row, rowstride) + (kchunk ? 16u * lcc : 0u));
                nv[i] = *reinterpret_cast<const q_u32x4*>(vseq + __umul24((unsigned)row, rowstride_v) + (vchunk ? 16u * lcc : 0u));
            }
        };
        auto stash = [&](int kt, int stage) __attribute__((always_inline)) {
            unsigned char* kd = kst[stage] + lrow * KS + 16 * lcc;
            unsigned char* vd = vst[stage] + lrow * VS + 16 * lcc;
            if (!UNEVEN && (kt + 1) * FBN <= kend) {   // wave-uniform: every row of the tile exists
#pragma unroll
                for (int i = 0; i < NCH; i++) {
                    *reinterpret_cast<q_u32x4*>(kd + (256 / CPR) * i * KS) = nk[i];
                    *reinterpret_cast<q_u32x4*>(vd + (256 / CPR) * i * VS) = nv[i];
                }
            } else {
                // the last tile: zero rows past the end (S = 0 gives P = 0, and 0 * V must not meet a NaN)
#pragma unroll
                for (int i = 0; i < NCH; i++) {
                    const bool ok = kt * FBN + lrow + (256 / CPR) * i < kend;
                    const q_u32x4 z = {0, 0, 0, 0};
                    *reinterpret_cast<q_u32x4*>(kd + (256 / CPR) * i * KS) = ok && kchunk ? nk[i] : z;
                    *reinterpret_cast<q_u32x4*>(vd + (256 / CPR) * i * VS) = ok && vchunk ? nv[i] : z;
                }
            }
        };
        __syncthreads();   // every wave is done with the stages of the previous tile
        if (ntk > 0) {
            fetch(0);
            stash(0, 0);
        }
        __syncthreads();

        for (int kt = 0; kt < ntk; kt++) {
            const int stage = kt & 1;
            const int k0 = kt * FBN;
            if (kt + 1 < ntk) fetch(kt + 1);
            // visibility class of the two 32-key blocks (wave-uniform).  A block past the K extent holds zero rows (P = 0
            // without a mask); a block the causal mask hides completely is masked like one it cuts (all bytes to zero), so
            // that the tile is straight-line code
            int cls[2];
            bool any = false;
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
                const int c0 = k0 + 32 * kb;
                const int c = (c0 >= kend || !tril) ? FBLK_ALL : fp8_classify(s, tgs, r0, c0);
                any |= c0 < kend && c != FBLK_SKIP;
                cls[kb] = c == FBLK_SKIP ? FBLK_CAUSAL : c;
            }
            if (any) {
                const unsigned char* kt_lds = kst[stage];
                const unsigned char* vt_lds = vst[stage];
                // ---- S^T of both blocks: all K fragments are requested before the first product
                q_i32x8 kf[2][D / 64];
#pragma unroll
                for (int kb = 0; kb < 2; kb++)
#pragma unroll
                    for (int t = 0; t < D / 64; t++) {
                        const unsigned char* at = kt_lds + 32 * kb * KS + kfrag_off + 64 * t;
                        const q_u32x4 x0 = *reinterpret_cast<const q_u32x4*>(at);
                        const q_u32x4 x1 = *reinterpret_cast<const q_u32x4*>(at + 16);
                        kf[kb][t] = (q_i32x8){(int)x0[0], (int)x0[1], (int)x0[2], (int)x0[3], (int)x1[0], (int)x1[1], (int)x1[2], (int)x1[3]};
                    }
                q_f32x16 sacc[2];
#pragma unroll
                for (int kb = 0; kb < 2; kb++) {
#pragma unroll
                    for (int r = 0; r < 16; r++) sacc[kb][r] = 0.f;
#pragma unroll
                    for (int t = 0; t < D / 64; t++)
                        sacc[kb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kf[kb][t], qf[t], sacc[kb], 0, 0, 0, 0, 0, 0);
                }
                // V^T fragments: at head dim 64 requested now and used after the SiLU pass; the wider ones have no registers to
                // hold them that long
                q_i32x2 vq[D / 32][4];
                if (D <= 64) {
#pragma unroll
                    for (int db = 0; db < D / 32; db++)
#pragma unroll
                        for (int c = 0; c < 4; c++)
                            vq[db][c] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(FP8_LDS_PTR(q_i32x2, vt_lds + 16 * c * VS + vfrag_off + 32 * db));
                }
                // ---- P = x * sigmoid(alpha * x) * alpha * silu_scale = x / ((1 + e) / (alpha * silu_scale)), to e4m3: register
                // 8u + i of block kb -> byte i of step 2 kb + u
                unsigned pq[8];   // P of this lane's Q row: byte 8c + i = key k0 + 16c + 8g + i
#pragma unroll
                for (int kb = 0; kb < 2; kb++) {
#pragma unroll
                    for (int x = 0; x < 4; x++) {
                        float pv[4];
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const float sc = sacc[kb][4 * x + i];
                            const float e = __builtin_amdgcn_exp2f(sc * a.exp_scale);
                            pv[i] = sc * __builtin_amdgcn_rcpf(__builtin_fmaf(e, inv_scale, inv_scale));
                        }
                        // both halves of the word are written: its initial value is irrelevant, and a live register saves a move
                        int word = __builtin_amdgcn_cvt_pk_fp8_f32(pv[0], pv[1], __builtin_bit_cast(int, pv[0]), false);
                        word = __builtin_amdgcn_cvt_pk_fp8_f32(pv[2], pv[3], word, true);
                        pq[4 * kb + x] = (unsigned)word;
                    }
                    // word x of the block covers keys c0 + 16 * (x / 2) + 8g + 4 * (x % 2) .. + 3
                    const int c0 = k0 + 32 * kb;
                    if (cls[kb] == FBLK_CAUSAL) {
#pragma unroll
                        for (int x = 0; x < 4; x++) {
                            const int lim = qi + s.delta - (c0 + 16 * (x >> 1) + 8 * g + 4 * (x & 1));   // key offset o of the word is visible iff o <= lim
                            pq[4 * kb + x] &= lim >= 3 ? 0xffffffffu : (lim < 0 ? 0u : (0xffffffffu >> (8 * (3 - lim))));
                        }
                    } else if (cls[kb] == FBLK_PRED) {
                        // branch-free form of builtin_visible()
                        const bool ctx_row = s.ctx > 0 && qi < s.ctx;
                        const bool tgt_row = tgs > 0 && s.tgt > 0 && qi >= s.hist_q;
                        const int left = tgt_row ? s.hist_k + ((qi - s.hist_q) / tgs) * tgs : 0;   // first visible target column
                        const int jmax = qi + s.delta;
#pragma unroll
                        for (int x = 0; x < 4; x++) {
                            unsigned m = 0;
#pragma unroll
                            for (int i = 0; i < 4; i++) {
                                const int j = c0 + 16 * (x >> 1) + 8 * g + 4 * (x & 1) + i;
                                const bool vis = (ctx_row & (j < s.hist_k)) | ((j <= jmax) & !(tgt_row & (j >= s.hist_k) & (j < left)));
                                m |= vis ? (0xffu << (8 * i)) : 0u;
                            }
                            pq[4 * kb + x] &= m;
                        }
                    }
                }
                const q_i32x8 pb = {(int)pq[0], (int)pq[1], (int)pq[2], (int)pq[3], (int)pq[4], (int)pq[5], (int)pq[6], (int)pq[7]};
                // ---- O^T += V^T P^T: 64 keys per instruction
#pragma unroll
                for (int db = 0; db < D / 32; db++) {
                    if (D > 64) {
#pragma unroll
                        for (int c = 0; c < 4; c++)
                            vq[db][c] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(FP8_LDS_PTR(q_i32x2, vt_lds + 16 * c * VS + vfrag_off + 32 * db));
                    }
                    const q_i32x8 va = {vq[db][0][0], vq[db][0][1], vq[db][1][0], vq[db][1][1], vq[db][2][0], vq[db][2][1], vq[db][3][0], vq[db][3][1]};
                    oacc[db] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(va, pb, oacc[db], 0, 0, 0, 0, 0, 0);
                }
            }
            if (kt + 1 < ntk) stash(kt + 1, stage ^ 1);
            __syncthreads();
        }

        // epilogue: O^T accumulator register r of block db holds d = 32 * db + 8 * (r / 4) + 4g + r % 4 of row qi
        if (qvalid) {
            _Float16* op = obase + ((s.q_start + qi) * p.heads_q + h) * (int64_t)dv_real + 4 * g;
#pragma unroll
            for (int db = 0; db < D / 32; db++) {
#pragma unroll
                for (int rr = 0; rr < 4; rr++) {
                    q_f16x2 lo, hi;
                    lo[0] = (_Float16)oacc[db][4 * rr]; lo[1] = (_Float16)oacc[db][4 * rr + 1];
                    hi[0] = (_Float16)oacc[db][4 * rr + 2]; hi[1] = (_Float16)oacc[db][4 * rr + 3];
                    const q_u32x2 o = {__builtin_bit_cast(unsigned, lo), __builtin_bit_cast(unsigned, hi)};
                    if (!UNEVEN || 32 * db + 8 * rr + 4 * g < dv_real) *reinterpret_cast<q_u32x2*>(op + 32 * db + 8 * rr) = o;
                }
            }
        }
    }

    // rows past the last offset are zero (the reference zero-fills its output: hstu_jagged.cpp:56-59)
    if (owned_rows < p.total_q) {
        const int64_t n = (p.total_q - owned_rows) * p.heads_q * (int64_t)dv_real;
        _Float16* o = obase + owned_rows * p.heads_q * (int64_t)dv_real;
        for (int64_t e = (int64_t)blockIdx.x * 256 + tid; e < n; e += (int64_t)gridDim.x * 256) o[e] = (_Float16)0.f;
    }
}

// head dims the padded variant takes: multiples of 16 up to 256 other than 64 / 128 / 256 for both q.k and v
static bool fp8_uneven(const hstu_fwd_params& p) {
    return p.dim_qk != p.dim_v || (p.dim_qk != 64 && p.dim_qk != 128 && p.dim_qk != 256);
}
static int fp8_padded_dim(const hstu_fwd_params& p) {
    const int d = p.dim_qk > p.dim_v ? p.dim_qk : p.dim_v;
    return d <= 64 ? 64 : (d <= 128 ? 128 : 256);
}

bool mfma_fp8_supported(const KArgs& a, const char** name) {
    const hstu_fwd_params& p = a.p;
    *name = nullptr;
    if (p.dtype != HSTU_FP8_E4M3 || a.op == OP_PAGED) return false;
    int d = p.dim_qk;
    const bool uneven = fp8_uneven(p);
    if (uneven) {
        if (p.dim_qk % 16 || p.dim_v % 16 || p.dim_qk > 256 || p.dim_v > 256) return false;
        d = fp8_padded_dim(p);
    }
    if (p.attn_bias || p.pos_table || p.ts_table || p.mask_type == HSTU_MASK_CUSTOM) return false;   // the plain kernel's
    const uintptr_t all = reinterpret_cast<uintptr_t>(p.q) | reinterpret_cast<uintptr_t>(p.k) | reinterpret_cast<uintptr_t>(p.v) |
                          reinterpret_cast<uintptr_t>(p.out);
    if (all & 15) return false;   // rows are read 16 bytes at a time
    *name = uneven ? (d == 64 ? "mfma_fp8_d64_padded" : (d == 128 ? "mfma_fp8_d128_padded" : "mfma_fp8_d256_padded"))
                   : (d == 64 ? "mfma_fp8_d64" : (d == 128 ? "mfma_fp8_d128" : "mfma_fp8_d256"));
    return true;
}

uint64_t mfma_fp8_workspace_bytes(const KArgs& a) { return work_list_shape(a.p).bytes; }

// launches without the schedule kernel: the conditions of the 16-bit kernels (mfma_self_scheduled)
bool mfma_fp8_self_scheduled(const KArgs& a) {
    const hstu_fwd_params& p = a.p;
    return a.op == OP_JAGGED && p.batch >= 1 && p.batch <= 128 && p.seq_offset_q && p.seq_offset_k && p.total_q == p.total_k && !p.num_context &&
           (p.mask_type == HSTU_MASK_TRIL || p.mask_type == HSTU_MASK_NONE) && p.max_seq_len_q == p.max_seq_len_k && p.max_seq_len_q <= 63 * FBM &&
           !(p.flags & HSTU_FLAG_REUSE_WORKSPACE);
}

hipError_t launch_mfma_fp8(const KArgs& a, void* workspace, hipStream_t stream) {
    const hstu_fwd_params& p = a.p;
    unsigned* ws = reinterpret_cast<unsigned*>(workspace);
    const dim3 grid(work_list_shape(p).grid), block(256);
    if (!fp8_uneven(p) && mfma_fp8_self_scheduled(a)) {
        switch (p.dim_qk) {
            case 64: hipLaunchKernelGGL((hstu_mfma_fp8_kernel<64, false, true>), grid, block, 0, stream, a, ws); break;
            case 128: hipLaunchKernelGGL((hstu_mfma_fp8_kernel<128, false, true>), grid, block, 0, stream, a, ws); break;
            default: hipLaunchKernelGGL((hstu_mfma_fp8_kernel<256, false, true>), grid, block, 0, stream, a, ws); break;
        }
        return hipGetLastError();
    }
    if (!(p.flags & HSTU_FLAG_REUSE_WORKSPACE)) {
        const hipError_t e = launch_work_list(a, ws, true, stream);
        if (e != hipSuccess) return e;
    }
    if (fp8_uneven(p)) {
        switch (fp8_padded_dim(p)) {
            case 64: hipLaunchKernelGGL((hstu_mfma_fp8_kernel<64, true>), grid, block, 0, stream, a, ws); break;
            case 128: hipLaunchKernelGGL((hstu_mfma_fp8_kernel<128, true>), grid, block, 0, stream, a, ws); break;
            default: hipLaunchKernelGGL((hstu_mfma_fp8_kernel<256, true>), grid, block, 0, stream, a, ws); break;
        }
        return hipGetLastError();
    }
    switch (p.dim_qk) {
        case 64: hipLaunchKernelGGL((hstu_mfma_fp8_kernel<64, false>), grid, block, 0, stream, a, ws); break;
        case 128: hipLaunchKernelGGL((hstu_mfma_fp8_kernel<128, false>), grid, block, 0, stream, a, ws); break;
        default: hipLaunchKernelGGL((hstu_mfma_fp8_kernel<256, false>), grid, block, 0, stream, a, ws); break;
    }
    return hipGetLastError();
}

}  // namespace hstu
