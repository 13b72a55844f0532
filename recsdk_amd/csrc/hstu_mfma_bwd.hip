// Jagged HSTU backward on the gfx950 matrix cores (bf16 / fp16, head dim 32, 64, 128 or 256, built-in mask, optional dense attn_bias
// with its gradient).
//
// Three kernels from one template, each a variation of the forward kernel's scheme: the rows a wave owns sit in
// registers as B operands, the other side streams through LDS in 64-row tiles, the 32x32 score block is produced by
// MFMAs with the owned rows as columns, so that its accumulator layout is the B-operand layout of the GEMM that
// follows and the block never leaves the registers:
//   MODE_DQ  owns 128 Q rows (and their dO rows); streams K, V:   S^T = K Q^T, G^T = V dO^T, dS^T = f(S^T, G^T),
//                                                                  dQ^T += K^T dS^T
//   MODE_DK  owns 128 K rows (and their V rows); streams Q, dO:   S = Q K^T, G = dO V^T, dS = f(S, G), dK^T += Q^T dS
//   MODE_DV  owns 128 K rows; streams Q, dO:                      S = Q K^T, P = silu(S), dV^T += dO^T P
//   MODE_DKV (head dim 32 / 64: both accumulators fit) the two K-side kernels in one: S, G, dS and P once per block
// with f = G * sigmoid(x) * (1 + x * (1 - sigmoid(x))), x = alpha * S (golden: build/presmoke/hstu/hstu_common.py:446-452).
// alpha * silu_scale factors out of the sums and is applied once to the fp32 accumulators; P and dS are rounded to the
// I/O dtype when they are packed for the second GEMM, as P in the forward.  Every gradient element has one producing
// workgroup (with GQA the K-side kernels loop over the query heads of their K/V head): no atomics, deterministic.
// With a dense attn_bias (BIAS) the scores are S + bias, read from [batch, heads, max_q, max_k] next to every block, and
// the dQ kernel, which owns whole Q rows, also writes dBias = dS (hstu_jagged.cpp:69-138: the only case that produces it)
// into a buffer that a fill kernel has zeroed: blocks the mask hides are never visited.
#include <cstdlib>
#include <mutex>
#include "hstu_device.h"

namespace hstu {

typedef __attribute__((ext_vector_type(8))) __bf16 b_bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 b_f16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 b_bf16x2;
typedef __attribute__((ext_vector_type(2))) _Float16 b_f16x2;
typedef __attribute__((ext_vector_type(16))) float b_f32x16;
typedef __attribute__((ext_vector_type(4))) short b_s16x4;
typedef __attribute__((ext_vector_type(8))) short b_s16x8;
typedef __attribute__((ext_vector_type(4))) unsigned int b_u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int b_u32x2;

#define BWD_LDS_PTR(type, p) ((__attribute__((address_space(3))) type*)(p))

template <typename T> struct BMM;
template <> struct BMM<__bf16> {
    typedef b_bf16x8 v8;
    static __device__ __forceinline__ b_f32x16 mfma(v8 a, v8 b, b_f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ unsigned pack2(float x, float y) {
        b_bf16x2 r; r[0] = (__bf16)x; r[1] = (__bf16)y; return __builtin_bit_cast(unsigned, r);
    }
};
template <> struct BMM<_Float16> {
    typedef b_f16x8 v8;
    static __device__ __forceinline__ b_f32x16 mfma(v8 a, v8 b, b_f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ unsigned pack2(float x, float y) {
        b_f16x2 r; r[0] = (_Float16)x; r[1] = (_Float16)y; return __builtin_bit_cast(unsigned, r);
    }
};

enum { MODE_DQ = 0, MODE_DK = 1, MODE_DV = 2, MODE_DKV = 3 };
constexpr int WBM = 128;   // rows a workgroup owns
constexpr int WBN = 64;    // rows of the other side per step

// Zeroes of the bias gradient ahead of the dQ kernel, which writes every 32 x 32 block it visits: [batch * heads, max_q,
// max_k], one row per workgroup step, 16 bytes per lane.  Under the plain causal mask (no context rows, no targets) the
// blocks that lie wholly below the diagonal of a wave's first row are always visited, so their columns are left out;
// everything else is zeroed, also what the dQ kernel overwrites later (it runs behind this kernel on the stream).
template <typename T> __global__ __launch_bounds__(256) void hstu_bwd_zero_bias_kernel(const BArgs a) {
    const hstu_fwd_params& p = a.f.p;
    const int plane = blockIdx.y, b = plane / p.heads_q;
    const Seq s = load_seq(a.f, b);
    const bool plain = p.mask_type == HSTU_MASK_TRIL && s.ctx <= 0 && s.tgt <= 0;
    const b_u32x4 z = {0, 0, 0, 0};
    T* base = reinterpret_cast<T*>(a.grad_bias) + (int64_t)plane * p.max_seq_len_q * (int64_t)p.max_seq_len_k;
    const int nchunk = p.max_seq_len_k / 8;
    for (int i = blockIdx.x; i < p.max_seq_len_q; i += gridDim.x) {
        int first = 0;
        if (plain && i < s.lq) {
            const int v = i / 32 * 32 + s.delta + 1;   // columns the first row of this wave's 32 rows sees
            first = v > 0 ? min(v / 32 * 32, p.max_seq_len_k) : 0;
        }
        b_u32x4* row = reinterpret_cast<b_u32x4*>(base + (int64_t)i * p.max_seq_len_k);
        for (int c = first / 8 + threadIdx.x; c < nchunk; c += 256) row[c] = z;
    }
}

// 16-bit half `hi` (0 / 1) of a 32-bit word as float
template <typename T> __device__ __forceinline__ float bwd_half(unsigned w, int hi);
template <> __device__ __forceinline__ float bwd_half<__bf16>(unsigned w, int hi) { return __builtin_bit_cast(float, hi ? (w & 0xffff0000u) : (w << 16)); }
template <> __device__ __forceinline__ float bwd_half<_Float16>(unsigned w, int hi) { return (float)__builtin_bit_cast(b_f16x2, w)[hi]; }

template <typename T, int D, int MODE, int XK>
// (head dim 256 keeps 32 operand fragments and a 32 x 256 accumulator per wave: one wave per SIMD)
// waves per SIMD: one at head dim 256 (see above), three where the registers allow it (head dim 32; at head dim 64 the
// kernels with one accumulator, since their tiles are copied straight into LDS), four for the dQ kernel at head dim 32
// (108 registers), else two
#define BWD_WAVES(D, MODE) ((D) == 256 ? 1 : ((D) == 32 && (MODE) == MODE_DQ) ? 4 : ((D) == 32 || ((D) == 64 && (MODE) != MODE_DKV)) ? 3 : 2)
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(BWD_WAVES(D, MODE), BWD_WAVES(D, MODE))))
void hstu_bwd_mfma_kernel(const BArgs a, const unsigned* __restrict__ ws) {
    typedef typename BMM<T>::v8 v8;
    const hstu_fwd_params& p = a.f.p;
    // XK: 0 = scores as they are, 1 = a dense attn_bias is added (and its gradient written), 2 = a custom mask multiplies P and
    // dS (mask_type 3: [batch, heads, max_q, max_k] like the bias and read the same way; the built-in mask is then off)
    constexpr bool BIAS = XK == 1, XMASK = XK == 2, XLOAD = XK != 0;
    // row strides of the LDS tiles in elements: +16 bytes keeps the 16-byte row-wise reads of 16 rows on distinct banks,
    // +64 bytes does the same for the 4-row transposing reads; a tile that is read both ways (K for dQ, Q for dK) takes a
    // stride of 12 banks modulo 64 (52 at head dim 64), under which the 16 rows of a row-wise read start on 16 different
    // multiples of 4 banks and the 4 rows of a transposing read lie at least 8 banks apart
    constexpr int BOTH = D + (D == 64 ? 40 : 24);
    constexpr int TS1 = MODE == MODE_DV ? D + 8 : BOTH;
    constexpr int TS2 = MODE == MODE_DV ? D + 32 : (MODE == MODE_DKV ? BOTH : D + 8);
    constexpr int NCH = D / 32;          // 16-byte chunks per thread and tile
    constexpr bool TWO = MODE != MODE_DV;   // a second score-shaped GEMM (dO V^T)
    // two stages: the tiles of the next step are fetched into registers while this step computes, and written to the
    // other stage afterwards (one barrier per step)
    // Head dims 64 and 128: the streamed tiles are copied global -> LDS by buffer loads with the LDS destination (no
    // registers in between).  One wave instruction fills 1024 contiguous bytes = 4 rows of head dim 128 (8 of 64), so a tile
    // is a sequence of such blocks, 16 bytes of padding behind each; inside a block row rho keeps its 16-byte chunk c in slot
    // (c + 4 rho) % 16 (head dim 64: (c + 2 (rho / 2)) % 8).  The 16 rows of a row-wise fragment read then start on 16
    // different multiples of 4 banks and the rows of a transposing read do not meet, so one layout serves the tile that is
    // read both ways.  Two stages in separate arrays: the compiler then does not make the reads of one stage wait for the
    // copy in flight into the other.
    // (not the dV kernel, which has half the matrix work per tile to hide the copies behind and measured 20 % slower with them)
    constexpr bool BDMA = (D == 128 || D == 64 || D == 32) && MODE != MODE_DV;
    constexpr int RPB = 512 / D;                     // rows per block: what one copy instruction (1 KB) brings
    constexpr int CPR = D / 8;                       // 16-byte chunks per row
    constexpr int DBLK = 1040, DTILE = (WBN / RPB) * DBLK;
    auto slot_of = [](int c, int rho) __attribute__((always_inline)) -> int { return D == 128 ? ((c + 4 * rho) & 15) : (D == 64 ? ((c + 2 * (rho >> 1)) & 7) : ((c + (rho >> 2)) & 3)); };
    __shared__ __attribute__((aligned(16))) char d1a[BDMA ? DTILE : 16];
    __shared__ __attribute__((aligned(16))) char d1b[BDMA ? DTILE : 16];
    __shared__ __attribute__((aligned(16))) char d2a[BDMA ? DTILE : 16];
    __shared__ __attribute__((aligned(16))) char d2b[BDMA ? DTILE : 16];
    __shared__ __attribute__((aligned(16))) T t1s[BDMA ? 1 : 2][BDMA ? 8 : WBN * TS1];
    // K-side kernels with a bias: per wave 16 rows x 32 columns of the bias, parked as they lie in memory and read back
    // transposed (row stride 72 bytes)
    constexpr int BTS = 72;
    constexpr bool BIAS_T = XLOAD && MODE != MODE_DQ;
    __shared__ __attribute__((aligned(16))) char bias_tile[BIAS_T ? 4 * 16 * BTS : 16];
    __shared__ __attribute__((aligned(16))) T t2s[BDMA ? 1 : 2][BDMA ? 8 : WBN * TS2];

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 5, l32 = lane & 31;
    // Workgroup -> item of the work list (built on the device from the sequence lengths: tiles of the sequences sorted
    // by length, (sequence, head) groups dealt to the XCDs, a group's tiles next to each other, no empty workgroups
    // ahead of real work).  The K-side kernels use a list built with the roles of Q and K swapped: its "Q tiles" are
    // their K tiles and its heads the K/V heads; only the indices of a record are used, the geometry is read again.
    const unsigned item = ws[WORK_HEADER_WORDS + WORK_RECORD_WORDS * (size_t)blockIdx.x];
    const bool idle = item == WORK_ITEM_EMPTY;
    const int b = idle ? 0 : (int)(item & 0xfff), ho = idle ? 0 : (int)((item >> 12) & 0xf);
    const int tl0 = idle ? 0 : (int)((item >> 16) & 0xff);
    const int tl_last = idle ? -1 : (((item >> 24) & 1) ? 0x7fffff : tl0 + (int)((item >> 25) & 7));
    const Seq s = load_seq(a.f, b);
    const int ratio = a.f.head_ratio;
    const bool tril = p.mask_type == HSTU_MASK_TRIL;
    const int tgs = p.target_group_size;
    const T* qb = reinterpret_cast<const T*>(p.q);
    const T* kb_ = reinterpret_cast<const T*>(p.k);
    const T* vb = reinterpret_cast<const T*>(p.v);
    const T* gb = reinterpret_cast<const T*>(a.grad_out);

    const int own_len = MODE == MODE_DQ ? s.lq : s.lk;
    // tiles beyond the grid (sequences longer than the max_seq_len attribute) are taken by the same workgroups
    for (int tl = tl0; tl <= tl_last && tl * WBM < own_len; tl++) {
        // the list starts a group with its last tile, which is the heavy one for Q tiles (it sees the most K columns);
        // the heavy K tile is the first (the most Q rows see it), so the K-side kernels count from the other end
        const int ntl = (own_len + WBM - 1) / WBM;
        const int tile = MODE == MODE_DQ ? tl : ntl - 1 - tl;
        const int o0 = tile * WBM;
        const int r0 = o0 + 32 * w, orow = r0 + l32;
        const bool ovalid = orow < own_len;
        const int hk = MODE == MODE_DQ ? ho / ratio : ho;
        // owned rows as B operands: column = owned row, k = head-dim index
        v8 xf[D / 16], yf[TWO ? D / 16 : 1];
        {
            const int rr = min(orow, own_len - 1);
            const T* xp = MODE == MODE_DQ ? qb + ((s.q_start + rr) * p.heads_q + ho) * (int64_t)D : kb_ + ((s.k_start + rr) * p.heads_k + hk) * (int64_t)D;
            const T* yp = MODE == MODE_DQ ? gb + ((s.q_start + rr) * p.heads_q + ho) * (int64_t)D : vb + ((s.k_start + rr) * p.heads_k + hk) * (int64_t)D;
            const b_u32x4 z = {0, 0, 0, 0};
#pragma unroll
            for (int ds = 0; ds < D / 16; ds++) {
                const b_u32x4 x = *reinterpret_cast<const b_u32x4*>(xp + 16 * ds + 8 * g);
                xf[ds] = __builtin_bit_cast(v8, ovalid ? x : z);
                if (TWO) {
                    const b_u32x4 y = *reinterpret_cast<const b_u32x4*>(yp + 16 * ds + 8 * g);
                    yf[ds] = __builtin_bit_cast(v8, ovalid ? y : z);
                }
            }
        }
        b_f32x16 oacc[D / 32], oacc2[MODE == MODE_DKV ? D / 32 : 1];   // (the fused K-side kernel: dK and dV)
#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                oacc[db][r] = 0.f;
                if constexpr (MODE == MODE_DKV) oacc2[db][r] = 0.f;
            }

        // range of the streamed side
        int t_begin = 0, t_end;
        if (MODE == MODE_DQ) {
            t_end = s.lk > 0 ? k_extent(a.f, s, o0, min(o0 + WBM, s.lq)) : 0;
        } else {
            t_end = s.lq;
            // first Q row that can see one of these K rows: causal -> j <= i + delta; context rows see the whole history
            if (tril && s.ctx <= 0) t_begin = max(0, o0 - s.delta) / WBN * WBN;
        }
        const int nheads = MODE == MODE_DQ ? 1 : ratio;
        for (int hq = 0; hq < nheads; hq++) {
            const int h = MODE == MODE_DQ ? ho : ho * ratio + hq;
            b_u32x4 n1[BDMA ? 1 : NCH], n2[BDMA ? 1 : NCH];
            // direct copies of the tile that starts at streamed row t0: wave w fills blocks 4 w .. 4 w + 3 of both tiles; lane L
            // brings slot L % 16 of row L / 16 of a block, i.e. chunk (slot - 4 rho) % 16 of that row; rows past the end get
            // an offset past the view and arrive as zeros
            auto dma = [&](int t0, char* d1, char* d2) __attribute__((always_inline)) {
                if constexpr (BDMA) {
                    const int sheads = MODE == MODE_DQ ? p.heads_k : p.heads_q, shead = MODE == MODE_DQ ? hk : h;
                    const unsigned rowstride = (unsigned)sheads * D * 2;
                    const int64_t first = ((MODE == MODE_DQ ? s.k_start : s.q_start) * (int64_t)sheads + shead) * D;
                    __amdgpu_buffer_rsrc_t r1 = __builtin_amdgcn_make_buffer_rsrc((void*)((MODE == MODE_DQ ? kb_ : qb) + first), 0, 0x7fffffff, 0x00020000);
                    __amdgpu_buffer_rsrc_t r2 = __builtin_amdgcn_make_buffer_rsrc((void*)((MODE == MODE_DQ ? vb : gb) + first), 0, 0x7fffffff, 0x00020000);
                    const int rho = lane / CPR;
                    const unsigned chunk = (unsigned)(D == 128 ? ((lane % CPR) - 4 * rho) & 15 : (D == 64 ? ((lane % CPR) - 2 * (rho >> 1)) & 7 : ((lane % CPR) - (rho >> 2)) & 3)) << 4;
                    constexpr int BPW = WBN / RPB / 4;   // blocks per wave and tile
#pragma unroll
                    for (int i = 0; i < BPW; i++) {
                        const int blk = BPW * w + i;
                        const int row = t0 + RPB * blk + rho;
                        const unsigned off = row < t_end ? (unsigned)row * rowstride + chunk : 0x80000000u;
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(r1, BWD_LDS_PTR(void, d1 + blk * DBLK), 16, off, 0, 0, 0);
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(r2, BWD_LDS_PTR(void, d2 + blk * DBLK), 16, off, 0, 0, 0);
                    }
                }
            };
            auto fetch = [&](int t0) __attribute__((always_inline)) {
#pragma unroll
                for (int i = 0; i < (BDMA ? 0 : NCH); i++) {
                    const int c = tid + 256 * i;
                    const int row = c / (D / 8), cc = c % (D / 8);
                    const int64_t grow = (MODE == MODE_DQ ? s.k_start : s.q_start) + min(t0 + row, t_end - 1);
                    const int64_t e = MODE == MODE_DQ ? (grow * p.heads_k + hk) * (int64_t)D : (grow * p.heads_q + h) * (int64_t)D;
                    // nothing here waits for the data: rows past the end are zeroed when the tile is written to LDS
                    n1[i] = *reinterpret_cast<const b_u32x4*>((MODE == MODE_DQ ? kb_ : qb) + e + cc * 8);
                    n2[i] = *reinterpret_cast<const b_u32x4*>((MODE == MODE_DQ ? vb : gb) + e + cc * 8);
                }
            };
            auto stash = [&](int t0, int stage) __attribute__((always_inline)) {
#pragma unroll
                for (int i = 0; i < (BDMA ? 0 : NCH); i++) {
                    const int c = tid + 256 * i;
                    const int row = c / (D / 8), cc = c % (D / 8);
                    const bool ok = t0 + row < t_end;
                    const b_u32x4 z = {0, 0, 0, 0};
                    *reinterpret_cast<b_u32x4*>(t1s[stage] + row * TS1 + cc * 8) = ok ? n1[i] : z;
                    *reinterpret_cast<b_u32x4*>(t2s[stage] + row * TS2 + cc * 8) = ok ? n2[i] : z;
                }
            };
            __syncthreads();   // every wave is done with the stages of the previous head / tile
            if (t_begin < t_end) {
                if constexpr (BDMA) {
                    dma(t_begin, d1a, d2a);
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                } else {
                    fetch(t_begin);
                    stash(t_begin, 0);
                }
            }
            __syncthreads();
            int stage = 0;
            for (int t0 = t_begin; t0 < t_end; t0 += WBN, stage ^= 1) {
                const T* t1 = t1s[BDMA ? 0 : stage];
                const T* t2 = t2s[BDMA ? 0 : stage];
                const char* c1 = stage ? d1b : d1a;
                const char* c2 = stage ? d2b : d2a;
                const bool more = t0 + WBN < t_end;
                if constexpr (BDMA) {
                    // the other stage was last read before the barrier that ended the previous step
                    if (more) dma(t0 + WBN, stage ? d1a : d1b, stage ? d2a : d2b);
                } else {
                    if (more) fetch(t0 + WBN);
                }
                // fragment reads: rows as A operands (row 32 kb + l32, head-dim chunk g + 2 ds), and transposed (4 streamed rows
                // 32 kb + 8 j + 4 g .. + 3 of head-dim column 32 db + l32 per lane)
                auto rd_row = [&](const T* tp, const char* tc, int ts, int kb, int ds) __attribute__((always_inline)) -> v8 {
                    if constexpr (BDMA)
                        return *reinterpret_cast<const v8*>(tc + ((32 / RPB) * kb + l32 / RPB) * DBLK + (l32 % RPB) * (2 * D) + (slot_of(g + 2 * ds, l32 % RPB) << 4));
                    else
                        return *reinterpret_cast<const v8*>(tp + (32 * kb + l32) * ts + 8 * g + 16 * ds);
                };
                auto rd_tr = [&](const T* tp, const char* tc, int ts, int kb, int db, int j) __attribute__((always_inline)) -> b_s16x4 {
                    const int trho = (lane & 15) >> 2;
                    if constexpr (BDMA) {
                        const int chunk = 4 * db + 2 * (l32 >> 4) + ((lane & 3) >> 1);
                        const int r = 8 * j + 4 * g + trho;     // row of the 32-row block
                        const char* at = tc + ((32 / RPB) * kb + r / RPB) * DBLK + (r % RPB) * (2 * D) + (slot_of(chunk, r % RPB) << 4) + 8 * (lane & 1);
                        return __builtin_amdgcn_ds_read_tr16_b64_v4i16(BWD_LDS_PTR(b_s16x4, at));
                    } else {
                        const T* vp = tp + (32 * kb + 4 * g + trho + 8 * j) * ts + 16 * (l32 >> 4) + 4 * (lane & 3) + 32 * db;
                        return __builtin_amdgcn_ds_read_tr16_b64_v4i16(BWD_LDS_PTR(b_s16x4, vp));
                    }
                };
#pragma unroll
                for (int kb = 0; kb < WBN / 32; kb++) {
                    const int c0 = t0 + 32 * kb;   // first streamed row of this block
                    // Q rows [i_lo, i_lo + 32) against K rows [j_lo, j_lo + 32) of this block (wave-uniform)
                    const int i_lo = MODE == MODE_DQ ? r0 : c0, j_lo = MODE == MODE_DQ ? c0 : r0;
                    bool pred = false, diag = false;   // full predicate (context rows / targets) or only the causal compare
                    if (tril) {
                        const bool has_ctx = s.ctx > 0 && i_lo < s.ctx;
                        const bool has_tgt = s.tgt > 0 && tgs > 0 && i_lo + 31 >= s.hist_q && j_lo + 31 >= s.hist_k;
                        if (!has_ctx && j_lo > i_lo + 31 + s.delta) continue;   // nothing visible
                        pred = has_ctx || has_tgt;
                        diag = !pred && j_lo + 31 > i_lo + s.delta;
                    }
                    if (c0 >= t_end) continue;
                    // Dense bias of this block, requested before the MFMAs and without a branch (an element outside the
                    // [max_q, max_k] square reads offset 0 and becomes 0).  The dQ kernel owns rows: four 8-byte pieces of
                    // its row.  The K-side kernels own columns: the block comes in as it lies in memory, two times 16 rows of
                    // 64 bytes (lane L: row L / 4, 16-byte piece L % 4), and is turned in LDS further down.
                    const T* bias_bh = reinterpret_cast<const T*>(XMASK ? p.mask : p.attn_bias) + ((int64_t)b * p.heads_q + h) * p.max_seq_len_q * (int64_t)p.max_seq_len_k;
                    b_u32x4 braw_q[(XLOAD && MODE == MODE_DQ) ? 2 : 1];
                    b_u32x4 braw_k[BIAS_T ? 2 : 1];
                    if (XLOAD && MODE == MODE_DQ) {
                        // 16 bytes per lane: columns c0 + 16 pr + 8 g .. + 7 of its row (the two lanes of a row then cover 32
                        // contiguous bytes per load); the halves are exchanged between the lanes further down
#pragma unroll
                        for (int pr = 0; pr < 2; pr++) {
                            const int j = c0 + 16 * pr + 8 * g;
                            const bool ok = orow < p.max_seq_len_q && j < p.max_seq_len_k;
                            const b_u32x4 x = *reinterpret_cast<const b_u32x4*>(bias_bh + (ok ? (unsigned)orow * (unsigned)p.max_seq_len_k + (unsigned)j : 0u));
                            braw_q[pr] = ok ? x : b_u32x4{0, 0, 0, 0};
                        }
                    }
                    if (BIAS_T) {
                        const int jcol = r0 + 8 * (lane & 3);
#pragma unroll
                        for (int hf = 0; hf < 2; hf++) {
                            const int i = c0 + 16 * hf + (lane >> 2);
                            const bool ok = i < p.max_seq_len_q && jcol < p.max_seq_len_k;
                            const b_u32x4 x = *reinterpret_cast<const b_u32x4*>(bias_bh + (ok ? (unsigned)i * (unsigned)p.max_seq_len_k + (unsigned)jcol : 0u));
                            braw_k[hf] = ok ? x : b_u32x4{0, 0, 0, 0};
                        }
                    }
                    b_f32x16 sacc, gacc;
#pragma unroll
                    for (int r = 0; r < 16; r++) { sacc[r] = 0.f; gacc[r] = 0.f; }
#pragma unroll
                    for (int ds = 0; ds < D / 16; ds++) {
                        const v8 f1 = rd_row(t1, c1, TS1, kb, ds);
                        sacc = BMM<T>::mfma(f1, xf[ds], sacc);
                    }
                    if (TWO) {
#pragma unroll
                        for (int ds = 0; ds < D / 16; ds++) {
                            const v8 f2 = rd_row(t2, c2, TS2, kb, ds);
                            gacc = BMM<T>::mfma(f2, yf[ds], gacc);
                        }
                    }
                    // accumulator register r holds streamed row c0 + 8*(r/4) + 4*g + r%4 for the owned row of this lane
                    // the bias of this lane's 16 elements as 8 words of two 16-bit values (pair x = elements 2x, 2x + 1), widened
                    // where they are used
                    unsigned bias_w[XLOAD ? 8 : 1];
                    if (XLOAD && MODE == MODE_DQ) {
                        // score registers 4 q .. 4 q + 3 are columns 8 q + 4 g .. + 3: of the 8 columns a lane loaded for q = 2 pr
                        // and 2 pr + 1, the lane with g = 0 keeps the first four and takes the first four of its partner
                        // (lane + 32), the lane with g = 1 takes the partner's last four and keeps its own: v_permlane32_swap
                        // exchanges the upper half of one register with the lower half of another
#pragma unroll
                        for (int pr = 0; pr < 2; pr++) {
                            const b_u32x2 s0 = __builtin_amdgcn_permlane32_swap(braw_q[pr][0], braw_q[pr][2], false, false);
                            const b_u32x2 s1 = __builtin_amdgcn_permlane32_swap(braw_q[pr][1], braw_q[pr][3], false, false);
                            bias_w[4 * pr] = s0[0]; bias_w[4 * pr + 1] = s1[0];
                            bias_w[4 * pr + 2] = s0[1]; bias_w[4 * pr + 3] = s1[1];
                        }
                    }
                    if (BIAS_T) {
                        char* bt = bias_tile + w * (16 * BTS);
#pragma unroll
                        for (int hf = 0; hf < 2; hf++) {
                            char* wp = bt + (lane >> 2) * BTS + (lane & 3) * 16;
                            *reinterpret_cast<b_u32x2*>(wp) = b_u32x2{braw_k[hf][0], braw_k[hf][1]};
                            *reinterpret_cast<b_u32x2*>(wp + 8) = b_u32x2{braw_k[hf][2], braw_k[hf][3]};
                            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                            __builtin_amdgcn_wave_barrier();
                            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                            // a 16-lane group reads 4 rows x 16 columns and every lane receives 4 consecutive rows of its column:
                            // streamed rows 16 hf + 8 qq + 4 g + 0..3 = score registers 4 (2 hf + qq) + 0..3
#pragma unroll
                            for (int qq = 0; qq < 2; qq++) {
                                const char* rp = bt + (8 * qq + 4 * g + ((lane & 15) >> 2)) * BTS + (16 * (l32 >> 4) + 4 * (lane & 3)) * 2;
                                const b_s16x4 t4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(BWD_LDS_PTR(b_s16x4, rp));
                                const b_u32x2 t2 = __builtin_bit_cast(b_u32x2, t4);
                                bias_w[2 * (2 * hf + qq)] = t2[0];
                                bias_w[2 * (2 * hf + qq) + 1] = t2[1];
                            }
                            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                            __builtin_amdgcn_wave_barrier();
                            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                        }
                    }
                    float wv[16], pv[MODE == MODE_DKV ? 16 : 1];
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const float sv = BIAS ? sacc[r] + bwd_half<T>(bias_w[r >> 1], r & 1) : sacc[r];
                        const float e = __builtin_amdgcn_exp2f(sv * a.f.exp_scale);
                        const float sg = __builtin_amdgcn_rcpf(1.0f + e);
                        if (TWO) {
                            const float x = sv * p.alpha;
                            wv[r] = gacc[r] * sg * __builtin_fmaf(x, 1.0f - sg, 1.0f);
                            if constexpr (MODE == MODE_DKV) pv[r] = sv * sg;
                        } else {
                            wv[r] = sv * sg;
                        }
                        if constexpr (XMASK) {
                            // P = silu(x) * scale * mask, so the mask value multiplies P and, through it, dS (elements outside the
                            // [max_q, max_k] square were read as 0: masked, as in the forward)
                            const float mv = bwd_half<T>(bias_w[r >> 1], r & 1);
                            wv[r] *= mv;
                            if constexpr (MODE == MODE_DKV) pv[r] *= mv;
                        }
                    }
                    b_u32x4 pk0, pk1, qk0, qk1;   // dS (or, in the dV kernel, P); P of the fused kernel
#pragma unroll
                    for (int x = 0; x < 4; x++) {
                        pk0[x] = BMM<T>::pack2(wv[2 * x], wv[2 * x + 1]);
                        pk1[x] = BMM<T>::pack2(wv[8 + 2 * x], wv[8 + 2 * x + 1]);
                        if constexpr (MODE == MODE_DKV) {
                            qk0[x] = BMM<T>::pack2(pv[2 * x], pv[2 * x + 1]);
                            qk1[x] = BMM<T>::pack2(pv[8 + 2 * x], pv[8 + 2 * x + 1]);
                        }
                    }
                    // visibility of this lane's 16 elements as masks of the packed pairs: applied to them at once, kept only where
                    // dBias needs them too (holding them in every variant costs the dK kernel 70 spilled registers)
                    constexpr bool KEEP_MASK = BIAS && MODE == MODE_DQ;
                    b_u32x4 m0 = {~0u, ~0u, ~0u, ~0u}, m1 = m0;
                    if (diag) {
                        // visible iff j <= i + delta; t runs over this lane's 16 streamed rows
                        auto vis = [&](int r) __attribute__((always_inline)) -> bool {
                            const int t = c0 + 8 * (r >> 2) + 4 * g + (r & 3);
                            return MODE == MODE_DQ ? t <= orow + s.delta : orow <= t + s.delta;
                        };
#pragma unroll
                        for (int x = 0; x < 4; x++) {
                            const unsigned v0 = (vis(2 * x) ? 0xffffu : 0u) | (vis(2 * x + 1) ? 0xffff0000u : 0u);
                            const unsigned v1 = (vis(8 + 2 * x) ? 0xffffu : 0u) | (vis(9 + 2 * x) ? 0xffff0000u : 0u);
                            pk0[x] &= v0;
                            pk1[x] &= v1;
                            if constexpr (MODE == MODE_DKV) { qk0[x] &= v0; qk1[x] &= v1; }
                            if (KEEP_MASK) { m0[x] = v0; m1[x] = v1; }
                        }
                    } else if (pred) {
                        // branch-free form of builtin_visible() for this lane's 16 elements
                        auto vis = [&](int r) __attribute__((always_inline)) -> bool {
                            const int t = c0 + 8 * (r >> 2) + 4 * g + (r & 3);
                            const int i = MODE == MODE_DQ ? orow : t, j = MODE == MODE_DQ ? t : orow;
                            const bool ctx_row = s.ctx > 0 && i < s.ctx;
                            const bool tgt_row = tgs > 0 && s.tgt > 0 && i >= s.hist_q;
                            const int left = tgt_row ? s.hist_k + ((i - s.hist_q) / tgs) * tgs : 0;
                            return (ctx_row & (j < s.hist_k)) | ((j <= i + s.delta) & !(tgt_row & (j >= s.hist_k) & (j < left)));
                        };
#pragma unroll
                        for (int x = 0; x < 4; x++) {
                            const unsigned v0 = (vis(2 * x) ? 0xffffu : 0u) | (vis(2 * x + 1) ? 0xffff0000u : 0u);
                            const unsigned v1 = (vis(8 + 2 * x) ? 0xffffu : 0u) | (vis(9 + 2 * x) ? 0xffff0000u : 0u);
                            pk0[x] &= v0;
                            pk1[x] &= v1;
                            if constexpr (MODE == MODE_DKV) { qk0[x] &= v0; qk1[x] &= v1; }
                            if (KEEP_MASK) { m0[x] = v0; m1[x] = v1; }
                        }
                    }
                    if (BIAS && MODE == MODE_DQ) {
                        // dBias = dS with its scale, rounded once, zero where the mask hides the element and behind the sequence;
                        // pair x of the first half holds this lane's streamed rows 8*(x/2) + 2*(x%2) and + 1, the second half 16 more
                        T* gbias = reinterpret_cast<T*>(a.grad_bias) + ((int64_t)b * p.heads_q + h) * p.max_seq_len_q * (int64_t)p.max_seq_len_k;
                        const float sc = a.f.out_scale;
#pragma unroll
                        for (int pr = 0; pr < 2; pr++) {
                            // the pieces of q = 2 pr and 2 pr + 1 go back through the same exchange and leave as 16 bytes per lane
                            const b_u32x4& mm = pr == 0 ? m0 : m1;
                            unsigned o[4];
#pragma unroll
                            for (int x = 0; x < 4; x++) o[x] = BMM<T>::pack2(wv[8 * pr + 2 * x] * sc, wv[8 * pr + 2 * x + 1] * sc) & mm[x];
                            const b_u32x2 s0 = __builtin_amdgcn_permlane32_swap(o[0], o[2], false, false);
                            const b_u32x2 s1 = __builtin_amdgcn_permlane32_swap(o[1], o[3], false, false);
                            const b_u32x4 out4 = {s0[0], s1[0], s0[1], s1[1]};
                            const int j = c0 + 16 * pr + 8 * g;
                            if (ovalid && orow < p.max_seq_len_q && j < p.max_seq_len_k) *reinterpret_cast<b_u32x4*>(gbias + ((unsigned)orow * (unsigned)p.max_seq_len_k + (unsigned)j)) = out4;
                        }
                    }
                    // OUT^T += (tile)^T W: transposing LDS reads, 4 streamed rows of one head-dim column per lane
                    const T* tt = MODE == MODE_DV ? t2 : t1;
                    const char* ct = MODE == MODE_DV ? c2 : c1;
                    constexpr int TT = MODE == MODE_DV ? TS2 : TS1;
#pragma unroll
                    for (int db = 0; db < D / 32; db++) {
                        const b_s16x4 a0 = rd_tr(tt, ct, TT, kb, db, 0);
                        const b_s16x4 a1 = rd_tr(tt, ct, TT, kb, db, 1);
                        const b_s16x4 a2 = rd_tr(tt, ct, TT, kb, db, 2);
                        const b_s16x4 a3 = rd_tr(tt, ct, TT, kb, db, 3);
                        const b_s16x8 lo = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
                        const b_s16x8 hi = {a2[0], a2[1], a2[2], a2[3], a3[0], a3[1], a3[2], a3[3]};
                        oacc[db] = BMM<T>::mfma(__builtin_bit_cast(v8, lo), __builtin_bit_cast(v8, pk0), oacc[db]);
                        oacc[db] = BMM<T>::mfma(__builtin_bit_cast(v8, hi), __builtin_bit_cast(v8, pk1), oacc[db]);
                    }
                    if constexpr (MODE == MODE_DKV) {
                        // dV^T += dO^T P from the other tile
#pragma unroll
                        for (int db = 0; db < D / 32; db++) {
                            const b_s16x4 a0 = rd_tr(t2, c2, TS2, kb, db, 0);
                            const b_s16x4 a1 = rd_tr(t2, c2, TS2, kb, db, 1);
                            const b_s16x4 a2 = rd_tr(t2, c2, TS2, kb, db, 2);
                            const b_s16x4 a3 = rd_tr(t2, c2, TS2, kb, db, 3);
                            const b_s16x8 lo = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
                            const b_s16x8 hi = {a2[0], a2[1], a2[2], a2[3], a3[0], a3[1], a3[2], a3[3]};
                            oacc2[db] = BMM<T>::mfma(__builtin_bit_cast(v8, lo), __builtin_bit_cast(v8, qk0), oacc2[db]);
                            oacc2[db] = BMM<T>::mfma(__builtin_bit_cast(v8, hi), __builtin_bit_cast(v8, qk1), oacc2[db]);
                        }
                    }
                }
                if constexpr (BDMA) {
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's part of the next tile has arrived
                } else {
                    if (more) stash(t0 + WBN, stage ^ 1);
                }
                __syncthreads();
            }
        }
        // accumulator register r of block db holds head-dim index 32*db + 8*(r/4) + 4*g + r%4 for the owned row: the two lanes
        // of a row hold alternating 8-byte pieces of it; they exchange halves (v_permlane32_swap: upper half of one register
        // with the lower half of another) and store 16 bytes each
        {
            const int64_t orc = ovalid ? orow : 0;
            const float sc = a.f.out_scale;   // alpha * silu_scale
            auto store_rows = [&](T* out, const b_f32x16* acc) __attribute__((always_inline)) {
#pragma unroll
                for (int db = 0; db < D / 32; db++) {
#pragma unroll
                    for (int pr = 0; pr < 2; pr++) {
                        unsigned o[4];
#pragma unroll
                        for (int x = 0; x < 4; x++) o[x] = BMM<T>::pack2(acc[db][8 * pr + 2 * x] * sc, acc[db][8 * pr + 2 * x + 1] * sc);
                        const b_u32x2 s0 = __builtin_amdgcn_permlane32_swap(o[0], o[2], false, false);
                        const b_u32x2 s1 = __builtin_amdgcn_permlane32_swap(o[1], o[3], false, false);
                        const b_u32x4 out4 = {s0[0], s1[0], s0[1], s1[1]};
                        if (ovalid) *reinterpret_cast<b_u32x4*>(out + 32 * db + 16 * pr + 8 * g) = out4;
                    }
                }
            };
            T* const out_q = reinterpret_cast<T*>(a.grad_q) + ((s.q_start + orc) * p.heads_q + ho) * (int64_t)D;
            T* const out_k = reinterpret_cast<T*>(a.grad_k) + ((s.k_start + orc) * p.heads_k + ho) * (int64_t)D;
            T* const out_v = reinterpret_cast<T*>(a.grad_v) + ((s.k_start + orc) * p.heads_k + ho) * (int64_t)D;
            store_rows(MODE == MODE_DQ ? out_q : (MODE == MODE_DV ? out_v : out_k), oacc);
            if constexpr (MODE == MODE_DKV) store_rows(out_v, oacc2);
        }
    }

    // rows past the last offset carry no gradient
    {
        const int is64 = p.index_type == HSTU_I64;
        const int64_t total = MODE == MODE_DQ ? p.total_q : p.total_k;
        const int heads = MODE == MODE_DQ ? p.heads_q : p.heads_k;
        const void* offs = MODE == MODE_DQ ? p.seq_offset_q : p.seq_offset_k;
        const int64_t tail = offs ? ld_idx(offs, p.batch, is64) : total;
        if (tail < total) {
            T* o = reinterpret_cast<T*>(MODE == MODE_DQ ? a.grad_q : (MODE == MODE_DV ? a.grad_v : a.grad_k)) + tail * heads * (int64_t)D;
            const int64_t n = (total - tail) * heads * (int64_t)D;
            for (int64_t e = (int64_t)blockIdx.x * 256 + tid; e < n; e += (int64_t)gridDim.x * 256) {
                o[e] = (T)0.f;
                if constexpr (MODE == MODE_DKV) reinterpret_cast<T*>(a.grad_v)[tail * heads * (int64_t)D + e] = (T)0.f;
            }
        }
    }
}

bool mfma_backward_supported(const BArgs& a) {
    const hstu_fwd_params& p = a.f.p;
    if (p.dtype != HSTU_BF16 && p.dtype != HSTU_F16) return false;
    if (p.dim_qk != p.dim_v || (p.dim_qk != 32 && p.dim_qk != 64 && p.dim_qk != 128 && p.dim_qk != 256)) return false;
    // a custom mask is read like a dense bias (8 bytes at a time along its rows); with a bias next to it: the plain kernels
    if (p.mask_type == HSTU_MASK_CUSTOM &&
        (p.attn_bias || !p.mask || p.max_seq_len_k % 8 != 0 || (reinterpret_cast<uintptr_t>(p.mask) & 15))) return false;
    // a dense bias is read 8 bytes at a time along its rows, its gradient written the same way
    if (p.attn_bias && (p.max_seq_len_k % 8 != 0 || ((reinterpret_cast<uintptr_t>(p.attn_bias) | reinterpret_cast<uintptr_t>(a.grad_bias)) & 15)))
        return false;
    // rows are read and written 16 bytes at a time: buffers that do not start on such a boundary take the plain kernels
    const uintptr_t all = reinterpret_cast<uintptr_t>(p.q) | reinterpret_cast<uintptr_t>(p.k) | reinterpret_cast<uintptr_t>(p.v) |
                          reinterpret_cast<uintptr_t>(a.grad_out) | reinterpret_cast<uintptr_t>(a.grad_q) |
                          reinterpret_cast<uintptr_t>(a.grad_k) | reinterpret_cast<uintptr_t>(a.grad_v);
    if (all & 15) return false;
    return true;
}

// two lists: Q tiles (dQ kernel) and K tiles (dK, dV kernels: the roles of Q and K swapped)
static KArgs swapped_roles(const KArgs& f) {
    KArgs k = f;
    k.p.seq_offset_q = f.p.seq_offset_k;
    k.p.seq_offset_k = f.p.seq_offset_q;
    k.p.total_q = f.p.total_k;
    k.p.total_k = f.p.total_q;
    k.p.heads_q = f.p.heads_k;
    k.p.max_seq_len_q = f.p.max_seq_len_k;
    k.p.max_seq_len_k = f.p.max_seq_len_q;
    k.p.num_context = nullptr;   // the list only orders the tiles; the kernels read the true geometry themselves
    k.p.num_target = nullptr;
    k.head_ratio = 1;
    return k;
}

// Self-attention without GQA (the .equal overload): K tile n-1-t has the work of Q tile t, so the Q list, read from
// the other end of each sequence, serves the K-side kernels as well (and pairs their two light tiles).
static bool one_list(const hstu_fwd_params& p) {
    return p.seq_offset_q == p.seq_offset_k && p.heads_q == p.heads_k && p.max_seq_len_q == p.max_seq_len_k;
}

uint64_t mfma_backward_workspace_bytes(const BArgs& a) {
    const uint64_t q = work_list_shape(a.f.p).bytes;
    return one_list(a.f.p) ? q : q + work_list_shape(swapped_roles(a.f).p).bytes;
}

// The dQ kernel and the K-side kernels are independent of each other (they read q, k, v, dO and the work lists and write
// different gradients), and each ends with a tail in which a few long items run while most of the chip idles.  They are
// therefore launched on three streams -- the caller's and two of the library's own per device, forked from and joined to
// the caller's stream by events -- so that the next kernel's workgroups fill the slots the previous one's tail leaves
// empty.  To the caller the call still is one piece of work on its stream (also under stream capture, where the events
// become edges of the graph).  Streams of default priority, events without timing, created on the first call on a device;
// if that fails everything runs on the caller's stream.
SideStreams* side_streams(hipStream_t caller) {
    constexpr int MAXDEV = 64, SETS = 8;
    struct Slot {
        SideStreams set;
        hipStream_t owner = nullptr;
        int state = 0;        // 0 = free, 1 = made, -1 = given up
        int failures = 0;
    };
    static std::mutex mu;
    static Slot slots[MAXDEV][SETS];
    static int serial = -1;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAXDEV) return nullptr;
    std::lock_guard<std::mutex> lock(mu);
    if (serial < 0) {
        const char* e = getenv("HSTU_HIP_SERIAL_BACKWARD");   // "1" keeps every backward on the caller's stream
        serial = (e && e[0] == '1') ? 1 : 0;
    }
    if (serial) return nullptr;
    Slot* slot = nullptr;
    for (int i = 0; i < SETS && !slot; i++)
        if (slots[dev][i].state == 1 && slots[dev][i].owner == caller) slot = &slots[dev][i];
    for (int i = 0; i < SETS && !slot; i++)
        if (slots[dev][i].state == 0) slot = &slots[dev][i];
    if (!slot) return slots[dev][SETS - 1].state == 1 ? &slots[dev][SETS - 1].set : nullptr;   // more caller streams than sets: share
    if (slot->state == 1) return &slot->set;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(caller, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return nullptr;    // not now: the next call outside a capture makes the set
    }
    SideStreams& f = slot->set;
    int ns = 0, ne = 0;
    bool ok = true;
    for (; ns < 2 && ok; ns++) ok = hipStreamCreateWithFlags(&f.side[ns], hipStreamNonBlocking) == hipSuccess;
    for (; ne < 3 && ok; ne++) ok = hipEventCreateWithFlags(&f.ev[ne], hipEventDisableTiming) == hipSuccess;
    if (!ok) {
        (void)hipGetLastError();
        // (the loops count the failed attempt too)
        for (int i = 0; i + 1 < ns; i++) (void)hipStreamDestroy(f.side[i]);
        for (int i = 0; i + 1 < ne; i++) (void)hipEventDestroy(f.ev[i]);
        if (++slot->failures >= 3) slot->state = -1;
        return nullptr;
    }
    slot->owner = caller;
    slot->state = 1;
    return &f;
}

template <typename T, int D>
static hipError_t launch_bwd_td(const BArgs& a, unsigned* ws, hipStream_t stream) {
    const KArgs kside = swapped_roles(a.f);
    const bool shared = one_list(a.f.p);
    const WorkList lq = work_list_shape(a.f.p), lk = shared ? lq : work_list_shape(kside.p);
    unsigned* wsq = ws;
    unsigned* wsk = shared ? ws : ws + lq.bytes / sizeof(unsigned);
    hipError_t e = launch_work_list(a.f, wsq, true, stream);
    if (e != hipSuccess) return e;
    if (!shared) {
        e = launch_work_list(kside, wsk, false, stream);   // tile costs are only roughly those of the K tiles: no pairs
        if (e != hipSuccess) return e;
    }
    // fork: the K-side kernels wait for the work lists only.  Worth it when the kernels are long against the few microseconds
    // the events cost: at 3840 items per kernel (B = 32, h = 8, S = 2048) -2 .. -7 %, at 1440 (the headline batch) +2 %
    SideStreams* fk = (lq.grid >= 3000 && !(a.f.p.flags & HSTU_FLAG_SERIAL_BACKWARD)) ? side_streams(stream) : nullptr;
    hipStream_t sk = stream, sv = stream;
    // a set can be shared (two host threads on one stream, or more caller streams than sets): from the first record to the
    // last wait of this call no other host thread may record its events (the calls below only enqueue work, so the lock is
    // held for microseconds)
    std::unique_lock<std::mutex> fork_lock;
    if (fk) fork_lock = std::unique_lock<std::mutex>(fk->mu);
    if (fk) {
        if (hipEventRecord(fk->ev[0], stream) == hipSuccess && hipStreamWaitEvent(fk->side[0], fk->ev[0], 0) == hipSuccess &&
            hipStreamWaitEvent(fk->side[1], fk->ev[0], 0) == hipSuccess) {
            sk = fk->side[0];
            sv = fk->side[1];
        } else {
            (void)hipGetLastError();
            fk = nullptr;
        }
    }
    auto join = [&](hipError_t err) -> hipError_t {
        if (fk) {
            // (also after a failed launch: the caller's stream must not run ahead of what did get launched)
            const bool ok = hipEventRecord(fk->ev[1], sk) == hipSuccess && hipEventRecord(fk->ev[2], sv) == hipSuccess &&
                            hipStreamWaitEvent(stream, fk->ev[1], 0) == hipSuccess && hipStreamWaitEvent(stream, fk->ev[2], 0) == hipSuccess;
            if (!ok && err == hipSuccess) err = hipGetLastError();
        }
        return err;
    };
    if (a.f.p.attn_bias) {
        // dBias: zero everywhere, then the dQ kernel writes the blocks the mask lets it visit
        const hstu_fwd_params& p = a.f.p;
        const unsigned zrows = (unsigned)(p.max_seq_len_q < 512 ? p.max_seq_len_q : 512);   // max_seq_len_k % 8 == 0
        hipLaunchKernelGGL(hstu_bwd_zero_bias_kernel<T>, dim3(zrows, (unsigned)(p.batch * p.heads_q)), dim3(256), 0, stream, a);
        e = hipGetLastError();
        if (e != hipSuccess) return join(e);
        hipLaunchKernelGGL((hstu_bwd_mfma_kernel<T, D, MODE_DQ, 1>), dim3(lq.grid), dim3(256), 0, stream, a, wsq);
        e = hipGetLastError();
        if (e != hipSuccess) return join(e);
        if constexpr (D <= 64) {
            hipLaunchKernelGGL((hstu_bwd_mfma_kernel<T, D, MODE_DKV, 1>), dim3(lk.grid), dim3(256), 0, sk, a, wsk);
            return join(hipGetLastError());
        }
        hipLaunchKernelGGL((hstu_bwd_mfma_kernel<T, D, MODE_DK, 1>), dim3(lk.grid), dim3(256), 0, sk, a, wsk);
        e = hipGetLastError();
        if (e != hipSuccess) return join(e);
        hipLaunchKernelGGL((hstu_bwd_mfma_kernel<T, D, MODE_DV, 1>), dim3(lk.grid), dim3(256), 0, sv, a, wsk);
        return join(hipGetLastError());
    }
    if (a.f.p.mask_type == HSTU_MASK_CUSTOM) {
        hipLaunchKernelGGL((hstu_bwd_mfma_kernel<T, D, MODE_DQ, 2>), dim3(lq.grid), dim3(256), 0, stream, a, wsq);
        e = hipGetLastError();
        if (e != hipSuccess) return join(e);
        if constexpr (D <= 64) {
            hipLaunchKernelGGL((hstu_bwd_mfma_kernel<T, D, MODE_DKV, 2>), dim3(lk.grid), dim3(256), 0, sk, a, wsk);
            return join(hipGetLastError());
        }
        hipLaunchKernelGGL((hstu_bwd_mfma_kernel<T, D, MODE_DK, 2>), dim3(lk.grid), dim3(256), 0, sk, a, wsk);
        e = hipGetLastError();
        if (e != hipSuccess) return join(e);
        hipLaunchKernelGGL((hstu_bwd_mfma_kernel<T, D, MODE_DV, 2>), dim3(lk.grid), dim3(256), 0, sv, a, wsk);
        return join(hipGetLastError());
    }
    hipLaunchKernelGGL((hstu_bwd_mfma_kernel<T, D, MODE_DQ, 0>), dim3(lq.grid), dim3(256), 0, stream, a, wsq);
    e = hipGetLastError();
    if (e != hipSuccess) return join(e);
    if constexpr (D <= 64) {
        // both K-side accumulators fit: S, G, dS and P once per block
        hipLaunchKernelGGL((hstu_bwd_mfma_kernel<T, D, MODE_DKV, 0>), dim3(lk.grid), dim3(256), 0, sk, a, wsk);
        return join(hipGetLastError());
    }
    hipLaunchKernelGGL((hstu_bwd_mfma_kernel<T, D, MODE_DK, 0>), dim3(lk.grid), dim3(256), 0, sk, a, wsk);
    e = hipGetLastError();
    if (e != hipSuccess) return join(e);
    if (D == 128 && shared && reversed_forward_supported(a.f.p)) {
        // plain causal self-attention: dV[j] = sum over i >= j of P[i][j] dO[i] is the forward with K as q, Q as k and
        // dO as v on rows taken in reverse order, and the forward's kernel for this head dim (direct copies into LDS,
        // 32-row tiles, three workgroups per CU) is the faster one
        KArgs r = a.f;
        r.p.q = a.f.p.k; r.p.k = a.f.p.q; r.p.v = a.grad_out; r.p.out = a.grad_v;
        return join(launch_reversed_forward(r, wsq, sv));
    }
    hipLaunchKernelGGL((hstu_bwd_mfma_kernel<T, D, MODE_DV, 0>), dim3(lk.grid), dim3(256), 0, sv, a, wsk);
    return join(hipGetLastError());
}

hipError_t launch_backward_mfma(const BArgs& a, void* workspace, hipStream_t stream) {
    const hstu_fwd_params& p = a.f.p;
    unsigned* ws = reinterpret_cast<unsigned*>(workspace);
    if (p.dtype == HSTU_BF16) {
        switch (p.dim_qk) {
            case 32: return launch_bwd_td<__bf16, 32>(a, ws, stream);
            case 64: return launch_bwd_td<__bf16, 64>(a, ws, stream);
            case 128: return launch_bwd_td<__bf16, 128>(a, ws, stream);
            default: return launch_bwd_td<__bf16, 256>(a, ws, stream);
        }
    }
    switch (p.dim_qk) {
        case 32: return launch_bwd_td<_Float16, 32>(a, ws, stream);
        case 64: return launch_bwd_td<_Float16, 64>(a, ws, stream);
        case 128: return launch_bwd_td<_Float16, 128>(a, ws, stream);
        default: return launch_bwd_td<_Float16, 256>(a, ws, stream);
    }
}

}  // namespace hstu
