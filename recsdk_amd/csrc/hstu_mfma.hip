// HSTU forward on the gfx950 matrix cores (bf16 / fp16 I/O, head dim 32, 64, 128 or 256).
//
// One workgroup (4 waves) owns a 128-row Q tile of one (sequence, head); wave w owns rows 32w..32w+31.
// K and V tiles of 64 columns (32 in the plain head-dim-128 variant, see Shape) stream through LDS, double buffered,
// one barrier per tile.
// Per tile and wave:
//     S^T = K Q^T           v_mfma_f32_32x32x16 with A = K fragment (ds_read_b128), B = Q fragment (registers)
//     P   = s*sigmoid(a*s)  in registers (v_exp_f32 + v_rcp_f32), mask/bias fused, packed to 16 bit
//     O^T += V^T P^T        A = V^T fragment (ds_read_b64_tr_b16 transposing loads), B = P straight from
//                           the S accumulator registers -- the accumulator layout of S^T is exactly the
//                           B-operand layout PV needs, so the score matrix never leaves the registers.
// alpha*silu_scale is applied once to the fp32 accumulator in the epilogue (it factors out of the sum).
// Element-wise order follows the reference (vector_score_inter.h:299-323): x = alpha*(S+bias), SiLU,
// then scale*mask; P is rounded to the I/O dtype before PV as there (vector_score_inter.h:177-184),
// S itself stays in fp32.
#include <type_traits>

#include "hstu_device.h"
#include "hstu_self_sched.h"

namespace hstu {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

#define LDS_PTR(type, p) ((__attribute__((address_space(3))) type*)(p))

template <typename T> struct MM;
template <> struct MM<__bf16> {
    typedef bf16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ unsigned pack2(float x, float y) {
        bf16x2 r; r[0] = (__bf16)x; r[1] = (__bf16)y; return __builtin_bit_cast(unsigned, r);
    }
};
template <> struct MM<_Float16> {
    typedef f16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ unsigned pack2(float x, float y) {
        f16x2 r; r[0] = (_Float16)x; r[1] = (_Float16)y; return __builtin_bit_cast(unsigned, r);
    }
};

// 16-bit half `hi` (0 / 1) of a 32-bit word as float
template <typename T> __device__ __forceinline__ float half_to_float(unsigned w, int hi);
template <> __device__ __forceinline__ float half_to_float<__bf16>(unsigned w, int hi) { return __builtin_bit_cast(float, hi ? (w & 0xffff0000u) : (w << 16)); }
template <> __device__ __forceinline__ float half_to_float<_Float16>(unsigned w, int hi) {
    const f16x2 v = __builtin_bit_cast(f16x2, w);
    return (float)v[hi];
}

constexpr int BM = 128;  // Q rows per workgroup
constexpr int BN = 64;   // K columns per step
constexpr int NT = 256;  // threads

template <int D> struct Tile {
    static constexpr int KS = D + 8;    // K row stride in elements: +16 B keeps ds_read_b128 of 16 rows on distinct banks
    static constexpr int VS = D + 32;   // V row stride: +64 B spreads the 4-row transposing reads over the banks
    static constexpr int NCH = D / 32;  // 16-byte chunks per thread and tile
    static constexpr int K_ELEMS = BN * KS;
    static constexpr int V_ELEMS = BN * VS;
    static constexpr int LDS_BYTES = 2 * (K_ELEMS + V_ELEMS) * 2;
};

// Source of one K or V row for the tile loader.
template <typename T, bool PAGED>
struct RowRef {
    const void* ptr;
    float scale;
    bool fp8;
};

// pages of one user whose ids (and fp8 scales) are kept in LDS: the reference's longest sequence (20480) in its smallest pages
// (32 rows, tiling_policy_paged.cpp:218-221); half of that in the head-dim-128 variants whose tiles go through registers
// (64-key tiles: the larger copy would leave one workgroup per CU)
constexpr int MAXP_ALL = 640, MAXP_HALF = 320;

template <typename T, bool PAGED>
__device__ __forceinline__ RowRef<T, PAGED> kv_row_ref(const KArgs& a, const Seq& s, int which, int j, int hk, int D,
                                                       const int* lds_pid, const float* lds_psc, int MAXP = MAXP_ALL) {
    const hstu_fwd_params& p = a.p;
    RowRef<T, PAGED> r;
    r.scale = 1.f;
    r.fp8 = false;
    if (!PAGED) {
        // (D is the row width in elements: dim_qk for k, dim_v for v -- the same for all variants but the uneven one)
        r.ptr = reinterpret_cast<const T*>(which ? p.v : p.k) + ((s.k_start + j) * p.heads_k + hk) * (int64_t)D;
        return r;
    }
    // Branch-free: both sources are addressed and one is selected, so the loads that follow stay in
    // straight-line code.  Page ids (and fp8 scales) come from the LDS copy made at the start of the tile;
    // the host only selects this kernel when every page index of a sequence fits that copy.
    const int ps = p.page_size;
    const bool pow2 = (ps & (ps - 1)) == 0;
    const bool hist = j < s.hist_k;
    const int jh = hist ? j : 0;
    const int pidx = pow2 ? (jh >> (31 - __builtin_clz(ps))) : jh / ps;
    const int slot = pow2 ? (jh & (ps - 1)) : jh - pidx * ps;
    const int pc = min(pidx, MAXP - 1);
    const int64_t page = lds_pid[pc];
    // one 64-bit multiply per row: page * (elements per page); everything inside a page is 32-bit
    const unsigned plane = (unsigned)ps * p.heads_k * D;  // elements of the K (or V) half of a page
    const int64_t e = page * (int64_t)(2u * plane) + (unsigned)(which * plane + (slot * p.heads_k + hk) * D);
    const bool fp8 = p.cache_dtype == HSTU_FP8_E4M3;
    const char* cache_ptr = reinterpret_cast<const char*>(p.kv_cache) + (fp8 ? e : e * (int64_t)sizeof(T));
    const int64_t row = s.cand_row + (j - s.hist_k);
    const char* in_ptr = reinterpret_cast<const char*>(which ? p.v : p.k) + ((row * p.heads_k + hk) * (int64_t)D) * (int64_t)sizeof(T);
    r.ptr = hist ? cache_ptr : in_ptr;
    r.fp8 = hist && fp8;
    r.scale = r.fp8 ? lds_psc[2 * pc + which] : 1.f;
    return r;
}

// Issue the load of one 8-element chunk.  fp8 rows are fetched raw (8 bytes) and converted when they are
// written to LDS, so that nothing waits on the load here.
template <typename T, bool PAGED>
__device__ __forceinline__ u32x4 load_chunk(const RowRef<T, PAGED>& r, int cc) {
    if (PAGED && r.fp8) {
        u32x2 raw = *reinterpret_cast<const u32x2*>(reinterpret_cast<const uint8_t*>(r.ptr) + cc * 8);
        u32x4 o = {raw[0], raw[1], 0u, 0u};
        return o;
    }
    return *reinterpret_cast<const u32x4*>(reinterpret_cast<const T*>(r.ptr) + cc * 8);
}

// e4m3 -> fp32 (exact), times the fp32 scale, rounded once to the I/O dtype.  The scaled pack-convert
// instruction only honours the exponent of its scale operand, so it is not used.
template <typename T>
__device__ __forceinline__ u32x4 dequant_chunk(u32x4 raw, float scale) {
    u32x4 o;
#pragma unroll
    for (int x = 0; x < 4; x++) {
        f32x2 f = (x & 1) ? __builtin_amdgcn_cvt_pk_f32_fp8(raw[x >> 1], true) : __builtin_amdgcn_cvt_pk_f32_fp8(raw[x >> 1], false);
        o[x] = MM<T>::pack2(f[0] * scale, f[1] * scale);
    }
    return o;
}

// visibility class of a 32x32 block (rows r0.., columns c0..) under the built-in mask
enum { BLK_ALL = 0, BLK_CAUSAL = 1, BLK_PRED = 2, BLK_SKIP = 3 };

__device__ __forceinline__ int classify_block(const Seq& s, int tgs, int r0, int c0) {
    const bool has_ctx = s.ctx > 0 && r0 < s.ctx;
    const bool has_tgt = s.tgt > 0 && tgs > 0 && r0 + 31 >= s.hist_q && c0 + 31 >= s.hist_k;
    if (!has_ctx && c0 > r0 + 31 + s.delta) return BLK_SKIP;
    if (has_ctx || has_tgt) return BLK_PRED;
    if (c0 + 31 <= r0 + s.delta) return BLK_ALL;
    return BLK_CAUSAL;
}

// ---- work list ------------------------------------------------------------------------------------------
// The hardware dispatches workgroups in index order and a workgroup that finds no work still costs a slot, so
// the grid is driven by a list that a one-workgroup kernel builds first from the sequence lengths:
//   * one item = one 128-row Q tile of one (sequence, head) (or one of its 2-4 K ranges, see sched_dims): a record
//     of 8 words -- seq | head << 12 | tile << 16 | sweep << 24 | K range << 25 | ranges << 28, then the sequence's geometry (q_start, lq, k_start, lk, num_context, num_target, first page
//     entry), so that a workgroup needs one scalar load to know its work
//   * the first two Q tiles of a long sequence are one item (bits 25..27 of an unsplit item count the further tiles
//     it covers): they see few K columns and would mostly pay a workgroup's start and end
//   * sequences are sorted by K length (longest first) and their (sequence, head) groups are dealt to the
//     8 XCDs in snake order; a group's tiles sit next to each other in its XCD's list, last tile first, so that
//     the workgroups that share one K/V run at the same time on CUs that share one L2
//   * workgroup i runs on XCD i % 8 and takes entry i / 8 of that XCD's list: record i
//   * items beyond a list's capacity are parked in an overflow list and then moved to the free slots at the end
//     of the other lists
// Layout of the workspace (uint32): [0] number of items that were moved, [2..3] rows the sequences own (int64),
// from word 16 the 8*cap records of the
// interleaved lists, then the parking area of the overflow list.  The main kernel only reads it.
constexpr unsigned ITEM_EMPTY = 0xffffffffu;
constexpr int SCHED_NT = 1024;
constexpr int WS_HEADER = 16;
constexpr int REC = 8;   // words per record

struct SchedDims {
    int ntiles_attr;   // Q tiles the max_seq_len_q attribute covers
    unsigned cap;      // entries per XCD list
    unsigned bound;    // upper bound of the number of items (= entries of the overflow list)
    int nsplit;        // K ranges per Q tile (1 = none); each range is an item of its own
    int pair;          // 1: the first two Q tiles of a long sequence may become one item
    int interleave;    // 1: four neighbouring groups of a list with equal entry counts are written entry by entry in turn
    int level_slots;   // > 0: workgroups a CU holds; lists of at most 32 times as many entries are levelled over the CUs (see hstu_schedule_kernel)
};

// head dims the matrix-core kernels take through the padded variant (EXTRA 11): multiples of 16 up to 256 that are not one
// of 32 / 64 / 128 / 256 for both q.k and v
static bool uneven_dims(const hstu_fwd_params& p) {
    const int d = p.dim_qk;
    return d != p.dim_v || (d != 32 && d != 64 && d != 128 && d != 256);
}
static int padded_dim(const hstu_fwd_params& p) {
    const int d = p.dim_qk > p.dim_v ? p.dim_qk : p.dim_v;
    return d <= 32 ? 32 : (d <= 64 ? 64 : (d <= 128 ? 128 : 256));
}

static SchedDims sched_dims(const hstu_fwd_params& p, bool whole_tiles = false) {
    SchedDims d;
    d.pair = 1;
    d.interleave = 0;
    d.level_slots = 0;
    d.ntiles_attr = (p.max_seq_len_q + BM - 1) / BM;
    // sum over sequences of min(ceil(lq / BM), ntiles_attr) <= min(total_q / BM + batch, batch * ntiles_attr)
    const int64_t by_rows = p.total_q / BM + p.batch, by_attr = (int64_t)p.batch * d.ntiles_attr;
    d.bound = (unsigned)((by_rows < by_attr ? by_rows : by_attr) * p.heads_q);
    // Few Q tiles but long K (serving: a handful of users, candidates against a long history): split the K range of
    // every tile over up to 4 workgroups so that the CUs hold 2-3 of them; the partial sums (HSTU has no softmax, so
    // they simply add up) go through the workspace and a small reduction kernel.
    d.nsplit = 1;
    const int ktiles = (p.max_seq_len_k + BN - 1) / BN;
    if (!whole_tiles && !(p.flags & FLAG_WHOLE_TILES) && !uneven_dims(p) && d.bound < 384 && ktiles >= 16) {
        int s = 768 / (int)(d.bound ? d.bound : 1);
        if (s > 4) s = 4;
        if (s > ktiles / 4) s = ktiles / 4;
        if (s > 1) d.nsplit = s;
    }
    d.bound *= (unsigned)d.nsplit;
    d.cap = (d.bound + 7) / 8 + (unsigned)(d.ntiles_attr * d.nsplit);
    return d;
}

static uint64_t list_bytes(const SchedDims& d) {
    const uint64_t b = (uint64_t)(WS_HEADER + REC * (8 * (uint64_t)d.cap + d.bound)) * sizeof(uint32_t);
    return (b + 255) / 256 * 256;
}

uint64_t mfma_workspace_bytes(const KArgs& a) {
    if (a.p.dtype == HSTU_FP8_E4M3) return mfma_fp8_workspace_bytes(a);
    const SchedDims d = sched_dims(a.p);
    uint64_t b = list_bytes(d);
    if (d.nsplit > 1) b += (uint64_t)d.nsplit * a.p.total_q * a.p.heads_q * a.p.dim_v * sizeof(float);   // partial sums
    return b;
}

// The work list for kernels other than the forward (the backward's): every Q tile is one item (no K ranges; the
// first two tiles of a long sequence become one item only if `pair`).
WorkList work_list_shape(const hstu_fwd_params& p) {
    const SchedDims d = sched_dims(p, true);
    WorkList w;
    w.grid = 8 * d.cap;
    w.bytes = list_bytes(d);
    return w;
}


__device__ __forceinline__ int xcd_of_group(unsigned r) { return (r & 8) ? 7 - (int)(r & 7) : (int)(r & 7); }

__global__ __launch_bounds__(SCHED_NT)
void hstu_schedule_kernel(const KArgs a, const SchedDims d, unsigned* __restrict__ ws) {
    const hstu_fwd_params& p = a.p;
    __shared__ unsigned short s_tiles[HSTU_MAX_BATCH];    // tiles of a sequence, by batch index
    __shared__ unsigned short s_order[HSTU_MAX_BATCH];    // batch index, by rank
    __shared__ unsigned char s_key[HSTU_MAX_BATCH];
    __shared__ unsigned char s_sweep[HSTU_MAX_BATCH];     // bit 0: the last item sweeps the tiles behind the attribute; bit 1: tiles 0 and 1 are one item
    __shared__ unsigned s_hist[256], s_base[256];
    __shared__ unsigned s_val[SCHED_NT], s_gpos[SCHED_NT];
    __shared__ unsigned s_wtot[(SCHED_NT / 64) * 16];   // per wave: entries of each residue class (group index % 16)
    __shared__ unsigned s_w4[4], s_len[8], s_ovf;
    __shared__ int s_geo[7][HSTU_MAX_BATCH];              // q_start, lq, k_start, lk, ctx, tgt, first page entry
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nthr = blockDim.x;   // 256, 512 or 1024: small batches run with fewer waves (cheaper barriers)
    unsigned* list = ws + WS_HEADER;
    unsigned* ovf = list + REC * 8 * (size_t)d.cap;

    for (size_t i = tid; i < 8 * (size_t)d.cap; i += nthr) list[REC * i] = ITEM_EMPTY;
    if (tid < 256) s_hist[tid] = 0;
    if (tid == 0) s_ovf = 0;
    __syncthreads();
    // sort key: number of 64-column K tiles (work of a Q tile grows with it), longest first
    for (int b = tid; b < p.batch; b += nthr) {
        const Seq s = load_seq(a, b);
        s_geo[0][b] = (int)s.q_start; s_geo[1][b] = s.lq; s_geo[2][b] = (int)s.k_start; s_geo[3][b] = s.lk;
        s_geo[4][b] = s.ctx; s_geo[5][b] = s.tgt; s_geo[6][b] = (int)s.page0;
        const int t = (s.lq + BM - 1) / BM;
        const int nt = min(t, d.ntiles_attr);
        s_tiles[b] = (unsigned short)nt;
        // The two first Q tiles of a long sequence see few K columns; as items of their own they mostly pay the start and
        // end of a workgroup.  They become one item when together they stay under 70 % of the sequence's last tile.
        bool pair = false;
        if (d.pair && d.nsplit == 1 && t == nt && nt >= 3) {
            const int c0 = (k_extent(a, s, 0, BM) + 63) / 64, c1 = (k_extent(a, s, BM, min(2 * BM, s.lq)) + 63) / 64;
            const int ctop = (k_extent(a, s, (nt - 1) * BM, s.lq) + 63) / 64;
            pair = 10 * (c0 + c1) <= 7 * ctop;
        }
        s_sweep[b] = (t > d.ntiles_attr ? 1 : 0) | (pair ? 2 : 0);
        const int key = 255 - min(255, (s.lk + BN - 1) / BN);
        s_key[b] = (unsigned char)key;
        atomicAdd(&s_hist[key], 1u);
    }
    __syncthreads();
    if (p.batch <= 32) {
        // small batch: rank by counting (ties by batch index, so the order is reproducible), one barrier
        if (tid < p.batch) {
            const unsigned mine = s_key[tid];
            unsigned rank = 0;
            for (int i = 0; i < p.batch; i++) {
                const unsigned k = s_key[i];
                rank += (k < mine) || (k == mine && i < tid);
            }
            s_order[rank] = (unsigned short)tid;
        }
        __syncthreads();
    } else {
        // exclusive scan of the 256 key counts: shuffles inside each of the first four waves, then the waves' totals
        unsigned hcount = 0, hincl = 0;
        if (tid < 256) {
            hcount = s_hist[tid];
            hincl = hcount;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const unsigned t = __shfl_up(hincl, off, 64);
                if (lane >= off) hincl += t;
            }
            if (lane == 63) s_w4[wave] = hincl;
        }
        __syncthreads();
        if (tid < 256) {
            unsigned before = 0;
            for (int ww = 0; ww < wave; ww++) before += s_w4[ww];
            s_base[tid] = before + hincl - hcount;
        }
        __syncthreads();
        for (int b = tid; b < p.batch; b += nthr) s_order[atomicAdd(&s_base[s_key[b]], 1u)] = (unsigned short)b;
        __syncthreads();
    }
    // groups r = rank * heads + head; exclusive prefix of the tile counts inside each XCD's list.  A chunk of
    // 1024 consecutive groups is scanned with stride 16 (one scan per residue class r % 16); XCD x owns the
    // classes x and 15 - x, class x first.
    const unsigned H = (unsigned)p.heads_q, G = (unsigned)p.batch * H;
    const int j = tid & 15, nwaves = nthr >> 6;
    unsigned cb = 0;   // entries of the classes j and 15 - j in the chunks before this one
    for (unsigned c0 = 0; c0 < G; c0 += nthr) {
        const unsigned r = c0 + tid;
        const unsigned rank = r / H, h = r - rank * H;
        const int b = r < G ? (int)s_order[rank] : 0;
        const unsigned ns = (unsigned)d.nsplit;
        const unsigned v = r < G ? (s_tiles[b] - ((s_sweep[b] >> 1) & 1)) * ns : 0u;   // entries of this group: (tile, K range) pairs
        // inclusive scan with stride 16: two shuffles inside the wave, then the totals of the waves before
        unsigned incl = v;
        unsigned t = __shfl_up(incl, 16, 64);
        if (lane >= 16) incl += t;
        t = __shfl_up(incl, 32, 64);
        if (lane >= 32) incl += t;
        if (lane >= 48) s_wtot[wave * 16 + (lane - 48)] = incl;
        __syncthreads();
        unsigned before = 0, chunk = 0;
        for (int ww = 0; ww < nwaves; ww++) {
            const unsigned mine = s_wtot[ww * 16 + j], other = s_wtot[ww * 16 + 15 - j];
            if (ww < wave) before += mine;
            chunk += mine + other;
        }
        incl += before;
        const int tp = (lane & ~15) | (15 - j);
        const unsigned pincl = __shfl(incl, tp, 64), pv = __shfl(v, tp, 64);
        unsigned pos = cb + (incl - v);
        pos += j < 8 ? pincl - pv : pincl;
        cb += chunk;
        // the records of a group are written by `sub` threads side by side (a group has up to 160 * 4 of them)
        s_gpos[tid] = pos;
        s_val[tid] = v;
        if (tid < 8) s_len[tid] = cb;   // entries of list x so far (all of them when the groups fit one chunk)
        __syncthreads();
        const unsigned gcount = min((unsigned)nthr, G - c0);
        unsigned sub = 1;
        while (sub * 2 * gcount <= (unsigned)nthr) sub *= 2;
        const unsigned gi = tid / sub, first = tid - gi * sub;
        if (gi < gcount) {
            const unsigned gr = c0 + gi, grank = gr / H, gh = gr - grank * H;
            const int gb = (int)s_order[grank];
            const unsigned gv = s_val[gi], gpos = s_gpos[gi];
            const int x = xcd_of_group(gr);
            const u32x4 hi = {(unsigned)s_geo[3][gb], (unsigned)s_geo[4][gb], (unsigned)s_geo[5][gb], (unsigned)s_geo[6][gb]};
            u32x4 lo = {0u, (unsigned)s_geo[0][gb], (unsigned)s_geo[1][gb], (unsigned)s_geo[2][gb]};
            const bool sw = s_sweep[gb] & 1, pair = s_sweep[gb] & 2;   // pair implies ns == 1
            // Four groups that follow each other in an XCD's list (r = 16 u + x, 16 u + 15 - x, 16 (u + 1) + x, 16 (u + 1) + 15 - x
            // with u even: all inside this chunk) and have the same number of entries are written interleaved, entry i
            // of the j-th of them at 4 i + j.  The hardware hands the workgroups of an XCD to its four shader engines in
            // turn and in order and waits when the engine whose turn it is has no room: four streams of equal cost keep the
            // engines level, so that none holds the others' free slots up.  It also moves the tiles of a group apart in time,
            // which costs the kernels that lean on the L2 for a group's K/V rows more than it gives them: measured on one
            // box, -6 .. -7 % for the plain variants at head dims 32 and 256, +1 .. +3 % for the dense-bias variant, the paged
            // variant with split K ranges and the backward kernels; the host asks for it accordingly.
            // When every workgroup of a launch is resident at once, the hardware places entries p, p + 32, p + 64 .. of an
            // XCD's list on the same CU (32 CUs, taken in a fixed order).  With the list in falling order of cost all
            // through, the CU of entry 0 then holds the dearest item of every round of 32 and ends last.  Writing the
            // rounds after the first in rising order levels the CUs.
            const unsigned level_n = (d.level_slots > 0 && G <= (unsigned)nthr && s_len[x] <= min(d.cap, 32u * (unsigned)d.level_slots)) ? s_len[x] : 0u;
            unsigned stride = 1, pos0 = gpos;
            if (d.interleave) {
                const unsigned u0 = (gr >> 5) << 1, cx = (unsigned)x;
                const unsigned r4[4] = {16u * u0 + cx, 16u * u0 + 15u - cx, 16u * (u0 + 1) + cx, 16u * (u0 + 1) + 15u - cx};
                if (r4[3] < G && r4[2] < G) {
                    const bool same = s_val[r4[0] - c0] == gv && s_val[r4[1] - c0] == gv && s_val[r4[2] - c0] == gv && s_val[r4[3] - c0] == gv;
                    if (same) {
                        stride = 4;
                        pos0 = s_gpos[r4[0] - c0] + (gr == r4[0] ? 0u : (gr == r4[1] ? 1u : (gr == r4[2] ? 2u : 3u)));
                    }
                }
            }
            for (unsigned i = first; i < gv; i += sub) {
                // last tile first; with `pair` the last entry is tile 0 and covers one more tile (the field that numbers the
                // K ranges of a split tile then holds the count of further tiles)
                const bool both = pair && i == gv - 1;
                const unsigned tile = both ? 0u : (gv - 1 - i) / ns + (pair ? 1u : 0u), part = both ? 1u : i % ns;
                lo[0] = (unsigned)gb | gh << 12 | tile << 16 | ((i < ns && sw) ? 1u << 24 : 0u) | part << 25 | ns << 28;
                unsigned at = pos0 + stride * i;
                if (level_n && at >= 32u) {
                    const unsigned r0 = at & ~31u;
                    at = r0 + (min(32u, level_n - r0) - 1u - (at & 31u));
                }
                unsigned* rec = at < d.cap ? list + REC * (8 * (size_t)at + x) : ovf + REC * (size_t)atomicAdd(&s_ovf, 1u);
                *reinterpret_cast<u32x4*>(rec) = lo;
                *reinterpret_cast<u32x4*>(rec + 4) = hi;
            }
        }
    }
    if (tid < 8) s_len[tid] = cb;   // entries of list x = classes x and 15 - x
    __syncthreads();
    // items that did not fit their XCD's list move to the free slots at the end of the other lists
    const unsigned novf = s_ovf;
    for (unsigned i = tid; i < novf; i += nthr) {
        unsigned k = i;
        for (int x = 0; x < 8; x++) {
            const unsigned len = min(s_len[x], d.cap), free = d.cap - len;
            if (k < free) {
                unsigned* rec = list + REC * (8 * (size_t)(len + k) + x);
                *reinterpret_cast<u32x4*>(rec) = *reinterpret_cast<const u32x4*>(ovf + REC * (size_t)i);
                *reinterpret_cast<u32x4*>(rec + 4) = *reinterpret_cast<const u32x4*>(ovf + REC * (size_t)i + 4);
                break;
            }
            k -= free;
        }
    }
    if (tid == 0) {
        ws[0] = novf;
        // rows the sequences own (the main kernel zero-fills the rows behind them)
        const int64_t owned = p.seq_offset_q ? ld_idx(p.seq_offset_q, p.batch, p.index_type == HSTU_I64) : p.total_q;
        *reinterpret_cast<int64_t*>(ws + 2) = owned;
    }
}


#ifdef HSTU_ITEM_TIMING
// Diagnostics build only (lib/libhstu_hip_timeline.so; the product library is built without it): every workgroup of the
// main kernel leaves {start, time to its first K/V tile in LDS, time to its end, hardware id, K tiles, item word, time to
// its record, time to the end of its last K loop} in 10 ns ticks of the constant clock.
__device__ unsigned g_item_times[8 * 32768];
}  // namespace hstu
extern "C" int hstu_hip_timeline_read(void* dst, size_t bytes) {
    return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(hstu::g_item_times), bytes);
}
namespace hstu {
#endif

// EXTRA: 5 / 6 / 7 = a dense bias / a custom mask / both, rows on 16-byte boundaries, and nothing else: the general
// variant's per-score code carries every option as a run-time test and runs 2.7 x slower than these on the same input;
// 0 = no bias / built-in mask only, 1 = dense bias and/or custom mask (tables, if any, gathered from
// global memory), 2 / 3 / 4 = bias tables only, gathered from LDS-resident copies: position table / time table /
// both (compile-time so that the per-score code is branch-free)
// The plain variant (head dim 128, built-in mask, no bias, rows straight from k/v) fits 168 registers and 34 KB of
// LDS with 32-column K/V tiles: three workgroups per CU (3 waves/SIMD), which overlaps the MFMA, SiLU and LDS phases of
// the waves better than two (measured -8 %).  The head-dim-64 variants other than the dense-bias one fit three per CU
// with 64-column tiles (-10..15 %).  The rest run 64-column tiles at two workgroups per CU.
// EXTRA 8 (paged only) = no bias like 0, with 2-byte pages of a multiple of 4 rows copied straight into LDS; 9 = the same
// for fp8 pages of a multiple of 8 rows: the raw bytes are copied into a staging area and widened from there.
template <int D, int EXTRA, bool PAGED> struct Shape {
    static constexpr bool PDMA8 = PAGED && EXTRA == 9 && D == 128;
    static constexpr bool PDMA = PAGED && (EXTRA == 8 || EXTRA == 9) && D == 128;
    // EXTRA 11: the plain variant (built-in mask, no bias) for head dims that are multiples of 16 other than D, and for
    // dim_qk != dim_v: D is the next of 32 / 64 / 128 / 256 above both, rows come in through registers and the columns
    // past the real dims are zeros in the fragments and in LDS, the output keeps its dim_v columns.
    static constexpr bool UNEVEN = EXTRA == 11;
    static constexpr int MAXP = (PAGED && D == 128 && EXTRA != 8 && EXTRA != 9) ? MAXP_HALF : MAXP_ALL;
    static constexpr bool DMA = (!PAGED && D == 128 && !UNEVEN) || PDMA;
    // head dim 64, rows straight from k / v, no dense bias or custom mask: direct copies too, 8 rows per instruction
    static constexpr bool DMA64 = !PAGED && D == 64 && (EXTRA == 0 || (EXTRA >= 2 && EXTRA <= 7));
    // head dim 32, plain variant: 16 rows of 64 bytes per instruction
    static constexpr bool DMA32 = !PAGED && D == 32 && (EXTRA == 0 || (EXTRA >= 5 && EXTRA <= 7));
    static constexpr bool LEAN = DMA && (EXTRA == 0 || EXTRA == 8 || EXTRA == 9 || EXTRA == 10);
    // EXTRA 10: the plain variant on sequences whose rows are taken in reverse order (row i of q / k / v / out is row
    // L - 1 - i of its sequence in memory).  With K in the place of q, Q in the place of k and dO in the place of v the
    // causal forward then computes dV of the backward: dV[j] = sum over i >= j of P[i][j] dO[i].
    static constexpr bool REV = EXTRA == 10;
    // a dense bias (or, without one, a custom mask) next to direct K/V copies: its blocks are copied into LDS the same way, one tile ahead
    static constexpr bool XDMA = (DMA || DMA64 || DMA32) && EXTRA >= 5 && EXTRA <= 7;
    static constexpr bool RDMA = DMA && REV;
    static constexpr int BNT = (LEAN || XDMA) ? 32 : 64;     // K columns per step
    // waves per SIMD; head dim 256 needs the registers of a whole SIMD lane for its 32 x 256 accumulator and Q fragments
    // (the variants with a bias or a mask copied by DMA fit three at the price of 7 spilled registers: 2 % faster than two;
    // the plain variants at head dims 32 and 64 need 81 / 113 registers and 16 / 34 KB of LDS and run four: 5 % / 1 % faster
    // than three -- at head dim 64 only since its tiles are copied straight into LDS; with the register loader it took 135
    // registers and lost 5 % to AGPR copies under the cap of 128.  Five and six at head dim 32: no faster, 1.5 % slower)
        static constexpr int WAVES = D == 256 ? 1 : (UNEVEN && D == 128) ? 2 : ((D <= 64 && EXTRA == 0 && !PAGED) ? 4 : ((LEAN || (D <= 64 && EXTRA != 1) || (XDMA && EXTRA != 7)) ? 3 : 2));
};

// SELF: no schedule kernel.  For small batches of plain causal self-attention (at most 128 sequences, one set of offsets
// for q and k) every wave of a workgroup derives the workgroup's record from the offsets themselves (self_record), which
// costs a workgroup about a microsecond and saves the call a kernel and the gap between two kernels.
template <typename T, int D, int EXTRA, bool PAGED, bool SELF = false>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(Shape<D, EXTRA, PAGED>::WAVES, Shape<D, EXTRA, PAGED>::WAVES)))
void hstu_mfma_kernel(const KArgs a, const unsigned* __restrict__ ws, const float* part_base) {
    typedef Tile<D> TL;
    typedef Shape<D, EXTRA, PAGED> SH;
    constexpr int MAXP = SH::MAXP;
    constexpr int BNT = SH::BNT;
    constexpr bool LEAN = SH::WAVES >= 3;          // register-tight variants read V fragments right before use
    constexpr bool PARK_OUT = LEAN;                // output tiles leave through LDS as whole rows
    constexpr int NBLK4 = BNT / 4;                 // 4-row blocks per tile
    typedef typename MM<T>::v8 v8;
    const hstu_fwd_params& p = a.p;
    // K/V tiles of head dim 128 that come straight from q-like [rows, heads, D] tensors are copied global -> LDS
    // by buffer loads with the LDS destination (no register staging).  One wave instruction fills 1024
    // contiguous LDS bytes = 4 rows, so a tile is a sequence of 4-row blocks (K blocks padded by 64 B); inside
    // a block row rho keeps its 16-byte chunk c at position (c + rho) % 16 (K) or (c + 4 rho) % 16 (V), which
    // spreads the fragment reads below over all banks.  Everything else goes through registers into padded rows.
    constexpr bool DMA = SH::DMA;
    constexpr int KBLK = 1088, VBLK = 1024;              // bytes per 4-row block
    // Head dim 64: one instruction fills 8 rows of 128 bytes; blocks of 8 rows, 1040 bytes apart, row rho keeping its chunk c
    // in slot (c + 2 (rho / 2)) % 8 -- one layout for K (read row-wise) and V (read transposed): the 16 rows of a row-wise
    // read start on 16 different multiples of 4 banks, the 4 rows of a transposing read lie 16 banks apart.
    constexpr bool DMA64 = SH::DMA64;
    constexpr int B64 = 1040, NBLK8 = BNT / 8;
    // Head dim 32: blocks of 16 rows = 1024 bytes, row rho keeping its chunk c in slot (c + rho / 4) % 4: the 16 rows of a
    // row-wise read then fall on 16 different groups of 4 banks, and a transposing read covers 4 whole consecutive rows.
    constexpr bool DMA32 = SH::DMA32;
    constexpr int NBLK16 = BNT / 16;
    constexpr int STAGE_BYTES = DMA ? NBLK4 * (KBLK + VBLK) : (DMA64 ? 2 * NBLK8 * B64 : (DMA32 ? 2 * NBLK16 * 1024 : (TL::K_ELEMS + TL::V_ELEMS) * 2));
    constexpr bool ANY_DMA = DMA || DMA64 || DMA32;
    // two separate arrays: reads of one tile are then independent of the copy in flight into the other
    __shared__ __attribute__((aligned(1024))) char lds0[STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) char lds1[STAGE_BYTES];
    // table mode: per K tile a window of the position table and the key timestamps (double buffered with the
    // K/V tiles), plus the whole time table and its bucket bounds as (lower, upper) pairs
    constexpr int PW = BM + BN;   // window entries: (j - k0) - (qi - i0) + BM - 1 in [0, BM + BN - 2]
    constexpr bool TAB = EXTRA >= 2 && EXTRA <= 4, tab_pos = EXTRA == 2 || EXTRA == 4, tab_ts = EXTRA == 3 || EXTRA == 4;
    // the dense-only variants: attn_bias (XB) and / or custom mask (XM) given, rows on 16-byte boundaries, no tables (host-checked)
    constexpr bool DENSE_ONLY = EXTRA >= 5 && EXTRA <= 7, XB = EXTRA == 5 || EXTRA == 7, XM = EXTRA == 6 || EXTRA == 7;
    __shared__ float lds_pos[tab_pos ? 2 * PW : 1];
    __shared__ __attribute__((aligned(8))) double lds_tk[tab_ts ? 2 * BN : 1];
    __shared__ __attribute__((aligned(16))) double lds_tkr[tab_ts ? 2 * (BN / 32) * 2 : 2];   // per stage and 32-key block: earliest, latest key time
    __shared__ __attribute__((aligned(16))) float lds_tkf[tab_ts ? 2 * BN : 4];   // key times relative to the earliest one of their block

    // The time table, indexed by the top bits of (float)|dt| itself (exponent and three mantissa bits, counted from 1.0f):
    // cell c covers the values whose bits start with 0x3f8 + c, a range no wider than a factor 1.125, so at most one
    // bucket bound falls inside it (host-checked through the spacing the hint promises).  Entry {that bound or the next
    // one above the cell, table[bucket below it], table[bucket from it on], the bound after that one}: one read and one
    // comparison give the bias.
    constexpr int TS_CELLS = 512;
    __shared__ __attribute__((aligned(16))) float lds_tsq[tab_ts ? 4 * TS_CELLS : 4];
    // paged: page ids of this user and, for an fp8 cache, the (K, V) scales of this kv head
    // fp8 pages by direct copies: raw rows of the next tile (32 keys x 128 bytes of K, then of V; wave w owns keys 8w..8w+7)
    __shared__ __attribute__((aligned(1024))) char lds_raw[SH::PDMA8 ? 2 * 4096 : 16];
    __shared__ int lds_pid[PAGED ? MAXP : 1];
    __shared__ float lds_psc[PAGED ? 2 * MAXP : 1];
    // dense bias / custom mask: every wave takes its 32 x 32 block in as whole 64-byte row pieces (16 bytes per lane, four
    // lanes per row) and reads it back from this private tile in the layout of the score registers; loading it in that
    // layout directly would touch 64 cache lines per instruction.  Row stride 72 bytes.
    constexpr int XRS = 72;
    constexpr bool XTILE = (EXTRA == 1 || DENSE_ONLY) && !PAGED;   // (the paged variant with a dense bias has no registers or LDS to spare for it)
    __shared__ __attribute__((aligned(16))) char lds_x[XTILE ? 4 * 32 * XRS : 16];
    // Direct copies of the bias (or, without a bias, the mask) block of every wave: 32 rows x 32 columns = 2 KB per wave and
    // K tile, two stages.  One wave instruction copies 16 rows of 64 bytes (lane L: row L / 4, 16-byte slot L % 4); slot s of
    // row r holds piece s ^ (r / 4 % 4) of the row, which spreads the 8-byte reads in register layout below over all banks.
    constexpr bool XDMA = SH::XDMA;
    // Two stages in two separate arrays, like the K/V tiles: the compiler then does not make the reads of one stage wait for
    // the copy in flight into the other.
    constexpr int XDW = 2048, XDS = 4 * XDW;   // bytes per wave and per stage
    __shared__ __attribute__((aligned(1024))) char lds_xd0[XDMA ? XDS : 16];
    __shared__ __attribute__((aligned(1024))) char lds_xd1[XDMA ? XDS : 16];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave index, kept in a scalar register
    const int g = lane >> 5, l32 = lane & 31;

#ifdef HSTU_ITEM_TIMING
    const unsigned long long it0 = __builtin_amdgcn_s_memrealtime();
    unsigned long long it1 = it0, it_loop = it0, it_rec = it0;
    int it_ntk = 0;
#endif
    // blockIdx -> record of the work list (see above)
    unsigned rw[REC];
    int64_t owned_rows;
    if constexpr (SELF) {
        // every wave derives the record by itself: no exchange through LDS, no barrier
        __shared__ unsigned lds_hist[4 * 64];
        unsigned rv[REC];
        if (p.seq_offset_k == p.seq_offset_q) self_record<EXTRA != 5, false>(a, (p.max_seq_len_q + BM - 1) / BM, lane, lds_hist + 64 * w, rv, owned_rows);
        else self_record<EXTRA != 5, true>(a, (p.max_seq_len_q + BM - 1) / BM, lane, lds_hist + 64 * w, rv, owned_rows);
#pragma unroll
        for (int i = 0; i < REC; i++) rw[i] = __builtin_amdgcn_readfirstlane(rv[i]);
        // the record also goes where the schedule kernel would have put it, so that the caller's workspace holds the list
        // afterwards and later calls on this geometry can pass HSTU_FLAG_REUSE_WORKSPACE
        if (tid < REC) {
            const unsigned val = tid == 0 ? rw[0] : ((tid == 1 || tid == 3) ? rw[1] : ((tid == 2 || tid == 4) ? rw[2] : (tid == 6 ? rw[6] : 0u)));
            const_cast<unsigned*>(ws)[WS_HEADER + REC * (size_t)blockIdx.x + tid] = val;
        }
        if (blockIdx.x == 0 && tid == 0) {
            const_cast<unsigned*>(ws)[0] = 0u;
            *reinterpret_cast<int64_t*>(const_cast<unsigned*>(ws) + 2) = owned_rows;
        }
    } else {
        const unsigned* rec = ws + WS_HEADER + REC * (size_t)blockIdx.x;
#pragma unroll
        for (int i = 0; i < REC; i++) rw[i] = rec[i];
        // rows the sequences own, for the zero fill at the end: requested here so that nothing waits for it there
        owned_rows = *reinterpret_cast<const int64_t*>(ws + 2);
    }
    asm volatile("" : "+s"(owned_rows));
    const unsigned item = rw[0];
#ifdef HSTU_ITEM_TIMING
    asm volatile("" :: "s"(item));
    it_rec = __builtin_amdgcn_s_memrealtime();
#endif
    const bool active = item != ITEM_EMPTY;
    const int b = active ? (int)(item & 0xfff) : 0, h = active ? (int)((item >> 12) & 0xf) : 0;
    const int tile0 = (int)((item >> 16) & 0xff);
    const bool sweep = (item >> 24) & 1;   // last tile the max_seq_len_q attribute covers of a sequence that is longer
    // bits 25..27: K range of the tile when it is split (bits 28..30 = ranges > 1), else further tiles of the sequence that
    // this item covers after its first one
    const int nsplit = active ? (int)((item >> 28) & 7) : 1;
    const int pfield = active ? (int)((item >> 25) & 7) : 0;
    const int part = nsplit > 1 ? pfield : 0;
    const int tile_last = sweep ? 0x7fffff : tile0 + (nsplit > 1 ? 0 : pfield);
    const int hk = h / a.head_ratio;
    Seq s;
    s.q_start = active ? (int)rw[1] : 0; s.lq = active ? (int)rw[2] : 0;
    s.k_start = active ? (int)rw[3] : 0; s.lk = active ? (int)rw[4] : 0;
    s.ctx = active ? (int)rw[5] : 0; s.tgt = active ? (int)rw[6] : 0; s.page0 = active ? (int)rw[7] : 0;
    s.delta = s.lk - s.lq; s.hist_q = s.lq - s.tgt; s.hist_k = s.lk - s.tgt; s.cand_row = s.q_start + s.hist_q;
    const bool tril = p.mask_type == HSTU_MASK_TRIL;
    const int tgs = p.target_group_size;
    // rows of attn_bias / mask start on 16-byte boundaries
    const bool x_rows16 = DENSE_ONLY || XTILE && p.max_seq_len_k % 8 == 0 && ((reinterpret_cast<uintptr_t>(p.attn_bias) | reinterpret_cast<uintptr_t>(p.mask)) & 15) == 0;
    const bool x_mask = XM || (EXTRA == 1 && p.mask_type == HSTU_MASK_CUSTOM);
    // the direct copies (head dim 128) carry the bias, or the mask of the variant without a bias; with both the mask keeps the tile path
    constexpr bool xd_bias = XDMA && XB, xd_mask = XDMA && !XB;
    const unsigned xd_plane_bytes = (unsigned)p.max_seq_len_q * (unsigned)p.max_seq_len_k * (unsigned)sizeof(T);   // <= 20480^2 * 2
    const char* xd_plane = reinterpret_cast<const char*>(xd_bias ? p.attn_bias : p.mask) + ((int64_t)b * p.heads_q + h) * (int64_t)xd_plane_bytes;
    const T* qbase = reinterpret_cast<const T*>(p.q);
    T* obase = reinterpret_cast<T*>(p.out);

    // loop-invariant per-lane byte offsets of the direct-copy layout
    const unsigned rowstride = (unsigned)p.heads_k * D * 2;   // bytes between consecutive K (or V) rows
    const int lrho = lane >> 4, lpos = lane & 15;             // loader: lane L fills slot L of a 4-row block
    const unsigned ldK = lrho * rowstride + (((lpos - lrho) & 15) << 4);
    const unsigned ldV = lrho * rowstride + (((lpos - 4 * lrho) & 15) << 4);
    const int krho = l32 & 3;                                 // K fragment: row l32 of a 32-key block
    const int kfrag_off = (l32 >> 2) * KBLK + krho * 256;
    const int q4 = (lane & 15) >> 2, u16 = l32 >> 4, piece = lane & 3;   // V transposing reads
    int voff[4];
#pragma unroll
    for (int db = 0; db < 4; db++)
        voff[db] = NBLK4 * KBLK + g * VBLK + q4 * 256 + ((4 * ((db + q4) & 3) + 2 * u16 + (piece >> 1)) << 4) + 8 * (piece & 1);

    for (int tile = tile0; active && tile * BM < s.lq; tile++) {
        const int i0 = tile * BM;
        const int kend = (s.lk > 0) ? k_extent(a, s, i0, min(i0 + BM, s.lq)) : 0;
        const int ntk = (kend + BNT - 1) / BNT;
        const int r0 = i0 + 32 * w;      // first row of this wave
        const int qi = r0 + l32;         // this lane's Q row
        const bool qvalid = qi < s.lq;

        // Q fragment (B operand of S^T = K Q^T): column = Q row, k = head-dim index
        v8 qf[D / 16];
        {
            const int qrow = SH::REV ? s.lq - 1 - min(qi, s.lq - 1) : min(qi, s.lq - 1);
            const int dq_real = SH::UNEVEN ? p.dim_qk : D;
            const T* qp = qbase + ((s.q_start + qrow) * p.heads_q + h) * (int64_t)dq_real + 8 * g;
#pragma unroll
            for (int ds = 0; ds < D / 16; ds++) {
                const u32x4 z = {0, 0, 0, 0};
                const bool have = !SH::UNEVEN || 16 * ds < dq_real;
                const u32x4 x = *reinterpret_cast<const u32x4*>(qp + (have ? 16 * ds : 0));
                qf[ds] = __builtin_bit_cast(v8, qvalid && have ? x : z);
            }
        }
        f32x16 oacc[D / 32];
#pragma unroll
        for (int db = 0; db < D / 32; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[db][r] = 0.f;

        int64_t tq = 0;
        if (EXTRA && EXTRA <= 4 && p.ts_table && qvalid && qi + s.delta >= 0) tq = p.timestamps[s.k_start + qi + s.delta];
        // LDS-table mode works on timestamps relative to the first one of the sequence, held as doubles: the
        // difference of two of them and its rounding to fp32 equal (float)|t_i - t_j| of the int64 values as long as
        // the timestamps of one sequence span less than 2^53
        int64_t tbase = 0;
        if (tab_ts && s.lk > 0) tbase = p.timestamps[s.k_start];
        const double tqd = (double)(tq - tbase);
        // values from the last bound on share the last bucket: |dt| is clamped to it (and to the last cell)
        float ts_top = 1.0f;
        if (tab_ts) {
            ts_top = fminf(p.ts_bounds[p.num_buckets], __builtin_bit_cast(float, 0x3f800000u + ((unsigned)(TS_CELLS - 1) << 20)));
        }
        float pw_reg = 0.f;
        double tk_reg = 0;
        if (PAGED) {
            const int is64 = p.index_type == HSTU_I64;
            const int np = min((s.hist_k + p.page_size - 1) / p.page_size, MAXP);
            for (int i = tid; i < np; i += NT) {
                const int64_t page = ld_idx(p.page_ids, s.page0 + i, is64);
                lds_pid[i] = (int)page;
                // (the variant that copies raw fp8 rows reads the scales behind the request for its first tile, see below)
                if (!SH::PDMA8 && p.cache_dtype == HSTU_FP8_E4M3) {
                    lds_psc[2 * i] = p.kv_scales[(page * 2 + 0) * p.heads_k + hk];
                    lds_psc[2 * i + 1] = p.kv_scales[(page * 2 + 1) * p.heads_k + hk];
                }
            }
            __syncthreads();
        }
        float kscale[TL::NCH], vscale[TL::NCH];
        unsigned fp8mask = 0;

        // Loader.  Register path: loads are unconditional (rows past the visible range are clamped to the last
        // visible row and zeroed when written to LDS) so that they stay in straight-line code and only the LDS
        // write waits for them.  Direct path: a buffer view of this (sequence, kv head) that ends with the last
        // visible row, so rows past it read as zeros.
        u32x4 kreg[ANY_DMA ? 1 : TL::NCH], vreg[ANY_DMA ? 1 : TL::NCH];
        const char* kview = reinterpret_cast<const char*>(p.k) + ((int64_t)s.k_start * p.heads_k + hk) * D * 2;
        const char* vview = reinterpret_cast<const char*>(p.v) + ((int64_t)s.k_start * p.heads_k + hk) * D * 2;
        const unsigned view_bytes = kend > 0 ? (unsigned)(kend - 1) * rowstride + D * 2 : 0;
        auto fetch = [&](int kt, char* dst) __attribute__((always_inline)) {
            const int k0 = kt * BNT;
            if constexpr (SH::PDMA) {
                // Paged rows by direct copies.  A block of 4 rows lies in one page (page_size % 4 == 0, host-checked) or behind
                // the history, in the candidate rows of k / v; lanes of a block that straddles the two take their side under
                // the execution mask.  Rows past the visible range get an offset past the view and arrive as zeros.
                const int ps = p.page_size;
                const unsigned plane_bytes = (unsigned)ps * rowstride;     // the K (or V) half of a page
                const char* cand_k = reinterpret_cast<const char*>(p.k) + ((int64_t)s.cand_row * p.heads_k + hk) * D * 2;
                const char* cand_v = reinterpret_cast<const char*>(p.v) + ((int64_t)s.cand_row * p.heads_k + hk) * D * 2;
                const unsigned chunkK = ((lpos - lrho) & 15) << 4, chunkV = ((lpos - 4 * lrho) & 15) << 4;
#pragma unroll
                for (int i = 0; i < NBLK4 / 4; i++) {
                    const int blk = (NBLK4 / 4) * w + i;
                    const int j0 = k0 + 4 * blk, j = j0 + lrho;            // first key of the block, this lane's key
                    const int pq = j0 / ps, slot0 = j0 - pq * ps;          // page of the block in the user's list, its first slot (wave-uniform)
                    const int pidx = min(pq, MAXP - 1);
                    const int64_t page = __builtin_amdgcn_readfirstlane(lds_pid[j0 < s.hist_k ? pidx : 0]);
                    const char* pk = reinterpret_cast<const char*>(p.kv_cache) + page * (int64_t)(2u * plane_bytes) + (unsigned)hk * D * 2;
                    __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc((void*)pk, 0, 0x7fffffff, 0x00020000);
                    __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc((void*)(pk + plane_bytes), 0, 0x7fffffff, 0x00020000);
                    __amdgpu_buffer_rsrc_t ck = __builtin_amdgcn_make_buffer_rsrc((void*)cand_k, 0, 0x7fffffff, 0x00020000);
                    __amdgpu_buffer_rsrc_t cv = __builtin_amdgcn_make_buffer_rsrc((void*)cand_v, 0, 0x7fffffff, 0x00020000);
                    char* kd = dst + blk * KBLK;
                    char* vd = dst + NBLK4 * KBLK + blk * VBLK;
                    if constexpr (SH::PDMA8) {
                        // only the candidate rows (k / v inputs) come in here; the history rows follow below
                        if (j >= s.hist_k) {
                            const unsigned row = (unsigned)(j - s.hist_k) * rowstride;
                            const unsigned ok = j < kend ? 0u : 0x80000000u;
                            __builtin_amdgcn_raw_ptr_buffer_load_lds(ck, LDS_PTR(void, kd), 16, (row + chunkK) | ok, 0, 0, 0);
                            __builtin_amdgcn_raw_ptr_buffer_load_lds(cv, LDS_PTR(void, vd), 16, (row + chunkV) | ok, 0, 0, 0);
                        }
                    } else if (j < s.hist_k) {
                        const unsigned row = (unsigned)(slot0 + lrho) * rowstride;
                        const unsigned ok = j < kend ? 0u : 0x80000000u;
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, LDS_PTR(void, kd), 16, (row + chunkK) | ok, 0, 0, 0);
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, LDS_PTR(void, vd), 16, (row + chunkV) | ok, 0, 0, 0);
                    } else {
                        const unsigned row = (unsigned)(j - s.hist_k) * rowstride;
                        const unsigned ok = j < kend ? 0u : 0x80000000u;
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(ck, LDS_PTR(void, kd), 16, (row + chunkK) | ok, 0, 0, 0);
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(cv, LDS_PTR(void, vd), 16, (row + chunkV) | ok, 0, 0, 0);
                    }
                }
                if constexpr (SH::PDMA8) {
                    // raw fp8 history rows of this wave's 8 keys (one page: page_size % 8 == 0): lane L = row L / 8, bytes 16 (L % 8) .. + 15
                    const int j0 = k0 + 8 * w;
                    if (j0 < s.hist_k) {
                        const int pq = j0 / ps, slot0 = j0 - pq * ps;
                        const int64_t page = __builtin_amdgcn_readfirstlane(lds_pid[min(pq, MAXP - 1)]);
                        const unsigned row8 = (unsigned)p.heads_k * D;           // bytes between consecutive fp8 rows of a page
                        const unsigned plane8 = (unsigned)ps * row8;
                        const char* pk = reinterpret_cast<const char*>(p.kv_cache) + page * (int64_t)(2u * plane8) + (unsigned)hk * D;
                        __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc((void*)pk, 0, 0x7fffffff, 0x00020000);
                        __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc((void*)(pk + plane8), 0, 0x7fffffff, 0x00020000);
                        const unsigned off = (j0 + (lane >> 3) < s.hist_k) ? (unsigned)(slot0 + (lane >> 3)) * row8 + 16u * (lane & 7) : 0x80000000u;
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, LDS_PTR(void, lds_raw + 1024 * w), 16, off, 0, 0, 0);
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, LDS_PTR(void, lds_raw + 4096 + 1024 * w), 16, off, 0, 0, 0);
                    }
                }
            } else if constexpr (SH::RDMA) {
                // the view is the whole sequence; key j sits in row lk - 1 - j, a row before the sequence gets an offset
                // past the view and arrives as zeros
                const unsigned all_bytes = s.lk > 0 ? (unsigned)(s.lk - 1) * rowstride + D * 2 : 0;
                __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc((void*)kview, 0, (int)all_bytes, 0x00020000);
                __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc((void*)vview, 0, (int)all_bytes, 0x00020000);
#pragma unroll
                for (int i = 0; i < NBLK4 / 4; i++) {
                    const int blk = (NBLK4 / 4) * w + i;
                    const int prow = s.lk - 1 - (k0 + 4 * blk + lrho);
                    const unsigned ro = prow >= 0 ? (unsigned)prow * rowstride : 0x80000000u;
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, LDS_PTR(void, dst + blk * KBLK), 16, ro + (ldK - lrho * rowstride), 0, 0, 0);
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, LDS_PTR(void, dst + NBLK4 * KBLK + blk * VBLK), 16, ro + (ldV - lrho * rowstride), 0, 0, 0);
                }
            } else if constexpr (DMA) {
                const unsigned tile_off = (unsigned)k0 * rowstride;
                __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc((void*)(kview + tile_off), 0, (int)(view_bytes - tile_off), 0x00020000);
                __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc((void*)(vview + tile_off), 0, (int)(view_bytes - tile_off), 0x00020000);
#pragma unroll
                for (int i = 0; i < NBLK4 / 4; i++) {
                    const int blk = (NBLK4 / 4) * w + i;
                    const unsigned so = (unsigned)(4 * blk) * rowstride;
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, LDS_PTR(void, dst + blk * KBLK), 16, ldK + so, 0, 0, 0);
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, LDS_PTR(void, dst + NBLK4 * KBLK + blk * VBLK), 16, ldV + so, 0, 0, 0);
                }
            } else if constexpr (DMA64) {
                const unsigned tile_off = (unsigned)k0 * rowstride;
                __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc((void*)(kview + tile_off), 0, (int)(view_bytes - tile_off), 0x00020000);
                __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc((void*)(vview + tile_off), 0, (int)(view_bytes - tile_off), 0x00020000);
                const int rho = lane >> 3;
                const unsigned lo = (unsigned)rho * rowstride + ((((lane & 7) - 2 * (rho >> 1)) & 7) << 4);   // lane L fills slot L % 8 of row L / 8
#pragma unroll
                for (int i = 0; i < NBLK8 / 4; i++) {
                    const int blk = (NBLK8 / 4) * w + i;
                    const unsigned so = (unsigned)(8 * blk) * rowstride;
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, LDS_PTR(void, dst + blk * B64), 16, lo + so, 0, 0, 0);
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, LDS_PTR(void, dst + (NBLK8 + blk) * B64), 16, lo + so, 0, 0, 0);
                }
            } else if constexpr (DMA32) {
                const unsigned tile_off = (unsigned)k0 * rowstride;
                __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc((void*)(kview + tile_off), 0, (int)(view_bytes - tile_off), 0x00020000);
                __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc((void*)(vview + tile_off), 0, (int)(view_bytes - tile_off), 0x00020000);
                const int rho = lane >> 2;
                const unsigned lo = (unsigned)rho * rowstride + ((((lane & 3) - (rho >> 2)) & 3) << 4);   // lane L fills slot L % 4 of row L / 4
                static_assert(!DMA32 || NBLK16 == 4 || NBLK16 == 2, "one block of K and one of V per wave, or one block per wave");
                if constexpr (NBLK16 == 4) {
                    const unsigned so = (unsigned)(16 * w) * rowstride;
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, LDS_PTR(void, dst + w * 1024), 16, lo + so, 0, 0, 0);
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, LDS_PTR(void, dst + (NBLK16 + w) * 1024), 16, lo + so, 0, 0, 0);
                } else {
                    // tiles of 32 keys: waves 0 and 1 copy the two blocks of K, waves 2 and 3 those of V
                    const int b = w & 1;
                    const unsigned so = (unsigned)(16 * b) * rowstride;
                    if (w < 2) __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, LDS_PTR(void, dst + b * 1024), 16, lo + so, 0, 0, 0);
                    else __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, LDS_PTR(void, dst + (NBLK16 + b) * 1024), 16, lo + so, 0, 0, 0);
                }
            } else if (PAGED && p.page_size % BNT == 0 && k0 + BNT <= s.hist_k) {
                // the whole tile lies in one page of the history (pages hold a multiple of the tile's columns and the
                // history starts at column 0): one page lookup for the tile, rows at a fixed stride
                const int ps = p.page_size;
                const int pidx = min(k0 / ps, MAXP - 1);
                const int64_t page = __builtin_amdgcn_readfirstlane(lds_pid[pidx]);
                const bool fp8 = p.cache_dtype == HSTU_FP8_E4M3;
                const unsigned esz = fp8 ? 1u : (unsigned)sizeof(T);
                const unsigned plane = (unsigned)ps * p.heads_k * D;   // elements of the K (or V) half of a page
                const unsigned rowb = (unsigned)p.heads_k * D * esz;   // bytes between consecutive rows of a page
                const char* kb = reinterpret_cast<const char*>(p.kv_cache) + (page * (int64_t)(2u * plane) + (unsigned)(((k0 % ps) * p.heads_k + hk) * D)) * esz;
                const char* vb = kb + (size_t)plane * esz;
                const float ks = fp8 ? lds_psc[2 * pidx] : 1.f, vs = fp8 ? lds_psc[2 * pidx + 1] : 1.f;
                fp8mask = fp8 ? (1u << TL::NCH) - 1u : 0u;
#pragma unroll
                for (int i = 0; i < TL::NCH; i++) {
                    const int c = tid + NT * i;
                    const int row = c / (D / 8), cc = c % (D / 8);
                    const unsigned off = row * rowb + cc * (fp8 ? 8u : 16u);
                    if (fp8) {
                        const u32x2 kr = *reinterpret_cast<const u32x2*>(kb + off), vr = *reinterpret_cast<const u32x2*>(vb + off);
                        kreg[i] = (u32x4){kr[0], kr[1], 0u, 0u};
                        vreg[i] = (u32x4){vr[0], vr[1], 0u, 0u};
                    } else {
                        kreg[i] = *reinterpret_cast<const u32x4*>(kb + off);
                        vreg[i] = *reinterpret_cast<const u32x4*>(vb + off);
                    }
                    kscale[i] = ks;
                    vscale[i] = vs;
                }
            } else {
#pragma unroll
                for (int i = 0; i < TL::NCH; i++) {
                    const int c = tid + NT * i;
                    const int row = c / (D / 8), cc = c % (D / 8);
                    const int jl = min(k0 + row, kend - 1);
                    const int j = SH::REV ? s.lk - 1 - jl : jl;
                    RowRef<T, PAGED> rk = kv_row_ref<T, PAGED>(a, s, 0, j, hk, SH::UNEVEN ? p.dim_qk : D, lds_pid, lds_psc, MAXP);
                    RowRef<T, PAGED> rv = kv_row_ref<T, PAGED>(a, s, 1, j, hk, SH::UNEVEN ? p.dim_v : D, lds_pid, lds_psc, MAXP);
                    // (uneven dims: chunks past the real row width are read from chunk 0 and zeroed when written to LDS)
                    kreg[i] = load_chunk<T, PAGED>(rk, SH::UNEVEN && cc * 8 >= p.dim_qk ? 0 : cc);
                    vreg[i] = load_chunk<T, PAGED>(rv, SH::UNEVEN && cc * 8 >= p.dim_v ? 0 : cc);
                    if (PAGED) {
                        kscale[i] = rk.scale;
                        vscale[i] = rv.scale;
                        fp8mask = (fp8mask & ~(1u << i)) | ((rk.fp8 ? 1u : 0u) << i);
                    }
                }
            }
            if (TAB) {
                if (tab_pos && tid < PW - 1) {
                    // window entry e holds pos_table[(max_k - 1) + (k0 + e - (BM - 1) - i0) - delta]
                    const int idx = (p.max_seq_len_k - 1) + k0 + tid - (BM - 1) - i0 - s.delta;
                    pw_reg = (idx >= 0 && idx < 2 * p.max_seq_len_k - 1) ? p.pos_table[idx] : 0.f;
                }
                if (tab_ts && tid < BN) tk_reg = (double)(p.timestamps[s.k_start + min(k0 + tid, s.lk - 1)] - tbase);
            }
        };
        // direct copy of this wave's block of the bias (mask) for tile kt into a stage, unless the built-in mask hides the
        // block (wave-uniform).  Pieces outside the [max_q, max_k] square get an offset past the view and arrive as zeros.
        auto fetch_x = [&](int kt, char* xstage) __attribute__((always_inline)) -> bool {
            if constexpr (XDMA) {
                const int k0 = kt * BNT;
                if (!(xd_bias || xd_mask) || k0 >= kend || (tril && classify_block(s, tgs, i0 + 32 * w, k0) == BLK_SKIP)) return false;
                __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void*)xd_plane, 0, (int)xd_plane_bytes, 0x00020000);
                char* xdst = xstage + w * XDW;
#pragma unroll
                for (int n = 0; n < 2; n++) {
                    const int rr = 16 * n + (lane >> 2);                    // row of the block
                    const int row = i0 + 32 * w + rr, col = k0 + 8 * ((lane & 3) ^ ((rr >> 2) & 3));
                    const unsigned off = (row < p.max_seq_len_q && col < p.max_seq_len_k)
                                             ? ((unsigned)row * (unsigned)p.max_seq_len_k + (unsigned)col) * (unsigned)sizeof(T) : 0x80000000u;
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, LDS_PTR(void, xdst + n * 1024), 16, off, 0, 0, 0);
                }
                return true;
            }
            return false;
        };
        // second half of the register path, and the table windows; ends with the tile being complete in LDS
        auto stash = [&](int kt, char* dst) __attribute__((always_inline)) {
            const int k0 = kt * BNT;
            const int buf = kt & 1;
            if (!ANY_DMA && k0 < kend) {
                T* dk = reinterpret_cast<T*>(dst);
                T* dv = dk + TL::K_ELEMS;
#pragma unroll
                for (int i = 0; i < TL::NCH; i++) {
                    const int c = tid + NT * i;
                    const int row = c / (D / 8), cc = c % (D / 8);
                    const bool ok = k0 + row < kend;
                    const u32x4 z = {0, 0, 0, 0};
                    u32x4 kx = kreg[i], vx = vreg[i];
                    if (PAGED && ((fp8mask >> i) & 1)) {
                        kx = dequant_chunk<T>(kx, kscale[i]);
                        vx = dequant_chunk<T>(vx, vscale[i]);
                    }
                    *reinterpret_cast<u32x4*>(dk + row * TL::KS + cc * 8) = ok && (!SH::UNEVEN || cc * 8 < p.dim_qk) ? kx : z;
                    *reinterpret_cast<u32x4*>(dv + row * TL::VS + cc * 8) = ok && (!SH::UNEVEN || cc * 8 < p.dim_v) ? vx : z;
                }
            }
            if (TAB) {
                if (tab_pos && tid < PW - 1) lds_pos[buf * PW + tid] = pw_reg;
                if (tab_ts && tid < BN) {
                    lds_tk[buf * BN + tid] = tk_reg;
                    // earliest and latest key time of each 32-key block (lane t of the first wave holds key t)
                    double lo = tk_reg, hi = tk_reg;
#pragma unroll
                    for (int off = 1; off < 32; off <<= 1) {
                        const double a = __shfl_xor(lo, off, 64), b = __shfl_xor(hi, off, 64);
                        lo = a < lo ? a : lo;
                        hi = b > hi ? b : hi;
                    }
                    // relative to the earliest one the key times of a block are small integers: exact in fp32 below 2^24 (a block
                    // that spans more reports a latest time of +inf, which sends it down the general path)
                    lds_tkf[buf * BN + tid] = (float)(tk_reg - lo);
                    if ((tid & 31) == 0) {
                        lds_tkr[(buf * (BN / 32) + (tid >> 5)) * 2] = lo;
                        lds_tkr[(buf * (BN / 32) + (tid >> 5)) * 2 + 1] = hi - lo < 16777216.0 ? hi : __builtin_inf();
                    }
                }
            }
            if constexpr (ANY_DMA) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if constexpr (SH::PDMA8) {
                // widen this wave's staged history rows (e4m3 x the page's scale, rounded once to the I/O dtype) into the tile:
                // lane L holds 16 elements of key k0 + 8w + L / 8 = chunks 2 (L % 8) and + 1 of row rho = that key % 4
                const int j0 = k0 + 8 * w, j = j0 + (lane >> 3);
                if (k0 < kend && j < s.hist_k) {
                    const int pc = min(j0 / p.page_size, MAXP - 1);
                    const float ks = lds_psc[2 * pc], vs = lds_psc[2 * pc + 1];
                    const u32x4 rk = *reinterpret_cast<const u32x4*>(lds_raw + 1024 * w + 16 * lane);
                    const u32x4 rv = *reinterpret_cast<const u32x4*>(lds_raw + 4096 + 1024 * w + 16 * lane);
                    const int blk = 2 * w + (lane >> 5), rho = (lane >> 3) & 3, c = 2 * (lane & 7);
                    char* kd = dst + blk * KBLK + rho * 256;
                    char* vd = dst + NBLK4 * KBLK + blk * VBLK + rho * 256;
                    *reinterpret_cast<u32x4*>(kd + (((c + rho) & 15) << 4)) = dequant_chunk<T>((u32x4){rk[0], rk[1], 0u, 0u}, ks);
                    *reinterpret_cast<u32x4*>(kd + (((c + 1 + rho) & 15) << 4)) = dequant_chunk<T>((u32x4){rk[2], rk[3], 0u, 0u}, ks);
                    *reinterpret_cast<u32x4*>(vd + (((c + 4 * rho) & 15) << 4)) = dequant_chunk<T>((u32x4){rv[0], rv[1], 0u, 0u}, vs);
                    *reinterpret_cast<u32x4*>(vd + (((c + 1 + 4 * rho) & 15) << 4)) = dequant_chunk<T>((u32x4){rv[2], rv[3], 0u, 0u}, vs);
                }
            }
            __syncthreads();
        };
        // fragment reads
        auto read_kf = [&](const char* cur, int kb, int ds) __attribute__((always_inline)) -> v8 {
            if constexpr (DMA) {
                const int pos = (2 * ds + g + krho) & 15;   // chunk 2*ds + g of row l32, rotated by the row's rho
                return *reinterpret_cast<const v8*>(cur + kb * 8 * KBLK + kfrag_off + (pos << 4));
            } else if constexpr (DMA64) {
                const int rho = l32 & 7;   // row l32 of the 32-key block: block l32 / 8, chunk g + 2 ds
                return *reinterpret_cast<const v8*>(cur + (4 * kb + (l32 >> 3)) * B64 + rho * 128 + (((g + 2 * ds + 2 * (rho >> 1)) & 7) << 4));
            } else if constexpr (DMA32) {
                const int rho = l32 & 15;   // row l32 of the 32-key block: block l32 / 16, chunk g + 2 ds
                return *reinterpret_cast<const v8*>(cur + (2 * kb + (l32 >> 4)) * 1024 + rho * 64 + (((g + 2 * ds + (rho >> 2)) & 3) << 4));
            } else {
                return *reinterpret_cast<const v8*>(reinterpret_cast<const T*>(cur) + (32 * kb + l32) * TL::KS + 8 * g + 16 * ds);
            }
        };
        // 4 keys (rows 32*kb + 8*part + 4*g ..+3) of column 32*db + l32 % 32 for this lane
        auto read_vf = [&](const char* cur, int kb, int db, int part) __attribute__((always_inline)) -> s16x4 {
            if constexpr (DMA) {
                return __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, cur + (8 * kb + 2 * part) * VBLK + voff[db]));
            } else if constexpr (DMA64) {
                // row 8 part + 4 g + (lane % 16) / 4 of the 32-key block = row 4 g + .. of block 4 kb + part; 8 bytes of chunk
                // 4 db + 2 (l32 / 16) + (lane % 4) / 2
                const int rho = 4 * g + ((lane & 15) >> 2), chunk = 4 * db + 2 * (l32 >> 4) + ((lane & 3) >> 1);
                return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    LDS_PTR(s16x4, cur + (NBLK8 + 4 * kb + part) * B64 + rho * 128 + (((chunk + 2 * (rho >> 1)) & 7) << 4) + 8 * (lane & 1)));
            } else if constexpr (DMA32) {
                // row 8 part + 4 g + (lane % 16) / 4 of the 32-key block; 8 bytes of chunk 2 (l32 / 16) + (lane % 4) / 2
                const int r = 8 * part + 4 * g + ((lane & 15) >> 2), rho = r & 15, chunk = 2 * (l32 >> 4) + ((lane & 3) >> 1);
                return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    LDS_PTR(s16x4, cur + (NBLK16 + 2 * kb + (r >> 4)) * 1024 + rho * 64 + (((chunk + (rho >> 2)) & 3) << 4) + 8 * (lane & 1)));
            } else {
                const T* vp = reinterpret_cast<const T*>(cur) + TL::K_ELEMS + (32 * kb + 8 * part + 4 * g + ((lane & 15) >> 2)) * TL::VS + 16 * (l32 >> 4) + 4 * (lane & 3);
                return __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, vp + 32 * db));
            }
        };

        // K range of this workgroup: all tiles, or its share of them when the tile is split
        const int per = (ntk + nsplit - 1) / nsplit;
        const int kt0 = part * per, kt1 = min(ntk, kt0 + per);
        if (kt0 < kt1) fetch(kt0, lds0);
        if (XDMA && kt0 < kt1) fetch_x(kt0, lds_xd0);
        if constexpr (SH::PDMA8) {
            // the pages' scales, a read that depends on the page ids like the first tile's rows: requested behind them, the two
            // round trips overlap; the widening in stash() is the first to need them
            const int np = min((s.hist_k + p.page_size - 1) / p.page_size, MAXP);
            for (int i = tid; i < np; i += NT) {
                const int64_t page = lds_pid[i];
                lds_psc[2 * i] = p.kv_scales[(page * 2 + 0) * p.heads_k + hk];
                lds_psc[2 * i + 1] = p.kv_scales[(page * 2 + 1) * p.heads_k + hk];
            }
            __syncthreads();
        }
        if (tab_ts) {
            // the cells of the time table, built behind the request for the first K/V tile: the two dependent reads per cell
            // (bound, then values) then run while that tile is on its way; the barrier in stash() publishes them
            for (int c = tid; c < TS_CELLS; c += NT) {
                // bucket of the cell's lowest value: the rounded log estimate f or f - 1, the exact bound of f decides
                const float lo = __builtin_bit_cast(float, 0x3f800000u + ((unsigned)c << 20));
                const int f = min((int)(__builtin_amdgcn_logf(lo) * p.ts_log2_scale + 0.5f), p.num_buckets + 1);
                const int bk = max(min(lo >= p.ts_bounds[f] ? f : f - 1, p.num_buckets), 0);
                const f32x4 entry = {p.ts_bounds[bk + 1], p.ts_table[bk], p.ts_table[min(bk + 1, p.num_buckets)], p.ts_bounds[min(bk + 2, p.num_buckets + 1)]};
                *reinterpret_cast<f32x4*>(lds_tsq + 4 * c) = entry;
            }
        }
        stash(kt0, lds0);
#ifdef HSTU_ITEM_TIMING
        if (it1 == it0) it1 = __builtin_amdgcn_s_memrealtime();
        it_ntk += kt1 - kt0;
#endif

        auto iteration = [&](int kt, const char* cur, char* nxt, const char* xcur, char* xnxt) __attribute__((always_inline)) {
            const int buf = kt & 1;
            const int k0 = kt * BNT;
            if (kt + 1 < kt1) fetch(kt + 1, nxt);
            if (XDMA && kt + 1 < kt1) fetch_x(kt + 1, xnxt);

#pragma unroll
            for (int kb = 0; kb < BNT / 32; kb++) {
                const int c0 = k0 + 32 * kb;
                const int cls = tril ? classify_block(s, tgs, r0, c0) : BLK_ALL;
                if (cls == BLK_SKIP) continue;  // wave-uniform
                // ---- S^T block: 32 keys x 32 Q rows.  All K fragments are requested before the first
                // MFMA so that the LDS latency is paid once per block, not once per instruction.
                // dense bias / mask block: rows r0 + lane / 4 and 16 more, columns c0 + 8 * (lane % 4) .. + 7 per lane; requested
                // here, used after the S^T products.  (Requesting it one block ahead costs more in spilled registers than
                // the latency it hides: measured.)
                u32x4 xb[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}}, xm[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
                if (XTILE && x_rows16 && !(XDMA && !(XB && XM))) {
                    const int col = c0 + 8 * (lane & 3);
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        const int row = r0 + (lane >> 2) + 16 * i;
                        if (row < p.max_seq_len_q && col < p.max_seq_len_k) {   // outside the attribute's square: no bias, mask 0
                            const int64_t at = (((int64_t)b * p.heads_q + h) * p.max_seq_len_q + row) * (int64_t)p.max_seq_len_k + col;
                            if ((XB || (EXTRA == 1 && p.attn_bias)) && !xd_bias) xb[i] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const T*>(p.attn_bias) + at);
                            if (x_mask && !xd_mask) xm[i] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const T*>(p.mask) + at);
                        }
                    }
                }
                v8 kf[D / 16];
#pragma unroll
                for (int ds = 0; ds < D / 16; ds++) kf[ds] = read_kf(cur, kb, ds);
                f32x16 sacc;
#pragma unroll
                for (int r = 0; r < 16; r++) sacc[r] = 0.f;
#pragma unroll
                for (int ds = 0; ds < D / 16; ds++) sacc = MM<T>::mfma(kf[ds], qf[ds], sacc);
                // V^T fragments of the first 16-key step: requested now, consumed after the SiLU pass.
                // Transposing LDS read: a 16-lane group reads 4 key rows x 16 columns and every lane
                // receives 4 consecutive keys of one column.
                s16x4 vlo[D / 32], vhi[D / 32], wlo[D / 32], whi[D / 32];
                if (!LEAN) {
#pragma unroll
                    for (int db = 0; db < D / 32; db++) {
                        vlo[db] = read_vf(cur, kb, db, 0);
                        vhi[db] = read_vf(cur, kb, db, 1);
                    }
                }
                // the bias (and mask) block in the layout of the score registers: 4 consecutive keys per 8-byte read
                u32x2 xbr[4], xmr[4];
                if (XTILE && x_rows16) {
                    char* tile = lds_x + w * (32 * XRS);
                    auto through_tile = [&](const u32x4* in, u32x2* out) __attribute__((always_inline)) {
#pragma unroll
                        for (int i = 0; i < 2; i++) {
                            char* at = tile + ((lane >> 2) + 16 * i) * XRS + 16 * (lane & 3);
                            *reinterpret_cast<u32x2*>(at) = (u32x2){in[i][0], in[i][1]};
                            *reinterpret_cast<u32x2*>(at + 8) = (u32x2){in[i][2], in[i][3]};
                        }
                        __builtin_amdgcn_wave_barrier();
#pragma unroll
                        for (int q = 0; q < 4; q++) out[q] = *reinterpret_cast<const u32x2*>(tile + l32 * XRS + (8 * q + 4 * g) * 2);
                        __builtin_amdgcn_wave_barrier();
                    };
                    if ((XB || (EXTRA == 1 && p.attn_bias)) && !xd_bias) through_tile(xb, xbr);
                    if (x_mask && !xd_mask) through_tile(xm, xmr);
                }
                if constexpr (XDMA) {
                    // the copied block in register layout: piece q of row l32 sits in slot q ^ (l32 / 4 % 4)
                    const char* xt = xcur + w * XDW + l32 * 64 + 8 * g;
                    const int sw = (l32 >> 2) & 3;
                    if constexpr (xd_bias) {
#pragma unroll
                        for (int q = 0; q < 4; q++) xbr[q] = *reinterpret_cast<const u32x2*>(xt + 16 * (q ^ sw));
                    } else {
#pragma unroll
                        for (int q = 0; q < 4; q++) xmr[q] = *reinterpret_cast<const u32x2*>(xt + 16 * (q ^ sw));
                    }
                }
                // ---- P = s * sigmoid(alpha * s) (scale folded into the epilogue), masked
                // accumulator register r holds key c0 + 8*(r/4) + 4*g + r%4 for Q row qi
                constexpr bool POS_AHEAD = tab_pos && !tab_ts && D > 64;
                if (POS_AHEAD) {
                    // position bias alone, two workgroups per CU: all sixteen window entries of the lane are requested before the
                    // first is added (2.5 % on the skewed configuration; with the time table next to it the registers run out)
                    float posv[16];
#pragma unroll
                    for (int r = 0; r < 16; r++) posv[r] = lds_pos[buf * PW + 32 * kb + 8 * (r >> 2) + 4 * g + (r & 3) - (32 * w + l32) + (BM - 1)];
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int r = 0; r < 16; r++) sacc[r] += posv[r];
                }
                // Time-bucket bias of a block whose scores lie in at most two neighbouring buckets.  The rows of a wave and the keys
                // of a block are 32 positions each; away from the diagonal |dt| varies by less than the factor between two bucket
                // bounds over the block, so one table cell -- that of the lane's smallest |dt|, row time minus the latest key
                // time -- names the only bound b that can fall into the lane's range, the values on either side of it and the
                // bound after it.  When every lane's largest |dt| stays below that next bound (and no key is later than the
                // row), a score's bias is `dt >= b ? above : below`, and since fp32 rounding is monotone that comparison is
                // `key time <= row time - X` with X the smallest integer that rounds to at least b.  With key times relative
                // to the block's earliest one (integers below 2^24, exact in fp32) that is four 16-byte reads per block and
                // three instructions per score instead of two reads and seven instructions per score, with the same bucket
                // ids bit for bit.
                bool ts_fast = false;
                if constexpr (tab_ts) {
                    const double kmin = lds_tkr[(buf * (BN / 32) + kb) * 2], kmax = lds_tkr[(buf * (BN / 32) + kb) * 2 + 1];
                    const double dlo_d = tqd - kmax;
                    const float dlo = __builtin_amdgcn_fmed3f((float)dlo_d, 1.0f, ts_top), dhi = (float)(tqd - kmin);
                    const unsigned cell16 = ((__builtin_bit_cast(unsigned, dlo) >> 16) & 0xfff0u) - 0x3f80u;
                    const f32x4 ent = *reinterpret_cast<const f32x4*>(reinterpret_cast<const char*>(lds_tsq) + cell16);
                    const bool lane_ok = (dlo_d >= 0.0 && dhi < ent[3]) || !qvalid;
                    ts_fast = __all(lane_ok);
                    if (ts_fast) {
                            // key time <= row time - X, both relative to the block's earliest key: an integer; clamped to what the
                            // relative key times can be, fp32 holds it exactly (beyond 2^24 the rounded value still clamps right)
                            // X: integers x with RN_f32(x) >= b are those from the midpoint m of b and its predecessor on -- from
                            // m itself if it is an integer and b's mantissa is even (the tie goes to b), else from the next integer
                            const unsigned bb = __builtin_bit_cast(unsigned, ent[0]);
                            const double m = 0.5 * ((double)__builtin_bit_cast(float, bb - 1u) + (double)ent[0]);
                            const double cm = __builtin_ceil(m);
                            const double xmin = cm + ((cm == m && (bb & 1u)) ? 1.0 : 0.0);
                            const float thr = __builtin_amdgcn_fmed3f((float)((tqd - xmin) - kmin), -1.0f, 16777216.0f);
                            f32x4 kt[4];
#pragma unroll
                            for (int q = 0; q < 4; q++) kt[q] = *reinterpret_cast<const f32x4*>(lds_tkf + buf * BN + 32 * kb + 8 * q + 4 * g);
#pragma unroll
                            for (int r = 0; r < 16; r++) sacc[r] += kt[r >> 2][r & 3] <= thr ? ent[2] : ent[1];
                    }
                }
                if (tab_ts && D > 64 && !ts_fast) {
                    // time-bucket bias, a batch of scores at a time: all table reads of a batch are in flight before the first is
                    // used (one read right before its use leaves its whole latency exposed, sixteen times per block)
                    constexpr int TSB = 4;
#pragma unroll
                    for (int r8 = 0; r8 < 16; r8 += TSB) {
                        float dcv[TSB];
                        f32x4 ent[TSB];
#pragma unroll
                        for (int i = 0; i < TSB; i++) {
                            const int r = r8 + i;
                            const int jj = 32 * kb + 8 * (r >> 2) + 4 * g + (r & 3);        // j - k0
                            const float dt = (float)__builtin_fabs(tqd - lds_tk[buf * BN + jj]);
                            // the cell of the clamped value; its one bound decides between the two buckets that meet in it
                            dcv[i] = __builtin_amdgcn_fmed3f(dt, 1.0f, ts_top);
                            const unsigned cell16 = ((__builtin_bit_cast(unsigned, dcv[i]) >> 16) & 0xfff0u) - 0x3f80u;
                            ent[i] = *reinterpret_cast<const f32x4*>(reinterpret_cast<const char*>(lds_tsq) + cell16);
                        }
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int i = 0; i < TSB; i++) sacc[r8 + i] += dcv[i] >= ent[i][0] ? ent[i][2] : ent[i][1];
                    }
                }
                float pf[16];
                // (two copies of this loop where the time table is read score by score: with and without those reads)
                auto silu_pass = [&](auto inline_ts) __attribute__((always_inline)) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    float x = sacc[r];
                    const int j = c0 + 8 * (r >> 2) + 4 * g + (r & 3);
                    float mval = 1.f;
                    if (XB) x += half_to_float<T>(xbr[r >> 2][(r >> 1) & 1], r & 1);
                    if (XM) mval = half_to_float<T>(xmr[r >> 2][(r >> 1) & 1], r & 1);
                    if (EXTRA == 1) {
                        const bool in_attr = qi < p.max_seq_len_q && j < p.max_seq_len_k;
                        const int64_t bm = (((int64_t)b * p.heads_q + h) * p.max_seq_len_q + qi) * (int64_t)p.max_seq_len_k + j;
                        if (x_rows16) {
                            if (p.attn_bias) x += half_to_float<T>(xbr[r >> 2][(r >> 1) & 1], r & 1);
                        } else if (p.attn_bias && in_attr) {
                            x += to_float(reinterpret_cast<const T*>(p.attn_bias)[bm]);
                        }
                        if (p.pos_table) {
                            const int idx = (p.max_seq_len_k - 1) + j - (qi + s.delta);
                            if (idx >= 0 && idx < 2 * p.max_seq_len_k - 1) x += p.pos_table[idx];
                        }
                        if (p.ts_table && j < s.lk) {
                            float dt = abs_dt_as_float(tq, p.timestamps[s.k_start + j]);
                            x += p.ts_table[ts_bucket(p.ts_bounds, p.num_buckets, dt)];
                        }
                        if (x_mask) mval = x_rows16 ? half_to_float<T>(xmr[r >> 2][(r >> 1) & 1], r & 1) : (in_attr ? to_float(reinterpret_cast<const T*>(p.mask)[bm]) : 0.f);
                    }
                    if (TAB) {
                        const int jj = 32 * kb + 8 * (r >> 2) + 4 * g + (r & 3);        // j - k0
                        if (tab_pos && !POS_AHEAD) x += lds_pos[buf * PW + jj - (32 * w + l32) + (BM - 1)];
                        if constexpr (decltype(inline_ts)::value) {
                            // (three waves per SIMD leave no registers for reads in flight: one score at a time, between the
                            // transcendental instructions of its neighbours)
                            const float dt = (float)__builtin_fabs(tqd - lds_tk[buf * BN + jj]);
                            const float dc = __builtin_amdgcn_fmed3f(dt, 1.0f, ts_top);
                            const unsigned cell16 = ((__builtin_bit_cast(unsigned, dc) >> 16) & 0xfff0u) - 0x3f80u;
                            const f32x4 entry = *reinterpret_cast<const f32x4*>(reinterpret_cast<const char*>(lds_tsq) + cell16);
                            x += dc >= entry[0] ? entry[2] : entry[1];
                        }
                    }
                    float e = __builtin_amdgcn_exp2f(x * a.exp_scale);
                    float pv = x * __builtin_amdgcn_rcpf(1.0f + e);
                    if (EXTRA == 1 || XM) pv *= mval;
                    pf[r] = pv;
                }
                };
                if (tab_ts && D <= 64 && !ts_fast) silu_pass(std::true_type{});
                else silu_pass(std::false_type{});
                // The built-in mask: the two-per-CU variants zero the fp32 values; the register-tight ones mask the packed
                // pairs instead (fewer operations, and a fully visible block then needs no copies at the join)
                if (!LEAN) {
                    if (cls == BLK_CAUSAL) {
                        const int lim = qi + s.delta - (c0 + 4 * g);  // visible iff 8*(r/4) + r%4 <= lim
#pragma unroll
                        for (int r = 0; r < 16; r++) pf[r] = (8 * (r >> 2) + (r & 3) <= lim) ? pf[r] : 0.f;
                    } else if (cls == BLK_PRED) {
                        // branch-free form of builtin_visible(); j runs over this lane's 16 keys
                        const bool ctx_row = s.ctx > 0 && qi < s.ctx;
                        const bool tgt_row = tgs > 0 && s.tgt > 0 && qi >= s.hist_q;
                        const int left = tgt_row ? s.hist_k + ((qi - s.hist_q) / tgs) * tgs : 0;  // first visible target column
                        const int jmax = qi + s.delta;
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const int j = c0 + 8 * (r >> 2) + 4 * g + (r & 3);
                            const bool vis = (ctx_row & (j < s.hist_k)) | ((j <= jmax) & !(tgt_row & (j >= s.hist_k) & (j < left)));
                            pf[r] = vis ? pf[r] : 0.f;
                        }
                    }
                }
                // ---- O^T += V^T P^T : two 16-key steps per block
                u32x4 pk0, pk1;
#pragma unroll
                for (int x = 0; x < 4; x++) {
                    pk0[x] = MM<T>::pack2(pf[2 * x], pf[2 * x + 1]);
                    pk1[x] = MM<T>::pack2(pf[8 + 2 * x], pf[8 + 2 * x + 1]);
                }
                if (LEAN) {
                    // pair x of the first step holds this lane's key offsets 8*(x/2) + 2*(x%2) and + 1, the second step 16 more
                    if (cls == BLK_CAUSAL) {
                        const int lim = qi + s.delta - (c0 + 4 * g);  // key offset o of this lane is visible iff o <= lim
#pragma unroll
                        for (int x = 0; x < 4; x++) {
                            const int o = 8 * (x >> 1) + 2 * (x & 1);
                            pk0[x] &= o + 1 <= lim ? 0xffffffffu : (o <= lim ? 0xffffu : 0u);
                            pk1[x] &= o + 17 <= lim ? 0xffffffffu : (o + 16 <= lim ? 0xffffu : 0u);
                        }
                    } else if (cls == BLK_PRED) {
                        // branch-free form of builtin_visible() for this lane's 16 keys
                        const bool ctx_row = s.ctx > 0 && qi < s.ctx;
                        const bool tgt_row = tgs > 0 && s.tgt > 0 && qi >= s.hist_q;
                        const int left = tgt_row ? s.hist_k + ((qi - s.hist_q) / tgs) * tgs : 0;  // first visible target column
                        const int jmax = qi + s.delta;
                        auto vis = [&](int r) __attribute__((always_inline)) -> bool {
                            const int j = c0 + 8 * (r >> 2) + 4 * g + (r & 3);
                            return (ctx_row & (j < s.hist_k)) | ((j <= jmax) & !(tgt_row & (j >= s.hist_k) & (j < left)));
                        };
#pragma unroll
                        for (int x = 0; x < 4; x++) {
                            pk0[x] &= (vis(2 * x) ? 0xffffu : 0u) | (vis(2 * x + 1) ? 0xffff0000u : 0u);
                            pk1[x] &= (vis(8 + 2 * x) ? 0xffffu : 0u) | (vis(9 + 2 * x) ? 0xffff0000u : 0u);
                        }
                    }
                }
                if (LEAN) {   // fewer live registers: fragments are read right before the step that uses them
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int db = 0; db < D / 32; db++) {
                        vlo[db] = read_vf(cur, kb, db, 0);
                        vhi[db] = read_vf(cur, kb, db, 1);
                    }
                } else {
#pragma unroll
                    for (int db = 0; db < D / 32; db++) {   // second step's fragments fly while the first step multiplies
                        wlo[db] = read_vf(cur, kb, db, 2);
                        whi[db] = read_vf(cur, kb, db, 3);
                    }
                }
#pragma unroll
                for (int db = 0; db < D / 32; db++) {
                    s16x8 vv = {vlo[db][0], vlo[db][1], vlo[db][2], vlo[db][3], vhi[db][0], vhi[db][1], vhi[db][2], vhi[db][3]};
                    oacc[db] = MM<T>::mfma(__builtin_bit_cast(v8, vv), __builtin_bit_cast(v8, pk0), oacc[db]);
                }
                if (LEAN) {
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int db = 0; db < D / 32; db++) {
                        wlo[db] = read_vf(cur, kb, db, 2);
                        whi[db] = read_vf(cur, kb, db, 3);
                    }
                }
#pragma unroll
                for (int db = 0; db < D / 32; db++) {
                    s16x8 vv = {wlo[db][0], wlo[db][1], wlo[db][2], wlo[db][3], whi[db][0], whi[db][1], whi[db][2], whi[db][3]};
                    oacc[db] = MM<T>::mfma(__builtin_bit_cast(v8, vv), __builtin_bit_cast(v8, pk1), oacc[db]);
                }
            }

            stash(kt + 1, nxt);
        };
        for (int kt = kt0; kt < kt1; kt += 2) {
            iteration(kt, lds0, lds1, lds_xd0, lds_xd1);
            if (kt + 1 < kt1) iteration(kt + 1, lds1, lds0, lds_xd1, lds_xd0);
        }

#ifdef HSTU_ITEM_TIMING
        it_loop = __builtin_amdgcn_s_memrealtime();
#endif
        // ---- epilogue: O^T accumulator register r of block db holds d = 32*db + 8*(r/4) + 4*g + r%4 for row qi
        if (PARK_OUT && nsplit == 1) {
            // Through LDS, so that the stores are whole rows: each wave parks its 32 x D tile in the K/V stage that
            // is free now (every wave is past the last barrier of the K loop), row stride 2*D + 8 bytes, and writes
            // it out 16 bytes per lane, 64 / (D / 8) rows per instruction.
            constexpr int ORS = 2 * D + 8;
            // (head dim 64 with the bias blocks copied: a stage of 32 keys holds one output tile, the other two waves use
            // the stages of the bias blocks)
            constexpr bool PARK_TWO = 2 * 32 * ORS <= STAGE_BYTES;
            static_assert(PARK_TWO || (XDMA && 32 * ORS <= STAGE_BYTES && 32 * ORS <= XDS), "every wave parks its output tile in a stage that is free");
            char* park = PARK_TWO ? ((w & 2) ? lds1 : lds0) + (w & 1) * (32 * ORS)
                                  : ((w & 2) ? ((w & 1) ? lds_xd1 : lds_xd0) : ((w & 1) ? lds1 : lds0));
#pragma unroll
            for (int db = 0; db < D / 32; db++) {
#pragma unroll
                for (int rr = 0; rr < 4; rr++) {
                    u32x2 o;
                    o[0] = MM<T>::pack2(oacc[db][4 * rr] * a.out_scale, oacc[db][4 * rr + 1] * a.out_scale);
                    o[1] = MM<T>::pack2(oacc[db][4 * rr + 2] * a.out_scale, oacc[db][4 * rr + 3] * a.out_scale);
                    *reinterpret_cast<u32x2*>(park + l32 * ORS + (32 * db + 8 * rr + 4 * g) * 2) = o;
                }
            }
            __builtin_amdgcn_wave_barrier();
            constexpr int CPR = D / 8, RPI = 64 / CPR;   // 16-byte chunks per row, rows per instruction
            int elane = lane;
            asm volatile("" : "+v"(elane));   // keeps the address arithmetic below out of the K loop's live ranges
            const int orow = elane / CPR, ochunk = elane % CPR;
#pragma unroll
            for (int i = 0; i < 32 / RPI; i++) {
                const int row = RPI * i + orow;
                const u32x4 x = *reinterpret_cast<const u32x4*>(park + row * ORS + ochunk * 16);
                const int dv_real = SH::UNEVEN ? p.dim_v : D;
                if (r0 + row < s.lq && (!SH::UNEVEN || ochunk * 8 < dv_real)) {
                    const int out_row = SH::REV ? s.lq - 1 - (r0 + row) : r0 + row;
                    *reinterpret_cast<u32x4*>(obase + ((s.q_start + out_row) * p.heads_q + h) * (int64_t)dv_real + ochunk * 8) = x;
                }
            }
        } else if (nsplit == 1) {
            // the two lanes of a row hold alternating 8-byte pieces of it: they exchange halves (v_permlane32_swap: upper half of
            // one register with the lower half of another) and store 16 bytes each
            const int orow = qvalid ? (SH::REV ? s.lq - 1 - qi : qi) : 0;
            const int dv_real = SH::UNEVEN ? p.dim_v : D;
            T* op = obase + ((s.q_start + orow) * p.heads_q + h) * (int64_t)dv_real + 8 * g;
#pragma unroll
            for (int db = 0; db < D / 32; db++) {
#pragma unroll
                for (int pr = 0; pr < 2; pr++) {
                    unsigned o[4];
#pragma unroll
                    for (int x = 0; x < 4; x++) o[x] = MM<T>::pack2(oacc[db][8 * pr + 2 * x] * a.out_scale, oacc[db][8 * pr + 2 * x + 1] * a.out_scale);
                    const u32x2 s0 = __builtin_amdgcn_permlane32_swap(o[0], o[2], false, false);
                    const u32x2 s1 = __builtin_amdgcn_permlane32_swap(o[1], o[3], false, false);
                    const u32x4 out4 = {s0[0], s1[0], s0[1], s1[1]};
                    if (qvalid && (!SH::UNEVEN || 32 * db + 16 * pr < dv_real)) *reinterpret_cast<u32x4*>(op + 32 * db + 16 * pr) = out4;
                }
            }
        } else if (qvalid) {
            // partial sums of this K range, unscaled fp32, [range][row][head][D] behind the work list
            float* pp = const_cast<float*>(part_base) + (((int64_t)part * p.total_q + s.q_start + qi) * p.heads_q + h) * (int64_t)D + 4 * g;
#pragma unroll
            for (int db = 0; db < D / 32; db++) {
#pragma unroll
                for (int rr = 0; rr < 4; rr++) {
                    const f32x4 o = {oacc[db][4 * rr], oacc[db][4 * rr + 1], oacc[db][4 * rr + 2], oacc[db][4 * rr + 3]};
                    *reinterpret_cast<f32x4*>(pp + 32 * db + 8 * rr) = o;
                }
            }
        }
        if (tile >= tile_last) break;
        __syncthreads();   // the next tile's loads overwrite the stages the output tiles were parked in
    }

#ifdef HSTU_ITEM_TIMING
    if (tid == 0 && blockIdx.x < 32768) {
        const unsigned long long it2 = __builtin_amdgcn_s_memrealtime();
        unsigned* o = g_item_times + 8 * blockIdx.x;
        o[0] = (unsigned)it0; o[1] = (unsigned)(it1 - it0); o[2] = (unsigned)(it2 - it0);
        o[3] = __builtin_amdgcn_s_getreg((31 << 11) | 4);     // HW_ID: wave 3:0, SIMD 5:4, CU 11:8, SH 12, SE 15:13
        o[4] = (unsigned)it_ntk; o[5] = item;
        o[6] = (unsigned)(it_rec - it0);                      // time to the record
        o[7] = (unsigned)(it_loop - it0);
    }
#endif
    // rows past the last offset are zero (the reference zero-fills its output: hstu_jagged.cpp:56-59)
    if (owned_rows < p.total_q) {
        const int64_t n = (p.total_q - owned_rows) * p.heads_q * (int64_t)(SH::UNEVEN ? p.dim_v : D);
        T* o = obase + owned_rows * p.heads_q * (int64_t)(SH::UNEVEN ? p.dim_v : D);
        for (int64_t e = (int64_t)blockIdx.x * NT + tid; e < n; e += (int64_t)gridDim.x * NT) o[e] = (T)0.f;
    }
}

// out = (sum over the K ranges of the partial sums) * alpha * silu_scale, for the rows the sequences own
template <typename T>
__global__ __launch_bounds__(256)
void hstu_reduce_kernel(const KArgs a, const float* __restrict__ part, const int nsplit) {
    const hstu_fwd_params& p = a.p;
    const int is64 = p.index_type == HSTU_I64;
    const int64_t rows = p.seq_offset_q ? ld_idx(p.seq_offset_q, p.batch, is64) : p.total_q;
    const int64_t per_range = p.total_q * p.heads_q * (int64_t)p.dim_v;
    const int64_t n4 = rows * p.heads_q * (int64_t)p.dim_v / 4;
    T* out = reinterpret_cast<T*>(p.out);
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (int64_t)gridDim.x * 256) {
        f32x4 acc = *reinterpret_cast<const f32x4*>(part + 4 * i);
        for (int r = 1; r < nsplit; r++) {
            const f32x4 x = *reinterpret_cast<const f32x4*>(part + r * per_range + 4 * i);
            acc[0] += x[0]; acc[1] += x[1]; acc[2] += x[2]; acc[3] += x[3];
        }
        u32x2 o;
        o[0] = MM<T>::pack2(acc[0] * a.out_scale, acc[1] * a.out_scale);
        o[1] = MM<T>::pack2(acc[2] * a.out_scale, acc[3] * a.out_scale);
        *reinterpret_cast<u32x2*>(out + 4 * i) = o;
    }
}

bool mfma_supported(const KArgs& a, const char** name) {
    const hstu_fwd_params& p = a.p;
    *name = nullptr;
    if (p.dtype == HSTU_FP8_E4M3) return mfma_fp8_supported(a, name);
    if (p.dtype != HSTU_BF16 && p.dtype != HSTU_F16) return false;
    int d = p.dim_qk;
    const bool uneven = uneven_dims(p);
    if (uneven) {
        // other multiples of 16 up to 256, and dim_qk != dim_v (the reference's own benchmark list has (64, 32) and (128, 48),
        // cust_op/test/hstu_v2/test_forward_op_benchmark.py:192-193): the padded plain variant -- built-in mask or none, no
        // bias, no tables, rows straight from k / v
        if (p.dim_qk % 16 || p.dim_v % 16 || p.dim_qk > 256 || p.dim_v > 256) return false;
        if (a.op == OP_PAGED || p.attn_bias || p.mask_type == HSTU_MASK_CUSTOM || p.pos_table || p.ts_table) return false;
        d = padded_dim(p);
    }
    // rows are read and written 16 bytes at a time (vector loads, direct copies into LDS): buffers that do not start on
    // such a boundary take the plain kernel
    const uintptr_t all = reinterpret_cast<uintptr_t>(p.q) | reinterpret_cast<uintptr_t>(p.k) | reinterpret_cast<uintptr_t>(p.v) |
                          reinterpret_cast<uintptr_t>(p.out) | reinterpret_cast<uintptr_t>(p.kv_cache);
    if (all & 15) return false;
    if (a.op == OP_PAGED) {   // page ids of a user must fit the LDS copy of the variant the call takes
        const bool copies = d == 128 && !p.attn_bias && p.mask_type != HSTU_MASK_CUSTOM && !p.pos_table && !p.ts_table &&
                            ((p.cache_dtype == p.dtype && p.page_size % 4 == 0) || (p.cache_dtype == HSTU_FP8_E4M3 && p.page_size % 8 == 0));
        if ((p.max_seq_len_k + p.page_size - 1) / p.page_size > ((d == 128 && !copies) ? MAXP_HALF : MAXP_ALL)) return false;
    }
    const bool bf = p.dtype == HSTU_BF16;
    if (uneven) {
        *name = d == 32 ? (bf ? "mfma_bf16_d32_padded" : "mfma_f16_d32_padded") : d == 64 ? (bf ? "mfma_bf16_d64_padded" : "mfma_f16_d64_padded")
              : d == 128 ? (bf ? "mfma_bf16_d128_padded" : "mfma_f16_d128_padded") : (bf ? "mfma_bf16_d256_padded" : "mfma_f16_d256_padded");
        return true;
    }
    *name = d == 32 ? (bf ? "mfma_bf16_d32" : "mfma_f16_d32") : d == 64 ? (bf ? "mfma_bf16_d64" : "mfma_f16_d64")
          : d == 128 ? (bf ? "mfma_bf16_d128" : "mfma_f16_d128") : (bf ? "mfma_bf16_d256" : "mfma_f16_d256");
    return true;
}

// Which variant of the kernel (template argument EXTRA, before the paged / padded choices) the options of a call ask for.
static int forward_extra(const KArgs& a) {
    const hstu_fwd_params& p = a.p;
    const bool dense_extra = p.attn_bias || p.mask_type == HSTU_MASK_CUSTOM;
    // the time table is used from LDS when it fits and the search hint is there; else the general path searches the
    // bounds in global memory
    // the LDS time table: buckets at least a factor 2^(1/5) apart (wider than its cells) and the last bound below 2^62
    const bool ts_in_lds = p.ts_table && p.ts_log2_scale > 0.f && p.ts_log2_scale <= 5.0f && p.num_buckets <= 62.f * p.ts_log2_scale;
    // a dense bias and / or a custom mask alone, rows on 16-byte boundaries: the variants without the other options
    const bool custom = p.mask_type == HSTU_MASK_CUSTOM;
    const bool dense_only = dense_extra && !p.pos_table && !p.ts_table && a.op != OP_PAGED && p.max_seq_len_k % 8 == 0 &&
                            ((reinterpret_cast<uintptr_t>(p.attn_bias) | (custom ? reinterpret_cast<uintptr_t>(p.mask) : 0)) & 15) == 0;
    if (dense_only) return p.attn_bias ? (custom ? 7 : 5) : 6;
    if (dense_extra || (p.ts_table && !ts_in_lds)) return 1;
    if (p.pos_table && p.ts_table) return 4;
    if (p.ts_table) return 3;
    if (p.pos_table) return 2;
    return 0;
}

// Launches without a schedule kernel (see SELF): the variants with the built-in mask or none and at most the bias tables
// or a dense bias alone at head dims 64 and 128 (the plain and the dense-bias variants also at 32), one or two sequences per lane, at most 64 tile-count classes (63 tile counts and the class of longer
// sequences), and lists that cannot overflow (entries per group follow the Q tiles alone and fall along the order; K offsets in a
// tensor of their own are fine when q and k have as many rows in total, the sign of plain self-attention).
// A caller that already holds a list (HSTU_FLAG_REUSE_WORKSPACE) keeps using it.
bool mfma_self_scheduled(const KArgs& a) {
    const hstu_fwd_params& p = a.p;
    if (p.dtype == HSTU_FP8_E4M3) return p.dim_qk == p.dim_v && (p.dim_qk == 64 || p.dim_qk == 128 || p.dim_qk == 256) && mfma_fp8_self_scheduled(a);
    const int extra = forward_extra(a);
    // head dim 32 has the plain variant only; at head dim 256 a SIMD holds one wave and nothing hides the derivation
    // (level with the schedule kernel on small batches, slower on large ones)
    const bool tables_too = p.dim_qk == 128 || p.dim_qk == 64;
    return a.op == OP_JAGGED && (p.dtype == HSTU_BF16 || p.dtype == HSTU_F16) && p.dim_qk == p.dim_v &&
           (p.dim_qk == 32 || p.dim_qk == 64 || p.dim_qk == 128) &&
           p.batch >= 1 && p.batch <= 128 && p.seq_offset_q && p.seq_offset_k && p.total_q == p.total_k && !p.num_context &&
           (p.mask_type == HSTU_MASK_TRIL || p.mask_type == HSTU_MASK_NONE) && (extra == 0 || extra == 5 || (tables_too && extra >= 2 && extra <= 4)) &&
           p.max_seq_len_q == p.max_seq_len_k && p.max_seq_len_q <= 63 * BM &&
           !(p.flags & HSTU_FLAG_REUSE_WORKSPACE) && sched_dims(p).nsplit == 1;
}

hipError_t launch_work_list(const KArgs& a, unsigned* ws, bool pair, hipStream_t stream) {
    SchedDims d = sched_dims(a.p, true);
    d.pair = pair ? 1 : 0;
    const int groups = a.p.batch * a.p.heads_q;
    const int sched_threads = groups <= 128 ? 256 : (groups <= 512 ? 512 : SCHED_NT);
    hipLaunchKernelGGL(hstu_schedule_kernel, dim3(1), dim3(sched_threads), 0, stream, a, d, ws);
    return hipGetLastError();
}

template <typename T, int D>
static hipError_t launch_td(const KArgs& a, unsigned* ws, hipStream_t stream) {
    const hstu_fwd_params& p = a.p;
    const SchedDims d = sched_dims(p);
    const int extra = forward_extra(a);
    const bool paged = a.op == OP_PAGED;
    // (the order in which launch_td's schedule kernel writes four equal groups: see hstu_schedule_kernel)
    SchedDims dsched = d;
    dsched.interleave = (!paged && d.nsplit == 1 && (extra == 0 || (extra >= 2 && extra <= 4))) ? 1 : 0;
    dsched.level_slots = (paged && d.nsplit > 1) ? 3 : 0;   // the paged variants hold two or three workgroups per CU
    const int groups = p.batch * p.heads_q;
    const int sched_threads = groups <= 128 ? 256 : (groups <= 512 ? 512 : SCHED_NT);   // spare threads write a group's records side by side
    hipError_t e = hipSuccess;
    dim3 grid(8 * d.cap), block(NT);   // the overflow list starts at entry gridDim.x of the lists
    const float* part = reinterpret_cast<const float*>(reinterpret_cast<const char*>(ws) + list_bytes(d));
    if constexpr (D == 32) {
        if (!paged && !uneven_dims(p) && mfma_self_scheduled(a)) {
            if (extra == 0) hipLaunchKernelGGL((hstu_mfma_kernel<T, D, 0, false, true>), grid, block, 0, stream, a, ws, part);
            else hipLaunchKernelGGL((hstu_mfma_kernel<T, D, 5, false, true>), grid, block, 0, stream, a, ws, part);
            return hipGetLastError();
        }
    }
    if constexpr (D == 128 || D == 64) {
        // small batches: the workgroups find their items themselves, no schedule kernel
        if (!paged && mfma_self_scheduled(a)) {
            if (extra == 0) hipLaunchKernelGGL((hstu_mfma_kernel<T, D, 0, false, true>), grid, block, 0, stream, a, ws, part);
            else if (extra == 2) hipLaunchKernelGGL((hstu_mfma_kernel<T, D, 2, false, true>), grid, block, 0, stream, a, ws, part);
            else if (extra == 3) hipLaunchKernelGGL((hstu_mfma_kernel<T, D, 3, false, true>), grid, block, 0, stream, a, ws, part);
            else if (extra == 5) hipLaunchKernelGGL((hstu_mfma_kernel<T, D, 5, false, true>), grid, block, 0, stream, a, ws, part);
            else hipLaunchKernelGGL((hstu_mfma_kernel<T, D, 4, false, true>), grid, block, 0, stream, a, ws, part);
            return hipGetLastError();
        }
    }
    if (!(p.flags & HSTU_FLAG_REUSE_WORKSPACE)) {
        hipLaunchKernelGGL(hstu_schedule_kernel, dim3(1), dim3(sched_threads), 0, stream, a, dsched, ws);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
#define HSTU_LAUNCH(E, P) hipLaunchKernelGGL((hstu_mfma_kernel<T, D, E, P>), grid, block, 0, stream, a, ws, part)
    if (uneven_dims(p)) {
        HSTU_LAUNCH(11, false);
    } else if constexpr (D == 32 || D == 256) {
        // the head dims at the ends of the reference's sweep: plain and general variants only (bias tables are gathered
        // from global memory by the general one)
        if (paged && extra == 0) HSTU_LAUNCH(0, true);
        else if (paged) HSTU_LAUNCH(1, true);
        else if (extra == 0) HSTU_LAUNCH(0, false);
        else if (extra == 5) HSTU_LAUNCH(5, false);
        else if (extra == 6) HSTU_LAUNCH(6, false);
        else if (extra == 7) HSTU_LAUNCH(7, false);
        else HSTU_LAUNCH(1, false);
    } else if (paged) {
        // pages in the dtype of q with a multiple of 4 rows: rows are copied straight into LDS (head dim 128)
        const bool page_copies = D == 128 && p.cache_dtype == p.dtype && p.page_size % 4 == 0;
        const bool page_copies8 = D == 128 && p.cache_dtype == HSTU_FP8_E4M3 && p.page_size % 8 == 0;
        if (extra == 0 && page_copies) HSTU_LAUNCH(8, true);
        else if (extra == 0 && page_copies8) HSTU_LAUNCH(9, true);
        else if (extra == 0) HSTU_LAUNCH(0, true);
        else HSTU_LAUNCH(1, true);      // paged + bias: the general gather path
    } else {
        if (extra == 0) HSTU_LAUNCH(0, false);
        else if (extra == 1) HSTU_LAUNCH(1, false);
        else if (extra == 2) HSTU_LAUNCH(2, false);
        else if (extra == 3) HSTU_LAUNCH(3, false);
        else if (extra == 5) HSTU_LAUNCH(5, false);
        else if (extra == 6) HSTU_LAUNCH(6, false);
        else if (extra == 7) HSTU_LAUNCH(7, false);
        else HSTU_LAUNCH(4, false);
    }
#undef HSTU_LAUNCH
    e = hipGetLastError();
    if (e != hipSuccess || d.nsplit == 1) return e;
    const int64_t n4 = p.total_q * p.heads_q * (int64_t)p.dim_v / 4;
    const unsigned rgrid = (unsigned)((n4 + 255) / 256 < 2048 ? (n4 + 255) / 256 : 2048);
    hipLaunchKernelGGL(hstu_reduce_kernel<T>, dim3(rgrid ? rgrid : 1), dim3(256), 0, stream, a, part, d.nsplit);
    return hipGetLastError();
}

bool reversed_forward_supported(const hstu_fwd_params& p) {
    return p.dim_qk == 128 && p.dim_v == 128 && (p.dtype == HSTU_BF16 || p.dtype == HSTU_F16) && p.mask_type == HSTU_MASK_TRIL &&
           !p.num_context && !p.num_target && !p.attn_bias && !p.pos_table && !p.ts_table && p.heads_q == p.heads_k &&
           p.seq_offset_q == p.seq_offset_k && p.max_seq_len_q == p.max_seq_len_k && p.total_q == p.total_k;
}

hipError_t launch_reversed_forward(const KArgs& a, const unsigned* ws, hipStream_t stream) {
    const SchedDims d = sched_dims(a.p, true);
    dim3 grid(8 * d.cap), block(NT);
    const float* none = nullptr;
    if (a.p.dtype == HSTU_BF16) hipLaunchKernelGGL((hstu_mfma_kernel<__bf16, 128, 10, false>), grid, block, 0, stream, a, ws, none);
    else hipLaunchKernelGGL((hstu_mfma_kernel<_Float16, 128, 10, false>), grid, block, 0, stream, a, ws, none);
    return hipGetLastError();
}

hipError_t launch_mfma(const KArgs& a, void* workspace, hipStream_t stream) {
    const hstu_fwd_params& p = a.p;
    unsigned* ws = reinterpret_cast<unsigned*>(workspace);
    if (p.dtype == HSTU_FP8_E4M3) return launch_mfma_fp8(a, workspace, stream);
    const int d = uneven_dims(p) ? padded_dim(p) : p.dim_qk;
    if (p.dtype == HSTU_BF16) {
        switch (d) {
            case 32: return launch_td<__bf16, 32>(a, ws, stream);
            case 64: return launch_td<__bf16, 64>(a, ws, stream);
            case 128: return launch_td<__bf16, 128>(a, ws, stream);
            default: return launch_td<__bf16, 256>(a, ws, stream);
        }
    }
    switch (d) {
        case 32: return launch_td<_Float16, 32>(a, ws, stream);
        case 64: return launch_td<_Float16, 64>(a, ws, stream);
        case 128: return launch_td<_Float16, 128>(a, ws, stream);
        default: return launch_td<_Float16, 256>(a, ws, stream);
    }
}

}  // namespace hstu
