// Deriving a workgroup's work-list record inside the main kernel (launches without the schedule kernel), shared by the
// 16-bit and the fp8 matrix-core kernels.  Both use Q tiles of 128 rows and the record layout of hstu_internal.h.
#pragma once
#include "hstu_device.h"

namespace hstu {

// Inclusive prefix sum over the 64 lanes of a wave by data-parallel-primitive moves: four shifts inside each row of 16
// lanes, then lane 15 of rows 0 / 2 into rows 1 / 3 and lane 31 into rows 2 and 3.
__device__ __forceinline__ unsigned wave_inclusive_sum(unsigned v) {
    v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false);   // row_shr:1
    v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false);   // row_shr:2
    v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, false);   // row_shr:4
    v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, false);   // row_shr:8
    v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);   // row_bcast:15, rows 1 and 3
    v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false);   // row_bcast:31, rows 2 and 3
    return v;
}

// x / y for x < 2^20 / y: exact, because (x + 0.5) / y lies at least 0.5 / y away from every integer
__device__ __forceinline__ unsigned small_div(unsigned x, unsigned y) {
    return (unsigned)(((float)x + 0.5f) * __builtin_amdgcn_rcpf((float)y));
}

// The record of workgroup blockIdx.x without a work list, computed by one wave on its own (the caller guarantees
// batch <= 128, at most 63 Q tiles per sequence under the attribute, the same attribute for q and k, no context rows, the
// built-in causal mask or no mask; target rows are fine).  The order is the schedule kernel's with a coarser key: sequences by
// their number of Q tiles (longest first, then by batch index), (sequence, head) groups r = rank * heads + head dealt to
// the XCDs in snake order (XCD x owns r = 16 u + x and 16 u + 15 - x), a group's tiles last tile first (the tiles of four
// groups of one class in turn, see below), under the causal mask the first two tiles of a sequence of five or more tiles as one item.  Lane b first holds sequences b and b + 64, then lane k holds the
// class of the sequences with cmax - k tiles (a histogram in `hist`, 64 words of LDS private to the wave): the sequences
// and the list entries ahead of a class are two prefix sums over the lanes, so the cost does not grow with the number of
// classes.  No list can exceed the grid: with entries per group falling along r, the lists differ by at most one group's
// entries.
constexpr int SELF_TILE_ROWS = 128;

template <bool FOUR_STREAMS = true, bool OWN_K = false>
__device__ __forceinline__ void self_record(const KArgs& a, int ntiles_attr, int lane, unsigned* hist, unsigned (&rec)[WORK_RECORD_WORDS], int64_t& rows) {
    const hstu_fwd_params& p = a.p;
    const int B = p.batch, H = p.heads_q;
    const int is64 = p.index_type == HSTU_I64;
    // offsets b and b + 1 of a sequence in one load (two dependent loads would double the wait)
    struct __attribute__((aligned(8))) I64x2 { int64_t lo, hi; };
    struct __attribute__((aligned(4))) I32x2 { int lo, hi; };
    const int cmax = ntiles_attr + 1;
    int64_t o0[2], o1[2];
    int len[2], cls[2], tgt[2];
    // OWN_K: the K offsets are a tensor of their own (the order follows the Q tiles either way; the record carries the K
    // range).  A template argument, chosen by the caller ahead of everything: a test down here would split the loads below
    // into two round trips, and loading them always costs the common case 0.4 us per call.
    unsigned ks[OWN_K ? 2 : 1], kl[OWN_K ? 2 : 1];
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const bool mine = lane + 64 * u < B;
        const int mb = mine ? lane + 64 * u : 0;
        if (is64) {
            const I64x2 v = *reinterpret_cast<const I64x2*>(static_cast<const int64_t*>(p.seq_offset_q) + mb);
            o0[u] = v.lo; o1[u] = v.hi;
            if constexpr (OWN_K) {
                const I64x2 kv = *reinterpret_cast<const I64x2*>(static_cast<const int64_t*>(p.seq_offset_k) + mb);
                ks[u] = (unsigned)kv.lo; kl[u] = (unsigned)(kv.hi - kv.lo);
            }
        } else {
            const I32x2 v = *reinterpret_cast<const I32x2*>(static_cast<const int*>(p.seq_offset_q) + mb);
            o0[u] = v.lo; o1[u] = v.hi;
            if constexpr (OWN_K) {
                const I32x2 kv = *reinterpret_cast<const I32x2*>(static_cast<const int*>(p.seq_offset_k) + mb);
                ks[u] = (unsigned)kv.lo; kl[u] = (unsigned)(kv.hi - kv.lo);
            }
        }
        tgt[u] = p.num_target ? (int)ld_idx(p.num_target, mb, is64) : 0;
    }
#pragma unroll
    for (int u = 0; u < 2; u++) {
        len[u] = (int)(o1[u] - o0[u]);
        // class of a sequence = its tile count; sequences longer than the attribute covers form the class above
        cls[u] = lane + 64 * u < B ? min((len[u] + SELF_TILE_ROWS - 1) / SELF_TILE_ROWS, cmax) : 0;
    }
    // rows the sequences own = the last offset, which the lane of sequence batch - 1 holds (a scalar load of its own would make
    // every later wait for a kernel argument wait for a round trip to the L2 as well)
    {
        const int64_t last = B > 64 ? o1[1] : o1[0];
        const int ll = (B - 1) & 63;
        rows = (int64_t)(((uint64_t)(unsigned)__builtin_amdgcn_readlane((int)(last >> 32), ll) << 32) | (unsigned)__builtin_amdgcn_readlane((int)last, ll));
    }
    hist[lane] = 0u;
    __builtin_amdgcn_wave_barrier();
    if (cls[0] > 0) atomicAdd(&hist[cmax - cls[0]], 1u);
    if (cls[1] > 0) atomicAdd(&hist[cmax - cls[1]], 1u);
    __builtin_amdgcn_wave_barrier();
    const unsigned n = hist[lane];                       // sequences of class c
    const int c = cmax - lane;                           // (lanes from cmax on: n = 0)
    const unsigned x = blockIdx.x & 7u, pos = blockIdx.x >> 3;
    // r's of XCD x below m
    auto below = [&](unsigned m) -> unsigned { return 2u * (m >> 4) + ((m & 15u) > x ? 1u : 0u) + ((m & 15u) > 15u - x ? 1u : 0u); };
    // without a mask every tile of a sequence sees all of K: no pair of cheap first tiles to merge
    const bool pairs = p.mask_type == HSTU_MASK_TRIL;
    auto entries = [&](int cc) -> unsigned { return (unsigned)min(cc, ntiles_attr) - ((pairs && cc <= ntiles_attr && cc >= 5) ? 1u : 0u); };
    const unsigned seqs_incl = wave_inclusive_sum(n), seqs_before = seqs_incl - n;
    const unsigned g0 = below(seqs_before * (unsigned)H), g1 = below(seqs_incl * (unsigned)H);
    const unsigned span = n ? (g1 - g0) * entries(c) : 0u;
    const unsigned ent_incl = wave_inclusive_sum(span), ent_before = ent_incl - span;
    const unsigned long long hit = __ballot(pos >= ent_before && pos < ent_incl);
    if (hit == 0) {
        rec[0] = WORK_ITEM_EMPTY;
#pragma unroll
        for (int i = 1; i < WORK_RECORD_WORDS; i++) rec[i] = 0u;
        return;
    }
    const int fk = __builtin_ctzll(hit);
    const int found_cls = cmax - fk;
    const unsigned found_first = (unsigned)__builtin_amdgcn_readlane((int)seqs_before, fk);
    const unsigned d = pos - (unsigned)__builtin_amdgcn_readlane((int)ent_before, fk);
    const unsigned found_e = entries(found_cls);
    // Inside a class the entries of four consecutive groups are interleaved (tile by tile: entry 4 i + j of such a block is
    // entry i of its group j); the last one to three groups of the class follow one after the other.  The hardware hands
    // the workgroups of an XCD to its four shader engines in turn and in order, and waits when the engine whose turn it
    // is has no room: with four streams of equal cost the engines fill and drain together instead of holding each
    // other's free slots up.
    const unsigned g_first = (unsigned)__builtin_amdgcn_readlane((int)g0, fk), g_count = (unsigned)__builtin_amdgcn_readlane((int)g1, fk) - g_first;
    // (FOUR_STREAMS off: group by group, for the variants that lean on the L2 for the rows and bias planes a group shares)
    const unsigned in_blocks = FOUR_STREAMS ? (g_count >> 2) * 4u * found_e : 0u;     // entries of the whole blocks
    unsigned found_g, found_i;
    if (d < in_blocks) {
        const unsigned blk = small_div(d, 4u * found_e), rem = d - blk * 4u * found_e;
        found_i = rem >> 2;
        found_g = g_first + 4u * blk + (rem & 3u);
    } else {
        const unsigned td = d - in_blocks, gj = small_div(td, found_e);
        found_i = td - gj * found_e;
        found_g = g_first + (FOUR_STREAMS ? (g_count & ~3u) : 0u) + gj;
    }
    // group found_g of this XCD's list: r = 16 (g / 2) + (x or 15 - x); its sequence is the (rank - found_first)-th of its class
    const unsigned r = 16u * (found_g >> 1) + ((found_g & 1u) ? 15u - x : x);
    const unsigned rank = small_div(r, (unsigned)H), h = r - rank * (unsigned)H;
    // the nth sequence of the class in batch order: sequences 0..63 first, then 64..127
    const unsigned long long m0 = __ballot(cls[0] == found_cls), m1 = __ballot(cls[1] == found_cls);
    unsigned nth = rank - found_first;
    const unsigned in0 = (unsigned)__builtin_popcountll(m0);
    const bool second = nth >= in0;
    const unsigned long long m = second ? m1 : m0;
    if (second) nth -= in0;
    const unsigned before_me = __builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, 0u));
    const unsigned long long pick = __ballot(((m >> lane) & 1ull) && before_me == nth);
    const int fl = pick ? __builtin_ctzll(pick) : 0;
    const unsigned q0 = (unsigned)__builtin_amdgcn_readlane((int)(second ? o0[1] : o0[0]), fl);
    const unsigned lq = (unsigned)__builtin_amdgcn_readlane(second ? len[1] : len[0], fl);
    const unsigned tg = (unsigned)__builtin_amdgcn_readlane(second ? tgt[1] : tgt[0], fl);
    unsigned k0 = q0, lk = lq;
    if constexpr (OWN_K) {
        k0 = (unsigned)__builtin_amdgcn_readlane((int)(second ? ks[1] : ks[0]), fl);
        lk = (unsigned)__builtin_amdgcn_readlane((int)(second ? kl[1] : kl[0]), fl);
    }
    const unsigned fb = (unsigned)fl + (second ? 64u : 0u);
    const bool sw = found_cls > ntiles_attr, pr = pairs && !sw && found_cls >= 5;
    const bool both = pr && found_i == found_e - 1;
    const unsigned tile = both ? 0u : (found_e - 1 - found_i) + (pr ? 1u : 0u), part = both ? 1u : 0u;
    rec[0] = fb | h << 12 | tile << 16 | ((found_i == 0 && sw) ? 1u << 24 : 0u) | part << 25 | 1u << 28;
    rec[1] = q0; rec[2] = lq; rec[3] = k0; rec[4] = lk; rec[5] = 0u; rec[6] = tg; rec[7] = 0u;
}

}  // namespace hstu
