// Shared pieces of the selection kernels: packed codes, chunk loaders, per-sequence budgets, wave scan.
#pragma once

#include "ha_common.h"

namespace ha_sel {

constexpr int kSelThreads = 256;
constexpr int kSelWaves = kSelThreads / HA_WAVE;
constexpr int kBlock = 1024;      // codes per workgroup per block: 4 waves x 64 lanes x 4 codes
constexpr int kMaxBlocks = 4;     // blocks per chunk held in registers
constexpr int kMaxChunks = 1024;  // per row: sequences up to 4 Mi tokens, so an index fits the low 24 bits of a candidate entry

struct SelectPlan {
    int blocks;  // 1024-code blocks per chunk, 1..kMaxBlocks
    int nchunk;
};

inline SelectPlan select_plan(int B, int Hc, int max_seq_len) {
    SelectPlan p;
    p.blocks = kMaxBlocks;
    // prefer many small workgroups while the grid is short of ~8 workgroups per CU
    while (p.blocks > 1 && (int64_t)B * Hc * ((max_seq_len + p.blocks * kBlock - 1) / (p.blocks * kBlock)) < 2048) p.blocks /= 2;
    p.nchunk = (max_seq_len + p.blocks * kBlock - 1) / (p.blocks * kBlock);
    return p;
}

template <int W> struct Code;
template <> struct Code<1> {
    uint32_t w0;
    __device__ __forceinline__ int dist(const Code &q) const { return __popc(w0 ^ q.w0); }
};
template <> struct Code<2> {
    uint32_t w0, w1;
    __device__ __forceinline__ int dist(const Code &q) const { return __popc(w0 ^ q.w0) + __popc(w1 ^ q.w1); }
};

template <int W> __device__ __forceinline__ Code<W> load_code(const uint32_t *p, int64_t j) {
    if constexpr (W == 1) return Code<1>{p[j]};
    else {
        const uint2 v = reinterpret_cast<const uint2 *>(p)[j];
        return Code<2>{v.x, v.y};
    }
}

// Four consecutive codes j0..j0+3 (j0 % 4 == 0).  `vec`: the row is 16-byte aligned and padded to whole
// groups of four, so one (W=1) or two (W=2) 128-bit loads are safe; otherwise element loads, only for
// indices inside [beg, end).  Codes outside [beg, end) are returned as zero and must be masked by the caller.
template <int W>
__device__ __forceinline__ void load_code4(const uint32_t *kc, int j0, int beg, int end, bool vec, Code<W> (&k)[4]) {
    // plain loads on purpose: the codes are scanned again by a later pass or launch, and with the non-temporal hint the
    // step measured 4 - 8 us slower
    if (vec) {
        if constexpr (W == 1) {
            const uint4 v = reinterpret_cast<const uint4 *>(kc)[j0 >> 2];
            k[0].w0 = v.x; k[1].w0 = v.y; k[2].w0 = v.z; k[3].w0 = v.w;
        } else {
            const uint4 a = reinterpret_cast<const uint4 *>(kc)[(j0 >> 1)], b = reinterpret_cast<const uint4 *>(kc)[(j0 >> 1) + 1];
            k[0].w0 = a.x; k[0].w1 = a.y; k[1].w0 = a.z; k[1].w1 = a.w;
            k[2].w0 = b.x; k[2].w1 = b.y; k[3].w0 = b.z; k[3].w1 = b.w;
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int j = j0 + e;
            if (j >= beg && j < end) k[e] = load_code<W>(kc, j);
            else if constexpr (W == 1) k[e] = Code<1>{0u};
            else k[e] = Code<2>{0u, 0u};
        }
    }
}

template <int W> __device__ __forceinline__ Code<W> load_qcode(const uint32_t *qcodes, int64_t row) {
    if constexpr (W == 1) return Code<1>{qcodes[row]};
    else return Code<2>{qcodes[row * 2], qcodes[row * 2 + 1]};
}

__device__ __forceinline__ int lanes_below(uint64_t mask) {  // set bits of mask in lanes below this one
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// candidate range [lo, hi) and heavy budget of one sequence
struct RowBudget {
    int S, lo, hi, kk;
};
__device__ __forceinline__ RowBudget row_budget(int S, int init, int recent, double heavy_budget) {
    RowBudget r;
    r.S = S;
    r.lo = init < S ? init : S;
    r.hi = (S - recent > r.lo) ? S - recent : r.lo;
    int heavy = heavy_budget > 1.0 ? (int)heavy_budget : (int)((double)S * heavy_budget);
    if (heavy < 0) heavy = 0;
    const int ncand = r.hi - r.lo;
    r.kk = heavy < ncand ? heavy : ncand;
    return r;
}

// The chunk of a workgroup, fetched up front.  k[blk][e] is code j = j0(blk) + e.
template <int W> struct ChunkRegs {
    Code<W> k[kMaxBlocks][4];
    int j0[kMaxBlocks];
};
template <int W>
__device__ __forceinline__ void load_chunk(const uint32_t *kc, int chunk_start, int blocks, int beg, int end, bool vec, int wave, int lane,
                                           ChunkRegs<W> &cr) {
#pragma unroll
    for (int blk = 0; blk < kMaxBlocks; ++blk) {
        cr.j0[blk] = chunk_start + blk * kBlock + wave * (HA_WAVE * 4) + lane * 4;
        const bool live = blk < blocks && cr.j0[blk] + 4 > beg && cr.j0[blk] < end;
        if (live) load_code4<W>(kc, cr.j0[blk], beg, end, vec, cr.k[blk]);
        else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if constexpr (W == 1) cr.k[blk][e] = Code<1>{0u};
                else cr.k[blk][e] = Code<2>{0u, 0u};
            }
        }
    }
}

// wave64 inclusive scan of a u32 (two packed 16-bit counters ride along for free): Hillis-Steele inside
// each 16-lane DPP row, then the row totals are carried across rows with row_bcast15 / row_bcast31.
#define HA_DPP_ADD(v, ctrl, row_mask) \
    (v) += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(v), (ctrl), (row_mask), 0xF, true)
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v) {
    HA_DPP_ADD(v, 0x111, 0xF);  // row_shr:1
    HA_DPP_ADD(v, 0x112, 0xF);  // row_shr:2
    HA_DPP_ADD(v, 0x114, 0xF);  // row_shr:4
    HA_DPP_ADD(v, 0x118, 0xF);  // row_shr:8
    HA_DPP_ADD(v, 0x142, 0xA);  // row_bcast:15 into rows 1 and 3
    HA_DPP_ADD(v, 0x143, 0xC);  // row_bcast:31 into rows 2 and 3
    return v;
}
#undef HA_DPP_ADD


#ifdef __HIPCC__
// T (k-th smallest distance), r (how many of the tie bucket are taken) and the number of heavy tokens from a
// histogram `tot` whose levels above `top` are unknown.  false if the known levels do not hold k tokens.
__device__ __forceinline__ bool solve_threshold(const uint32_t *tot, int top, int NL, int kk, int mode, int depth, int &T, int &r,
                                                int &nheavy) {
    T = 0;
    r = 0;
    nheavy = 0;
    if (kk <= 0) return true;
    int cum = 0, l = 0, dmin = -1;
    for (; l <= top && l < NL; ++l) {
        const int t = (int)tot[l];
        if (dmin < 0 && t > 0) dmin = l;
        if (cum + t >= kk) break;
        cum += t;
    }
    if (l > top || l >= NL) return false;
    if (mode == HA_SELECT_SIMPLE) {
        T = l;
        r = kk - cum;
        nheavy = kk;
    } else {
        const int th = min(dmin + depth, l);
        T = th + 1;
        r = 0;
        for (int i = 0; i <= th; ++i) nheavy += (int)tot[i];
    }
    return true;
}

#endif

// ---- host side -----------------------------------------------------------------------------------
// rows start 16-byte aligned and hold whole groups of four codes: 128-bit loads never leave a row
inline bool rows_vectorisable(const uint32_t *kcodes, int64_t kc_sb, int64_t kc_sh, int W) {
    return ha_aligned(kcodes, 16) && kc_sb % (4 * W) == 0 && kc_sh % (4 * W) == 0;
}


// workspace of the histogram selection: per-chunk histograms, row meta {T, r, n_heavy, size of the tie bucket}, per-chunk prefixes
// {#d < T before the chunk, #d == T before the chunk}
struct SelectWorkspace {
    uint32_t *hist;
    int32_t *meta, *chunk_pre;
    size_t bytes;
};
inline SelectWorkspace carve_select_ws(void *base, int64_t rows, int nchunk, int W) {
    SelectWorkspace w;
    size_t off = 0;
    auto take = [&](size_t n) {
        size_t o = off;
        off += (n + 255) / 256 * 256;
        return o;
    };
    const size_t o_hist = take((size_t)rows * nchunk * (32 * W + 1) * 4);
    const size_t o_meta = take((size_t)rows * 4 * 4);
    const size_t o_pre = take((size_t)rows * nchunk * 2 * 4);
    w.hist = (uint32_t *)((char *)base + o_hist);
    w.meta = (int32_t *)((char *)base + o_meta);
    w.chunk_pre = (int32_t *)((char *)base + o_pre);
    w.bytes = off;
    return w;
}


// workspace of the sampled-threshold selection: T_hi per row, candidate count per (row, chunk), candidate segments
struct SampledWorkspace {
    int32_t *thi, *cand_cnt, *cand;
    int cap;  // entries per (row, chunk) segment: half a chunk
    size_t bytes;
};
inline SampledWorkspace carve_sampled_ws(void *base, int64_t rows, int nchunk, int blocks) {
    SampledWorkspace w;
    size_t off = 0;
    auto take = [&](size_t n) {
        size_t o = off;
        off += (n + 255) / 256 * 256;
        return o;
    };
    w.cap = blocks * kBlock / 2;
    const size_t o_thi = take((size_t)rows * 4);
    const size_t o_cnt = take((size_t)rows * nchunk * 4);
    const size_t o_cand = take((size_t)rows * nchunk * w.cap * 4);
    w.thi = (int32_t *)((char *)base + o_thi);
    w.cand_cnt = (int32_t *)((char *)base + o_cnt);
    w.cand = (int32_t *)((char *)base + o_cand);
    w.bytes = off;
    return w;
}
size_t sampled_workspace_bytes(int64_t rows, int nchunk, int blocks);
int launch_select_sampled(const uint32_t *kcodes, int64_t kc_sb, int64_t kc_sh, const uint32_t *qcodes, int B, int H, int Hc, int W,
                          int max_seq_len, const int32_t *seq_lens, int init, int recent, double heavy_budget, int mode, int depth,
                          int force_exact, int32_t *out_idx, int64_t idx_cap, int32_t *out_counts, void *workspace, hipStream_t s);

}  // namespace ha_sel
