// Decode attention kernels (gfx950, wave64): gather-only sparse attend, dense flash-decode, split merge.
//
// Row layout: one K or V row is 128 elements; a 16-lane quarter-wave ("row group") owns one row at
// a time, lane `sub` holding elements [8*sub, 8*sub+8) fetched with 128-bit loads, so one wave
// load instruction brings in four whole rows.  A workgroup of 256 threads runs 16 such row streams,
// each keeping its own online softmax (m, l, acc[8]) in registers in the log2 domain; the streams
// are merged through LDS at the end, and workgroups of one row's split are merged by
// merge_splits_kernel with the usual log-sum-exp algebra (launched only when a row is split at all).
// The sparse kernel is software-pipelined: the K/V rows of step i+1 and the indices of step i+2 are in
// flight while step i is reduced, so a wave always has 8 x 1 KiB of row data outstanding.
#include <stdlib.h>

#include "ha_select_common.h"

namespace {

constexpr int kAttThreads = 256;
constexpr int kStreams = kAttThreads / 16;  // 16 row streams per workgroup
constexpr int kUnroll = 4;                  // rows in flight per stream (K and V: 8 x 128-bit loads per lane)
constexpr float kLog2e = 1.4426950408889634f;

// sum over the 16 lanes of a DPP row; every lane ends with the total
__device__ __forceinline__ float row16_sum(float x) {
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x141, 0xF, 0xF, true));  // row_half_mirror
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x140, 0xF, 0xF, true));  // row_mirror
    return x;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

constexpr int kMinSplitRows = 64;

// Tuning overrides for experiments, compiled in only with -DHASHATTN_TUNING_ENV (read once): HASHATTN_SPARSE_SPLIT_ROWS =
// rows of the index list per workgroup (0 = whole list, no split merge), HASHATTN_SPARSE_THREADS = 256 or 512.  The
// library as shipped reads no environment variable.
inline int env_int(const char *name, int dflt) {
#ifdef HASHATTN_TUNING_ENV
    const char *e = getenv(name);
    return (e && *e) ? atoi(e) : dflt;
#else
    (void)name;
    return dflt;
#endif
}

struct SparsePlan {
    int threads;     // workgroup size: 256 (16 row streams) or 512 (32)
    int split_rows;  // selected rows per workgroup, multiple of 64
    int nsplit_max;
};
inline SparsePlan sparse_plan(int B, int H, int64_t idx_cap) {
    static const int env_split = env_int("HASHATTN_SPARSE_SPLIT_ROWS", -1);
    static const int env_threads = env_int("HASHATTN_SPARSE_THREADS", -1);
    SparsePlan p;
    const int64_t rows = (int64_t)B * H;
    p.threads = env_threads == 256 || env_threads == 512 ? env_threads : 512;
    // enough workgroups to keep 256 CUs busy (two 512-thread workgroups per CU), but no finer: when the
    // rows alone supply them a row is not split and the merge launch disappears
    int64_t want_splits = (512 + rows - 1) / rows;
    int64_t split = (idx_cap + want_splits - 1) / want_splits;
    if (env_split == 0) split = idx_cap;
    else if (env_split > 0) split = env_split;
    split = (split + kMinSplitRows - 1) / kMinSplitRows * kMinSplitRows;
    if (split < kMinSplitRows) split = kMinSplitRows;
    p.split_rows = (int)split;
    p.nsplit_max = (int)((idx_cap + split - 1) / split);
    if (p.nsplit_max < 1) p.nsplit_max = 1;
    return p;
}

struct DensePlan {
    int chunk;  // tokens per workgroup, multiple of 256
    int nsplit_max;
};
inline DensePlan dense_plan(int B, int Hkv, int max_seq_len) {
    DensePlan p;
    int want = (2048 + B * Hkv - 1) / (B * Hkv);
    if (want < 1) want = 1;
    int64_t chunk = ((int64_t)max_seq_len + want - 1) / want;
    chunk = (chunk + 255) / 256 * 256;
    if (chunk < 256) chunk = 256;
    p.chunk = (int)chunk;
    p.nsplit_max = (max_seq_len + p.chunk - 1) / p.chunk;
    if (p.nsplit_max < 1) p.nsplit_max = 1;
    return p;
}

// Merge the NS streams of a workgroup.  s_m/s_l [NS], s_acc [NS][128].  Thread e < 128 returns
// the merged (m, l, acc_e).
template <int NS>
__device__ __forceinline__ void merge_streams(const float *s_m, const float *s_l, const float *s_acc, int e, float &M, float &L,
                                              float &A) {
    M = -INFINITY;
#pragma unroll
    for (int s = 0; s < NS; ++s) M = fmaxf(M, s_m[s]);
    L = 0.f;
    A = 0.f;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const float w = (s_m[s] == -INFINITY) ? 0.f : fast_exp2(s_m[s] - M);
        L += w * s_l[s];
        A += w * s_acc[s * HA_HEAD_DIM + e];
    }
}

// ------------------------------------------------------------------------------------------------
// Selection fused into the attend kernel (FW = code words, 0 = the list comes from memory).  After
// ha_select_prepare the workspace holds, per row, the threshold T, the number r of ties taken and n_heavy, and per
// (row, chunk) how many tokens with d < T / d == T precede the chunk.  That is all a workgroup needs to rebuild its
// part of the ordered index list in LDS straight from the codes - the list never goes through memory, and the
// compaction launch disappears.  A workgroup owns `cps` consecutive chunks (all of them when rows are not split);
// the first also takes the sink window, the last the recent window.
constexpr int kFusedListCap = 8192;  // entries of the LDS list (32 KiB)
struct FusedSel {
    const uint32_t *kcodes;
    int64_t kc_sb, kc_sh;
    const uint32_t *qcodes;
    const int32_t *meta, *chunk_pre;
    int nchunk, chunk, cps, gq, init, recent, vec;
    // when `hist` is set the workspace holds only the per-chunk histograms (ha_select_histogram): the workgroup derives
    // its row's threshold and chunk prefixes itself (at most kFusedLocalChunks chunks) and writes the row's count
    const uint32_t *hist;
    double heavy_budget;
    int32_t *out_counts;
};
// Additive attention mask of a list-fed launch: values [B, len] fp32 (row stride stride_b), indexed by the token position
// of a list entry, or by the entry's place in the list (by_slot).
struct AttnMask {
    const float *values;
    int64_t stride_b;
    int len, by_slot;
    // fused launch only (kernel parameter LP): tokens [0, masked_prefix[b]) of sequence b score -inf - the additive mask of
    // a left-padded batch in the one form it takes there
    const int32_t *masked_prefix;
};
// Token -> slot map of a paged cache (the `Req_to_tokens` table of efficiency/kernels/flash_fwd_sparse.py:396-470): the K/V
// row of token j of sequence b is row slots[b * stride_b + j] of the cache.  slots == nullptr: the identity.
struct SlotMap {
    const int32_t *slots;
    int64_t stride_b;
    int max_slot;  // n_slots - 1: entries of the fused launch's LDS list are clamped to it
};
constexpr int kFusedLocalChunks = 64;
// chunk prefixes a workgroup keeps in LDS: those of the whole row up to this many chunks, of its own piece beyond (the host
// cuts longer rows into pieces of at most this many chunks)
constexpr int kFusedMaxChunks = 256;
constexpr int kFusedSortBatch = 128;  // ragged batches up to this size are planned in the kernel (order and piece size)
// a batch of equal lengths is cut into this many workgroups (one per CU): measured against 512 at 64K tokens, B = 6: 76.6
// against 82.3 us, B = 8: 76.7 against 81.2, B = 12: 107.1 against 125.5; B = 1 at 32K: 39.2 against 40.9; B = 4 at 128K: 84.1
// against 87.0 - the pieces are setup-bound, so fewer and larger ones win (measured again with pieces of equal work, 256 / 384 /
// 512 pieces: B = 1 at 32K 22.1 / 28.0 / 27.4 us, B = 4 at 128K 60.2 / 69.3 / 63.4, B = 8 at 64K 58.5 / 66.2 / 66.5)
constexpr int kFusedUniformPieces = 256;
constexpr int kFusedResident = 512;   // 512-thread workgroups resident at once: two on each of 256 CUs
constexpr int kChunkScanRows = 48;    // a chunk's scan takes about as long as gathering this many rows (pieces of equal work)

// NSLAB slabs of 256 codes of one chunk, four consecutive codes per lane and slab, for rows that do not take 128-bit loads
// (misaligned, or strides that are no multiples of four codes): element loads inside [beg, end), zeros outside.
template <int W, int NSLAB>
__device__ __forceinline__ void load_slabs_by_element(const uint32_t *kc, int j_first, int beg, int end, int lane,
                                                      ha_sel::Code<W> (&k)[NSLAB][4]) {
#pragma unroll
    for (int s = 0; s < NSLAB; ++s) ha_sel::load_code4<W>(kc, j_first + s * (HA_WAVE * 4) + lane * 4, beg, end, false, k[s]);
}

// A fused workgroup alternates scan rounds (fused_round: its waves place the selected tokens of the next few chunks in
// the LDS list) with as many steps of the attention loop as the list filled so far allows.  (Dedicated producer
// waves feeding the loop through LDS counters were tried: the loop's bandwidth follows the number of gathering
// waves, and giving two of eight to the scan cost more than the scan itself.  Building the whole list first costs
// the scan's ~15 us up front.)
struct FusedRow {
    // {#d < T, #d == T} before each chunk of the row, in LDS: worked out by the workgroup or copied from the workspace.  (Read
    // from either place through one pointer they would be flat loads, and a flat load in a scan round waits for every
    // outstanding request of the wave, rows on their way included.)
    const int32_t *pre;
    int pre_first;  // the chunk pre[0], pre[1] belong to (0 unless only the piece's prefixes were copied)
    __device__ __forceinline__ int pre_lt(int c) const { return pre[(c - pre_first) * 2]; }
    __device__ __forceinline__ int pre_eq(int c) const { return pre[(c - pre_first) * 2 + 1]; }
    int lo, hi, T, r, nheavy, neq, c0, nc, n;
    int nwin;   // window entries at the head of this workgroup's list (sink if it has the first chunk, recent if the last)
    int hbase;  // list position of a heavy token = hbase + (#d < T before it) + min(#d == T before it, r)
    int cstar;  // the chunk of this workgroup that holds the r-th tie (ties before it are taken, after it not), or -1
};

// The row's chunk histograms (ha_select_histogram's), requested when the kernel starts and parked in registers: by the time
// the threshold search wants them in LDS their round trip is over.
template <int W, int NTT> struct HistTileRegs {
    static constexpr int NL = 32 * W + 1;
    static constexpr int N = (kFusedLocalChunks * NL + NTT - 1) / NTT;
    uint32_t v[N];
    __device__ __forceinline__ void request(const FusedSel &f, int64_t row) {
        const uint32_t *hp = f.hist + row * f.nchunk * NL;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int at = (int)threadIdx.x + i * NTT;
            v[i] = 0;
            if (at < f.nchunk * NL) v[i] = hp[at];
        }
    }
    // the tile into LDS, and every counter added to its level's total (s_tot: NL words, zero)
    __device__ __forceinline__ void to_lds(const FusedSel &f, uint32_t *s_h, uint32_t *s_tot) const {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int at = (int)threadIdx.x + i * NTT;
            if (at < f.nchunk * NL) {
                s_h[at] = v[i];
                if (v[i]) atomicAdd(&s_tot[at % NL], v[i]);
            }
        }
    }
};

// Setup of a row whose thresholds are derived in the launch (the work of select_threshold_kernel for this row, plus what the
// workgroup needs of its own piece), two barriers: the histogram tile into LDS, every counter added to its level's total on
// the way (HistTileRegs::to_lds, by the caller); then ONE wave does the rest without leaving its registers - the threshold T and the tie remainder r (a level per lane: a wave scan
// of the totals, the first lane whose running total reaches the budget), the chunk prefixes {#d < T, #d == T} (a chunk per
// lane, two wave scans), the piece's chunk range by work (see fused_thresholds) and the chunk that holds the r-th tie (two
// ballots) - and leaves s_pre and s_meta = {T, r, n_heavy, #d == T, first chunk, end chunk, tie chunk}.  At most 64 chunks.
template <int W, int NTT>
__device__ __forceinline__ void local_thresholds(const FusedSel &f, int S, int sp, int row_pieces, int c0_even, int nc_even,
                                                 const uint32_t *s_h, int32_t *s_pre, int32_t *s_meta) {
    constexpr int NL = 32 * W + 1;
    const int tid = threadIdx.x;
    const uint32_t *s_tot = s_h + f.nchunk * NL;  // NL words behind the tile: the caller has stored the tile and added up the totals
    __syncthreads();
    if (tid < HA_WAVE) {
        const int lane = tid;
        const int kk = ha_sel::row_budget(S, f.init, f.recent, f.heavy_budget).kk;
        // ha_sel::solve_threshold, simple mode: T = the first level at which the running total reaches kk, r = what is still
        // missing in front of it; nothing (0, 0, 0) when the budget is empty
        const uint32_t mine = lane < NL ? s_tot[lane] : 0u;
        const uint32_t run = ha_sel::wave_inclusive_scan(mine);
        int T = 0, r = 0, nheavy = 0;
        if (kk > 0) {
            const unsigned long long reached = __ballot(lane < NL && (int)run >= kk);
            if (reached) {
                T = __ffsll((long long)reached) - 1;
                r = kk - __builtin_amdgcn_readlane((int)(run - mine), T);
                nheavy = kk;
            } else if (NL > HA_WAVE) {  // 64-bit codes: the one level beyond the lanes
                const int before = __builtin_amdgcn_readlane((int)run, HA_WAVE - 1);
                if (before + (int)s_tot[NL - 1] >= kk) {
                    T = NL - 1;
                    r = kk - before;
                    nheavy = kk;
                }
            }
        }
        const int neq = (int)s_tot[T];
        // chunk prefixes
        uint32_t lt = 0, eq = 0;
        if (lane < f.nchunk) {
            const uint32_t *mine_h = s_h + lane * NL;
            uint32_t a1 = 0, a2 = 0, a3 = 0;  // four sums: four reads on their way at a time, not one
            int l = 0;
            for (; l + 4 <= T; l += 4) lt += mine_h[l], a1 += mine_h[l + 1], a2 += mine_h[l + 2], a3 += mine_h[l + 3];
            for (; l < T; ++l) lt += mine_h[l];
            lt += a1 + a2 + a3;
            eq = mine_h[T];
        }
        const uint32_t ilt = ha_sel::wave_inclusive_scan(lt), ieq = ha_sel::wave_inclusive_scan(eq);
        const int pre_lt = (int)(ilt - lt), pre_eq = (int)(ieq - eq);
        if (lane < f.nchunk) {
            s_pre[lane * 2] = pre_lt;
            s_pre[lane * 2 + 1] = pre_eq;
        }
        // this piece's chunks: an even share of the row's work (fused_thresholds has the rule), or the even share of its chunks
        int c0 = c0_even, c1 = c0_even + nc_even;
        if (row_pieces > 1) {
            const int nc_row = min((S + f.chunk - 1) / f.chunk, f.nchunk);
            const int total = nheavy + kChunkScanRows * nc_row;
            const int wt = lane < nc_row ? pre_lt + min(pre_eq, r) + kChunkScanRows * lane : total;
            const int t0 = (int)((int64_t)sp * total / row_pieces), t1 = (int)((int64_t)(sp + 1) * total / row_pieces);
            const unsigned long long m0 = __ballot(wt >= t0), m1 = __ballot(wt >= t1);
            c0 = sp == 0 ? 0 : min(m0 ? __ffsll((long long)m0) - 1 : f.nchunk, f.nchunk);
            c1 = sp == row_pieces - 1 ? f.nchunk : min(m1 ? __ffsll((long long)m1) - 1 : f.nchunk, f.nchunk);
            c1 = max(c1, c0);
        }
        // the chunk of this piece in which the r-th tie lies: ties before it do not reach r, ties through it pass r
        const unsigned long long tie = __ballot(lane >= c0 && lane < c1 && lane < f.nchunk && pre_eq < r && r < (int)ieq);
        if (lane == 0) {
            s_meta[0] = T;
            s_meta[1] = r;
            s_meta[2] = nheavy;
            s_meta[3] = neq;
            s_meta[4] = c0;
            s_meta[5] = c1;
            s_meta[6] = tie ? __ffsll((long long)tie) - 1 : -1;
        }
    }
    __syncthreads();
}

// Setup, first half: what is known without any threshold - the row's window geometry, this workgroup's chunks, and the
// window entries at the head of its list (the loop can be primed on them while the second half runs).
template <int NTT>
__device__ __forceinline__ void fused_windows(const FusedSel &f, int S, int sp, int cps, int row_pieces, int32_t *s_list, FusedRow &fr,
                                              const int32_t *slot_row /* this sequence's token -> slot map, or nullptr */) {
    const int tid = threadIdx.x;
    fr.lo = min(f.init, S);
    fr.hi = max(S - f.recent, fr.lo);
    // workgroup sp of the row owns chunks [sp * cps, (sp + 1) * cps); the row has row_pieces such workgroups
    fr.c0 = min(sp * cps, f.nchunk);
    const int c1 = min(fr.c0 + cps, f.nchunk);
    fr.nc = c1 - fr.c0;
    // sink: first workgroup; recent: last workgroup of the row
    const int n_sink = sp == 0 ? fr.lo : 0, n_recent = sp == row_pieces - 1 ? S - fr.hi : 0;
    fr.nwin = min(n_sink + n_recent, kFusedListCap);
    // with a slot map the list holds slots: the window entries are translated here, the heavy ones by fused_round
    for (int i = tid; i < n_sink && i < fr.nwin; i += NTT) s_list[i] = slot_row ? slot_row[i] : i;
    for (int i = tid; i < n_recent; i += NTT)
        if (n_sink + i < fr.nwin) s_list[n_sink + i] = slot_row ? slot_row[fr.hi + i] : fr.hi + i;
    __syncthreads();
}

// Setup, second half: threshold, prefixes, list length, the chunk of the r-th tie.
// The pieces of a split row take equal shares of the row's WORK, not of its chunks: with ties broken by the lowest index
// the taken part of the tie bucket lies at the front of the sequence, so pieces of equal token ranges gather very
// different numbers of rows (B = 4 at 128K tokens: 2750 against 1350 rows, 56 against 43 us).  A piece's work is counted
// as its selected rows plus kChunkScanRows per chunk it scans (a chunk's scan takes about as long as gathering that many
// rows); piece i starts at the first chunk before which at least i / pieces of the row's work lies.  Every workgroup of
// the row derives the same boundaries from the same prefixes, whichever launch derived the thresholds.
template <int W, int NTT>
__device__ __forceinline__ void fused_thresholds(const FusedSel &f, int64_t row, int S, int sp, int row_pieces, int *s_cstar,
                                                 const uint32_t *s_h, int32_t *s_pre, int32_t *s_meta, FusedRow &fr) {
    const int tid = threadIdx.x;
    fr.pre = s_pre;
    fr.pre_first = 0;
    // heavy tokens of the row before chunk c
    auto rank = [&](int c) { return c >= f.nchunk ? fr.nheavy : fr.pre_lt(c) + min(fr.pre_eq(c), fr.r); };
    if (f.hist) {
        local_thresholds<W, NTT>(f, S, sp, row_pieces, fr.c0, fr.nc, s_h, s_pre, s_meta);
        fr.T = s_meta[0];
        fr.r = s_meta[1];
        fr.nheavy = s_meta[2];
        fr.neq = s_meta[3];
        fr.c0 = s_meta[4];
        fr.nc = s_meta[5] - fr.c0;
        fr.cstar = s_meta[6];
        if (sp == 0 && tid == 0 && f.out_counts) f.out_counts[row] = fr.lo + fr.nheavy + (S - fr.hi);
    } else {
        fr.T = f.meta[row * 4 + 0];
        fr.r = f.meta[row * 4 + 1];
        fr.nheavy = f.meta[row * 4 + 2];
        fr.neq = f.meta[row * 4 + 3];
        const int32_t *gp = f.chunk_pre + row * f.nchunk * 2;
        if (f.nchunk <= kFusedMaxChunks) {
            for (int i = tid; i < 2 * f.nchunk; i += NTT) s_pre[i] = gp[i];
        } else {  // a long row: this piece's chunks and the one behind them (no more than kFusedMaxChunks + 1: the host sees to it)
            fr.pre_first = fr.c0;
            const int n = min(fr.nc + 1, f.nchunk - fr.c0);
            for (int i = tid; i < 2 * n; i += NTT) s_pre[i] = gp[2 * fr.c0 + i];
        }
        if (tid == 0) *s_cstar = -1;
        __syncthreads();
        if (row_pieces > 1 && f.nchunk <= HA_WAVE) {
            if (tid < HA_WAVE) {  // nchunk <= 64: a chunk per lane
                const int c = tid;
                const int nc_row = min((S + f.chunk - 1) / f.chunk, f.nchunk);  // chunks that hold tokens of this row
                const int total = fr.nheavy + kChunkScanRows * nc_row;
                const int wt = c < nc_row ? fr.pre_lt(c) + min(fr.pre_eq(c), fr.r) + kChunkScanRows * c : total;
                const int t0 = (int)((int64_t)sp * total / row_pieces), t1 = (int)((int64_t)(sp + 1) * total / row_pieces);
                const unsigned long long m0 = __ballot(wt >= t0), m1 = __ballot(wt >= t1);
                if (tid == 0) {
                    s_meta[4] = sp == 0 ? 0 : min(m0 ? __ffsll((long long)m0) - 1 : f.nchunk, f.nchunk);
                    s_meta[5] = sp == row_pieces - 1 ? f.nchunk : min(m1 ? __ffsll((long long)m1) - 1 : f.nchunk, f.nchunk);
                }
            }
            __syncthreads();
            fr.c0 = s_meta[4];
            fr.nc = max(s_meta[5] - fr.c0, 0);
        }
        for (int i = tid; i < fr.nc; i += NTT) {
            const int c = fr.c0 + i;
            const int eq0 = fr.pre_eq(c), eq1 = c + 1 < f.nchunk ? fr.pre_eq(c + 1) : fr.neq;
            if (eq0 < fr.r && fr.r < eq1) *s_cstar = c;  // at most one chunk of the row
        }
        __syncthreads();
        fr.cstar = *s_cstar;
    }
    const int c1 = fr.c0 + fr.nc;
    fr.hbase = fr.nwin - rank(fr.c0);
    fr.n = min(fr.nwin + max(rank(c1) - rank(fr.c0), 0), kFusedListCap);
}

// Scan rounds work on staged codes: the codes of a wave's group travel from memory straight into a 4 KiB region of LDS that
// belongs to the wave (one 16-byte request per lane and instruction, lane l's bytes at l * 16 behind the address in M0), a
// round ahead, so they occupy no registers while the gather loop runs between the rounds and nobody waits for them when the
// next round starts.  (Requested inside the round that ranks them, every round waits a memory round trip with nothing else of
// the wave in flight; held in registers across the loop they cost 16 - 32 of its 128.)  The requests are inline assembly on
// purpose: the compiler does not see them.  Through the builtin it waits for every outstanding request in front of each LDS
// access it cannot tell from the staging space, and before each barrier.  Its own `s_waitcnt vmcnt(n)` stay safe, because
// requests return in order: unseen requests among the n youngest only make a wait cover more than it had to, which is why
// the codes are requested in front of a step's rows, not behind them.  The wave's own wait for its staged codes is written
// by hand (staged_codes_arrived): once at least eight later requests have been issued - one gather step or the loop's
// priming - "at most eight outstanding" means the codes are in LDS.
constexpr int kStageWaveWords = 1024;  // staging region of one wave: 1024 32-bit codes or 512 64-bit codes
__device__ __forceinline__ void request_16_bytes_to_lds(const uint32_t *src, const uint32_t *dst /* uniform over the wave */) {
    const uint32_t lds_byte_address = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)dst);
    uint32_t saved_m0;  // M0 is the compiler's: handed back as it was
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0)
                 : "v"(src), "s"(lds_byte_address)
                 : "memory");
}
// One 4-byte request per active lane: lane l's word lands at dst + l (dst uniform over the wave); inactive lanes write nothing.
__device__ __forceinline__ void request_4_bytes_to_lds(const int32_t *src, const int32_t *dst /* uniform over the wave */) {
    const uint32_t lds_byte_address = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)dst);
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %1, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0)
                 : "v"(src), "s"(lds_byte_address)
                 : "memory");
}
// What vmcnt(8) relies on, both stated where they are established: (a) at least eight vector-memory LOADS of the wave are
// younger than the requests waited for (a gather step or the loop's priming: the static_assert in sparse_attend_kernel),
// and (b) no global STORE of the wave is outstanding between those requests and this wait (loads and stores retire out of
// order with respect to each other; the kernel stores only behind its loops).  -DHASHATTN_STAGE_WAIT_ALL builds the
// conservative form, which must give the same bits.
__device__ __forceinline__ void staged_codes_arrived(bool eight_younger_requests) {
#ifdef HASHATTN_STAGE_WAIT_ALL
    (void)eight_younger_requests;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#else
    if (eight_younger_requests) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
}
// Requests the codes of this wave's group of scan round `round` (geometry as in fused_round).  Lanes past the end of the
// candidate range ask for the chunk's first codes instead (the range is not empty, so they exist); fused_round masks them.
// Rows that do not take 128-bit loads are not staged: fused_staged_codes loads their codes itself.
template <int W, int GS, int NW>
__device__ __forceinline__ void fused_round_stage(const FusedSel &f, const FusedRow &fr, int b, int h, int round, int n_groups,
                                                  const uint32_t *s_stage) {
    static_assert(GS * HA_WAVE * 4 * W == kStageWaveWords, "a group fills the wave's staging region");
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // the wave's number in scalar registers
    constexpr int GC = GS * HA_WAVE * 4;
    const int gpc = f.chunk / GC, gpc_log2 = __builtin_ctz((unsigned)gpc);  // a power of two
    const int g = round * NW + wave;
    if (g >= n_groups || !f.vec) return;
    const int c = fr.c0 + (g >> gpc_log2), gi = g & (gpc - 1);
    const int cb = c * f.chunk, j_first = cb + gi * GC;
    const int beg = max(fr.lo, cb), end = min(fr.hi, cb + f.chunk);
    if (beg >= end) return;
    const uint32_t *kc = f.kcodes + b * f.kc_sb + (h / f.gq) * f.kc_sh;
    const uint32_t *dst = s_stage + wave * kStageWaveWords;
#pragma unroll
    for (int s = 0; s < GS; ++s) {
        const int j0 = j_first + s * (HA_WAVE * 4) + lane * 4;
        const int64_t j = j0 < end ? j0 : cb;
        if constexpr (W == 1) {
            request_16_bytes_to_lds(kc + j, dst + s * 256);
        } else {
            request_16_bytes_to_lds(kc + j * 2, dst + s * 512);
            request_16_bytes_to_lds(kc + j * 2 + 4, dst + s * 512 + 256);
        }
    }
}
// The codes fused_round_stage requested for this wave, from its staging region into registers.
template <int W, int GS>
__device__ __forceinline__ void fused_staged_codes(const uint32_t *s_stage, bool eight_younger_requests, ha_sel::Code<W> (&k)[GS][4]) {
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // the wave's number in scalar registers
    staged_codes_arrived(eight_younger_requests);
    const uint4 *sw = reinterpret_cast<const uint4 *>(s_stage + wave * kStageWaveWords);
#pragma unroll
    for (int s = 0; s < GS; ++s) {
        if constexpr (W == 1) {
            const uint4 v = sw[s * HA_WAVE + lane];
            k[s][0].w0 = v.x, k[s][1].w0 = v.y, k[s][2].w0 = v.z, k[s][3].w0 = v.w;
        } else {
            const uint4 a = sw[s * 2 * HA_WAVE + lane], b2 = sw[(s * 2 + 1) * HA_WAVE + lane];
            k[s][0].w0 = a.x, k[s][0].w1 = a.y, k[s][1].w0 = a.z, k[s][1].w1 = a.w;
            k[s][2].w0 = b2.x, k[s][2].w1 = b2.y, k[s][3].w0 = b2.z, k[s][3].w1 = b2.w;
        }
    }
}

// One scan round of a fused workgroup: its NW waves take NW consecutive groups of GS slabs (a group is part of one
// chunk; a chunk's groups never straddle rounds), place the selected tokens of those groups in the list, and return
// how many leading list entries are in LDS afterwards.  Two workgroup barriers per round; called by all threads.
// The gather loop runs between rounds, so the scan's integer work sits in the shadow of the loop's memory waits
// instead of in front of it.  `q`: the row's query code; `s_stage`, `eight_younger_requests`: see fused_staged_codes.
template <int W, int GS, int NW>
__device__ __forceinline__ int fused_round(const FusedSel &f, const FusedRow &fr, int b, int h, const ha_sel::Code<W> &q, int round, int n_groups,
                                           uint32_t *s_cnt /* [NW] */, int *s_ready, int32_t *s_list, const uint32_t *s_stage,
                                           bool eight_younger_requests, const int32_t *slot_row) {
    using namespace ha_sel;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // the wave's number in scalar registers
    constexpr int GC = GS * HA_WAVE * 4;  // codes per group
    const int gpc = f.chunk / GC, gpc_log2 = __builtin_ctz((unsigned)gpc);  // groups per chunk: a power of two that divides NW
    const int g = round * NW + wave;
    const bool active = g < n_groups;
    const int c = fr.c0 + (active ? g >> gpc_log2 : 0), gi = active ? g & (gpc - 1) : 0;
    const int cb = c * f.chunk, j_first = cb + gi * GC;
    const int beg = max(fr.lo, cb), end = min(fr.hi, cb + f.chunk);
    const bool whole = f.vec && beg == cb && end == cb + f.chunk;

    // Slot map: the entries the previous round placed are being translated in place (below); those requests are older than
    // the staged codes' and every wave waits for its own here, so behind this round's first barrier the previous round's
    // entries hold slots for everybody.
    if (slot_row) staged_codes_arrived(eight_younger_requests);
    uint32_t lt = 0, le = 0;  // bit 4 s + e: code (slab s, element e) of this lane has d < T / d <= T
    if (active && beg < end && fr.nheavy > 0) {
        Code<W> k[GS][4];
        if (f.vec) {
            fused_staged_codes<W, GS>(s_stage, eight_younger_requests, k);
        } else {
            const uint32_t *kc = f.kcodes + b * f.kc_sb + (h / f.gq) * f.kc_sh;
            load_slabs_by_element<W, GS>(kc, j_first, beg, end, lane, k);
        }
        if (c == fr.cstar) {
            const int neg_t = -fr.T;
#pragma unroll
            for (int s = GS - 1; s >= 0; --s)
#pragma unroll
                for (int e = 3; e >= 0; --e) {
                    const int key = k[s][e].dist(q) + neg_t;  // sign bit: d < T; of key - 1: d <= T
                    lt = __builtin_amdgcn_alignbit(lt, (uint32_t)key, 31);
                    le = __builtin_amdgcn_alignbit(le, (uint32_t)(key - 1), 31);
                }
        } else {
            // any other chunk takes all of its ties (those before it do not reach r) or none: one compare per code, against
            // T + 1 or T, and the chunk counts no ties of its own
            const int neg_t = -(fr.T + (fr.pre_eq(c) < fr.r ? 1 : 0));
#pragma unroll
            for (int s = GS - 1; s >= 0; --s)
#pragma unroll
                for (int e = 3; e >= 0; --e) lt = __builtin_amdgcn_alignbit(lt, (uint32_t)(k[s][e].dist(q) + neg_t), 31);
            le = lt;
        }
        if (!whole) {
            uint32_t valid = 0;
#pragma unroll
            for (int s = 0; s < GS; ++s) {
                const int j0 = j_first + s * (HA_WAVE * 4) + lane * 4;
#pragma unroll
                for (int e = 0; e < 4; ++e) valid |= (j0 + e >= beg && j0 + e < end) ? (1u << (4 * s + e)) : 0u;
            }
            lt &= valid;
            le &= valid;
        }
    }
    const uint32_t eq = le & ~lt;
    const uint32_t cnt = (uint32_t)__popc(lt) | ((uint32_t)__popc(eq) << 16);
    const uint32_t incl = wave_inclusive_scan(cnt);
    const uint32_t tot = (uint32_t)__builtin_amdgcn_readlane((int)incl, HA_WAVE - 1);
    if (lane == 0) s_cnt[wave] = tot;
    __syncthreads();

    // tokens of the row with d < T / d == T before this group: the chunk's prefix plus the chunk's earlier groups,
    // which are the gi waves just below this one
    int a = fr.pre_lt(c), t = fr.pre_eq(c);
    for (int w2 = wave - gi; w2 < wave; ++w2) {
        const uint32_t v = s_cnt[w2];
        a += (int)(v & 0xFFFFu);
        t += (int)(v >> 16);
    }
    const int r = fr.r;
    if (active && tot != 0) {
        const int j_lane = j_first + lane * 4;
        if (c != fr.cstar) {
            // ties of the chunk all taken (t < r here and through the chunk) or none (t >= r): one mask, one scan
            const bool ties = t < r;
            uint32_t m = ties ? le : lt;
            const uint32_t excl = incl - cnt;
            int pos = fr.hbase + a + min(t, r) + (int)(excl & 0xFFFFu) + (ties ? (int)(excl >> 16) : 0);
            while (m) {
                const int bit = __ffs((int)m) - 1;
                m &= m - 1;
                if (pos >= 0 && pos < fr.n) s_list[pos] = j_lane + (bit >> 2) * (HA_WAVE * 4) + (bit & 3);
                ++pos;
            }
        } else {
            // the chunk of the r-th tie: ties in token order, slab by slab
            int n_lt = a, n_eq = t;
#pragma unroll
            for (int s = 0; s < GS; ++s) {
                const uint32_t lt4 = (lt >> (4 * s)) & 0xFu, eq4 = (eq >> (4 * s)) & 0xFu;
                const uint32_t c4 = (uint32_t)__popc(lt4) | ((uint32_t)__popc(eq4) << 16);
                const uint32_t in4 = wave_inclusive_scan(c4);
                const uint32_t ex4 = in4 - c4;
                int a2 = n_lt + (int)(ex4 & 0xFFFFu), t2 = n_eq + (int)(ex4 >> 16);
                const uint32_t em = t2 < r ? eq4 : 0u;  // past the r-th tie nothing more of the tie bucket is taken
                uint32_t todo = lt4 | em;
                while (todo) {
                    const int e = __ffs((int)todo) - 1;
                    todo &= todo - 1;
                    const bool is_eq = (em >> e) & 1u;
                    if (!is_eq || t2 < r) {
                        const int pos = fr.hbase + a2 + min(t2, r);
                        if (pos >= 0 && pos < fr.n) s_list[pos] = j_lane + s * (HA_WAVE * 4) + e;
                    }
                    a2 += is_eq ? 0 : 1;
                    t2 += is_eq ? 1 : 0;
                }
                const uint32_t t4 = (uint32_t)__builtin_amdgcn_readlane((int)in4, HA_WAVE - 1);
                n_lt += (int)(t4 & 0xFFFFu);
                n_eq += (int)(t4 >> 16);
            }
        }
    }
    // Slot map: the tokens this wave has just placed - one contiguous stretch of the list - are replaced by their slots, in
    // place and without a register: lane l asks for the map entry of the token at stretch position l, the answer lands on
    // that list entry (memory -> LDS).  The wave's LDS operations complete in order, so the tokens read back here are the
    // ones written above, and each request is issued after the read of the entry it overwrites.
    if (slot_row && active && tot != 0) {
        const int first = fr.hbase + a + min(t, r);
        const int p0 = max(first, 0);
        const int p1 = min(first - min(t, r) + (int)(tot & 0xFFFFu) + min(t + (int)(tot >> 16), r), fr.n);
        for (int pb = p0; pb < p1; pb += HA_WAVE) {
            const int p = pb + lane;
            if (p < p1) request_4_bytes_to_lds(slot_row + s_list[p], s_list + pb);
        }
    }
    // the last group of the round knows where the placed prefix ends
    const int last = min(n_groups - 1 - round * NW, NW - 1);
    if (wave == last && lane == 0) *s_ready = fr.hbase + a + (int)(tot & 0xFFFFu) + min(t + (int)(tot >> 16), r);
    __syncthreads();
    return *s_ready;
}

// ------------------------------------------------------------------------------------------------
// grid (nsplit_max, H, B).  Workgroup s of row (b, h) attends to idx[b, h, s*split_rows : (s+1)*split_rows).
// NT threads = NT/16 row streams; U rows per stream per step.
// MK: an additive term per list entry (AttnMask), natural-log units, added to the scaled score before the softmax; list-fed
// launches only.
// SL: the K/V rows are addressed through a token -> slot table (SlotMap); an instantiation of its own, so that launches
// without a table carry none of it (as a run-time switch it cost the plain launches 0.7 - 1.3 us at 64K tokens x 16).
// LP: fused launches of a left-padded batch: a list entry below amask.masked_prefix[b] scores -inf (it stays in the list and
// in the counts: the selection does not see the mask, hashattention_llama.py:593-598).  The token of a row being reduced is
// read back from the LDS list, so the gather loop carries no extra register.
template <typename E, int NT, int U, int FW, bool MK = false, bool SL = false, bool LP = false>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(4, 4))) void sparse_attend_kernel(const void *__restrict__ q, int64_t q_sb, int64_t q_sh,
                                                           const void *__restrict__ k, const void *__restrict__ v, int64_t kv_sb,
                                                           int64_t kv_sh, int64_t kv_ss, int H, int G,
                                                           const int32_t *__restrict__ idx, int64_t idx_cap,
                                                           const int32_t *__restrict__ counts, float scale_log2e, int split_rows,
                                                           int nsplit_max, float *__restrict__ part_acc,
                                                           float *__restrict__ part_ml, void *__restrict__ out,
                                                           const float *__restrict__ win_part, int win_init, int win_recent,
                                                           const int32_t *__restrict__ seq_lens, int max_S, const FusedSel fsel,
                                                           const AttnMask amask, int rows_per_seq, const SlotMap smap) {
    using EL = Elem<E>;
    static_assert(!MK || FW == 0, "the additive mask exists for list-fed launches only");
    static_assert(!LP || (FW > 0 && !SL), "the masked prefix exists for fused launches without a slot table");
    // staged_codes_arrived(true) waits with vmcnt(8): a gather step (and the loop's priming) must put at least eight
    // vector-memory loads per wave behind the staged codes' requests - U key rows and U value rows of 8 elements, one
    // 128-bit load per 16 bytes
    static_assert(FW == 0 || 2 * U * (Elem<E>::bytes * 8 / 16) >= 8, "fewer than eight row loads per gather step: vmcnt(8) would not cover the staged codes");
    constexpr int NS = NT / 16;  // row streams
    __shared__ float s_m[NS], s_l[NS];
    // the streams' partial results at the end of the kernel; before that, in a fused launch, the waves' staging regions (and,
    // for 64-bit codes, the histogram tile of the threshold search, which is over before the first codes are requested)
    constexpr int kStageWords = FW > 0 ? (NT / HA_WAVE) * kStageWaveWords : 0;
    constexpr int kRawWords = kStageWords > NS * HA_HEAD_DIM ? kStageWords : NS * HA_HEAD_DIM;
    constexpr bool kTileInRaw = FW == 2;
    __shared__ __attribute__((aligned(16))) uint32_t s_raw[kRawWords];
    float *s_acc = reinterpret_cast<float *>(s_raw);
    __shared__ int32_t s_list[FW > 0 ? kFusedListCap : 1];
    __shared__ uint32_t s_cnt[FW > 0 ? 64 : 1];
    __shared__ int s_cstar;
    __shared__ int s_plan[2];
    // in-kernel thresholds: the row's chunk histograms (+ their totals), chunk prefixes, {T, r, n_heavy, tie bucket}
    static_assert(!kTileInRaw || (kFusedLocalChunks + 1) * (32 * FW + 1) <= kRawWords, "the histogram tile fits the staging space");
    __shared__ uint32_t s_tile[FW > 0 && !kTileInRaw ? (kFusedLocalChunks + 1) * (32 * FW + 1) : 1];
    uint32_t *s_h = kTileInRaw ? s_raw : s_tile;
    __shared__ int32_t s_pre[FW > 0 ? 2 * (kFusedMaxChunks + 1) : 1];
    __shared__ int32_t s_meta[8];

    // Workgroups are handed to the 8 XCDs round-robin in launch order.  Walking blockIdx.y over
    // (head in group, group) instead of heads in order puts the query heads of one KV group 8*k apart when
    // there are 8 KV heads, i.e. on one XCD, so rows they share (the sink and recent windows, commonly
    // selected keys) are served by that XCD's L2 instead of being fetched from HBM once per XCD.
    const int Hkv = H / G;
    int sp = blockIdx.x, by = blockIdx.y, b = blockIdx.z;
    if constexpr (FW > 0) {
        // in-kernel plan (below): walk the grid piece index slowest, so that the first pieces of all rows are dispatched
        // first and spread over all XCDs, and the workgroups that turn out to own nothing come last
        if (seq_lens && (int)gridDim.z <= kFusedSortBatch && gridDim.x > 1) {
            const int lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z), per = gridDim.y * gridDim.z;
            sp = lin / per;
            by = (lin % per) % (int)gridDim.y;
            b = (lin % per) / (int)gridDim.y;
        }
    }
    const int h = (by % Hkv) * G + by / Hkv;
    const int tid = threadIdx.x, sub = tid & 15, stream = tid >> 4;
    const int slice = b;  // position of this workgroup's sequence in the walk over the batch
    int cps = fsel.cps, row_pieces = nsplit_max;  // chunks per workgroup, workgroups of this row that own chunks
    if constexpr (FW > 0) {
        // Ragged batch (lengths on the device, up to kFusedSortBatch sequences): every workgroup works out the same plan
        // from the lengths.  (1) Workgroups are dispatched in launch order, so the z-th slice of the grid takes the z-th
        // longest sequence (ties by index) and the long rows do not start last.  (2) One piece size for the batch: the
        // fewest chunks per workgroup for which all pieces of all rows are resident at once (kFusedResident workgroups),
        // so a long row is cut into more pieces than a short one and no second round of workgroups is needed.
        if (seq_lens && (int)gridDim.z <= kFusedSortBatch) {
            const int nb = gridDim.z;
            if (tid < nb) {
                const int mine = seq_lens[tid];
                int rank = 0;
                for (int u = 0; u < nb; ++u) {
                    const int o = seq_lens[u];
                    rank += (o > mine || (o == mine && u < tid)) ? 1 : 0;
                }
                if (rank == slice) s_plan[0] = tid;
            }
            if (tid >= 192 && tid < 256) {  // one candidate piece size per lane of the fourth wave
                const int cstep = (fsel.nchunk + 63) / 64;
                const int cand = (tid - 192 + 1) * cstep;
                int total = 0, longest = 1;
                for (int u = 0; u < nb; ++u) {
                    const int nc = min(max((min(seq_lens[u], max_S) + fsel.chunk - 1) / fsel.chunk, 1), fsel.nchunk);
                    total += (nc + cand - 1) / cand;
                    longest = max(longest, nc);
                }
                const unsigned long long ok = __ballot((int64_t)total * H <= kFusedResident);
                int pick = ok ? (__ffsll((long long)ok)) * cstep : 64 * cstep;
                pick = min(pick, kFusedMaxChunks);  // the chunk prefixes a workgroup keeps in LDS
                pick = max(pick, (longest + (int)gridDim.x - 1) / (int)gridDim.x);  // the grid has gridDim.x workgroups per row
                if (tid == 192) s_plan[1] = pick;
            }
            __syncthreads();
            b = s_plan[0];
            const int nc = min(max((min(seq_lens[b], max_S) + fsel.chunk - 1) / fsel.chunk, 1), fsel.nchunk);
            row_pieces = (nc + s_plan[1] - 1) / s_plan[1];
            cps = (nc + row_pieces - 1) / row_pieces;  // the row's chunks dealt evenly to its pieces
        }
    }
    const int64_t row = (int64_t)b * H + h;
    int r0, r1, nsplit;
    const int32_t *ix = nullptr;
    FusedRow fr = {};
    [[maybe_unused]] HistTileRegs<(FW > 0 ? FW : 1), NT> hist_tile;
    int j_max = 0;  // fused: last token of the sequence (list entries are clamped to it: a wrong entry must not become a wild address)
    [[maybe_unused]] int masked_below = 0;
    if constexpr (FW > 0) {
        int S = seq_lens ? seq_lens[b] : max_S;
        if (S > max_S) S = max_S;
        if constexpr (LP) masked_below = amask.masked_prefix[b];
        nsplit = nsplit_max;  // every workgroup of the grid owns chunks; an empty one leaves an empty partial
        if (sp >= row_pieces) {  // nothing of this row here (uniform over the workgroup): an empty partial
            if (tid < HA_HEAD_DIM) {
                const int64_t p = row * nsplit_max + sp;
                part_acc[p * HA_HEAD_DIM + tid] = 0.f;
                if (tid == 0) {
                    part_ml[p * 2] = -INFINITY;
                    part_ml[p * 2 + 1] = 0.f;
                }
            }
            return;
        }
        if (fsel.hist) {
            hist_tile.request(fsel, row);
            if (tid < 32 * FW + 1) s_h[fsel.nchunk * (32 * FW + 1) + tid] = 0;  // the level totals (local_thresholds)
        }
        fused_windows<NT>(fsel, S, sp, cps, row_pieces, s_list, fr, SL ? smap.slots + b * smap.stride_b : nullptr);
        j_max = SL ? smap.max_slot : max(S - 1, 0);
        r0 = 0;
        r1 = fr.nwin;  // until the thresholds are known the list is its windows
    } else {
        int64_t n = counts[b * H + h];
        if (n > idx_cap) n = idx_cap;
        // win_part: the sink and recent windows were attended by another launch; their entries (the first
        // min(init, S) and the last S - max(S - recent, min(init, S)) of the list) are skipped here and the
        // partial is merged at the end
        int skip_front = 0;
        if (win_part) {
            int S = seq_lens ? seq_lens[b] : max_S;
            if (S > max_S) S = max_S;
            const int lo = min(win_init, S), hi = max(S - win_recent, lo);
            skip_front = lo;
            n = max((int64_t)0, n - lo - (S - hi));
        }
        nsplit = n > 0 ? (int)((n + split_rows - 1) / split_rows) : 1;
        if (sp >= nsplit) return;
        if (n == 0 && !win_part) {  // empty sequence: defined as a zero output
            if (tid < HA_HEAD_DIM) EL::store1((char *)out + row * HA_HEAD_DIM * EL::bytes, tid, 0.f);
            return;
        }
        r0 = skip_front + sp * split_rows;
        r1 = (int)min((int64_t)r0 + split_rows, skip_front + n);
        ix = idx + row * idx_cap;
    }
    // rows_per_seq consecutive batch entries attend to the cache of one sequence (the rows of a chunk of tokens)
    // (list-fed launches only: in the fused instantiation the extra value would cost it a spilled register)
    int64_t b_kv = b;
    if constexpr (FW == 0) b_kv = rows_per_seq > 1 ? b / rows_per_seq : b;
    const char *kb = (const char *)k + (b_kv * kv_sb + (h / G) * kv_sh) * EL::bytes;
    const char *vb = (const char *)v + (b_kv * kv_sb + (h / G) * kv_sh) * EL::bytes;
    const int64_t row_bytes = kv_ss * EL::bytes;
    constexpr int STEP = NS * U;  // rows of the list consumed per step by the workgroup
    // this sequence's token -> slot map (nullptr: rows lie at their token positions)
    const int32_t *slot_row = nullptr;
    if constexpr (SL) slot_row = smap.slots + b_kv * smap.stride_b;

    // the query slice as it lies in memory: the score is dot8(q, k) * scale, two elements per instruction for 16-bit rows
    const Raw8<E> qraw = EL::load8((const char *)q + (b * q_sb + h * q_sh) * EL::bytes, sub);
    float m = -INFINITY, l = 0.f, acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;

    // list position of (step base, u) for this stream; positions >= r1 are padded with the split's first row
    auto list_index = [&](int base, int u) {
        const int r = base + stream + u * NS;
        if constexpr (FW > 0) return r < r1 ? min(max(s_list[r], 0), j_max) : 0;  // padding: token 0, always present
        else return ix[r < r1 ? r : r0];
    };
    int32_t j_next[U];   // indices of the step after the one in flight
    // list-fed launch with a slot map: j_next holds slots; the tokens of the step behind that one are loaded a step earlier
    // still, so that their map entries can be requested without waiting for them (t_after), and a mask by token position
    // keeps the tokens of the step after the one in flight (tok_next)
    [[maybe_unused]] int32_t t_after[U], tok_next[U];
    Raw8<E> kr[U], vr[U];
    int base = r0;
    // MK: the additive term of list position (step base, u), token j, in the log2 units of the scores.  The index is
    // clamped to the mask row, so a list entry beyond it reads the row's last value instead of a wild address.
    [[maybe_unused]] float mk[U], mk_next[U];
    [[maybe_unused]] auto mask_term = [&](int base_, int u, int32_t j) {
        const int r = base_ + stream + u * NS;
        const int64_t e = amask.by_slot ? (r < r1 ? r : r0) : j;
        return amask.values[b * amask.stride_b + min(max(e, (int64_t)0), (int64_t)amask.len - 1)] * kLog2e;
    };
    // needs list entries [base, base + 2 STEP)
    auto prime = [&]() {
        int32_t j0[U];
#pragma unroll
        for (int u = 0; u < U; ++u) j0[u] = list_index(base, u);
#pragma unroll
        for (int u = 0; u < U; ++u) j_next[u] = list_index(base + STEP, u);
        if constexpr (MK) {
#pragma unroll
            for (int u = 0; u < U; ++u) mk[u] = mask_term(base, u, j0[u]);
        }
        if constexpr (FW == 0 && SL) {
            {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    t_after[u] = list_index(base + 2 * STEP, u);
                    if constexpr (MK) tok_next[u] = j_next[u];
                    j0[u] = slot_row[j0[u]];
                    j_next[u] = slot_row[j_next[u]];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) kr[u] = EL::load8s(kb + j0[u] * row_bytes, sub);
#pragma unroll
        for (int u = 0; u < U; ++u) vr[u] = EL::load8s(vb + j0[u] * row_bytes, sub);
    };
    // consumes list entries [base, base + STEP); needs entries up to base + 3 STEP
    auto step = [&]() {
        // ---- issue the loads of the next step (harmless duplicates of a padding row past the end)
        Raw8<E> kn[U], vn[U];
        int32_t j_after[U];
#pragma unroll
        for (int u = 0; u < U; ++u) kn[u] = EL::load8s(kb + j_next[u] * row_bytes, sub);
#pragma unroll
        for (int u = 0; u < U; ++u) vn[u] = EL::load8s(vb + j_next[u] * row_bytes, sub);
        [[maybe_unused]] int32_t tok_after[U];
        constexpr bool translated = FW == 0 && SL;
        if constexpr (translated) {
            {  // tokens of step + 2 arrived a step ago -> their slots; tokens of step + 3 requested
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int32_t t = t_after[u];
                    j_after[u] = slot_row[t];
                    if constexpr (MK) tok_after[u] = t;
                    t_after[u] = list_index(base + 3 * STEP, u);
                }
            }
        }
        if constexpr (!translated) {
#pragma unroll
            for (int u = 0; u < U; ++u) j_after[u] = list_index(base + 2 * STEP, u);
        }
        if constexpr (MK) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if constexpr (translated) mk_next[u] = mask_term(base + STEP, u, tok_next[u]);
                else mk_next[u] = mask_term(base + STEP, u, j_next[u]);
            }
        }

        // ---- reduce the current step
        float sc[U], mloc = -INFINITY;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float d = row16_sum(EL::dot8(qraw, kr[u])) * scale_log2e;
            if constexpr (MK) d += mk[u];
            bool live = base + stream + u * NS < r1;
            if constexpr (LP) live = live && s_list[min(base + stream + u * NS, kFusedListCap - 1)] >= masked_below;
            sc[u] = live ? d : -INFINITY;
            mloc = fmaxf(mloc, sc[u]);
        }
        if (mloc > -INFINITY) {  // at least one live row in this stream's step
            const float m_new = fmaxf(m, mloc);
            const float alpha = fast_exp2(m - m_new);  // m == -inf on the first pass gives 0
            l *= alpha;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] *= alpha;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const float p = fast_exp2(sc[u] - m_new);
                float vf[8];
                EL::unpack(vr[u], vf);
                l += p;
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[i] = fmaf(p, vf[i], acc[i]);
            }
            m = m_new;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            kr[u] = kn[u];
            vr[u] = vn[u];
            j_next[u] = j_after[u];
            if constexpr (MK) {
                mk[u] = mk_next[u];
                if constexpr (translated) tok_next[u] = tok_after[u];
            }
        }
        base += STEP;
    };

    if constexpr (FW > 0) {
        // scan rounds and gather steps alternate: after a round the list is complete up to `ready`, and the loop runs
        // as far as its look-ahead (3 steps) allows.  Everything here is uniform over the workgroup.
        constexpr int NW = NT / HA_WAVE;
        constexpr int GS = kStageWaveWords / (HA_WAVE * 4 * FW);  // slabs per wave and round: a staging region's worth
        constexpr int gc = GS * HA_WAVE * 4;                      // codes per wave and round; divides every chunk size
        // the row's query code, once and in scalar registers: loaded in a scan round it would be the youngest request of the
        // wave there, and waiting for it would mean waiting for every row on its way
        // (requested here, moved to the scalar registers behind the threshold search: in front of it the move would wait a
        // memory round trip before the window rows and the first codes are even requested)
        ha_sel::Code<FW> qcode = ha_sel::load_qcode<FW>(fsel.qcodes, row);
        // the codes of the first round are requested before the thresholds are worked out, when the workgroup's chunks are
        // known by then (a row in one piece) and the histogram tile has a place of its own - and before the window rows:
        // the compiler's wait for the histogram tile (requested earlier still) counts the requests it knows, so unseen
        // requests behind the rows would make it wait for as many rows
        bool staged_early = false;
        if constexpr (!kTileInRaw) {
            if (row_pieces == 1) {
                fused_round_stage<FW, GS, NW>(fsel, fr, b, h, 0, fr.nc * (fsel.chunk / gc), s_raw);
                staged_early = true;
            }
        }
        // the windows alone fill the first two steps: their rows are requested before the thresholds are worked out too.
        // The histogram tile goes from its registers to LDS behind them, written out in either branch: placed behind the
        // branch, the compiler's wait for the tile would have to assume that no rows were requested and wait for all but two
        // of the requests it knows - for the window rows too.
        bool primed = false;
        if (fr.nwin >= 2 * STEP) {
            prime();
            primed = true;
            if (fsel.hist) hist_tile.to_lds(fsel, s_h, s_h + fsel.nchunk * (32 * FW + 1));
        } else {
            if (fsel.hist) hist_tile.to_lds(fsel, s_h, s_h + fsel.nchunk * (32 * FW + 1));
        }
        {
            int S = seq_lens ? seq_lens[b] : max_S;
            if (S > max_S) S = max_S;
            fused_thresholds<FW, NT>(fsel, row, S, sp, row_pieces, &s_cstar, s_h, s_pre, s_meta, fr);
        }
        r1 = fr.n;
        qcode.w0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)qcode.w0);
        if constexpr (FW == 2) qcode.w1 = (uint32_t)__builtin_amdgcn_readfirstlane((int)qcode.w1);
        const int n_groups = fr.nheavy > 0 ? fr.nc * (fsel.chunk / gc) : 0;
        const int rounds = (n_groups + NW - 1) / NW;
        // codes requested for a round that will not take place must not arrive in the partial results later
        if (staged_early && rounds == 0) staged_codes_arrived(false);
        if (nsplit == 1 && r1 == 0) {  // empty sequence: defined as a zero output (uniform over the workgroup)
            if (tid < HA_HEAD_DIM) EL::store1((char *)out + row * HA_HEAD_DIM * EL::bytes, tid, 0.f);
            return;
        }
        if (rounds > 0 && !staged_early) fused_round_stage<FW, GS, NW>(fsel, fr, b, h, 0, n_groups, s_raw);
        bool covered = false;  // eight row requests have been issued behind the staged codes' requests
        // Slot map: a round's entries are translated in place behind the round and hold slots for every wave once the next
        // round's first barrier has passed, so the loop runs one round behind the scan: `usable` = the entries placed by the
        // rounds before the last one (the windows were translated when they were written).
        int usable = fr.nwin, placed = fr.nwin;
        for (int k = 0; k < rounds; ++k) {
            int ready = fused_round<FW, GS, NW>(fsel, fr, b, h, qcode, k, n_groups, s_cnt, &s_cstar, s_list, s_raw, covered, slot_row);
            if constexpr (SL) {
                usable = placed;
                placed = min(ready, r1);
                ready = usable;
                if (k == rounds - 1) covered = false;  // the youngest requests are now this round's translations
            }
            if (k == rounds - 1) break;
            ready = min(ready, r1);
            fused_round_stage<FW, GS, NW>(fsel, fr, b, h, k + 1, n_groups, s_raw);
            covered = false;
            if (!primed && ready >= min(2 * STEP, r1)) {
                prime();
                primed = true;
                covered = true;
            }
            // Steps two at a time: a step's requests go to the registers its predecessor has just read, so after two
            // steps every row is where the loop expects it; after one, leaving the loop costs a copy of rows that are
            // still on their way, i.e. a wait for everything outstanding.
            while (primed && base + 4 * STEP <= ready) {
                step();
                step();
                covered = true;
            }
        }
        if (SL && rounds > 0) {
            // the last round's entries: run what the earlier rounds allow, then every wave waits for its own translations
            // and the waves meet
            if (!primed && usable >= min(2 * STEP, r1)) {
                prime();
                primed = true;
                covered = true;
            }
            while (primed && base + 4 * STEP <= usable) {
                step();
                step();
                covered = true;
            }
            staged_codes_arrived(covered);
            __syncthreads();
        }
        if (!primed) prime();
        while (base < r1) step();
    } else {
        prime();
        while (base < r1) step();
    }

    if (sub == 0) {
        s_m[stream] = m;
        s_l[stream] = l;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) s_acc[stream * HA_HEAD_DIM + sub * 8 + i] = acc[i];
    __syncthreads();
    if (tid < HA_HEAD_DIM) {
        float M, L, A;
        merge_streams<NS>(s_m, s_l, s_acc, tid, M, L, A);
        if (nsplit == 1) {
            if (win_part) {  // partial of the windows: acc[128], m, l
                const float *wp = win_part + row * (HA_HEAD_DIM + 2);
                const float wm = wp[HA_HEAD_DIM], wl = wp[HA_HEAD_DIM + 1];
                const float M2 = fmaxf(M, wm);
                const float sh = (M == -INFINITY) ? 0.f : fast_exp2(M - M2), sw = (wm == -INFINITY) ? 0.f : fast_exp2(wm - M2);
                A = A * sh + wp[tid] * sw;
                L = L * sh + wl * sw;
            }
            EL::store1((char *)out + row * HA_HEAD_DIM * EL::bytes, tid, L > 0.f ? A / L : 0.f);
        } else {
            const int64_t p = row * nsplit_max + sp;
            part_acc[p * HA_HEAD_DIM + tid] = A;
            if (tid == 0) {
                part_ml[p * 2] = M;
                part_ml[p * 2 + 1] = L;
            }
        }
    }
}

// grid (H, B), 128 threads: merge the split partials of a row.  `unit` = rows (sparse) or keys (dense) per
// split; counts is per (b, h) row, per sequence (per_batch), or absent (every row has count_cap units).
// Rows with a single split were finished by the attend kernel.
template <typename E>
__global__ __launch_bounds__(HA_HEAD_DIM) void merge_splits_kernel(const float *__restrict__ part_acc, const float *__restrict__ part_ml,
                                                                   const int32_t *__restrict__ counts, int per_batch,
                                                                   int64_t count_cap, int H, int unit, int nsplit_max,
                                                                   void *__restrict__ out, const float *__restrict__ win_part,
                                                                   int win_init, int win_recent,
                                                                   const int32_t *__restrict__ win_seq_lens, int win_max_S) {
    using EL = Elem<E>;
    const int h = blockIdx.x, b = blockIdx.y, e = threadIdx.x;
    const int64_t row = (int64_t)b * H + h;
    int64_t n = counts ? counts[per_batch ? b : row] : count_cap;
    if (n > count_cap) n = count_cap;
    if (win_part) {  // the attend kernel skipped the window entries of the list (see sparse_attend_kernel)
        int win_S = win_seq_lens ? win_seq_lens[b] : win_max_S;
        if (win_S > win_max_S) win_S = win_max_S;
        const int lo = min(win_init, win_S), hi = max(win_S - win_recent, lo);
        n = max((int64_t)0, n - lo - (win_S - hi));
    }
    const int nsplit = (int)((n + unit - 1) / unit);
    if (nsplit <= 1) return;
    const float *ml = part_ml + row * nsplit_max * 2;
    const float *pa = part_acc + row * nsplit_max * HA_HEAD_DIM + e;
    float M = -INFINITY;
#pragma unroll 8
    for (int s = 0; s < nsplit; ++s) M = fmaxf(M, ml[s * 2]);
    float L = 0.f, A = 0.f;
#pragma unroll 8
    for (int s = 0; s < nsplit; ++s) {
        const float w = (ml[s * 2] == -INFINITY) ? 0.f : fast_exp2(ml[s * 2] - M);  // an empty split leaves (m, l) = (-inf, 0)
        L += w * ml[s * 2 + 1];
        A += w * pa[(int64_t)s * HA_HEAD_DIM];
    }
    if (win_part) {
        const float *wp = win_part + row * (HA_HEAD_DIM + 2);
        const float wm = wp[HA_HEAD_DIM], M2 = fmaxf(M, wm);
        const float sh = (M == -INFINITY) ? 0.f : fast_exp2(M - M2), sw = (wm == -INFINITY) ? 0.f : fast_exp2(wm - M2);
        A = A * sh + wp[e] * sw;
        L = L * sh + wp[HA_HEAD_DIM + 1] * sw;
    }
    EL::store1((char *)out + row * HA_HEAD_DIM * EL::bytes, e, L > 0.f ? A / L : 0.f);
}

// ------------------------------------------------------------------------------------------------
// Dense flash-decode.  grid (nsplit_max, Hkv * passes, B).  A workgroup streams `chunk` consecutive keys of one
// KV head once and scores them against G query heads of its group of `group` heads: passes = ceil(group / G), and a
// group that is not 1, 2, 4 or 8 heads wide leaves the last slots of its last pass idle (24 query heads on 8 KV heads:
// G = 4, one pass, three slots used).
// WIN: the same over the sink and recent windows only (win_init, win_recent; grid (1, Hkv, B)): the result is
// left as an unnormalised partial (acc, m, l) per row for the sparse kernel to merge, so this small launch can
// run on another stream while the selection is still being computed.
template <typename E, int G, bool WIN>
__global__ __launch_bounds__(kAttThreads) void dense_attend_kernel(const void *__restrict__ q, int64_t q_sb, int64_t q_sh,
                                                                   const void *__restrict__ k, const void *__restrict__ v,
                                                                   int64_t kv_sb, int64_t kv_sh, int64_t kv_ss, int H, int group,
                                                                   int max_S, const int32_t *__restrict__ seq_lens, float scale_log2e,
                                                                   int chunk, int nsplit_max, float *__restrict__ part_acc,
                                                                   float *__restrict__ part_ml, void *__restrict__ out, int win_init,
                                                                   int win_recent) {
    using EL = Elem<E>;
    __shared__ float s_m[kStreams], s_l[kStreams];
    __shared__ float s_acc[kStreams * HA_HEAD_DIM];

    const int sp = blockIdx.x, b = blockIdx.z;
    const int passes = (group + G - 1) / G;
    const int hk = blockIdx.y / passes;
    const int h0 = hk * group + (blockIdx.y % passes) * G;  // query head of slot 0
    const int n_slots = min(G, (hk + 1) * group - h0);      // slots of this workgroup that hold a query head
    const int tid = threadIdx.x, sub = tid & 15, stream = tid >> 4;
    int S = seq_lens ? seq_lens[b] : max_S;
    if (S > max_S) S = max_S;
    // WIN: list position t < n_sink is token t, the others are tokens win_hi + (t - n_sink)
    const int n_sink = WIN ? min(win_init, S) : 0;
    const int win_hi = WIN ? max(S - win_recent, n_sink) : 0;
    const int n_rows = WIN ? n_sink + (S - win_hi) : S;
    const int nsplit = WIN ? 1 : (S > 0 ? (S + chunk - 1) / chunk : 1);
    if (sp >= nsplit) return;
    if (!WIN && S == 0) {
        if (tid < HA_HEAD_DIM)
            for (int g = 0; g < n_slots; ++g) EL::store1((char *)out + ((int64_t)b * H + h0 + g) * HA_HEAD_DIM * EL::bytes, tid, 0.f);
        return;
    }
    const int r0 = WIN ? 0 : sp * chunk, r1 = WIN ? n_rows : min(r0 + chunk, S);
    auto token = [&](int r) { return WIN ? (r < n_sink ? r : win_hi + (r - n_sink)) : r; };
    const char *kb = (const char *)k + (b * kv_sb + hk * kv_sh) * EL::bytes;
    const char *vb = (const char *)v + (b * kv_sb + hk * kv_sh) * EL::bytes;
    const int64_t row_bytes = kv_ss * EL::bytes;

    float qf[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float t[8];
        EL::unpack(EL::load8((const char *)q + (b * q_sb + (h0 + min(g, n_slots - 1)) * q_sh) * EL::bytes, sub), t);  // idle slots repeat the last head
#pragma unroll
        for (int i = 0; i < 8; ++i) qf[g][i] = t[i] * scale_log2e;
    }
    float m[G], l[G], acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m[g] = -INFINITY;
        l[g] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g][i] = 0.f;
    }

    for (int base = r0 + stream; base < r1; base += kStreams * kUnroll) {
        bool ok[kUnroll];
        Raw8<E> kr[kUnroll], vr[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int r = base + u * kStreams;
            ok[u] = r < r1;
            kr[u] = EL::load8s(kb + token(ok[u] ? r : base) * row_bytes, sub);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) vr[u] = EL::load8s(vb + token(ok[u] ? base + u * kStreams : base) * row_bytes, sub);

        float sc[G][kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            float kf[8];
            EL::unpack(kr[u], kf);
#pragma unroll
            for (int g = 0; g < G; ++g) {
                float d = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) d = fmaf(qf[g][i], kf[i], d);
                d = row16_sum(d);
                sc[g][u] = ok[u] ? d : -INFINITY;
            }
        }
        float p[G][kUnroll];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float mloc = sc[g][0];
#pragma unroll
            for (int u = 1; u < kUnroll; ++u) mloc = fmaxf(mloc, sc[g][u]);
            const float m_new = fmaxf(m[g], mloc);
            const float alpha = fast_exp2(m[g] - m_new);
            l[g] *= alpha;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[g][i] *= alpha;
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                p[g][u] = fast_exp2(sc[g][u] - m_new);
                l[g] += p[g][u];
            }
            m[g] = m_new;
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            float vf[8];
            EL::unpack(vr[u], vf);
#pragma unroll
            for (int g = 0; g < G; ++g)
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[g][i] = fmaf(p[g][u], vf[i], acc[g][i]);
        }
    }

#pragma unroll
    for (int g = 0; g < G; ++g) {
        __syncthreads();  // the previous head's merge has finished reading LDS
        if (sub == 0) {
            s_m[stream] = m[g];
            s_l[stream] = l[g];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) s_acc[stream * HA_HEAD_DIM + sub * 8 + i] = acc[g][i];
        __syncthreads();
        if (tid < HA_HEAD_DIM && g < n_slots) {
            float M, L, A;
            merge_streams<kStreams>(s_m, s_l, s_acc, tid, M, L, A);
            const int64_t row = (int64_t)b * H + h0 + g;
            if (WIN) {  // one record per row: acc[128], m, l
                part_acc[row * (HA_HEAD_DIM + 2) + tid] = A;
                if (tid == 0) {
                    part_acc[row * (HA_HEAD_DIM + 2) + HA_HEAD_DIM] = M;
                    part_acc[row * (HA_HEAD_DIM + 2) + HA_HEAD_DIM + 1] = L;
                }
            } else if (nsplit == 1) {
                EL::store1((char *)out + row * HA_HEAD_DIM * EL::bytes, tid, A / L);
            } else {
                const int64_t pi = row * nsplit_max + sp;
                part_acc[pi * HA_HEAD_DIM + tid] = A;
                if (tid == 0) {
                    part_ml[pi * 2] = M;
                    part_ml[pi * 2 + 1] = L;
                }
            }
        }
    }
}

// query-head slots per workgroup of the dense kernel for a group of `group` query heads per KV head
inline int dense_slots(int group) { return group <= 1 ? 1 : group <= 2 ? 2 : group <= 4 ? 4 : 8; }

int validate_qkv(const void *q, int64_t q_sb, int64_t q_sh, const void *k, const void *v, int kv_dtype, int64_t kv_sb, int64_t kv_sh,
                 int64_t kv_ss, int B, int H, int Hkv, const void *out) {
    HA_REQUIRE(q && k && v && out, HA_ERR_NULL_POINTER, "q/k/v/out is NULL");
    HA_REQUIRE(kv_dtype == HA_F32 || kv_dtype == HA_BF16 || kv_dtype == HA_F16, HA_ERR_BAD_DTYPE, "kv_dtype %d", kv_dtype);
    HA_REQUIRE(B > 0 && H > 0 && Hkv > 0 && B <= 65535 && H <= 65535, HA_ERR_BAD_SHAPE, "B, H, Hkv must be in 1..65535");
    HA_REQUIRE(H % Hkv == 0, HA_ERR_BAD_SHAPE, "H=%d not a multiple of Hkv=%d", H, Hkv);
    HA_REQUIRE(kv_ss >= HA_HEAD_DIM && kv_sh >= 0 && kv_sb >= 0 && q_sh >= HA_HEAD_DIM && q_sb >= 0, HA_ERR_BAD_SHAPE,
               "strides smaller than a 128-element row");
    const int eb = ha_dtype_bytes(kv_dtype);
    HA_REQUIRE(ha_aligned(q, 16) && ha_aligned(k, 16) && ha_aligned(v, 16) && ha_aligned(out, 16), HA_ERR_MISALIGNED,
               "q/k/v/out must be 16-byte aligned");
    HA_REQUIRE((kv_ss * eb) % 16 == 0 && (kv_sh * eb) % 16 == 0 && (kv_sb * eb) % 16 == 0 && (q_sh * eb) % 16 == 0 &&
                   (q_sb * eb) % 16 == 0,
               HA_ERR_MISALIGNED, "strides must keep rows 16-byte aligned");
    return HA_OK;
}

size_t part_bytes(int64_t rows, int nsplit_max) { return (size_t)rows * nsplit_max * (HA_HEAD_DIM + 2) * sizeof(float); }

}  // namespace

extern "C" {

size_t ha_sparse_decode_workspace_bytes(int B, int H, int64_t idx_cap) {
    if (B <= 0 || H <= 0 || idx_cap <= 0) return 0;
    // sized for the finest split any plan uses, so tuning overrides never outgrow a caller's buffer
    return part_bytes((int64_t)B * H, (int)((idx_cap + kMinSplitRows - 1) / kMinSplitRows));
}

static int sparse_decode_impl(const void *q, int64_t q_stride_b, int64_t q_stride_h, const void *k, const void *v, int kv_dtype,
                              int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, int B, int H, int Hkv,
                              const int32_t *idx, int64_t idx_cap, const int32_t *counts, float sm_scale, void *out, void *workspace,
                              size_t workspace_bytes, const float *win_part, int win_init, int win_recent, const int32_t *seq_lens,
                              int max_seq_len, const AttnMask amask, void *stream, int rows_per_seq = 1,
                              const SlotMap smap = SlotMap{}) {
    int st = validate_qkv(q, q_stride_b, q_stride_h, k, v, kv_dtype, kv_stride_b, kv_stride_h, kv_stride_s, B, H, Hkv, out);
    if (st) return st;
    HA_REQUIRE(rows_per_seq >= 1 && B % rows_per_seq == 0, HA_ERR_BAD_SHAPE, "rows_per_sequence=%d must divide the %d batch entries",
               rows_per_seq, B);
    HA_REQUIRE(idx && counts, HA_ERR_NULL_POINTER, "idx/counts is NULL");
    HA_REQUIRE(idx_cap > 0, HA_ERR_BAD_SHAPE, "idx_cap must be positive");
    const size_t need = ha_sparse_decode_workspace_bytes(B, H, idx_cap);
    HA_REQUIRE(workspace && workspace_bytes >= need, HA_ERR_WORKSPACE, "sparse decode workspace: need %zu bytes, got %zu", need,
               workspace ? workspace_bytes : (size_t)0);
    HA_REQUIRE(ha_aligned(workspace, 256), HA_ERR_MISALIGNED, "workspace must be 256-byte aligned");
    if ((st = ha_require_device())) return st;

    const SparsePlan plan = sparse_plan(B, H, idx_cap);
    const int64_t rows = (int64_t)B * H;
    float *part_acc = (float *)workspace;
    float *part_ml = part_acc + rows * plan.nsplit_max * HA_HEAD_DIM;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(plan.nsplit_max, H, B), mgrid(H, B);
    const float sl2 = sm_scale * kLog2e;
    const int G = H / Hkv;
#define HA_SPARSE_LAUNCH(E_, NT_, U_, MK_, SL_)                                                                                      \
    do {                                                                                                                          \
        hipLaunchKernelGGL((sparse_attend_kernel<E_, NT_, U_, 0, MK_, SL_>), grid, dim3(NT_), 0, s, q, q_stride_b, q_stride_h, k, v, \
                           kv_stride_b, kv_stride_h, kv_stride_s, H, G, idx, idx_cap, counts, sl2, plan.split_rows,               \
                           plan.nsplit_max, part_acc, part_ml, out, win_part, win_init, win_recent, seq_lens, max_seq_len,        \
                           FusedSel{}, amask, rows_per_seq, smap);                                                                \
        HA_CHECK_LAUNCH("sparse_attend_kernel");                                                                                  \
        if (plan.nsplit_max > 1) {                                                                                                \
            hipLaunchKernelGGL(merge_splits_kernel<E_>, mgrid, dim3(HA_HEAD_DIM), 0, s, part_acc, part_ml, counts, 0, idx_cap, H, \
                               plan.split_rows, plan.nsplit_max, out, win_part, win_init, win_recent, seq_lens, max_seq_len);     \
            HA_CHECK_LAUNCH("merge_splits_kernel");                                                                               \
        }                                                                                                                         \
    } while (0)
    // (256-thread workgroups exist as a tuning override only; a table takes the 512-thread form)
#ifdef HASHATTN_TUNING_ENV
#define HA_SPARSE_NT(E_, U_, MK_)                                                         \
    do {                                                                                  \
        if (smap.slots) HA_SPARSE_LAUNCH(E_, 512, U_, MK_, true);                         \
        else if (plan.threads == 512) HA_SPARSE_LAUNCH(E_, 512, U_, MK_, false);          \
        else HA_SPARSE_LAUNCH(E_, 256, U_, MK_, false);                                   \
    } while (0)
#else
#define HA_SPARSE_NT(E_, U_, MK_)                                                         \
    do {                                                                                  \
        if (smap.slots) HA_SPARSE_LAUNCH(E_, 512, U_, MK_, true);                         \
        else HA_SPARSE_LAUNCH(E_, 512, U_, MK_, false);                                   \
    } while (0)
#endif
#define HA_SPARSE_DISPATCH(E_, U_)                 \
    do {                                           \
        if (amask.values) HA_SPARSE_NT(E_, U_, true); \
        else HA_SPARSE_NT(E_, U_, false);          \
    } while (0)
    if (kv_dtype == HA_BF16) HA_SPARSE_DISPATCH(ElemBF16, 4);
    else if (kv_dtype == HA_F16) HA_SPARSE_DISPATCH(ElemF16, 4);
    else HA_SPARSE_DISPATCH(ElemF32, 2);
#undef HA_SPARSE_DISPATCH
#undef HA_SPARSE_NT
#undef HA_SPARSE_LAUNCH
    return HA_OK;
}

int ha_sparse_decode(const void *q, int64_t q_stride_b, int64_t q_stride_h, const void *k, const void *v, int kv_dtype,
                     int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, int B, int H, int Hkv, const int32_t *idx,
                     int64_t idx_cap, const int32_t *counts, float sm_scale, void *out, void *workspace, size_t workspace_bytes,
                     void *stream) {
    return sparse_decode_impl(q, q_stride_b, q_stride_h, k, v, kv_dtype, kv_stride_b, kv_stride_h, kv_stride_s, B, H, Hkv, idx, idx_cap,
                              counts, sm_scale, out, workspace, workspace_bytes, nullptr, 0, 0, nullptr, 0, AttnMask{}, stream);
}

int ha_sparse_decode_masked(const void *q, int64_t q_stride_b, int64_t q_stride_h, const void *k, const void *v, int kv_dtype,
                            int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, int B, int H, int Hkv, const int32_t *idx,
                            int64_t idx_cap, const int32_t *counts, float sm_scale, const float *mask, int64_t mask_stride_b,
                            int mask_len, int mask_by_slot, void *out, void *workspace, size_t workspace_bytes, void *stream) {
    HA_REQUIRE(mask, HA_ERR_NULL_POINTER, "mask is NULL");
    HA_REQUIRE(mask_len > 0 && mask_stride_b >= 0, HA_ERR_BAD_SHAPE, "mask_len must be positive and mask_stride_b non-negative");
    HA_REQUIRE(mask_by_slot == 0 || mask_by_slot == 1, HA_ERR_BAD_SHAPE, "mask_by_slot must be 0 or 1");
    HA_REQUIRE(!mask_by_slot || mask_len >= idx_cap, HA_ERR_BAD_SHAPE, "a mask by list slot needs idx_cap=%lld values per row, got %d",
               (long long)idx_cap, mask_len);
    HA_REQUIRE(ha_aligned(mask, 4), HA_ERR_MISALIGNED, "mask misaligned");
    return sparse_decode_impl(q, q_stride_b, q_stride_h, k, v, kv_dtype, kv_stride_b, kv_stride_h, kv_stride_s, B, H, Hkv, idx, idx_cap,
                              counts, sm_scale, out, workspace, workspace_bytes, nullptr, 0, 0, nullptr, 0,
                              AttnMask{mask, mask_stride_b, mask_len, mask_by_slot}, stream);
}

int ha_sparse_decode_rows(const void *q, int64_t q_stride_b, int64_t q_stride_h, const void *k, const void *v, int kv_dtype,
                          int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, int B, int rows_per_sequence, int H, int Hkv,
                          const int32_t *idx, int64_t idx_cap, const int32_t *counts, float sm_scale, const float *mask,
                          int64_t mask_stride_b, int mask_len, void *out, void *workspace, size_t workspace_bytes, void *stream) {
    HA_REQUIRE(!mask || (mask_len > 0 && mask_stride_b >= 0 && ha_aligned(mask, 4)), HA_ERR_BAD_SHAPE,
               "mask_len must be positive, mask_stride_b non-negative, the mask 4-byte aligned");
    return sparse_decode_impl(q, q_stride_b, q_stride_h, k, v, kv_dtype, kv_stride_b, kv_stride_h, kv_stride_s, B, H, Hkv, idx, idx_cap,
                              counts, sm_scale, out, workspace, workspace_bytes, nullptr, 0, 0, nullptr, 0,
                              mask ? AttnMask{mask, mask_stride_b, mask_len, 0} : AttnMask{}, stream, rows_per_sequence);
}

int ha_sparse_decode_heavy(const void *q, int64_t q_stride_b, int64_t q_stride_h, const void *k, const void *v, int kv_dtype,
                           int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, int B, int H, int Hkv, const int32_t *idx,
                           int64_t idx_cap, const int32_t *counts, float sm_scale, void *out, void *workspace,
                           size_t workspace_bytes, const float *window_partial, int init_budget, int recent_budget,
                           int max_seq_len, const int32_t *seq_lens, void *stream) {
    HA_REQUIRE(window_partial, HA_ERR_NULL_POINTER, "window_partial is NULL");
    HA_REQUIRE(init_budget >= 0 && recent_budget >= 0 && max_seq_len > 0, HA_ERR_BAD_SHAPE, "bad window budgets or max_seq_len");
    return sparse_decode_impl(q, q_stride_b, q_stride_h, k, v, kv_dtype, kv_stride_b, kv_stride_h, kv_stride_s, B, H, Hkv, idx, idx_cap,
                              counts, sm_scale, out, workspace, workspace_bytes, window_partial, init_budget, recent_budget, seq_lens,
                              max_seq_len, AttnMask{}, stream);
}

// Chunks per workgroup of the fused path.  A batch of equal lengths: whole rows when there are at least
// kFusedUniformPieces rows, else that many workgroups in all.  With lengths on the device the kernel decides per row how
// many workgroups own chunks (kFusedResident in all), so the grid offers up to four times the uniform count per row (at
// most kFusedResident / H, the count a single sequence would get).
static int fused_chunks_per_split(int B, int H, int nchunk, bool ragged) {
    const int64_t rows = (int64_t)B * H;
    int64_t want = ((ragged && B > 1 ? kFusedResident : kFusedUniformPieces) + rows - 1) / rows;
    if (ragged && B > 1 && B <= kFusedSortBatch && rows < kFusedResident) want = std::min<int64_t>(4 * want, (kFusedResident + H - 1) / H);
    if (want > nchunk) want = nchunk;
    if (want < 1) want = 1;
    // no piece longer than the chunk prefixes a workgroup keeps in LDS
    return std::min((int)((nchunk + want - 1) / want), kFusedMaxChunks);
}

int ha_sparse_decode_fused_applies(int B, int H, int Hc, int W, int max_seq_len, int init_budget, int recent_budget, double heavy_budget,
                                   int mode) {
    if (B <= 0 || H <= 0 || Hc <= 0 || max_seq_len <= 0 || (W != 1 && W != 2) || H % Hc != 0) return 0;
    if (mode != HA_SELECT_SIMPLE || init_budget < 0 || recent_budget < 0 || heavy_budget < 0.0) return 0;
    // the heavy count as the selection takes it: truncated (int(k) above 1, int(S * fraction) otherwise)
    const double heavy = std::floor(heavy_budget > 1.0 ? heavy_budget : (double)max_seq_len * heavy_budget);
    return (double)init_budget + (double)recent_budget + heavy <= (double)kFusedListCap ? 1 : 0;
}

int ha_sparse_decode_fused_local_thresholds(int B, int Hc, int max_seq_len) {
    if (B <= 0 || Hc <= 0 || max_seq_len <= 0) return 0;
    return ha_sel::select_plan(B, Hc, max_seq_len).nchunk <= kFusedLocalChunks ? 1 : 0;
}

size_t ha_sparse_decode_fused_workspace_bytes(int B, int H, int Hc, int max_seq_len) {
    if (B <= 0 || H <= 0 || Hc <= 0 || max_seq_len <= 0) return 0;
    const ha_sel::SelectPlan plan = ha_sel::select_plan(B, Hc, max_seq_len);
    return part_bytes((int64_t)B * H, plan.nchunk);
}

static int sparse_decode_fused_impl(const void *q, int64_t q_stride_b, int64_t q_stride_h, const void *k, const void *v, int kv_dtype,
                           int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, const uint32_t *kcodes, int64_t kc_stride_b,
                           int64_t kc_stride_h, const uint32_t *qcodes, int B, int H, int Hkv, int Hc, int W, int max_seq_len,
                           const int32_t *seq_lens, int init_budget, int recent_budget, double heavy_budget,
                           const void *select_workspace, size_t select_workspace_bytes, int thresholds_ready, int32_t *out_counts,
                           float sm_scale, void *out, void *workspace, size_t workspace_bytes, void *stream, const SlotMap smap,
                           const int32_t *masked_prefix = nullptr) {
    int st = validate_qkv(q, q_stride_b, q_stride_h, k, v, kv_dtype, kv_stride_b, kv_stride_h, kv_stride_s, B, H, Hkv, out);
    if (st) return st;
    HA_REQUIRE(kcodes && qcodes && select_workspace, HA_ERR_NULL_POINTER, "kcodes/qcodes/select_workspace is NULL");
    HA_REQUIRE(Hc > 0 && H % Hc == 0 && (W == 1 || W == 2) && max_seq_len > 0, HA_ERR_BAD_SHAPE, "bad Hc, W or max_seq_len");
    HA_REQUIRE(kc_stride_h >= (int64_t)max_seq_len * W && kc_stride_b >= kc_stride_h, HA_ERR_BAD_SHAPE,
               "code strides smaller than the rows they span");
    HA_REQUIRE(ha_sparse_decode_fused_applies(B, H, Hc, W, max_seq_len, init_budget, recent_budget, heavy_budget, HA_SELECT_SIMPLE),
               HA_ERR_BAD_SHAPE, "selection larger than the %d-entry list of the fused path: use ha_select + ha_sparse_decode",
               kFusedListCap);
    HA_REQUIRE(select_workspace_bytes >= ha_select_workspace_bytes(B, H, Hc, W, max_seq_len), HA_ERR_WORKSPACE,
               "select workspace smaller than ha_select_workspace_bytes");
    const size_t need = ha_sparse_decode_fused_workspace_bytes(B, H, Hc, max_seq_len);
    HA_REQUIRE(workspace && workspace_bytes >= need, HA_ERR_WORKSPACE, "fused decode workspace: need %zu bytes, got %zu", need,
               workspace ? workspace_bytes : (size_t)0);
    HA_REQUIRE(ha_aligned(workspace, 256) && ha_aligned(select_workspace, 256) && ha_aligned(kcodes, 4 * W) && ha_aligned(qcodes, 4),
               HA_ERR_MISALIGNED, "workspaces must be 256-byte aligned, codes aligned to their word count");
    if ((st = ha_require_device())) return st;

    const ha_sel::SelectPlan plan = ha_sel::select_plan(B, Hc, max_seq_len);
    const ha_sel::SelectWorkspace sw = ha_sel::carve_select_ws(const_cast<void *>(select_workspace), (int64_t)B * H, plan.nchunk, W);
    FusedSel f;
    f.kcodes = kcodes;
    f.kc_sb = kc_stride_b;
    f.kc_sh = kc_stride_h;
    f.qcodes = qcodes;
    f.meta = sw.meta;
    f.chunk_pre = sw.chunk_pre;
    f.nchunk = plan.nchunk;
    f.chunk = plan.blocks * ha_sel::kBlock;
    f.cps = fused_chunks_per_split(B, H, plan.nchunk, seq_lens != nullptr);
    f.gq = H / Hc;
    f.init = init_budget;
    f.recent = recent_budget;
    f.vec = ha_sel::rows_vectorisable(kcodes, kc_stride_b, kc_stride_h, W) ? 1 : 0;
    f.hist = nullptr;
    f.heavy_budget = heavy_budget;
    f.out_counts = out_counts;
    if (!thresholds_ready) {
        HA_REQUIRE(plan.nchunk <= kFusedLocalChunks, HA_ERR_BAD_SHAPE,
                   "rows of more than %d chunks need their thresholds from ha_select_prepare", kFusedLocalChunks);
        f.hist = sw.hist;
    }
    const int nsplit = (plan.nchunk + f.cps - 1) / f.cps;
    const int64_t rows = (int64_t)B * H;
    float *part_acc = (float *)workspace;
    float *part_ml = part_acc + rows * nsplit * HA_HEAD_DIM;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(nsplit, H, B), mgrid(H, B);
    const float sl2 = sm_scale * kLog2e;
    const int G = H / Hkv;
    HA_REQUIRE(!(masked_prefix && smap.slots), HA_ERR_BAD_SHAPE, "a masked prefix and a slot table cannot be combined");
    const AttnMask amask{nullptr, 0, 0, 0, masked_prefix};
#define HA_FUSED_LAUNCH_SL(E_, U_, FW_, SL_, LP_)                                                                                 \
    do {                                                                                                                          \
        hipLaunchKernelGGL((sparse_attend_kernel<E_, 512, U_, FW_, false, SL_, LP_>), grid, dim3(512), 0, s, q, q_stride_b, q_stride_h, k, v, \
                           kv_stride_b, kv_stride_h, kv_stride_s, H, G, nullptr, (int64_t)kFusedListCap, nullptr, sl2, 0, nsplit, \
                           part_acc, part_ml, out, nullptr, 0, 0, seq_lens, max_seq_len, f, amask, 1, smap);                      \
        HA_CHECK_LAUNCH("sparse_attend_kernel (fused selection)");                                                                \
        if (nsplit > 1) {                                                                                                         \
            hipLaunchKernelGGL(merge_splits_kernel<E_>, mgrid, dim3(HA_HEAD_DIM), 0, s, part_acc, part_ml, nullptr, 0,            \
                               (int64_t)nsplit, H, 1, nsplit, out, nullptr, 0, 0, nullptr, 0);                                    \
            HA_CHECK_LAUNCH("merge_splits_kernel");                                                                               \
        }                                                                                                                         \
    } while (0)
#define HA_FUSED_LAUNCH(E_, U_, FW_)                                          \
    do {                                                                      \
        if (smap.slots) HA_FUSED_LAUNCH_SL(E_, U_, FW_, true, false);         \
        else if (masked_prefix) HA_FUSED_LAUNCH_SL(E_, U_, FW_, false, true); \
        else HA_FUSED_LAUNCH_SL(E_, U_, FW_, false, false);                   \
    } while (0)
    if (W == 1) {
        if (kv_dtype == HA_BF16) HA_FUSED_LAUNCH(ElemBF16, 4, 1);
        else if (kv_dtype == HA_F16) HA_FUSED_LAUNCH(ElemF16, 4, 1);
        else HA_FUSED_LAUNCH(ElemF32, 2, 1);
    } else {
        if (kv_dtype == HA_BF16) HA_FUSED_LAUNCH(ElemBF16, 4, 2);
        else if (kv_dtype == HA_F16) HA_FUSED_LAUNCH(ElemF16, 4, 2);
        else HA_FUSED_LAUNCH(ElemF32, 2, 2);
    }
#undef HA_FUSED_LAUNCH
#undef HA_FUSED_LAUNCH_SL
    return HA_OK;
}

int ha_sparse_decode_fused(const void *q, int64_t q_stride_b, int64_t q_stride_h, const void *k, const void *v, int kv_dtype,
                           int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, const uint32_t *kcodes, int64_t kc_stride_b,
                           int64_t kc_stride_h, const uint32_t *qcodes, int B, int H, int Hkv, int Hc, int W, int max_seq_len,
                           const int32_t *seq_lens, int init_budget, int recent_budget, double heavy_budget,
                           const void *select_workspace, size_t select_workspace_bytes, int thresholds_ready, int32_t *out_counts,
                           float sm_scale, void *out, void *workspace, size_t workspace_bytes, void *stream) {
    return sparse_decode_fused_impl(q, q_stride_b, q_stride_h, k, v, kv_dtype, kv_stride_b, kv_stride_h, kv_stride_s, kcodes, kc_stride_b,
                                    kc_stride_h, qcodes, B, H, Hkv, Hc, W, max_seq_len, seq_lens, init_budget, recent_budget, heavy_budget,
                                    select_workspace, select_workspace_bytes, thresholds_ready, out_counts, sm_scale, out, workspace,
                                    workspace_bytes, stream, SlotMap{});
}

int ha_sparse_decode_fused_prefix_masked(const void *q, int64_t q_stride_b, int64_t q_stride_h, const void *k, const void *v, int kv_dtype,
                                         int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, const uint32_t *kcodes,
                                         int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes, int B, int H, int Hkv, int Hc,
                                         int W, int max_seq_len, const int32_t *seq_lens, int init_budget, int recent_budget,
                                         double heavy_budget, const void *select_workspace, size_t select_workspace_bytes,
                                         int thresholds_ready, int32_t *out_counts, const int32_t *masked_prefix, float sm_scale,
                                         void *out, void *workspace, size_t workspace_bytes, void *stream) {
    HA_REQUIRE(masked_prefix, HA_ERR_NULL_POINTER, "masked_prefix is NULL");
    HA_REQUIRE(ha_aligned(masked_prefix, 4), HA_ERR_MISALIGNED, "masked_prefix misaligned");
    return sparse_decode_fused_impl(q, q_stride_b, q_stride_h, k, v, kv_dtype, kv_stride_b, kv_stride_h, kv_stride_s, kcodes, kc_stride_b,
                                    kc_stride_h, qcodes, B, H, Hkv, Hc, W, max_seq_len, seq_lens, init_budget, recent_budget, heavy_budget,
                                    select_workspace, select_workspace_bytes, thresholds_ready, out_counts, sm_scale, out, workspace,
                                    workspace_bytes, stream, SlotMap{}, masked_prefix);
}

static int validate_slot_map(const int32_t *slot_of_token, int64_t slot_stride_b, int64_t n_slots) {
    HA_REQUIRE(slot_of_token, HA_ERR_NULL_POINTER, "slot_of_token is NULL");
    HA_REQUIRE(slot_stride_b >= 0, HA_ERR_BAD_SHAPE, "slot_stride_b must not be negative");
    HA_REQUIRE(n_slots > 0 && n_slots <= 2147483647LL, HA_ERR_BAD_SHAPE, "n_slots=%lld, must be in 1..2^31-1", (long long)n_slots);
    HA_REQUIRE(ha_aligned(slot_of_token, 4), HA_ERR_MISALIGNED, "slot_of_token misaligned");
    return HA_OK;
}

int ha_sparse_decode_paged(const void *q, int64_t q_stride_b, int64_t q_stride_h, const void *k, const void *v, int kv_dtype,
                           int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, int B, int rows_per_sequence, int H, int Hkv,
                           const int32_t *idx, int64_t idx_cap, const int32_t *counts, float sm_scale, const float *mask,
                           int64_t mask_stride_b, int mask_len, int mask_by_slot, const int32_t *slot_of_token, int64_t slot_stride_b,
                           int64_t n_slots, void *out, void *workspace, size_t workspace_bytes, void *stream) {
    int st = validate_slot_map(slot_of_token, slot_stride_b, n_slots);
    if (st) return st;
    if (mask) {
        HA_REQUIRE(mask_len > 0 && mask_stride_b >= 0, HA_ERR_BAD_SHAPE, "mask_len must be positive and mask_stride_b non-negative");
        HA_REQUIRE(mask_by_slot == 0 || mask_by_slot == 1, HA_ERR_BAD_SHAPE, "mask_by_slot must be 0 or 1");
        HA_REQUIRE(!mask_by_slot || mask_len >= idx_cap, HA_ERR_BAD_SHAPE, "a mask by list slot needs idx_cap=%lld values per row, got %d",
                   (long long)idx_cap, mask_len);
        HA_REQUIRE(ha_aligned(mask, 4), HA_ERR_MISALIGNED, "mask misaligned");
    }
    return sparse_decode_impl(q, q_stride_b, q_stride_h, k, v, kv_dtype, kv_stride_b, kv_stride_h, kv_stride_s, B, H, Hkv, idx, idx_cap,
                              counts, sm_scale, out, workspace, workspace_bytes, nullptr, 0, 0, nullptr, 0,
                              mask ? AttnMask{mask, mask_stride_b, mask_len, mask_by_slot} : AttnMask{}, stream, rows_per_sequence,
                              SlotMap{slot_of_token, slot_stride_b, (int)(n_slots - 1)});
}

int ha_sparse_decode_fused_paged(const void *q, int64_t q_stride_b, int64_t q_stride_h, const void *k, const void *v, int kv_dtype,
                                 int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, const uint32_t *kcodes,
                                 int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes, int B, int H, int Hkv, int Hc, int W,
                                 int max_seq_len, const int32_t *seq_lens, int init_budget, int recent_budget, double heavy_budget,
                                 const void *select_workspace, size_t select_workspace_bytes, int thresholds_ready,
                                 int32_t *out_counts, const int32_t *slot_of_token, int64_t slot_stride_b, int64_t n_slots,
                                 float sm_scale, void *out, void *workspace, size_t workspace_bytes, void *stream) {
    int st = validate_slot_map(slot_of_token, slot_stride_b, n_slots);
    if (st) return st;
    return sparse_decode_fused_impl(q, q_stride_b, q_stride_h, k, v, kv_dtype, kv_stride_b, kv_stride_h, kv_stride_s, kcodes, kc_stride_b,
                                    kc_stride_h, qcodes, B, H, Hkv, Hc, W, max_seq_len, seq_lens, init_budget, recent_budget, heavy_budget,
                                    select_workspace, select_workspace_bytes, thresholds_ready, out_counts, sm_scale, out, workspace,
                                    workspace_bytes, stream, SlotMap{slot_of_token, slot_stride_b, (int)(n_slots - 1)});
}

size_t ha_window_partial_bytes(int B, int H) {
    if (B <= 0 || H <= 0) return 0;
    return (size_t)B * H * (HA_HEAD_DIM + 2) * sizeof(float);
}

int ha_window_partial(const void *q, int64_t q_stride_b, int64_t q_stride_h, const void *k, const void *v, int kv_dtype,
                      int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, int B, int H, int Hkv, int max_seq_len,
                      const int32_t *seq_lens, int init_budget, int recent_budget, float sm_scale, float *window_partial,
                      void *stream) {
    HA_REQUIRE(window_partial, HA_ERR_NULL_POINTER, "window_partial is NULL");
    int st = validate_qkv(q, q_stride_b, q_stride_h, k, v, kv_dtype, kv_stride_b, kv_stride_h, kv_stride_s, B, H, Hkv, window_partial);
    if (st) return st;
    HA_REQUIRE(init_budget >= 0 && recent_budget >= 0 && max_seq_len > 0, HA_ERR_BAD_SHAPE, "bad window budgets or max_seq_len");
    const int group = H / Hkv;
    const int G = dense_slots(group);
    HA_REQUIRE((int64_t)Hkv * ((group + G - 1) / G) <= 65535, HA_ERR_BAD_SHAPE, "too many heads");
    if ((st = ha_require_device())) return st;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(1, Hkv * ((group + G - 1) / G), B);
    const float sl2 = sm_scale * kLog2e;
#define HA_WIN_LAUNCH(E_, G_)                                                                                                      \
    do {                                                                                                                           \
        hipLaunchKernelGGL((dense_attend_kernel<E_, G_, true>), grid, dim3(kAttThreads), 0, s, q, q_stride_b, q_stride_h, k, v,    \
                           kv_stride_b, kv_stride_h, kv_stride_s, H, group, max_seq_len, seq_lens, sl2, 0, 1, window_partial,      \
                           (float *)nullptr, (void *)nullptr, init_budget, recent_budget);                                         \
        HA_CHECK_LAUNCH("dense_attend_kernel<window>");                                                                            \
    } while (0)
#define HA_WIN_DISPATCH(E_)                    \
    do {                                       \
        if (G == 1) HA_WIN_LAUNCH(E_, 1);      \
        else if (G == 2) HA_WIN_LAUNCH(E_, 2); \
        else if (G == 4) HA_WIN_LAUNCH(E_, 4); \
        else HA_WIN_LAUNCH(E_, 8);             \
    } while (0)
    if (kv_dtype == HA_BF16) HA_WIN_DISPATCH(ElemBF16);
    else if (kv_dtype == HA_F16) HA_WIN_DISPATCH(ElemF16);
    else HA_WIN_DISPATCH(ElemF32);
#undef HA_WIN_DISPATCH
#undef HA_WIN_LAUNCH
    return HA_OK;
}

size_t ha_dense_decode_workspace_bytes(int B, int H, int max_seq_len) {
    if (B <= 0 || H <= 0 || max_seq_len <= 0) return 0;
    // the plan depends on Hkv only through the workgroup count; size for the worst case over Hkv
    int worst = 1;
    for (int hkv = 1; hkv <= H; hkv *= 2) {
        const int ns = dense_plan(B, hkv, max_seq_len).nsplit_max;
        if (ns > worst) worst = ns;
    }
    return part_bytes((int64_t)B * H, worst);
}

int ha_dense_decode(const void *q, int64_t q_stride_b, int64_t q_stride_h, const void *k, const void *v, int kv_dtype,
                    int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, int B, int H, int Hkv, int max_seq_len,
                    const int32_t *seq_lens, float sm_scale, void *out, void *workspace, size_t workspace_bytes, void *stream) {
    int st = validate_qkv(q, q_stride_b, q_stride_h, k, v, kv_dtype, kv_stride_b, kv_stride_h, kv_stride_s, B, H, Hkv, out);
    if (st) return st;
    HA_REQUIRE(max_seq_len > 0, HA_ERR_BAD_SHAPE, "max_seq_len must be positive");
    const int group = H / Hkv;
    const int G = dense_slots(group), passes = (group + G - 1) / G;
    HA_REQUIRE((int64_t)Hkv * passes <= 65535, HA_ERR_BAD_SHAPE, "too many heads");
    const DensePlan plan = dense_plan(B, Hkv, max_seq_len);
    const size_t need = part_bytes((int64_t)B * H, plan.nsplit_max);
    HA_REQUIRE(workspace && workspace_bytes >= need, HA_ERR_WORKSPACE, "dense decode workspace: need %zu bytes, got %zu", need,
               workspace ? workspace_bytes : (size_t)0);
    HA_REQUIRE(ha_aligned(workspace, 256), HA_ERR_MISALIGNED, "workspace must be 256-byte aligned");
    if ((st = ha_require_device())) return st;

    const int64_t rows = (int64_t)B * H;
    float *part_acc = (float *)workspace;
    float *part_ml = part_acc + rows * plan.nsplit_max * HA_HEAD_DIM;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(plan.nsplit_max, Hkv * passes, B), mgrid(H, B);
    const float sl2 = sm_scale * kLog2e;
#define HA_DENSE_LAUNCH(E_, G_)                                                                                                    \
    do {                                                                                                                           \
        hipLaunchKernelGGL((dense_attend_kernel<E_, G_, false>), grid, dim3(kAttThreads), 0, s, q, q_stride_b, q_stride_h, k, v,   \
                           kv_stride_b, kv_stride_h, kv_stride_s, H, group, max_seq_len, seq_lens, sl2, plan.chunk,                \
                           plan.nsplit_max, part_acc, part_ml, out, 0, 0);                                                         \
        HA_CHECK_LAUNCH("dense_attend_kernel");                                                                                    \
        if (plan.nsplit_max > 1) {                                                                                                 \
            hipLaunchKernelGGL(merge_splits_kernel<E_>, mgrid, dim3(HA_HEAD_DIM), 0, s, part_acc, part_ml, seq_lens, 1,            \
                               (int64_t)max_seq_len, H, plan.chunk, plan.nsplit_max, out, (const float *)nullptr, 0, 0,            \
                               (const int32_t *)nullptr, 0);                                                                       \
            HA_CHECK_LAUNCH("merge_splits_kernel");                                                                                \
        }                                                                                                                          \
    } while (0)
#define HA_DENSE_DISPATCH(E_)                    \
    do {                                         \
        if (G == 1) HA_DENSE_LAUNCH(E_, 1);      \
        else if (G == 2) HA_DENSE_LAUNCH(E_, 2); \
        else if (G == 4) HA_DENSE_LAUNCH(E_, 4); \
        else HA_DENSE_LAUNCH(E_, 8);             \
    } while (0)
    if (kv_dtype == HA_BF16) HA_DENSE_DISPATCH(ElemBF16);
    else if (kv_dtype == HA_F16) HA_DENSE_DISPATCH(ElemF16);
    else HA_DENSE_DISPATCH(ElemF32);
#undef HA_DENSE_DISPATCH
#undef HA_DENSE_LAUNCH
    return HA_OK;
}

}  // extern "C"
