// Hamming scoring and heavy-token selection over the packed code cache (gfx950, wave64).
//
// Selection never sorts.  Distances take only NL = 32*W + 1 values, so the k-th smallest distance
// T of a row follows from a histogram, and "the k nearest, lowest index first" is
//     { j : d_j < T }  union  the first r = k - #{d < T} tokens with d_j == T in index order.
// Three launches per call:
//   1. select_hist_kernel       grid (chunk, code head, sequence): per-chunk histograms of the distances
//                               of every query head of the group, one streaming pass over the codes
//   2. select_threshold_kernel  grid (head, sequence): T, r, per-chunk output offsets, window indices, counts
//   3. select_compact_kernel    grid as 1: ordered compaction (bit masks + one DPP scan) into ascending index lists
// Pass 3 re-reads the codes (4*W bytes per token) from L2 / Infinity Cache.
//
// Both streaming kernels fetch all codes of their chunk before using any (128-bit loads, up to 16 codes
// per lane), so a workgroup has its whole chunk in flight at once instead of paying one memory round
// trip per tile.
#include <mutex>

#include "ha_select_common.h"

using namespace ha_sel;

// Scratch of ha_select_static: the selection's workspace (chunk histograms, row meta, chunk prefixes) for callers that
// cannot allocate.  Every GPU the library runs on holds its own copy at its own address until the process ends.  In host
// code the name `scratch` is only a handle: the array's device address on the current GPU comes from
// hipGetSymbolAddress (static_scratch below, once per device), and that pointer is what the kernels are given.  Nothing
// in it has to start at zero: the histogram launch writes every counter of every (row, chunk) it is launched for, the
// threshold launch every meta and prefix entry, before the next launch reads them.  Calls that overlap in time on one
// GPU (two streams, two threads) would share the array and race.
constexpr size_t kStaticScratchBytes = (size_t)8 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

// ------------------------------------------------------------------------------------------------
template <int W>
__global__ __launch_bounds__(256) void hamming_score_kernel(const uint32_t *__restrict__ kcodes, int64_t kc_sb, int64_t kc_sh,
                                                            const uint32_t *__restrict__ qcodes, int H, int Hc, int max_S,
                                                            const int32_t *__restrict__ seq_lens, uint8_t *__restrict__ scores) {
    const int b = blockIdx.z, h = blockIdx.y;
    const int S = seq_lens ? seq_lens[b] : max_S;
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= S || j >= max_S) return;
    const Code<W> q = load_qcode<W>(qcodes, (int64_t)b * H + h);
    const uint32_t *kc = kcodes + b * kc_sb + (h / (H / Hc)) * kc_sh;
    scores[((int64_t)b * H + h) * max_S + j] = (uint8_t)load_code<W>(kc, j).dist(q);
}

// Workgroups go to the 8 XCDs round-robin in launch order.  Walking a grid (chunk, code head, sequence) code head fastest
// puts every chunk of a (sequence, code head) row on XCD = code head % 8 when the code heads come in multiples of 8:
// with 8 code heads that is the XCD on which the attention launch places the query heads of the KV group, so the codes
// a later pass or launch scans again are already in that L2 (whole step at B = 16, 64K tokens: 120.4 -> 118.9 us).
__device__ __forceinline__ void walk_code_head_fastest(int &c, int &hc, int &b) {
    c = blockIdx.x, hc = blockIdx.y, b = blockIdx.z;
    if (gridDim.y % 8 == 0) {
        const int lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
        hc = lin % (int)gridDim.y;
        c = (lin / (int)gridDim.y) % (int)gridDim.x;
        b = lin / (int)(gridDim.y * gridDim.x);
    }
}

// ------------------------------------------------------------------------------------------------
// Pass 1.  grid (nchunk, Hc, B).  hist[b, h, chunk, level] = #candidates of the chunk at that distance.
// The LDS histogram is replicated REP times (replica = lane % REP, which is also the bank) so that the
// few hot levels of a binomial-like distance distribution do not serialise the ds_add.
template <int W, int GQ, int REP>
__global__ __launch_bounds__(kSelThreads) void select_hist_kernel(const uint32_t *__restrict__ kcodes, int64_t kc_sb, int64_t kc_sh,
                                                                  const uint32_t *__restrict__ qcodes, int H, int max_S,
                                                                  const int32_t *__restrict__ seq_lens, int init, int recent,
                                                                  int blocks, int nchunk, int vec, uint32_t *__restrict__ hist,
                                                                  int rows_per_seq) {
    constexpr int NL = 32 * W + 1;
    __shared__ uint32_t lh[GQ * NL * REP];
    int c, hc, b;
    walk_code_head_fastest(c, hc, b);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int S = seq_lens ? seq_lens[b] : max_S;
    if (S > max_S) S = max_S;
    const int lo = init < S ? init : S;
    const int hi = (S - recent > lo) ? S - recent : lo;
    const int chunk = blocks * kBlock;
    const int beg = max(lo, c * chunk), end = min(hi, (c + 1) * chunk);

    ChunkRegs<W> cr;
    // rows_per_seq consecutive batch entries are queries against the codes of one sequence (the rows of a chunk of tokens)
    if (beg < end)
        load_chunk<W>(kcodes + (b / rows_per_seq) * kc_sb + hc * kc_sh, c * chunk, blocks, beg, end, vec != 0, wave, lane, cr);
    for (int i = tid; i < GQ * NL * REP; i += kSelThreads) lh[i] = 0;
    __syncthreads();

    if (beg < end) {
        Code<W> q[GQ];
#pragma unroll
        for (int g = 0; g < GQ; ++g) q[g] = load_qcode<W>(qcodes, (int64_t)b * H + hc * GQ + g);
        const int rep = tid % REP;
        const bool whole = beg == c * chunk && end == (c + 1) * chunk;  // uniform: every code of the chunk is a candidate
#pragma unroll
        for (int blk = 0; blk < kMaxBlocks; ++blk) {
            if (blk >= blocks) break;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int j = cr.j0[blk] + e;
                if (whole || (j >= beg && j < end)) {
#pragma unroll
                    for (int g = 0; g < GQ; ++g) atomicAdd(&lh[(g * NL + cr.k[blk][e].dist(q[g])) * REP + rep], 1u);
                }
            }
        }
    }
    __syncthreads();
    for (int p = tid; p < GQ * NL; p += kSelThreads) {
        uint32_t s = 0;
#pragma unroll 8
        for (int r = 0; r < REP; ++r) s += lh[p * REP + ((r + tid) % REP)];
        const int g = p / NL, l = p % NL;
        hist[(((int64_t)b * H + hc * GQ + g) * nchunk + c) * NL + l] = s;
    }
}

// ------------------------------------------------------------------------------------------------
// Pass 2.  grid (H, B), 256 threads.  meta[row] = {T, r, n_heavy, #tokens with d == T}; chunk_pre[row][c] = {#selected with
// d < T in chunks before c, #tokens with d == T in chunks before c}.  Also writes the sink and recent
// window indices and the row's count.
template <int W>
__global__ __launch_bounds__(kSelThreads) void select_threshold_kernel(const uint32_t *__restrict__ hist, int H, int max_S,
                                                                       const int32_t *__restrict__ seq_lens, int init, int recent,
                                                                       double heavy_budget, int mode, int depth, int nchunk,
                                                                       int32_t *__restrict__ meta, int32_t *__restrict__ chunk_pre,
                                                                       int32_t *__restrict__ out_idx, int64_t idx_cap,
                                                                       int32_t *__restrict__ out_counts) {
    constexpr int NL = 32 * W + 1;
    constexpr int TC = 32;  // chunks per LDS tile
    __shared__ uint32_t s_tile[TC * NL];
    __shared__ uint32_t s_tot[NL];
    __shared__ int s_T, s_nheavy, s_carry_lt, s_carry_eq;

    const int h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const int64_t row = (int64_t)b * H + h;
    int S = seq_lens ? seq_lens[b] : max_S;
    if (S > max_S) S = max_S;
    const RowBudget rb = row_budget(S, init, recent, heavy_budget);
    const uint32_t *hp = hist + row * nchunk * NL;

    if (tid < NL) s_tot[tid] = 0;
    for (int c0 = 0; c0 < nchunk; c0 += TC) {
        const int n = min(TC, nchunk - c0) * NL;
        __syncthreads();
        for (int i = tid; i < n; i += kSelThreads) s_tile[i] = hp[(int64_t)c0 * NL + i];
        __syncthreads();
        if (tid < NL) {
            uint32_t s = 0;
            for (int cc = 0; cc * NL < n; ++cc) s += s_tile[cc * NL + tid];
            s_tot[tid] += s;
        }
    }
    __syncthreads();
    if (tid == 0) {
        int T, r, nheavy;
        solve_threshold(s_tot, NL - 1, NL, rb.kk, mode, depth, T, r, nheavy);
        s_T = T;
        s_nheavy = nheavy;
        s_carry_lt = 0;
        s_carry_eq = 0;
        meta[row * 4 + 0] = T;
        meta[row * 4 + 1] = r;
        meta[row * 4 + 2] = nheavy;
        meta[row * 4 + 3] = (T >= 0 && T < NL) ? (int)s_tot[T] : 0;  // size of the tie bucket
    }
    __syncthreads();
    const int T = s_T, nheavy = s_nheavy;

    // exclusive prefix over chunks of (#d < T, #d == T); wave 0 scans a tile of 32 chunks at a time
    for (int c0 = 0; c0 < nchunk; c0 += TC) {
        const int nc = min(TC, nchunk - c0);
        __syncthreads();
        for (int i = tid; i < nc * NL; i += kSelThreads) s_tile[i] = hp[(int64_t)c0 * NL + i];
        __syncthreads();
        if (tid < HA_WAVE) {
            int a = 0, e = 0;
            if (tid < nc) {
                for (int l = 0; l < T && l < NL; ++l) a += (int)s_tile[tid * NL + l];
                if (T < NL) e = (int)s_tile[tid * NL + T];
            }
            int ia = a, ie = e;  // inclusive scan over lanes 0..31
#pragma unroll
            for (int off = 1; off < TC; off <<= 1) {
                const int ta = __shfl_up(ia, off), te = __shfl_up(ie, off);
                if (tid >= off) {
                    ia += ta;
                    ie += te;
                }
            }
            const int base_lt = s_carry_lt, base_eq = s_carry_eq;
            if (tid < nc) {
                chunk_pre[(row * nchunk + c0 + tid) * 2 + 0] = base_lt + ia - a;
                chunk_pre[(row * nchunk + c0 + tid) * 2 + 1] = base_eq + ie - e;
            }
            if (tid == nc - 1) {
                s_carry_lt = base_lt + ia;
                s_carry_eq = base_eq + ie;
            }
        }
    }

    // windows and count
    int32_t *o = out_idx + row * idx_cap;
    const int n_recent = rb.S - rb.hi;
    const int64_t rbase = (int64_t)rb.lo + nheavy;
    if (out_idx) {
        for (int i = tid; i < rb.lo; i += kSelThreads)
            if (i < idx_cap) o[i] = i;
        for (int i = tid; i < n_recent; i += kSelThreads)
            if (rbase + i < idx_cap) o[rbase + i] = rb.hi + i;
    }
    if (tid == 0) out_counts[row] = (int32_t)(rbase + n_recent);
}

// ------------------------------------------------------------------------------------------------
// Pass 3.  grid (nchunk, Hc, B).  A wave owns a contiguous quarter of the chunk and a lane 4*blocks
// consecutive codes of it, so "wave, lane, element" is ascending token order.  Per head a lane turns its
// codes into two bit masks (d < T, d == T); one packed DPP scan gives every lane the number of such tokens
// before it, and only the set bits are visited when the indices are written.
template <int W, int GQ>
__global__ __launch_bounds__(kSelThreads) void select_compact_kernel(const uint32_t *__restrict__ kcodes, int64_t kc_sb, int64_t kc_sh,
                                                                     const uint32_t *__restrict__ qcodes, int H, int max_S,
                                                                     const int32_t *__restrict__ seq_lens, int init, int recent,
                                                                     int blocks, int nchunk, int vec, const int32_t *__restrict__ meta,
                                                                     const int32_t *__restrict__ chunk_pre,
                                                                     int32_t *__restrict__ out_idx, int64_t idx_cap, int rows_per_seq) {
    constexpr int CPL = 4 * kMaxBlocks;  // codes per lane at most
    __shared__ uint32_t s_wtot[kSelWaves][GQ];

    int c, hc, b;
    walk_code_head_fastest(c, hc, b);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int S = seq_lens ? seq_lens[b] : max_S;
    if (S > max_S) S = max_S;
    const int lo = init < S ? init : S;
    const int hi = (S - recent > lo) ? S - recent : lo;
    const int chunk = blocks * kBlock;
    const int beg = max(lo, c * chunk), end = min(hi, (c + 1) * chunk);
    if (beg >= end) return;  // uniform over the workgroup

    const int cpl = 4 * blocks;
    const int j_lane = c * chunk + (wave * HA_WAVE + lane) * cpl;
    const uint32_t *kc = kcodes + (b / rows_per_seq) * kc_sb + hc * kc_sh;
    Code<W> k[CPL];
    uint32_t vmask;  // bit e: code j_lane + e is a candidate of this chunk
    if (vec && blocks == kMaxBlocks && beg == c * chunk && end == (c + 1) * chunk) {
        // the common case, uniform over the workgroup: a full chunk strictly inside the candidate range of a
        // 16-byte aligned row
#pragma unroll
        for (int i = 0; i < kMaxBlocks; ++i) {
            Code<W> k4[4];
            load_code4<W>(kc, j_lane + 4 * i, beg, end, true, k4);
#pragma unroll
            for (int e = 0; e < 4; ++e) k[4 * i + e] = k4[e];
        }
        vmask = 0xFFFFu;
    } else {
        vmask = 0;
#pragma unroll
        for (int i = 0; i < kMaxBlocks; ++i) {
            const int j0 = j_lane + 4 * i;
            const bool live = i < blocks && j0 + 4 > beg && j0 < end;
            Code<W> k4[4];
            if (live) load_code4<W>(kc, j0, beg, end, vec != 0, k4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (live) k[4 * i + e] = k4[e];
                else if constexpr (W == 1) k[4 * i + e] = Code<1>{0u};
                else k[4 * i + e] = Code<2>{0u, 0u};
                if (live && j0 + e >= beg && j0 + e < end) vmask |= 1u << (4 * i + e);
            }
        }
    }

    Code<W> q[GQ];
    int T[GQ], r[GQ], lt_pre[GQ], eq_pre[GQ];
    bool any = false;
#pragma unroll
    for (int g = 0; g < GQ; ++g) {
        const int64_t row = (int64_t)b * H + hc * GQ + g;
        q[g] = load_qcode<W>(qcodes, row);
        T[g] = meta[row * 4 + 0];
        r[g] = meta[row * 4 + 1];
        any = any || meta[row * 4 + 2] > 0;
        lt_pre[g] = chunk_pre[(row * nchunk + c) * 2 + 0];
        eq_pre[g] = chunk_pre[(row * nchunk + c) * 2 + 1];
    }
    if (!any) return;  // uniform: nothing heavy to write for this group

    uint32_t ltm[GQ], eqm[GQ], incl[GQ];
#pragma unroll
    for (int g = 0; g < GQ; ++g) {
        // sign bit of (d - T) is "d < T", of (d - T - 1) is "d <= T"; v_alignbit shifts each into its mask.
        // Elements are visited from the last to the first so that element e lands on bit e.
        uint32_t lt = 0, le = 0;
        const int neg_t = -T[g];
#pragma unroll
        for (int e = CPL - 1; e >= 0; --e) {
            const int key = k[e].dist(q[g]) + neg_t;
            lt = __builtin_amdgcn_alignbit(lt, (uint32_t)key, 31);
            le = __builtin_amdgcn_alignbit(le, (uint32_t)(key - 1), 31);
        }
        const uint32_t eq = le & ~lt;
        ltm[g] = lt & vmask;
        eqm[g] = eq & vmask;
        incl[g] = wave_inclusive_scan((uint32_t)__popc(ltm[g]) | ((uint32_t)__popc(eqm[g]) << 16));
        if (lane == HA_WAVE - 1) s_wtot[wave][g] = incl[g];
    }
    __syncthreads();

#pragma unroll
    for (int g = 0; g < GQ; ++g) {
        const uint32_t excl = incl[g] - ((uint32_t)__popc(ltm[g]) | ((uint32_t)__popc(eqm[g]) << 16));
        int n_lt = lt_pre[g] + (int)(excl & 0xFFFFu), n_eq = eq_pre[g] + (int)(excl >> 16);
        for (int w = 0; w < wave; ++w) {
            const uint32_t t = s_wtot[w][g];
            n_lt += (int)(t & 0xFFFFu);
            n_eq += (int)(t >> 16);
        }
        const int rg = r[g];
        int32_t *o = out_idx + ((int64_t)b * H + hc * GQ + g) * idx_cap;
        const uint32_t em = n_eq < rg ? eqm[g] : 0u;  // past the r-th tie nothing more of the tie bucket is taken
        uint32_t todo = ltm[g] | em;
        while (todo) {
            const int e = __ffs((int)todo) - 1;
            todo &= todo - 1;
            const bool is_eq = (em >> e) & 1u;
            if (!is_eq || n_eq < rg) {
                const uint32_t pos = (uint32_t)(lo + n_lt + min(n_eq, rg));  // < S: fits 32 bits, uniform base `o`
                if ((int64_t)pos < idx_cap) o[pos] = j_lane + e;
            }
            n_lt += is_eq ? 0 : 1;
            n_eq += is_eq ? 1 : 0;
        }
    }
}

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

// Address of `scratch` on the current device (resolved at the first call on that device).
int static_scratch(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) HA_FAIL(HA_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(e));
    HA_REQUIRE(dev >= 0 && dev < kMaxDevices, HA_ERR_NO_DEVICE, "device ordinal %d outside 0..%d", dev, kMaxDevices - 1);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) HA_FAIL(HA_ERR_HIP, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return HA_OK;
}

// ------------------------------------------------------------------------------------------------
int validate_codes(const uint32_t *kcodes, int64_t kc_sb, int64_t kc_sh, const uint32_t *qcodes, int B, int H, int Hc, int W,
                   int max_seq_len, bool any_group = false) {
    HA_REQUIRE(kcodes && qcodes, HA_ERR_NULL_POINTER, "kcodes/qcodes is NULL");
    HA_REQUIRE(B > 0 && H > 0 && Hc > 0 && max_seq_len > 0, HA_ERR_BAD_SHAPE, "B, H, Hc, max_seq_len must be positive");
    HA_REQUIRE(B <= 65535 && H <= 65535, HA_ERR_BAD_SHAPE, "B and H are limited to 65535");
    HA_REQUIRE(W == 1 || W == 2, HA_ERR_BAD_SHAPE, "code words W=%d, must be 1 or 2", W);
    HA_REQUIRE(H % Hc == 0, HA_ERR_BAD_SHAPE, "H=%d not a multiple of Hc=%d", H, Hc);
    const int gq = H / Hc;
    HA_REQUIRE(any_group || gq == 1 || gq == 2 || gq == 4 || gq == 8, HA_ERR_BAD_SHAPE, "H/Hc=%d, must be 1, 2, 4 or 8", gq);
    HA_REQUIRE(kc_sh >= (int64_t)max_seq_len * W && (kc_sb >= kc_sh || kc_sb == 0), HA_ERR_BAD_SHAPE,
               "code strides smaller than the rows they span");
    HA_REQUIRE((int64_t)max_seq_len <= (int64_t)kMaxChunks * kMaxBlocks * kBlock, HA_ERR_BAD_SHAPE, "max_seq_len above %d",
               kMaxChunks * kMaxBlocks * kBlock);
    HA_REQUIRE(ha_aligned(kcodes, 4 * W) && ha_aligned(qcodes, 4) && (W == 1 || (kc_sb % 2 == 0 && kc_sh % 2 == 0)),
               HA_ERR_MISALIGNED, "codes must be aligned to their word count");
    return HA_OK;
}

}  // namespace

extern "C" {

int ha_hamming_score(const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes, int B, int H,
                     int Hc, int W, int max_seq_len, const int32_t *seq_lens, uint8_t *scores, void *stream) {
    int st = validate_codes(kcodes, kc_stride_b, kc_stride_h, qcodes, B, H, Hc, W, max_seq_len, true);
    if (st) return st;
    HA_REQUIRE(scores, HA_ERR_NULL_POINTER, "scores is NULL");
    if ((st = ha_require_device())) return st;
    dim3 grid((max_seq_len + 255) / 256, H, B);
    if (W == 1)
        hipLaunchKernelGGL(hamming_score_kernel<1>, grid, dim3(256), 0, (hipStream_t)stream, kcodes, kc_stride_b, kc_stride_h, qcodes, H,
                           Hc, max_seq_len, seq_lens, scores);
    else
        hipLaunchKernelGGL(hamming_score_kernel<2>, grid, dim3(256), 0, (hipStream_t)stream, kcodes, kc_stride_b, kc_stride_h, qcodes, H,
                           Hc, max_seq_len, seq_lens, scores);
    HA_CHECK_LAUNCH("hamming_score_kernel");
    return HA_OK;
}

size_t ha_select_workspace_bytes(int B, int H, int Hc, int W, int max_seq_len) {
    if (B <= 0 || H <= 0 || Hc <= 0 || max_seq_len <= 0 || (W != 1 && W != 2)) return 0;
    const SelectPlan p = select_plan(B, Hc, max_seq_len);
    // large enough for either algorithm
    const size_t exact = carve_select_ws(nullptr, (int64_t)B * H, p.nchunk, W).bytes;
    const size_t sampled = sampled_workspace_bytes((int64_t)B * H, p.nchunk, p.blocks);
    return exact > sampled ? exact : sampled;
}

#define HA_SELECT_LAUNCH(W_, GQ_, REP_)                                                                                           \
    do {                                                                                                                          \
        hipLaunchKernelGGL((select_hist_kernel<W_, GQ_, REP_>), grid, dim3(kSelThreads), 0, s, kcodes, kc_stride_b, kc_stride_h,  \
                           qcodes, H, max_seq_len, seq_lens, init_budget, recent_budget, plan.blocks, plan.nchunk, vec, ws.hist,   \
                           rows_per_seq);                                                                                         \
        HA_CHECK_LAUNCH("select_hist_kernel");                                                                                    \
        if (!out_counts) break; /* ha_select_histogram: chunk histograms only */                                                  \
        hipLaunchKernelGGL(select_threshold_kernel<W_>, dim3(H, B), dim3(kSelThreads), 0, s, ws.hist, H, max_seq_len, seq_lens,   \
                           init_budget, recent_budget, heavy_budget, mode, depth, plan.nchunk, ws.meta, ws.chunk_pre, out_idx,    \
                           idx_cap, out_counts);                                                                                  \
        HA_CHECK_LAUNCH("select_threshold_kernel");                                                                               \
        if (!out_idx) break; /* ha_select_prepare: thresholds and offsets only */                                                 \
        hipLaunchKernelGGL((select_compact_kernel<W_, GQ_>), grid, dim3(kSelThreads), 0, s, kcodes, kc_stride_b, kc_stride_h,     \
                           qcodes, H, max_seq_len, seq_lens, init_budget, recent_budget, plan.blocks, plan.nchunk, vec, ws.meta,  \
                           ws.chunk_pre, out_idx, idx_cap, rows_per_seq);                                                         \
        HA_CHECK_LAUNCH("select_compact_kernel");                                                                                 \
    } while (0)

static int select_impl(const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes, int B, int H, int Hc,
                       int W, int max_seq_len, const int32_t *seq_lens, int init_budget, int recent_budget, double heavy_budget,
                       int mode, int depth, int algo, int32_t *out_idx, int64_t idx_cap, int32_t *out_counts, void *workspace,
                       size_t workspace_bytes, void *stream, bool prepare_only, bool use_static_scratch = false,
                       int rows_per_seq = 1) {
    int st = validate_codes(kcodes, kc_stride_b, kc_stride_h, qcodes, B, H, Hc, W, max_seq_len);
    if (st) return st;
    HA_REQUIRE(rows_per_seq >= 1 && B % rows_per_seq == 0, HA_ERR_BAD_SHAPE, "rows_per_sequence=%d must divide the %d batch entries",
               rows_per_seq, B);
    HA_REQUIRE(rows_per_seq == 1 || algo == HA_SELECT_ALGO_AUTO || algo == HA_SELECT_ALGO_HISTOGRAM, HA_ERR_BAD_SHAPE,
               "several rows per sequence take the histogram method");
    if (rows_per_seq > 1) algo = HA_SELECT_ALGO_HISTOGRAM;
    HA_REQUIRE(prepare_only || (out_idx && out_counts), HA_ERR_NULL_POINTER, "out_idx/out_counts is NULL");
    HA_REQUIRE(init_budget >= 0 && recent_budget >= 0 && heavy_budget >= 0.0 && depth >= 0, HA_ERR_BAD_SHAPE,
               "budgets and depth must be non-negative");
    HA_REQUIRE(heavy_budget < 2147483647.0, HA_ERR_BAD_SHAPE, "heavy_budget too large");
    HA_REQUIRE(mode == HA_SELECT_SIMPLE || mode == HA_SELECT_THRESHOLD, HA_ERR_BAD_SHAPE, "unknown select mode %d", mode);
    HA_REQUIRE(algo >= HA_SELECT_ALGO_AUTO && algo <= HA_SELECT_ALGO_SAMPLED_EXACT_ROWS, HA_ERR_BAD_SHAPE, "unknown select algo %d", algo);
    HA_REQUIRE(idx_cap > 0, HA_ERR_BAD_SHAPE, "idx_cap must be positive");
    if (use_static_scratch) {
        // the histogram method's own need (the sampled method parks candidates in a far larger workspace)
        const size_t need = carve_select_ws(nullptr, (int64_t)B * H, select_plan(B, Hc, max_seq_len).nchunk, W).bytes;
        HA_REQUIRE(need <= kStaticScratchBytes, HA_ERR_WORKSPACE,
                   "ha_select_static: this shape needs %zu bytes of scratch, the built-in buffer holds %zu: use ha_select with a "
                   "workspace of ha_select_workspace_bytes()", need, kStaticScratchBytes);
        if ((st = ha_require_device())) return st;
        if ((st = static_scratch(&workspace))) return st;
        algo = HA_SELECT_ALGO_HISTOGRAM;
    } else {
        const size_t need = ha_select_workspace_bytes(B, H, Hc, W, max_seq_len);
        HA_REQUIRE(workspace && workspace_bytes >= need, HA_ERR_WORKSPACE, "select workspace: need %zu bytes, got %zu", need,
                   workspace ? workspace_bytes : (size_t)0);
        HA_REQUIRE(ha_aligned(workspace, 256), HA_ERR_MISALIGNED, "select workspace must be 256-byte aligned");
        if ((st = ha_require_device())) return st;
    }

    if (prepare_only) algo = HA_SELECT_ALGO_HISTOGRAM;
    if (algo == HA_SELECT_ALGO_AUTO) {
        // Measured on MI355X (16 x 64K-token rows, 1/32 kept): histogram 33.7 us, sampled 36.9 us.  Both are
        // bound by per-launch latency chains at these sizes, so the simpler method is the default.
        algo = HA_SELECT_ALGO_HISTOGRAM;
    }
    if (algo != HA_SELECT_ALGO_HISTOGRAM)
        return launch_select_sampled(kcodes, kc_stride_b, kc_stride_h, qcodes, B, H, Hc, W, max_seq_len, seq_lens, init_budget,
                                     recent_budget, heavy_budget, mode, depth, algo == HA_SELECT_ALGO_SAMPLED_EXACT_ROWS ? 1 : 0,
                                     out_idx, idx_cap, out_counts, workspace, (hipStream_t)stream);
    const SelectPlan plan = select_plan(B, Hc, max_seq_len);
    const SelectWorkspace ws = carve_select_ws(workspace, (int64_t)B * H, plan.nchunk, W);
    const int vec = rows_vectorisable(kcodes, kc_stride_b, kc_stride_h, W) ? 1 : 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(plan.nchunk, Hc, B);
    const int gq = H / Hc;
    // replicas of the LDS histogram.  With four query heads per code head 16 replicas beat 32: the launch is bound by the
    // LDS atomics either way, but the smaller histogram is cleared and summed faster and, for 64-bit codes (65 levels,
    // 33 KB with 32 replicas), lets all workgroups be resident at once (ten launches back to back: 21.3 -> 14.3 us at 8
    // sequences of 115K tokens with 64-bit codes; 8.2 -> 7.4 us at 4 x 128K with 32-bit codes; 8 replicas: 12.2 us against
    // 10.2 at 16 x 64K)
    if (W == 1) {
        if (gq == 1) HA_SELECT_LAUNCH(1, 1, 32);
        else if (gq == 2) HA_SELECT_LAUNCH(1, 2, 32);
        else if (gq == 4) HA_SELECT_LAUNCH(1, 4, 16);
        else HA_SELECT_LAUNCH(1, 8, 16);
    } else {
        if (gq == 1) HA_SELECT_LAUNCH(2, 1, 32);
        else if (gq == 2) HA_SELECT_LAUNCH(2, 2, 32);
        else if (gq == 4) HA_SELECT_LAUNCH(2, 4, 16);
        else HA_SELECT_LAUNCH(2, 8, 16);
    }
    return HA_OK;
}

int ha_select(const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes, int B, int H, int Hc, int W,
              int max_seq_len, const int32_t *seq_lens, int init_budget, int recent_budget, double heavy_budget, int mode,
              int depth, int algo, int32_t *out_idx, int64_t idx_cap, int32_t *out_counts, void *workspace,
              size_t workspace_bytes, void *stream) {
    return select_impl(kcodes, kc_stride_b, kc_stride_h, qcodes, B, H, Hc, W, max_seq_len, seq_lens, init_budget, recent_budget,
                       heavy_budget, mode, depth, algo, out_idx, idx_cap, out_counts, workspace, workspace_bytes, stream, false);
}

size_t ha_select_static_max_bytes(void) { return kStaticScratchBytes; }

int ha_select_static(const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes, int B, int H, int Hc,
                     int W, int max_seq_len, const int32_t *seq_lens, int init_budget, int recent_budget, double heavy_budget,
                     int mode, int depth, int32_t *out_idx, int64_t idx_cap, int32_t *out_counts, void *stream) {
    return select_impl(kcodes, kc_stride_b, kc_stride_h, qcodes, B, H, Hc, W, max_seq_len, seq_lens, init_budget, recent_budget,
                       heavy_budget, mode, depth, HA_SELECT_ALGO_HISTOGRAM, out_idx, idx_cap, out_counts, nullptr, 0, stream, false,
                       true);
}

int ha_select_rows(const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes, int B, int rows_per_sequence,
                   int H, int Hc, int W, int max_seq_len, const int32_t *seq_lens, int init_budget, int recent_budget,
                   double heavy_budget, int mode, int depth, int32_t *out_idx, int64_t idx_cap, int32_t *out_counts, void *workspace,
                   size_t workspace_bytes, void *stream) {
    HA_REQUIRE(seq_lens, HA_ERR_NULL_POINTER, "ha_select_rows needs one length per row");
    return select_impl(kcodes, kc_stride_b, kc_stride_h, qcodes, B, H, Hc, W, max_seq_len, seq_lens, init_budget, recent_budget,
                       heavy_budget, mode, depth, HA_SELECT_ALGO_HISTOGRAM, out_idx, idx_cap, out_counts, workspace, workspace_bytes,
                       stream, false, false, rows_per_sequence);
}

int ha_select_histogram(const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes, int B, int H, int Hc,
                        int W, int max_seq_len, const int32_t *seq_lens, int init_budget, int recent_budget, void *workspace,
                        size_t workspace_bytes, void *stream) {
    return select_impl(kcodes, kc_stride_b, kc_stride_h, qcodes, B, H, Hc, W, max_seq_len, seq_lens, init_budget, recent_budget, 0.0,
                       HA_SELECT_SIMPLE, 0, HA_SELECT_ALGO_HISTOGRAM, nullptr, 1, nullptr, workspace, workspace_bytes, stream, true);
}

int ha_select_prepare(const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes, int B, int H, int Hc,
                      int W, int max_seq_len, const int32_t *seq_lens, int init_budget, int recent_budget, double heavy_budget,
                      int mode, int depth, int32_t *out_counts, void *workspace, size_t workspace_bytes, void *stream) {
    HA_REQUIRE(out_counts, HA_ERR_NULL_POINTER, "out_counts is NULL");
    return select_impl(kcodes, kc_stride_b, kc_stride_h, qcodes, B, H, Hc, W, max_seq_len, seq_lens, init_budget, recent_budget,
                       heavy_budget, mode, depth, HA_SELECT_ALGO_HISTOGRAM, nullptr, 1, out_counts, workspace, workspace_bytes, stream,
                       true);
}

}  // extern "C"
