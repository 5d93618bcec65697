// Hamming scoring and heavy-token selection over the packed code cache (gfx950, wave64).
//
// Selection never sorts.  Distances take only NL = 32*W + 1 values, so the k-th smallest distance
// T of a row follows from a histogram, and "the k nearest, lowest index first" is
//     { j : d_j < T }  union  the first r = k - #{d < T} tokens with d_j == T in index order.
// Two streaming passes over the codes of a (sequence, code head):
//   1. select_hist_kernel     per-chunk histograms of the distances of every query head of the group
//   2. select_compact_kernel  T and r from the summed histograms, then an ordered wave-ballot
//                             compaction that writes ascending index lists (sink | heavy | recent)
// The second pass re-reads the codes (4*W bytes per token) from L2 / Infinity Cache.
#include "ha_common.h"

namespace {

constexpr int kSelThreads = 256;
constexpr int kSelWaves = kSelThreads / HA_WAVE;
constexpr int kMaxChunks = 32;

struct SelectPlan {
    int chunk;   // tokens per workgroup, multiple of 1024
    int nchunk;  // <= kMaxChunks
};

inline SelectPlan select_plan(int max_seq_len) {
    SelectPlan p;
    int64_t per = ((int64_t)max_seq_len + kMaxChunks - 1) / kMaxChunks;
    p.chunk = (int)((per + 1023) / 1024) * 1024;
    if (p.chunk < 1024) p.chunk = 1024;
    p.nchunk = (max_seq_len + p.chunk - 1) / p.chunk;
    if (p.nchunk < 1) p.nchunk = 1;
    return p;
}

template <int W> struct Code;
template <> struct Code<1> {
    uint32_t w0;
    __device__ static __forceinline__ Code load(const uint32_t *p, int64_t j) { return Code{p[j]}; }
    __device__ __forceinline__ int dist(const Code &q) const { return __popc(w0 ^ q.w0); }
};
template <> struct Code<2> {
    uint32_t w0, w1;
    __device__ static __forceinline__ Code load(const uint32_t *p, int64_t j) {
        uint2 v = reinterpret_cast<const uint2 *>(p)[j];
        return Code{v.x, v.y};
    }
    __device__ __forceinline__ int dist(const Code &q) const { return __popc(w0 ^ q.w0) + __popc(w1 ^ q.w1); }
};

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
    int ncand = r.hi - r.lo;
    r.kk = heavy < ncand ? heavy : ncand;
    return r;
}

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
    scores[((int64_t)b * H + h) * max_S + j] = (uint8_t)Code<W>::load(kc, j).dist(q);
}

// ------------------------------------------------------------------------------------------------
// Pass 1.  grid (nchunk, Hc, B).  hist[b, h, chunk, level] = #candidates of the chunk at that distance.
// The LDS histogram is replicated REP times (bank = lane % REP) so that the ~10 hot levels of a
// binomial-like distance distribution do not serialise the ds_add.
template <int W, int GQ, int REP>
__global__ __launch_bounds__(kSelThreads) void select_hist_kernel(const uint32_t *__restrict__ kcodes, int64_t kc_sb, int64_t kc_sh,
                                                                  const uint32_t *__restrict__ qcodes, int H, int max_S,
                                                                  const int32_t *__restrict__ seq_lens, int init, int recent,
                                                                  int chunk, int nchunk, uint32_t *__restrict__ hist) {
    constexpr int NL = 32 * W + 1;
    __shared__ uint32_t lh[GQ * NL * REP];
    const int c = blockIdx.x, hc = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x;
    int S = seq_lens ? seq_lens[b] : max_S;
    if (S > max_S) S = max_S;
    const int lo = init < S ? init : S;
    const int hi = (S - recent > lo) ? S - recent : lo;
    const int beg = max(lo, c * chunk), end = min(hi, (c + 1) * chunk);

    for (int i = tid; i < GQ * NL * REP; i += kSelThreads) lh[i] = 0;
    __syncthreads();

    if (beg < end) {
        Code<W> q[GQ];
#pragma unroll
        for (int g = 0; g < GQ; ++g) q[g] = load_qcode<W>(qcodes, (int64_t)b * H + hc * GQ + g);
        const uint32_t *kc = kcodes + b * kc_sb + hc * kc_sh;
        const int rep = tid % REP;
        for (int j = c * chunk + tid; j < end; j += kSelThreads) {
            if (j < beg) continue;
            const Code<W> k = Code<W>::load(kc, j);
#pragma unroll
            for (int g = 0; g < GQ; ++g) atomicAdd(&lh[(g * NL + k.dist(q[g])) * REP + rep], 1u);
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
// Pass 2.  grid (nchunk, Hc, B).  Each wave owns a contiguous quarter of the chunk, so output order
// is chunk-major, wave-major, tile-major, lane-major = ascending token index.
template <int W, int GQ>
__global__ __launch_bounds__(kSelThreads) void select_compact_kernel(const uint32_t *__restrict__ kcodes, int64_t kc_sb, int64_t kc_sh,
                                                                     const uint32_t *__restrict__ qcodes, int H, int max_S,
                                                                     const int32_t *__restrict__ seq_lens, int init, int recent,
                                                                     double heavy_budget, int mode, int depth, int chunk, int nchunk,
                                                                     const uint32_t *__restrict__ hist, int32_t *__restrict__ out_idx,
                                                                     int64_t idx_cap, int32_t *__restrict__ out_counts) {
    constexpr int NL = 32 * W + 1;
    __shared__ uint32_t s_tot[GQ][NL], s_pre[GQ][NL];
    __shared__ int s_T[GQ], s_r[GQ], s_ltpre[GQ], s_eqpre[GQ], s_nheavy[GQ];
    __shared__ int s_wcnt[kSelWaves][GQ][2];

    const int c = blockIdx.x, hc = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int S = seq_lens ? seq_lens[b] : max_S;
    if (S > max_S) S = max_S;
    const RowBudget rb = row_budget(S, init, recent, heavy_budget);

    // ---- chunk-summed histograms and the part that lies in earlier chunks
    for (int p = tid; p < GQ * NL; p += kSelThreads) {
        const int g = p / NL, l = p % NL;
        const uint32_t *hp = hist + ((int64_t)b * H + hc * GQ + g) * nchunk * NL + l;
        uint32_t tot = 0, pre = 0;
        for (int cc = 0; cc < nchunk; ++cc) {
            const uint32_t v = hp[(int64_t)cc * NL];
            tot += v;
            if (cc < c) pre += v;
        }
        s_tot[g][l] = tot;
        s_pre[g][l] = pre;
    }
    __syncthreads();
    if (tid < GQ) {
        const int g = tid;
        int T = 0, r = 0, nheavy = 0;
        if (rb.kk > 0) {
            int cum = 0, l = 0, dmin = -1;
            for (; l < NL; ++l) {
                const int t = (int)s_tot[g][l];
                if (dmin < 0 && t > 0) dmin = l;
                if (cum + t >= rb.kk) break;
                cum += t;
            }
            if (l >= NL) l = NL - 1;  // unreachable when the histograms cover all candidates
            if (mode == HA_SELECT_SIMPLE) {
                T = l;
                r = rb.kk - cum;
                nheavy = rb.kk;
            } else {
                const int th = min(dmin + depth, l);
                T = th + 1;  // every distance <= th, no partial tie bucket
                r = 0;
                for (int i = 0; i <= th; ++i) nheavy += (int)s_tot[g][i];
            }
        }
        int ltpre = 0;
        for (int i = 0; i < T && i < NL; ++i) ltpre += (int)s_pre[g][i];
        s_T[g] = T;
        s_r[g] = r;
        s_ltpre[g] = ltpre;
        s_eqpre[g] = (T < NL) ? (int)s_pre[g][T] : 0;
        s_nheavy[g] = nheavy;
    }
    __syncthreads();

    // ---- windows and counts: written once per row, by the workgroup of chunk 0
    if (c == 0) {
        const int n_recent = rb.S - rb.hi;
#pragma unroll
        for (int g = 0; g < GQ; ++g) {
            int32_t *o = out_idx + ((int64_t)b * H + hc * GQ + g) * idx_cap;
            const int64_t rbase = (int64_t)rb.lo + s_nheavy[g];
            for (int i = tid; i < rb.lo; i += kSelThreads)
                if (i < idx_cap) o[i] = i;
            for (int i = tid; i < n_recent; i += kSelThreads)
                if (rbase + i < idx_cap) o[rbase + i] = rb.hi + i;
            if (tid == 0) out_counts[b * H + hc * GQ + g] = (int32_t)(rbase + n_recent);
        }
    }

    const int beg = max(rb.lo, c * chunk), end = min(rb.hi, (c + 1) * chunk);
    if (beg >= end || rb.kk == 0) return;  // uniform over the workgroup

    Code<W> q[GQ];
    int T[GQ], cnt_lt[GQ], cnt_eq[GQ];
#pragma unroll
    for (int g = 0; g < GQ; ++g) {
        q[g] = load_qcode<W>(qcodes, (int64_t)b * H + hc * GQ + g);
        T[g] = s_T[g];
        cnt_lt[g] = cnt_eq[g] = 0;
    }
    const uint32_t *kc = kcodes + b * kc_sb + hc * kc_sh;
    const int seg = chunk / kSelWaves;
    const int wbeg = c * chunk + wave * seg, wend = min(wbeg + seg, end);

    // ---- pass A: per-wave counts
    for (int j0 = wbeg; j0 < wend; j0 += HA_WAVE) {
        const int j = j0 + lane;
        const bool valid = j >= beg && j < wend;
        Code<W> k = q[0];
        if (valid) k = Code<W>::load(kc, j);
#pragma unroll
        for (int g = 0; g < GQ; ++g) {
            const int d = k.dist(q[g]);
            cnt_lt[g] += __popcll(__ballot(valid && d < T[g]));
            cnt_eq[g] += __popcll(__ballot(valid && d == T[g]));
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int g = 0; g < GQ; ++g) {
            s_wcnt[wave][g][0] = cnt_lt[g];
            s_wcnt[wave][g][1] = cnt_eq[g];
        }
    }
    __syncthreads();

    int run_sel[GQ], run_eq[GQ], r[GQ];
#pragma unroll
    for (int g = 0; g < GQ; ++g) {
        int lt_before = s_ltpre[g], eq_before = s_eqpre[g];
        for (int w = 0; w < wave; ++w) {
            lt_before += s_wcnt[w][g][0];
            eq_before += s_wcnt[w][g][1];
        }
        r[g] = s_r[g];
        run_eq[g] = eq_before;
        run_sel[g] = rb.lo + lt_before + min(eq_before, r[g]);
    }

    // ---- pass B: ordered compaction
    for (int j0 = wbeg; j0 < wend; j0 += HA_WAVE) {
        const int j = j0 + lane;
        const bool valid = j >= beg && j < wend;
        Code<W> k = q[0];
        if (valid) k = Code<W>::load(kc, j);
#pragma unroll
        for (int g = 0; g < GQ; ++g) {
            const int d = k.dist(q[g]);
            const bool is_lt = valid && d < T[g];
            const bool is_eq = valid && d == T[g];
            const uint64_t bal_eq = __ballot(is_eq);
            const bool sel = is_lt || (is_eq && run_eq[g] + lanes_below(bal_eq) < r[g]);
            const uint64_t bal_sel = __ballot(sel);
            if (sel) {
                const int64_t pos = (int64_t)run_sel[g] + lanes_below(bal_sel);
                if (pos < idx_cap) out_idx[((int64_t)b * H + hc * GQ + g) * idx_cap + pos] = j;
            }
            run_eq[g] += __popcll(bal_eq);
            run_sel[g] += __popcll(bal_sel);
        }
    }
}

int validate_codes(const uint32_t *kcodes, int64_t kc_sb, int64_t kc_sh, const uint32_t *qcodes, int B, int H, int Hc, int W,
                   int max_seq_len) {
    HA_REQUIRE(kcodes && qcodes, HA_ERR_NULL_POINTER, "kcodes/qcodes is NULL");
    HA_REQUIRE(B > 0 && H > 0 && Hc > 0 && max_seq_len > 0, HA_ERR_BAD_SHAPE, "B, H, Hc, max_seq_len must be positive");
    HA_REQUIRE(B <= 65535 && H <= 65535, HA_ERR_BAD_SHAPE, "B and H are limited to 65535");
    HA_REQUIRE(W == 1 || W == 2, HA_ERR_BAD_SHAPE, "code words W=%d, must be 1 or 2", W);
    HA_REQUIRE(H % Hc == 0, HA_ERR_BAD_SHAPE, "H=%d not a multiple of Hc=%d", H, Hc);
    const int gq = H / Hc;
    HA_REQUIRE(gq == 1 || gq == 2 || gq == 4 || gq == 8, HA_ERR_BAD_SHAPE, "H/Hc=%d, must be 1, 2, 4 or 8", gq);
    HA_REQUIRE(kc_sh >= (int64_t)max_seq_len * W && kc_sb >= kc_sh, HA_ERR_BAD_SHAPE, "code strides smaller than the rows they span");
    HA_REQUIRE(ha_aligned(kcodes, 4 * W) && ha_aligned(qcodes, 4) && (W == 1 || (kc_sb % 2 == 0 && kc_sh % 2 == 0)),
               HA_ERR_MISALIGNED, "codes must be aligned to their word count");
    return HA_OK;
}

}  // namespace

extern "C" {

int ha_hamming_score(const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes, int B, int H,
                     int Hc, int W, int max_seq_len, const int32_t *seq_lens, uint8_t *scores, void *stream) {
    int st = validate_codes(kcodes, kc_stride_b, kc_stride_h, qcodes, B, H, Hc, W, max_seq_len);
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
    (void)Hc;
    if (B <= 0 || H <= 0 || max_seq_len <= 0 || (W != 1 && W != 2)) return 0;
    const SelectPlan p = select_plan(max_seq_len);
    return (size_t)B * H * p.nchunk * (32 * W + 1) * sizeof(uint32_t);
}

#define HA_SELECT_LAUNCH(W_, GQ_, REP_)                                                                                           \
    do {                                                                                                                          \
        hipLaunchKernelGGL((select_hist_kernel<W_, GQ_, REP_>), grid, dim3(kSelThreads), 0, s, kcodes, kc_stride_b, kc_stride_h,  \
                           qcodes, H, max_seq_len, seq_lens, init_budget, recent_budget, plan.chunk, plan.nchunk, hist);          \
        HA_CHECK_LAUNCH("select_hist_kernel");                                                                                    \
        hipLaunchKernelGGL((select_compact_kernel<W_, GQ_>), grid, dim3(kSelThreads), 0, s, kcodes, kc_stride_b, kc_stride_h,     \
                           qcodes, H, max_seq_len, seq_lens, init_budget, recent_budget, heavy_budget, mode, depth, plan.chunk,   \
                           plan.nchunk, hist, out_idx, idx_cap, out_counts);                                                      \
        HA_CHECK_LAUNCH("select_compact_kernel");                                                                                 \
    } while (0)

int ha_select(const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes, int B, int H, int Hc, int W,
              int max_seq_len, const int32_t *seq_lens, int init_budget, int recent_budget, double heavy_budget, int mode,
              int depth, int32_t *out_idx, int64_t idx_cap, int32_t *out_counts, void *workspace, size_t workspace_bytes,
              void *stream) {
    int st = validate_codes(kcodes, kc_stride_b, kc_stride_h, qcodes, B, H, Hc, W, max_seq_len);
    if (st) return st;
    HA_REQUIRE(out_idx && out_counts, HA_ERR_NULL_POINTER, "out_idx/out_counts is NULL");
    HA_REQUIRE(init_budget >= 0 && recent_budget >= 0 && heavy_budget >= 0.0 && depth >= 0, HA_ERR_BAD_SHAPE,
               "budgets and depth must be non-negative");
    HA_REQUIRE(heavy_budget < 2147483647.0, HA_ERR_BAD_SHAPE, "heavy_budget too large");
    HA_REQUIRE(mode == HA_SELECT_SIMPLE || mode == HA_SELECT_THRESHOLD, HA_ERR_BAD_SHAPE, "unknown select mode %d", mode);
    HA_REQUIRE(idx_cap > 0, HA_ERR_BAD_SHAPE, "idx_cap must be positive");
    const size_t need = ha_select_workspace_bytes(B, H, Hc, W, max_seq_len);
    HA_REQUIRE(workspace && workspace_bytes >= need, HA_ERR_WORKSPACE, "select workspace: need %zu bytes, got %zu", need,
               workspace ? workspace_bytes : (size_t)0);
    HA_REQUIRE(ha_aligned(workspace, 256), HA_ERR_MISALIGNED, "select workspace must be 256-byte aligned");
    if ((st = ha_require_device())) return st;

    const SelectPlan plan = select_plan(max_seq_len);
    uint32_t *hist = (uint32_t *)workspace;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(plan.nchunk, Hc, B);
    const int gq = H / Hc;
    if (W == 1) {
        if (gq == 1) HA_SELECT_LAUNCH(1, 1, 32);
        else if (gq == 2) HA_SELECT_LAUNCH(1, 2, 32);
        else if (gq == 4) HA_SELECT_LAUNCH(1, 4, 32);
        else HA_SELECT_LAUNCH(1, 8, 16);
    } else {
        if (gq == 1) HA_SELECT_LAUNCH(2, 1, 32);
        else if (gq == 2) HA_SELECT_LAUNCH(2, 2, 32);
        else if (gq == 4) HA_SELECT_LAUNCH(2, 4, 32);
        else HA_SELECT_LAUNCH(2, 8, 16);
    }
    return HA_OK;
}

}  // extern "C"
