// Selection with a sampled threshold guess (gfx950).  Same result as the two-pass histogram selection of
// ha_select.hip, bit for bit, with one cheap pass over the codes instead of two expensive ones.
//
// The exact method spends its time on per-(code, query head) work it does not need: it histograms and then
// ranks every token, although only the ~k nearest matter.  Here
//   1. select_sample_kernel    per (sequence, code head): distances of <= 4096 evenly spread candidates give,
//                              per query head, a level T_hi that bounds the true threshold T from above with
//                              overwhelming probability (5 sigma of the sampling error on top of k);
//   2. select_filter_kernel    one pass over all codes: three VALU ops per (code, head) decide d <= T_hi, and
//                              only those few percent of the tokens are written, in index order, to a per-chunk
//                              candidate segment;
//   3. select_finalize_kernel  per row: exact histogram of the candidates, exact T and r, ordered compaction of
//                              the candidates, windows and count.
// Nothing rests on the guess being right: if a row's candidates do not contain k tokens, or a segment
// overflows, select_finalize_kernel redoes that row exactly from the codes (slow, rare, same kernel: no
// round trip to the host).
#include <type_traits>

#include "ha_select_common.h"

using namespace ha_sel;

namespace {

constexpr int kFinThreads = 512;
constexpr int kFinWaves = kFinThreads / HA_WAVE;
constexpr int kMaxSample = 4096;  // sampled candidates per (sequence, code head)

// ------------------------------------------------------------------------------------------------
// grid (Hc, B), 256 threads.  thi[row] = T_hi, -1 when the row has no heavy budget, -2 = "take the exact path".
template <int W, int GQ>
__global__ __launch_bounds__(kSelThreads) void select_sample_kernel(const uint32_t *__restrict__ kcodes, int64_t kc_sb, int64_t kc_sh,
                                                                    const uint32_t *__restrict__ qcodes, int H, int max_S,
                                                                    const int32_t *__restrict__ seq_lens, int init, int recent,
                                                                    double heavy_budget, int force_exact, int32_t *__restrict__ thi) {
    constexpr int NL = 32 * W + 1;
    constexpr int REP = (GQ * NL * 32 * 4 <= 40000) ? 32 : 16;
    __shared__ uint32_t lh[GQ * NL * REP];
    __shared__ uint32_t s_h[GQ][NL];
    const int hc = blockIdx.x, b = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int S = seq_lens ? seq_lens[b] : max_S;
    if (S > max_S) S = max_S;
    const RowBudget rb = row_budget(S, init, recent, heavy_budget);
    const int ncand = rb.hi - rb.lo;
    if (rb.kk == 0 || force_exact) {  // uniform
        if (tid < GQ) thi[(int64_t)b * H + hc * GQ + tid] = force_exact && rb.kk > 0 ? -2 : -1;
        return;
    }
    for (int i = tid; i < GQ * NL * REP; i += kSelThreads) lh[i] = 0;
    __syncthreads();

    Code<W> q[GQ];
#pragma unroll
    for (int g = 0; g < GQ; ++g) q[g] = load_qcode<W>(qcodes, (int64_t)b * H + hc * GQ + g);
    const uint32_t *kc = kcodes + b * kc_sb + hc * kc_sh;
    const int rep = tid % REP;
    const bool whole = ncand <= kMaxSample;  // small rows: the "sample" is every candidate
    const int n_samp = whole ? ncand : kMaxSample;
    constexpr int PER = kMaxSample / kSelThreads;  // 16 samples per thread
    Code<W> k[PER];
    bool have[PER];
#pragma unroll
    for (int t = 0; t < PER; ++t) {
        int j;
        if (whole) {
            j = rb.lo + t * kSelThreads + tid;
            have[t] = t * kSelThreads + tid < ncand;
        } else {  // 64 segments of 64 consecutive codes, evenly spread over the candidates
            const int seg = wave + kSelWaves * t;
            j = rb.lo + (int)(((int64_t)seg * (ncand - 64)) / 63) + lane;
            have[t] = true;
        }
        if (have[t]) k[t] = load_code<W>(kc, j);
        else k[t] = q[0];
    }
#pragma unroll
    for (int t = 0; t < PER; ++t) {
        if (have[t]) {
#pragma unroll
            for (int g = 0; g < GQ; ++g) atomicAdd(&lh[(g * NL + k[t].dist(q[g])) * REP + rep], 1u);
        }
    }
    __syncthreads();
    for (int p = tid; p < GQ * NL; p += kSelThreads) {
        uint32_t s = 0;
#pragma unroll 8
        for (int r = 0; r < REP; ++r) s += lh[p * REP + ((r + tid) % REP)];
        s_h[p / NL][p % NL] = s;
    }
    __syncthreads();
    if (tid < GQ) {
        // tokens the sample must hold below T_hi so that the whole row holds k of them, 5 sigma of the
        // sampling error included; an exhaustive "sample" needs exactly k
        int need = rb.kk;
        if (!whole) {
            const double mean = (double)rb.kk * (double)n_samp / (double)ncand;
            need = (int)ceil(mean + 5.0 * sqrt(mean) + 1.0);
        }
        int cum = 0, t_hi = NL - 1;
        for (int l = 0; l < NL; ++l) {
            cum += (int)s_h[tid][l];
            if (cum >= need) {
                t_hi = l;
                break;
            }
        }
        thi[(int64_t)b * H + hc * GQ + tid] = t_hi;
    }
}

// ------------------------------------------------------------------------------------------------
// grid (nchunk, Hc, B), 256 threads; chunk layout as select_compact_kernel (a lane owns 4*blocks consecutive codes).
// cand[row][chunk][0..cap) = the chunk's candidates with d <= T_hi in ascending index order, each entry
// (d << 24) | index (so the last kernel never has to gather codes again); cand_cnt = their number (the true
// one, also when it exceeds cap).  The lane's codes are parked in LDS so that the few set bits can look
// their code up by a run-time element number.
template <int W, int GQ>
__global__ __launch_bounds__(kSelThreads) void select_filter_kernel(const uint32_t *__restrict__ kcodes, int64_t kc_sb, int64_t kc_sh,
                                                                    const uint32_t *__restrict__ qcodes, int H, int max_S,
                                                                    const int32_t *__restrict__ seq_lens, int init, int recent,
                                                                    int blocks, int nchunk, int vec, const int32_t *__restrict__ thi,
                                                                    int cap, int32_t *__restrict__ cand,
                                                                    int32_t *__restrict__ cand_cnt) {
    constexpr int CPL = 4 * kMaxBlocks;
    constexpr int NP = (GQ + 1) / 2;  // packed scan words: two 16-bit counters each
    __shared__ uint32_t s_wtot[kSelWaves][NP];
    __shared__ uint32_t s_codes[CPL * W * kSelThreads];  // [element][word][thread]: bank = thread % 32 for every access

    const int c = blockIdx.x, hc = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int S = seq_lens ? seq_lens[b] : max_S;
    if (S > max_S) S = max_S;
    const int lo = init < S ? init : S;
    const int hi = (S - recent > lo) ? S - recent : lo;
    const int chunk = blocks * kBlock;
    const int beg = max(lo, c * chunk), end = min(hi, (c + 1) * chunk);

    int t_hi[GQ];
    bool any = false;
#pragma unroll
    for (int g = 0; g < GQ; ++g) {
        t_hi[g] = thi[(int64_t)b * H + hc * GQ + g];
        any = any || t_hi[g] >= 0;
    }
    if (beg >= end || !any) {  // uniform: an empty chunk, or rows that take another path
        if (tid < GQ) cand_cnt[((int64_t)b * H + hc * GQ + tid) * nchunk + c] = 0;
        return;
    }

    const int cpl = 4 * blocks;
    const int j_lane = c * chunk + (wave * HA_WAVE + lane) * cpl;
    const uint32_t *kc = kcodes + b * kc_sb + hc * kc_sh;
    Code<W> k[CPL];
    uint32_t vmask;  // bit e: code j_lane + e is a candidate of this chunk
    if (vec && blocks == kMaxBlocks && beg == c * chunk && end == (c + 1) * chunk) {
        // the common case, uniform over the workgroup: a full chunk strictly inside the candidate range
        // of a 16-byte aligned row: four (eight) 128-bit loads and no per-element bounds
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

#pragma unroll
    for (int e = 0; e < CPL; ++e) {
        s_codes[(e * W) * kSelThreads + tid] = k[e].w0;
        if constexpr (W == 2) s_codes[(e * W + 1) * kSelThreads + tid] = k[e].w1;
    }
    uint32_t lem[GQ], packed[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) packed[p] = 0;
    Code<W> qh[GQ];
#pragma unroll
    for (int g = 0; g < GQ; ++g) {
        qh[g] = load_qcode<W>(qcodes, (int64_t)b * H + hc * GQ + g);
        const Code<W> q = qh[g];
        uint32_t le = 0;
        const int off = -t_hi[g] - 1;  // sign of d - T_hi - 1 is "d <= T_hi"; T_hi < 0 leaves it clear
#pragma unroll
        for (int e = CPL - 1; e >= 0; --e) le = __builtin_amdgcn_alignbit(le, (uint32_t)(k[e].dist(q) + off), 31);
        lem[g] = t_hi[g] >= 0 ? (le & vmask) : 0u;
        packed[g >> 1] |= (uint32_t)__popc(lem[g]) << (16 * (g & 1));
    }
    uint32_t incl[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        incl[p] = wave_inclusive_scan(packed[p]);
        if (lane == HA_WAVE - 1) s_wtot[wave][p] = incl[p];
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < GQ; ++g) {
        const int sh = 16 * (g & 1);
        int pos = (int)(((incl[g >> 1] - packed[g >> 1]) >> sh) & 0xFFFFu), total = 0;
        for (int w = 0; w < kSelWaves; ++w) {
            const int t = (int)((s_wtot[w][g >> 1] >> sh) & 0xFFFFu);
            if (w < wave) pos += t;
            total += t;
        }
        const int64_t row = (int64_t)b * H + hc * GQ + g;
        int32_t *seg = cand + (row * nchunk + c) * cap;  // uniform base, 32-bit lane offsets
        uint32_t todo = lem[g];
        uint32_t upos = (uint32_t)pos;
        while (todo) {
            const int e = __ffs((int)todo) - 1;
            todo &= todo - 1;
            Code<W> ce;
            ce.w0 = s_codes[(e * W) * kSelThreads + tid];
            if constexpr (W == 2) ce.w1 = s_codes[(e * W + 1) * kSelThreads + tid];
            if (upos < (uint32_t)cap) seg[upos] = (ce.dist(qh[g]) << 24) | (j_lane + e);
            ++upos;
        }
        if (tid == 0) cand_cnt[row * nchunk + c] = total;
    }
}

// ------------------------------------------------------------------------------------------------
// 512-thread exclusive scan of two ints; s_a/s_b hold one total per wave.  Two barriers.
__device__ __forceinline__ void block_scan2(int a, int b, uint32_t *s_a, uint32_t *s_b, int &ex_a, int &ex_b, int &tot_a, int &tot_b) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t ia = wave_inclusive_scan((uint32_t)a), ib = wave_inclusive_scan((uint32_t)b);
    __syncthreads();  // previous use of s_a/s_b is over
    if (lane == HA_WAVE - 1) {
        s_a[wave] = ia;
        s_b[wave] = ib;
    }
    __syncthreads();
    ex_a = (int)ia - a;
    ex_b = (int)ib - b;
    tot_a = tot_b = 0;
#pragma unroll
    for (int w = 0; w < kFinWaves; ++w) {
        if (w < wave) {
            ex_a += (int)s_a[w];
            ex_b += (int)s_b[w];
        }
        tot_a += (int)s_a[w];
        tot_b += (int)s_b[w];
    }
}

// grid (H, B), 512 threads.
template <int W>
__global__ __launch_bounds__(kFinThreads) void select_finalize_kernel(const uint32_t *__restrict__ kcodes, int64_t kc_sb, int64_t kc_sh,
                                                                      const uint32_t *__restrict__ qcodes, int H, int Hc, int max_S,
                                                                      const int32_t *__restrict__ seq_lens, int init, int recent,
                                                                      double heavy_budget, int mode, int depth, int nchunk,
                                                                      const int32_t *__restrict__ thi, int cap,
                                                                      const int32_t *__restrict__ cand,
                                                                      const int32_t *__restrict__ cand_cnt,
                                                                      int32_t *__restrict__ out_idx, int64_t idx_cap,
                                                                      int32_t *__restrict__ out_counts) {
    constexpr int NL = 32 * W + 1;
    constexpr int REP = 32;  // histogram replicas (replica = lane % 32 = bank): the candidates sit on a dozen levels
    static_assert(kMaxChunks <= 2 * kFinThreads, "the chunk prefix is scanned two entries per thread");
    __shared__ int s_pre[kMaxChunks + 1];
    __shared__ uint32_t s_rep[NL * REP];
    __shared__ uint32_t s_hist[NL];
    __shared__ uint32_t s_sa[kFinWaves], s_sb[kFinWaves];
    __shared__ int s_T, s_r, s_nheavy, s_ok;

    const int h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const int64_t row = (int64_t)b * H + h;
    int S = seq_lens ? seq_lens[b] : max_S;
    if (S > max_S) S = max_S;
    const RowBudget rb = row_budget(S, init, recent, heavy_budget);
    const uint32_t *kc = kcodes + b * kc_sb + (h / (H / Hc)) * kc_sh;
    const Code<W> q = load_qcode<W>(qcodes, row);
    int32_t *o = out_idx + row * idx_cap;
    const int t_hi = thi[row];
    const int32_t *cnt = cand_cnt + row * nchunk;
    const int32_t *seg0 = cand + row * nchunk * cap;

    int nheavy = 0;
    if (rb.kk > 0) {  // uniform
        // ---- candidates per chunk -> exclusive prefix (two chunks per thread, one block scan)
        if (tid == 0) s_ok = t_hi >= 0 ? 1 : 0;
        for (int i = tid; i < NL * REP; i += kFinThreads) s_rep[i] = 0;
        int c0 = 0, c1 = 0;
        if (t_hi >= 0) {
            if (tid < nchunk) c0 = cnt[tid];
            if (tid + kFinThreads < nchunk) c1 = cnt[tid + kFinThreads];
        }
        __syncthreads();
        if (c0 > cap || c1 > cap) s_ok = 0;  // a segment overflowed (benign race: every writer stores 0)
        {
            int ex0, ex1, tot0, tot1;
            block_scan2(min(c0, cap), min(c1, cap), s_sa, s_sb, ex0, ex1, tot0, tot1);
            if (tid < nchunk) s_pre[tid] = ex0;
            if (tid + kFinThreads < nchunk) s_pre[tid + kFinThreads] = tot0 + ex1;
            if (tid == 0) s_pre[nchunk] = tot0 + tot1;
        }
        __syncthreads();
        const int ntot = t_hi >= 0 ? s_pre[nchunk] : 0;
        // chunk that holds entry i of the row's candidate list: binary search in the prefix
        auto chunk_of = [&](int i) {
            int lo_c = 0, hi_c = nchunk - 1;
            while (lo_c < hi_c) {
                const int mid = (lo_c + hi_c + 1) >> 1;
                if (s_pre[mid] <= i) lo_c = mid;
                else hi_c = mid - 1;
            }
            return lo_c;
        };
        // A thread owns a contiguous run of the candidate list, handled in batches of RB entries held in
        // registers (index and distance come in one word): the loads of a batch are independent of each other.
        // RB is picked per row from the run length, so short runs do not pay for a long unrolled body.
        const int R = (ntot + kFinThreads - 1) / kFinThreads;
        const int i0 = min(tid * R, ntot), i1 = min(i0 + R, ntot);
        auto from_candidates = [&](auto rb_tag) {
            constexpr int RB = decltype(rb_tag)::value;
            const int nbatch = (R + RB - 1) / RB;  // uniform
            int jreg[RB], dreg[RB];
            auto load_batch = [&](int first) {  // entries [first, first + RB) of the run -> jreg / dreg (d = NL when absent)
                int c = first < i1 ? chunk_of(first) : 0;
                int seg_end = s_pre[c + 1];
                const int32_t *src = seg0 + (int64_t)c * cap - s_pre[c];  // entry i of the list is src[i] while i < seg_end
#pragma unroll
                for (int t = 0; t < RB; ++t) {
                    const int i = first + t;
                    jreg[t] = -1;
                    if (i < i1) {
                        if (i >= seg_end) {  // the run crosses into a later chunk's segment
                            while (i >= s_pre[c + 1]) ++c;
                            seg_end = s_pre[c + 1];
                            src = seg0 + (int64_t)c * cap - s_pre[c];
                        }
                        jreg[t] = src[i];
                    }
                }
#pragma unroll
                for (int t = 0; t < RB; ++t) {
                    dreg[t] = jreg[t] >= 0 ? (int)((uint32_t)jreg[t] >> 24) : NL;
                    jreg[t] &= 0xFFFFFF;
                }
            };
            // ---- exact histogram of the candidates
            for (int bt = 0; bt < nbatch; ++bt) {
                load_batch(i0 + bt * RB);
#pragma unroll
                for (int t = 0; t < RB; ++t)
                    if (dreg[t] < NL) atomicAdd(&s_rep[dreg[t] * REP + (tid % REP)], 1u);
            }
            __syncthreads();
            if (tid < NL) {
                uint32_t sum = 0;
#pragma unroll 8
                for (int rr = 0; rr < REP; ++rr) sum += s_rep[tid * REP + ((rr + tid) % REP)];
                s_hist[tid] = sum;
            }
            __syncthreads();
            if (tid == 0) {
                int T, r, nh;
                const bool ok = solve_threshold(s_hist, t_hi, NL, rb.kk, mode, depth, T, r, nh);
                s_T = T;
                s_r = r;
                s_nheavy = nh;
                s_ok = ok ? 1 : 0;
            }
            __syncthreads();
            if (!s_ok) return;  // uniform: the candidates do not hold k tokens
            // ---- ordered compaction of the candidate list
            const int T = s_T, r = s_r;
            int nlt = 0, neq = 0;
            for (int bt = 0; bt < nbatch; ++bt) {
                if (nbatch > 1) load_batch(i0 + bt * RB);  // a single batch is still in registers
#pragma unroll
                for (int t = 0; t < RB; ++t) {
                    nlt += dreg[t] < T ? 1 : 0;
                    neq += dreg[t] == T ? 1 : 0;
                }
            }
            int ex_lt, ex_eq, tot_lt, tot_eq;
            block_scan2(nlt, neq, s_sa, s_sb, ex_lt, ex_eq, tot_lt, tot_eq);
            for (int bt = 0; bt < nbatch; ++bt) {
                if (nbatch > 1) load_batch(i0 + bt * RB);
#pragma unroll
                for (int t = 0; t < RB; ++t) {
                    const int d = dreg[t];
                    if (d < T || (d == T && ex_eq < r)) {
                        const int64_t pos = (int64_t)rb.lo + ex_lt + min(ex_eq, r);
                        if (pos < idx_cap) o[pos] = jreg[t];
                    }
                    ex_lt += d < T ? 1 : 0;
                    ex_eq += d == T ? 1 : 0;
                }
            }
        };
        if (s_ok) {
            if (R <= 8) from_candidates(std::integral_constant<int, 8>{});
            else if (R <= 16) from_candidates(std::integral_constant<int, 16>{});
            else from_candidates(std::integral_constant<int, 32>{});
        }
        if (s_ok) {
            nheavy = s_nheavy;
        } else {
            // ---- exact path from the codes: the guess was too low, a segment overflowed, or it was asked for
            __syncthreads();
            if (tid < NL) s_hist[tid] = 0;
            __syncthreads();
            for (int j = rb.lo + tid; j < rb.hi; j += kFinThreads) atomicAdd(&s_hist[load_code<W>(kc, j).dist(q)], 1u);
            __syncthreads();
            if (tid == 0) {
                int T, r, nh;
                solve_threshold(s_hist, NL - 1, NL, rb.kk, mode, depth, T, r, nh);
                s_T = T;
                s_r = r;
                s_nheavy = nh;
            }
            __syncthreads();
            const int T = s_T, r = s_r;
            int run_lt = 0, run_eq = 0;
            for (int base = rb.lo; base < rb.hi; base += kFinThreads) {
                const int j = base + tid;
                int d = NL;
                if (j < rb.hi) d = load_code<W>(kc, j).dist(q);
                const int is_lt = d < T ? 1 : 0, is_eq = d == T ? 1 : 0;
                int ex_lt, ex_eq, tot_lt, tot_eq;
                block_scan2(is_lt, is_eq, s_sa, s_sb, ex_lt, ex_eq, tot_lt, tot_eq);
                if (is_lt || (is_eq && run_eq + ex_eq < r)) {
                    const int64_t pos = (int64_t)rb.lo + run_lt + ex_lt + min(run_eq + ex_eq, r);
                    if (pos < idx_cap) o[pos] = j;
                }
                run_lt += tot_lt;
                run_eq += tot_eq;
            }
            nheavy = s_nheavy;
        }
    }

    // ---- windows and count
    const int n_recent = rb.S - rb.hi;
    const int64_t rbase = (int64_t)rb.lo + nheavy;
    for (int i = tid; i < rb.lo; i += kFinThreads)
        if (i < idx_cap) o[i] = i;
    for (int i = tid; i < n_recent; i += kFinThreads)
        if (rbase + i < idx_cap) o[rbase + i] = rb.hi + i;
    if (tid == 0) out_counts[row] = (int32_t)(rbase + n_recent);
}

}  // namespace

namespace ha_sel {

size_t sampled_workspace_bytes(int64_t rows, int nchunk, int blocks) {
    return carve_sampled_ws(nullptr, rows, nchunk, blocks).bytes;
}

int launch_select_sampled(const uint32_t *kcodes, int64_t kc_sb, int64_t kc_sh, const uint32_t *qcodes, int B, int H, int Hc, int W,
                          int max_seq_len, const int32_t *seq_lens, int init, int recent, double heavy_budget, int mode, int depth,
                          int force_exact, int32_t *out_idx, int64_t idx_cap, int32_t *out_counts, void *workspace, hipStream_t s) {
    const SelectPlan plan = select_plan(B, Hc, max_seq_len);
    const SampledWorkspace ws = carve_sampled_ws(workspace, (int64_t)B * H, plan.nchunk, plan.blocks);
    const int vec = rows_vectorisable(kcodes, kc_sb, kc_sh, W) ? 1 : 0;
    const dim3 grid(plan.nchunk, Hc, B);
    const int gq = H / Hc;
#define HA_SAMPLED_LAUNCH(W_, GQ_)                                                                                                 \
    do {                                                                                                                          \
        hipLaunchKernelGGL((select_sample_kernel<W_, GQ_>), dim3(Hc, B), dim3(kSelThreads), 0, s, kcodes, kc_sb, kc_sh, qcodes, H, \
                           max_seq_len, seq_lens, init, recent, heavy_budget, force_exact, ws.thi);                               \
        HA_CHECK_LAUNCH("select_sample_kernel");                                                                                  \
        hipLaunchKernelGGL((select_filter_kernel<W_, GQ_>), grid, dim3(kSelThreads), 0, s, kcodes, kc_sb, kc_sh, qcodes, H,       \
                           max_seq_len, seq_lens, init, recent, plan.blocks, plan.nchunk, vec, ws.thi, ws.cap, ws.cand,           \
                           ws.cand_cnt);                                                                                          \
        HA_CHECK_LAUNCH("select_filter_kernel");                                                                                  \
        hipLaunchKernelGGL(select_finalize_kernel<W_>, dim3(H, B), dim3(kFinThreads), 0, s, kcodes, kc_sb, kc_sh, qcodes, H, Hc,  \
                           max_seq_len, seq_lens, init, recent, heavy_budget, mode, depth, plan.nchunk, ws.thi, ws.cap, ws.cand,  \
                           ws.cand_cnt, out_idx, idx_cap, out_counts);                                                            \
        HA_CHECK_LAUNCH("select_finalize_kernel");                                                                                \
    } while (0)
    if (W == 1) {
        if (gq == 1) HA_SAMPLED_LAUNCH(1, 1);
        else if (gq == 2) HA_SAMPLED_LAUNCH(1, 2);
        else if (gq == 4) HA_SAMPLED_LAUNCH(1, 4);
        else HA_SAMPLED_LAUNCH(1, 8);
    } else {
        if (gq == 1) HA_SAMPLED_LAUNCH(2, 1);
        else if (gq == 2) HA_SAMPLED_LAUNCH(2, 2);
        else if (gq == 4) HA_SAMPLED_LAUNCH(2, 4);
        else HA_SAMPLED_LAUNCH(2, 8);
    }
#undef HA_SAMPLED_LAUNCH
    return HA_OK;
}

}  // namespace ha_sel
