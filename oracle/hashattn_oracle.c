/*
 * Plain-C restatement of HashAttention's sparse decode stages.  TEST INFRASTRUCTURE ONLY:
 * the checker for the HIP kernels at sizes where the Python oracle is too slow, and a
 * timed CPU baseline.  Nothing in the shipped library links or loads this file.
 *
 * It follows the same reference lines as oracle/hashattn_oracle.py but with different
 * algorithms from the GPU code, so agreement is evidence and not tautology:
 *   orc_hamming        popcount(q ^ k)                efficiency/kernels/bit_count_uint32.py:4-12,
 *                                                     efficiency/kernels/torchatt.py:58-62
 *   orc_select         full sort of (distance, index) hashattention/hashattention_llama.py:423-438
 *                      keys, then the first k          (canonical tie-break: lowest index)
 *   orc_encode         Linear/SiLU chain + sign pack   hashattention_llama.py:99-128, 168-173;
 *                                                     torchatt.py:55-56, 159
 *   orc_sparse_attend  gather, fp32 -> double softmax  efficiency/kernels/sparse.py:190-214
 *   orc_dense_attend   all keys of a sequence          efficiency/kernels/torchatt.py:17-30
 *
 * Build: gcc -O2 -fopenmp -shared -fPIC -o libhashattn_oracle.so hashattn_oracle.c -lm
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static int popc32(uint32_t x) {           /* bit-by-bit on purpose: independent of __builtin_popcount */
    int c = 0;
    while (x) { x &= x - 1; ++c; }
    return c;
}

/* kcodes [B, Hc, S_stride, W], qcodes [B, H, W], out [B, H, S_stride] (uint8), rows >= seq_len untouched */
void orc_hamming(const uint32_t *kcodes, const uint32_t *qcodes, int B, int H, int Hc, int64_t S_stride, int W,
                 const int32_t *seq_lens, uint8_t *out) {
    int G = H / Hc;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int b = 0; b < B; ++b)
        for (int h = 0; h < H; ++h) {
            const uint32_t *kc = kcodes + ((int64_t)b * Hc + h / G) * S_stride * W;
            const uint32_t *qc = qcodes + ((int64_t)b * H + h) * W;
            uint8_t *o = out + ((int64_t)b * H + h) * S_stride;
            int S = seq_lens[b];
            for (int j = 0; j < S; ++j) {
                int d = 0;
                for (int w = 0; w < W; ++w) d += popc32(kc[(int64_t)j * W + w] ^ qc[w]);
                o[j] = (uint8_t)d;
            }
        }
}

static int cmp_u64(const void *a, const void *b) {
    uint64_t x = *(const uint64_t *)a, y = *(const uint64_t *)b;
    return (x > y) - (x < y);
}
static int cmp_i32(const void *a, const void *b) {
    int32_t x = *(const int32_t *)a, y = *(const int32_t *)b;
    return (x > y) - (x < y);
}

/*
 * q_len == 1 selection.  Candidates are j in [init, S - recent); the k_eff = min(heavy, #cand)
 * of them with the smallest distance are kept, ties going to the lowest index, together with the
 * sink [0, init) and recent [S - recent, S) windows.  heavy = (hb > 1) ? (int)hb : (int)(S * hb)
 * in double arithmetic, as Python's int(k * heavy_budget) (hashattention_llama.py:431-434).
 * mode 1 (threshold): keep every candidate with distance <= min(d_min + depth, d_(k_eff)) (:439-443).
 * out_idx [B, H, idx_cap] ascending; out_counts [B, H] holds the full count even beyond idx_cap.
 */
void orc_select(const uint32_t *kcodes, const uint32_t *qcodes, int B, int H, int Hc, int64_t S_stride, int W,
                const int32_t *seq_lens, int init, int recent, double heavy_budget, int mode, int depth,
                int32_t *out_idx, int64_t idx_cap, int32_t *out_counts) {
    int G = H / Hc;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int b = 0; b < B; ++b)
        for (int h = 0; h < H; ++h) {
            int S = seq_lens[b];
            int lo = init < S ? init : S;
            int hi = S - recent > lo ? S - recent : lo;
            int ncand = hi - lo;
            int heavy = heavy_budget > 1.0 ? (int)heavy_budget : (int)((double)S * heavy_budget);
            int kk = heavy < ncand ? heavy : ncand;
            const uint32_t *kc = kcodes + ((int64_t)b * Hc + h / G) * S_stride * W;
            const uint32_t *qc = qcodes + ((int64_t)b * H + h) * W;
            int32_t *o = out_idx + ((int64_t)b * H + h) * idx_cap;
            int64_t n = 0;
            for (int j = 0; j < lo; ++j) { if (n < idx_cap) o[n] = j; ++n; }
            if (ncand > 0 && kk > 0) {
                uint64_t *keys = (uint64_t *)malloc(sizeof(uint64_t) * (size_t)ncand);
                for (int j = lo; j < hi; ++j) {
                    int d = 0;
                    for (int w = 0; w < W; ++w) d += popc32(kc[(int64_t)j * W + w] ^ qc[w]);
                    keys[j - lo] = ((uint64_t)d << 32) | (uint32_t)j;
                }
                qsort(keys, (size_t)ncand, sizeof(uint64_t), cmp_u64);
                int take = kk;
                if (mode == 1) {
                    int dmin = (int)(keys[0] >> 32), dk = (int)(keys[kk - 1] >> 32);
                    int th = dmin + depth < dk ? dmin + depth : dk;
                    take = 0;
                    while (take < ncand && (int)(keys[take] >> 32) <= th) ++take;
                }
                int32_t *sel = (int32_t *)malloc(sizeof(int32_t) * (size_t)take);
                for (int i = 0; i < take; ++i) sel[i] = (int32_t)(keys[i] & 0xFFFFFFFFu);
                qsort(sel, (size_t)take, sizeof(int32_t), cmp_i32);
                for (int i = 0; i < take; ++i) { if (n < idx_cap) o[n] = sel[i]; ++n; }
                free(sel);
                free(keys);
            }
            for (int j = hi; j < S; ++j) { if (n < idx_cap) o[n] = j; ++n; }
            out_counts[b * H + h] = (int32_t)n;
        }
}

/*
 * Hash MLP of one head over n rows in the fixed fp32 arithmetic of the GPU's exact encoder: the inputs
 * of a Linear are split in four contiguous quarters, each reduced by an ascending fmaf chain from 0,
 * y = (((b[o] + p0) + p1) + p2) + p3; SiLU(y) = y / (1 + expf(-y)).  Input widths are multiples of 4.
 * W is nn.Linear layout [out, in].  logits [n, final] (may be NULL), codes [n, final/32].
 */
void orc_encode(const float *x, int64_t n, int n_layers, const int32_t *dims /* n_layers+1 */,
                const float *const *Wl, const float *const *bl, float *logits, uint32_t *codes) {
    int maxd = 0;
    for (int l = 0; l <= n_layers; ++l) if (dims[l] > maxd) maxd = dims[l];
    int D = dims[n_layers];
#pragma omp parallel
    {
        float *a = (float *)malloc(sizeof(float) * (size_t)maxd), *c = (float *)malloc(sizeof(float) * (size_t)maxd);
#pragma omp for schedule(static)
        for (int64_t r = 0; r < n; ++r) {
            memcpy(a, x + r * dims[0], sizeof(float) * (size_t)dims[0]);
            for (int l = 0; l < n_layers; ++l) {
                int in = dims[l], out = dims[l + 1];
                for (int o = 0; o < out; ++o) {
                    float acc = bl[l][o];
                    for (int s = 0; s < 4; ++s) {
                        float p = 0.0f;
                        for (int k = s * (in / 4); k < (s + 1) * (in / 4); ++k) p = fmaf(a[k], Wl[l][(int64_t)o * in + k], p);
                        acc += p;
                    }
                    if (l + 1 < n_layers) acc = acc / (1.0f + expf(-acc));
                    c[o] = acc;
                }
                float *t = a; a = c; c = t;
            }
            if (logits) memcpy(logits + r * D, a, sizeof(float) * (size_t)D);
            for (int w = 0; w < D / 32; ++w) {
                uint32_t word = 0;
                for (int i = 0; i < 32; ++i) if (a[w * 32 + i] > 0.0f) word |= 1u << i;
                codes[r * (D / 32) + w] = word;
            }
        }
        free(a); free(c);
    }
}

static float bf16_to_f32(uint16_t u) { uint32_t x = (uint32_t)u << 16; float f; memcpy(&f, &x, 4); return f; }
static float f16_to_f32(uint16_t h) {
    uint32_t s = (uint32_t)(h >> 15) << 31, e = (h >> 10) & 31, m = h & 1023, x;
    if (e == 0) { float f = ldexpf((float)m, -24); return s ? -f : f; }
    x = e == 31 ? s | 0x7F800000u | (m << 13) : s | ((e + 112) << 23) | (m << 13);
    float f; memcpy(&f, &x, 4); return f;
}
/* dtype: 0 fp32, 1 bf16, 2 fp16 */
static float ld(const void *p, int64_t i, int dtype) {
    return dtype == 0 ? ((const float *)p)[i] : dtype == 1 ? bf16_to_f32(((const uint16_t *)p)[i])
                                                           : f16_to_f32(((const uint16_t *)p)[i]);
}

/*
 * q [B, H, d]; k, v [B, Hkv, S_stride, d]; idx [B, H, idx_cap], counts [B, H]; out [B, H, d] fp32.
 * Scores in fp32 inputs, softmax and accumulation in double.
 */
void orc_sparse_attend(const void *q, const void *k, const void *v, int dtype, int B, int H, int Hkv, int64_t S_stride,
                       int d, const int32_t *idx, int64_t idx_cap, const int32_t *counts, double sm_scale, float *out) {
    int G = H / Hkv;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int b = 0; b < B; ++b)
        for (int h = 0; h < H; ++h) {
            int n = counts[b * H + h];
            if (n > idx_cap) n = (int)idx_cap;
            const int32_t *ix = idx + ((int64_t)b * H + h) * idx_cap;
            int64_t base = ((int64_t)b * Hkv + h / G) * S_stride * d, qb = ((int64_t)b * H + h) * d;
            double *s = (double *)malloc(sizeof(double) * (size_t)(n > 0 ? n : 1)), m = -INFINITY, l = 0;
            double *acc = (double *)calloc((size_t)d, sizeof(double));
            for (int i = 0; i < n; ++i) {
                double a = 0;
                for (int e = 0; e < d; ++e) a += (double)ld(q, qb + e, dtype) * (double)ld(k, base + (int64_t)ix[i] * d + e, dtype);
                s[i] = a * sm_scale;
                if (s[i] > m) m = s[i];
            }
            for (int i = 0; i < n; ++i) {
                double p = exp(s[i] - m);
                l += p;
                for (int e = 0; e < d; ++e) acc[e] += p * (double)ld(v, base + (int64_t)ix[i] * d + e, dtype);
            }
            for (int e = 0; e < d; ++e) out[qb + e] = n > 0 ? (float)(acc[e] / l) : 0.0f;
            free(s); free(acc);
        }
}

void orc_dense_attend(const void *q, const void *k, const void *v, int dtype, int B, int H, int Hkv, int64_t S_stride,
                      int d, const int32_t *seq_lens, double sm_scale, float *out) {
    int G = H / Hkv;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int b = 0; b < B; ++b)
        for (int h = 0; h < H; ++h) {
            int n = seq_lens[b];
            int64_t base = ((int64_t)b * Hkv + h / G) * S_stride * d, qb = ((int64_t)b * H + h) * d;
            double *s = (double *)malloc(sizeof(double) * (size_t)(n > 0 ? n : 1)), m = -INFINITY, l = 0;
            double *acc = (double *)calloc((size_t)d, sizeof(double));
            for (int i = 0; i < n; ++i) {
                double a = 0;
                for (int e = 0; e < d; ++e) a += (double)ld(q, qb + e, dtype) * (double)ld(k, base + (int64_t)i * d + e, dtype);
                s[i] = a * sm_scale;
                if (s[i] > m) m = s[i];
            }
            for (int i = 0; i < n; ++i) {
                double p = exp(s[i] - m);
                l += p;
                for (int e = 0; e < d; ++e) acc[e] += p * (double)ld(v, base + (int64_t)i * d + e, dtype);
            }
            for (int e = 0; e < d; ++e) out[qb + e] = n > 0 ? (float)(acc[e] / l) : 0.0f;
            free(s); free(acc);
        }
}
