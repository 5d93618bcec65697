// Bulk (prefill) hash-MLP encode on the gfx950 matrix cores.
//
// Per MLP head the work is a chain of dense GEMMs  Y^T = W . X^T  (W [out][in] as stored by
// nn.Linear, X one 128-feature row per cached key), so it is computed with
// v_mfma_f32_32x32x16_bf16: A = a 32-row block of W, B = 32 tokens, D = 32 outputs x 32 tokens.
//
// Chaining without shuffles.  In the 32x32 accumulator layout lane (t = lane%32, half = lane/32)
// holds, for output block ob, the 16 outputs o = 32*ob + 8*q + 4*half + i (q, i in 0..3) of token t.
// The next layer's B operand wants 8 k-values per lane per MFMA; since a dot product does not
// care about the order of k, the activated accumulators ARE the next B operand (k-slot j = 4*s + i
// of k-step 2*ob + p  <->  feature 32*ob + 16*p + 8*s + 4*half + i) provided the next layer's
// weights are laid out in LDS with the same permutation.  The LDS fill does that once per workgroup.
//
// Arithmetic = HA_ARITH_BF16: bf16 inputs and weights, fp32 accumulate, bias added in fp32, result
// rounded to bf16, SiLU evaluated in fp32 on the rounded value and rounded to bf16 again.
#include "ha_common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kMfThreads = 512;
constexpr int kMfWaves = kMfThreads / HA_WAVE;
constexpr int kTokPerWave = 64;  // two 32-token MFMA column blocks per wave: every A operand read from LDS is used twice
constexpr int kTile = kMfWaves * kTokPerWave;
constexpr int kDim = 128;
constexpr int kKSteps = kDim / 16;

// LDS bytes of one layer's permuted weights: [out/32][8 k-steps][64 lanes][8 bf16]
constexpr int wp_bytes(int out) { return (out / 32) * kKSteps * 64 * 16; }

// SiLU of a Linear output in bf16 arithmetic: the accumulator is rounded to bf16, y * sigmoid(y) is evaluated
// in fp32 with the hardware exp2 and reciprocal (1 ulp each, far below the bf16 rounding that follows in the
// caller).  Evaluated per activation it costs ~13 issue slots, two of them transcendentals, against the 72 MFMA
// cycles per (token, head) that 256 activations share: three times the matrix work.  The kernel uses it to build
// the table below.
__device__ __forceinline__ float silu_bf16(float acc) {
    const float y = (float)(__bf16)acc;
    const float t = __builtin_amdgcn_exp2f(y * -1.4426950408889634f);
    return y * __builtin_amdgcn_rcpf(1.0f + t);
}

// The activation as a table.  Its input is a bf16 value, so bf16(SiLU(y)) is a function of 16 bits: the workgroup keeps
// it in LDS for every |y| from 2^-20 up (all larger magnitudes, infinities and NaNs included), one 32-bit entry per
// magnitude: low half the result for +|y|, high half for -|y|, both computed with silu_bf16 itself, so the table gives
// what the formula gives.  Magnitudes below 2^-20 read the entry of 2^-20: an absolute error under 2^-21 on a value that
// is added to sums of order one in fp32.  A pair of activations then costs one packed conversion, a packed clamp, a few
// integer operations, two LDS reads and one byte permute instead of four transcendentals.
constexpr uint32_t kTabLo = 107u << 7;                    // bf16 bits of 2^-20
constexpr int kTabEntries = 0x8000 - (int)kTabLo;        // magnitudes kTabLo .. 0x7fff
constexpr int kTabBytes = kTabEntries * 4;

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void fill_silu_table(uint32_t *tab, int tid) {
    for (int i = tid; i < kTabEntries; i += kMfThreads) {
        const uint32_t mag = kTabLo + (uint32_t)i;
        uint32_t pos, neg;
        if (mag >= (134u << 7) && mag <= 0x7f80u) {      // |y| >= 2^7, not NaN: exp2 under- / overflows, SiLU(y) = y or -0
            pos = mag;
            neg = 0x8000u;
        } else {
            const float y = __uint_as_float(mag << 16);
            pos = __builtin_bit_cast(unsigned short, (__bf16)silu_bf16(y));
            neg = __builtin_bit_cast(unsigned short, (__bf16)silu_bf16(-y));
        }
        tab[i] = pos | (neg << 16);
    }
}

// bf16(SiLU(bf16(a0))) | bf16(SiLU(bf16(a1))) << 16 through the table
__device__ __forceinline__ uint32_t silu_pair_lut(float a0, float a1, const uint32_t *tab) {
    f32x2 a;
    a.x = a0, a.y = a1;
    const uint32_t p = __builtin_bit_cast(uint32_t, __builtin_convertvector(a, bf16x2));
    const u16x2 mag = __builtin_bit_cast(u16x2, p & 0x7fff7fffu);
    u16x2 lo;
    lo.x = (unsigned short)kTabLo, lo.y = (unsigned short)kTabLo;
    const uint32_t pc = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(mag, lo));
    const uint32_t d0 = tab[(int)(pc & 0xffffu) - (int)kTabLo];
    const uint32_t d1 = tab[(int)(pc >> 16) - (int)kTabLo];
    // result half k comes from entry k: its high half when activation k is negative, else its low half
    const uint32_t sel = 0x05040100u + ((p >> 15) & 0x00010001u) * 0x0202u;
    return __builtin_amdgcn_perm(d1, d0, sel);
}

// Copy W [out][128] (bf16, global) into the MFMA A-operand order.  c_perm selects the k permutation:
// false: natural (layer fed from global rows), true: accumulator order (layer fed from a previous layer).
__device__ __forceinline__ void fill_weights(uint2 *dst, const __bf16 *W, int out, bool c_perm, int tid) {
    const int chunks = (out / 32) * kKSteps * 64 * 2;
    for (int c = tid; c < chunks; c += kMfThreads) {
        const int s = c & 1, lane = (c >> 1) & 63, ks = (c >> 7) & 7, ob = c >> 10;
        const int o = 32 * ob + (lane & 31), half = lane >> 5;
        const int feat = c_perm ? 16 * ks + 8 * s + 4 * half : 16 * ks + 8 * half + 4 * s;
        dst[c] = *reinterpret_cast<const uint2 *>(W + (int64_t)o * kDim + feat);
    }
}

// One 128 -> 32*NOB layer for the wave's 64 tokens.  Bin[ks][nb]: B operands; Wp/bias in LDS.
// acc[ob][nb] returns bias + W x (fp32).
template <int NOB>
__device__ __forceinline__ void layer_mfma(const uint4 *Wp, const float *bias, const bf16x8 (&Bin)[kKSteps][2], f32x16 (&acc)[NOB][2],
                                           int lane) {
    const int half = lane >> 5;
#pragma unroll
    for (int ob = 0; ob < NOB; ++ob) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float4 bv = *reinterpret_cast<const float4 *>(bias + 32 * ob + 8 * q + 4 * half);
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                acc[ob][nb][4 * q + 0] = bv.x;
                acc[ob][nb][4 * q + 1] = bv.y;
                acc[ob][nb][4 * q + 2] = bv.z;
                acc[ob][nb][4 * q + 3] = bv.w;
            }
        }
#pragma unroll
        for (int ks = 0; ks < kKSteps; ++ks) {
            const uint4 raw = Wp[(ob * kKSteps + ks) * 64 + lane];
            const bf16x8 a = __builtin_bit_cast(bf16x8, raw);
            acc[ob][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, Bin[ks][0], acc[ob][0], 0, 0, 0);
            acc[ob][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, Bin[ks][1], acc[ob][1], 0, 0, 0);
        }
    }
}

// hidden layer: 128 -> 128 with SiLU (through the table); output is the next layer's B operand set
__device__ __forceinline__ void hidden_layer(const uint4 *Wp, const float *bias, const uint32_t *tab, const bf16x8 (&Bin)[kKSteps][2],
                                             bf16x8 (&Bout)[kKSteps][2], int lane) {
#pragma unroll
    for (int ob = 0; ob < 4; ++ob) {
        f32x16 acc[1][2];
        layer_mfma<1>(Wp + ob * kKSteps * 64, bias + 32 * ob, Bin, acc, lane);
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                uint32_t w[4];
#pragma unroll
                for (int m = 0; m < 4; ++m) w[m] = silu_pair_lut(acc[0][nb][8 * p + 2 * m], acc[0][nb][8 * p + 2 * m + 1], tab);
                Bout[2 * ob + p][nb] = __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3]));
            }
    }
}

template <int NL, int D> constexpr int lds_bytes() {
    return (NL - 1) * wp_bytes(kDim) + wp_bytes(D) + ((NL - 1) * kDim + D) * 4 + (NL > 1 ? kTabBytes : 0);
}

// grid (wg_per_seq, n_heads, B).  NL layers, final width D (32 or 64).
template <int NL, int D>
__global__ __launch_bounds__(kMfThreads) void encode_mfma_kernel(const __bf16 *__restrict__ x, int64_t x_sb, int64_t x_sh, int64_t x_st,
                                                                 int x_heads, int n_heads, int T, int tiles_per_wg,
                                                                 const __bf16 *__restrict__ wblob, int64_t per_head,
                                                                 uint32_t *__restrict__ codes, int64_t c_sb, int64_t c_sh, int pos0,
                                                                 const int32_t *__restrict__ pos_dev) {
    // one static LDS block per instantiation: every address in it is a compile-time constant, so a table read needs no
    // address arithmetic beyond the scaled index (the rest folds into the instruction's offset field)
    __shared__ __align__(16) unsigned char smem[lds_bytes<NL, D>()];
    constexpr int NOBF = D / 32;
    constexpr int W = D / 32;
    // LDS: hidden weights (NL-1) x 32 KB | final weights | biases fp32 [(NL-1)*128 + D] | SiLU table (NL > 1)
    unsigned char *sp = smem;
    uint4 *wp_hidden[NL > 1 ? NL - 1 : 1];
#pragma unroll
    for (int l = 0; l < NL - 1; ++l) wp_hidden[l] = reinterpret_cast<uint4 *>(sp + l * wp_bytes(kDim));
    uint4 *wp_final = reinterpret_cast<uint4 *>(sp + (NL - 1) * wp_bytes(kDim));
    float *s_bias = reinterpret_cast<float *>(sp + (NL - 1) * wp_bytes(kDim) + wp_bytes(D));
    uint32_t *s_tab = reinterpret_cast<uint32_t *>(s_bias + (NL - 1) * kDim + D);

    const int head = blockIdx.y, b = blockIdx.z, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int in_head = head / (n_heads / x_heads);
    const __bf16 *wh = wblob + head * per_head;
    {
        const __bf16 *w = wh;
#pragma unroll
        for (int l = 0; l < NL - 1; ++l) {
            fill_weights(reinterpret_cast<uint2 *>(wp_hidden[l]), w, kDim, l > 0, tid);
            for (int i = tid; i < kDim; i += kMfThreads) s_bias[l * kDim + i] = (float)w[kDim * kDim + i];
            w += kDim * kDim + kDim;
        }
        fill_weights(reinterpret_cast<uint2 *>(wp_final), w, D, NL > 1, tid);
        for (int i = tid; i < D; i += kMfThreads) s_bias[(NL - 1) * kDim + i] = (float)w[D * kDim + i];
        if constexpr (NL > 1) fill_silu_table(s_tab, tid);
    }
    __syncthreads();

    const int half = lane >> 5, tl = lane & 31;
    const __bf16 *xb = x + b * x_sb + in_head * x_sh;
    const int64_t pos = pos_dev ? pos_dev[b] : pos0;
    uint32_t *cb = codes + b * c_sb + head * c_sh + pos * W;

    for (int it = 0; it < tiles_per_wg; ++it) {
        const int64_t t0 = ((int64_t)blockIdx.x * tiles_per_wg + it) * kTile + wave * kTokPerWave;
        if (t0 >= T) break;  // uniform per wave; no workgroup barrier below this point

        bf16x8 Ba[kKSteps][2], Bb[kKSteps][2];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            int64_t t = t0 + nb * 32 + tl;
            if (t >= T) t = T - 1;
            const uint4 *row = reinterpret_cast<const uint4 *>(xb + t * x_st);
#pragma unroll
            for (int ks = 0; ks < kKSteps; ++ks) Ba[ks][nb] = __builtin_bit_cast(bf16x8, row[2 * ks + half]);
        }
        if constexpr (NL >= 2) hidden_layer(wp_hidden[0], s_bias, s_tab, Ba, Bb, lane);
        if constexpr (NL >= 3) hidden_layer(wp_hidden[1], s_bias + kDim, s_tab, Bb, Ba, lane);

        f32x16 acc[NOBF][2];
        if constexpr (NL == 2) layer_mfma<NOBF>(wp_final, s_bias + (NL - 1) * kDim, Bb, acc, lane);
        else layer_mfma<NOBF>(wp_final, s_bias + (NL - 1) * kDim, Ba, acc, lane);

#pragma unroll
        for (int ob = 0; ob < NOBF; ++ob)
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                uint32_t part = 0;
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int i = 0; i < 4; ++i) part |= (acc[ob][nb][4 * q + i] > 0.0f ? 1u : 0u) << (8 * q + 4 * half + i);
                const uint32_t word = part | (uint32_t)__shfl_xor((int)part, 32);
                const int64_t t = t0 + nb * 32 + tl;
                if (half == 0 && t < T) cb[t * W + ob] = word;
            }
    }
}

template <int NL, int D>
int launch_mfma(dim3 grid, hipStream_t s, const __bf16 *x, int64_t x_sb, int64_t x_sh, int64_t x_st, int x_heads, int n_heads, int T,
                int tiles_per_wg, const __bf16 *w, int64_t per_head, uint32_t *codes, int64_t c_sb, int64_t c_sh, int pos0,
                const int32_t *pos_dev) {
    hipLaunchKernelGGL((encode_mfma_kernel<NL, D>), grid, dim3(kMfThreads), 0, s, x, x_sb, x_sh, x_st, x_heads, n_heads, T, tiles_per_wg, w,
                       per_head, codes, c_sb, c_sh, pos0, pos_dev);
    HA_CHECK_LAUNCH("encode_mfma_kernel");
    return HA_OK;
}

}  // namespace

extern "C" int ha_encode_pack_prefill(const void *x, int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_t, int B, int x_heads,
                                      int n_heads, int T, const void *weights_bf16, int n_layers, int head_dim, int int_dim,
                                      int final_dim, uint32_t *codes, int64_t c_stride_b, int64_t c_stride_h, int pos0,
                                      const int32_t *pos_dev, void *stream) {
    HA_REQUIRE(x && weights_bf16 && codes, HA_ERR_NULL_POINTER, "x/weights/codes is NULL");
    HA_REQUIRE(B > 0 && x_heads > 0 && n_heads > 0 && T > 0 && B <= 65535 && n_heads <= 65535, HA_ERR_BAD_SHAPE,
               "B, x_heads, n_heads, T must be positive (B, n_heads <= 65535)");
    HA_REQUIRE(n_heads % x_heads == 0, HA_ERR_BAD_SHAPE, "n_heads=%d not a multiple of x_heads=%d", n_heads, x_heads);
    HA_REQUIRE(n_layers >= 1 && n_layers <= 3, HA_ERR_BAD_SHAPE, "n_layers=%d, must be 1..3", n_layers);
    HA_REQUIRE(head_dim == kDim && int_dim == kDim, HA_ERR_BAD_SHAPE, "the MFMA encoder needs head_dim == int_dim == 128");
    HA_REQUIRE(final_dim == 32 || final_dim == 64, HA_ERR_BAD_SHAPE, "final_dim=%d, must be 32 or 64", final_dim);
    HA_REQUIRE(pos0 >= 0 && c_stride_b >= 0 && c_stride_h >= 0, HA_ERR_BAD_SHAPE, "negative position or stride");
    HA_REQUIRE(ha_aligned(x, 16) && x_stride_b % 8 == 0 && x_stride_h % 8 == 0 && x_stride_t % 8 == 0 && x_stride_t >= kDim,
               HA_ERR_MISALIGNED, "x rows must be 16-byte aligned bf16 rows of 128");
    HA_REQUIRE(ha_aligned(weights_bf16, 8) && ha_aligned(codes, 4), HA_ERR_MISALIGNED, "weights/codes misaligned");
    {
        // tokens a (sequence, head) row of the code buffer spans, from its strides (a row nobody follows: unbounded)
        const int W = final_dim / 32;
        const int64_t c_cap = c_stride_h > 0 ? c_stride_h / W : (c_stride_b > 0 ? c_stride_b / W : INT64_MAX);
        HA_REQUIRE(pos_dev || (int64_t)pos0 + T <= c_cap, HA_ERR_BAD_SHAPE, "pos0 + T = %lld exceeds the %lld tokens of a code row",
                   (long long)pos0 + T, (long long)c_cap);
    }
    int st = ha_require_device();
    if (st) return st;

    const int64_t per_head = ha_usa_packed_floats(n_layers, head_dim, int_dim, final_dim);
    const int tiles = (T + kTile - 1) / kTile;
    // enough workgroups to fill 256 CUs a few times over, but several tiles each so the LDS fill (weights, table) amortises
    int tiles_per_wg = 1;
    while (tiles_per_wg < 16 && (int64_t)B * n_heads * ((tiles + 2 * tiles_per_wg - 1) / (2 * tiles_per_wg)) >= 1024) tiles_per_wg *= 2;
    const dim3 grid((tiles + tiles_per_wg - 1) / tiles_per_wg, n_heads, B);
    hipStream_t s = (hipStream_t)stream;
    const __bf16 *xp = (const __bf16 *)x, *wp = (const __bf16 *)weights_bf16;
#define HA_MFMA_CASE(NL_, D_)                                                                                                    \
    if (n_layers == NL_ && final_dim == D_)                                                                                      \
        return launch_mfma<NL_, D_>(grid, s, xp, x_stride_b, x_stride_h, x_stride_t, x_heads, n_heads, T, tiles_per_wg, wp,      \
                                    per_head, codes, c_stride_b, c_stride_h, pos0, pos_dev);
    HA_MFMA_CASE(3, 32)
    HA_MFMA_CASE(3, 64)
    HA_MFMA_CASE(2, 32)
    HA_MFMA_CASE(2, 64)
    HA_MFMA_CASE(1, 32)
    HA_MFMA_CASE(1, 64)
#undef HA_MFMA_CASE
    HA_FAIL(HA_ERR_BAD_SHAPE, "unsupported MLP shape");
}
