// Hash-MLP encode into packed sign codes (gfx950): the scalar-FMA kernel used at decode time
// (a handful of new keys and queries per step) and as the exact-arithmetic path.
//
// One workgroup = one MLP head x a tile of ROWS (1, 2 or 4) input rows, 512 threads.  A decode step has little
// work and a long dependency chain (three layers), so the kernel is built for latency: every thread
// owns one output neuron and one quarter of the reduction (thread = (o, segment)), fetches its 32
// weights of the NEXT layer before finishing the current one, and the quarters meet in LDS.
// Weights are read transposed ([in][out], coalesced over o).
//
// The arithmetic is fixed, so results are reproducible bit for bit (the C oracle mirrors it):
//   p_s = 0; for k ascending in segment s (a quarter of the inputs): p_s = fmaf(x[k], W[k][o], p_s)
//   y   = (((bias[o] + p_0) + p_1) + p_2) + p_3;          SiLU(y) = y / (1 + expf(-y))
// HA_ARITH_BF16 additionally rounds the input, every Linear output and every SiLU output to bf16,
// which is what a hash module kept in bf16 computes.
#include "ha_common.h"

namespace {

constexpr int kEncThreads = 512;
constexpr int kSeg = 4;        // reduction segments per output
constexpr int kMaxRows = 4;    // most input rows per workgroup (template parameter ROWS: 1, 2 or 4)
constexpr int kMaxDim = 256;
constexpr int kMaxPerSeg = kMaxDim / kSeg;

// One input tensor with its MLP heads and its destination in a code buffer.
struct EncSide {
    const void *x;
    int x_dtype;
    int64_t x_sb, x_sh, x_st;
    int x_heads, n_heads;
    const float *weights;
    uint32_t *codes;
    int64_t c_sb, c_sh;
    int pos0;
    const int32_t *pos_dev;
    float *logits;
    int pos_bias;  // added to pos_dev[b] (-1 when pos_dev holds sequence lengths and the row is the last one)
    int x_at_pos;  // T = 1: x is a cache and the row to hash sits at the position the code is written to
    // tokens a (sequence, head) row of `codes` can hold, from its strides: a position read from device memory that lies
    // beyond it is written nowhere instead of into the next row (0: unknown, no check)
    int64_t pos_cap;
};
// Up to two sides share one launch (the new keys and the queries of a decode step): blockIdx.y runs over
// the heads of side 0, then those of side 1.
// Optional front end of a decode step (T = 1, 128-wide heads): side 0 / side 1 read the raw key / query rows of a fused
// QKV projection, rotate them (rotate-half RoPE at the sequence's position), write the rotated key and the value row
// into the caches and the rotated query to q_out, and hash what they wrote.
struct EncRope {
    const float *inv_freq;  // [64]; nullptr (and no cos_tab): no front end, the sides read finished rows
    // the rotation given as tables instead: cos, sin [B, 128] of the element type (row stride cs_sb elements, 0 shares one
    // row), as transformers hands them to its attention layers; the arithmetic then follows its apply_rotary_pos_emb,
    // every product and the sum rounded to the element type
    const void *cos_tab, *sin_tab;
    int64_t cs_sb;
    const void *v_src;      // raw value rows [B, Hkv, 128], batch stride v_sb
    int64_t v_sb;
    void *q_out;            // [B, H, 128]
    void *k_cache, *v_cache;
    int64_t kv_sb, kv_sh, kv_ss;
    int pos;
    const int32_t *pos_dev;
    int64_t cache_len;      // tokens a (sequence, head) row of the caches holds: a device-side position beyond it writes nothing
};
struct EncArgs {
    EncSide side[2];
    int B, T, n_layers, d_in, d_int, d_out, arith;
    int64_t per_head;
    EncRope rope;
};

// Position of W[o][k] (k = input, o = output) inside a layer's block of the packed blob: inputs in groups of four,
// [in / 4][out][4], when the layer has a multiple of 16 inputs; plain W^T [in][out] otherwise.
__device__ __forceinline__ int64_t weight_index(int in, int out, int k, int o) {
    return (in & 15) == 0 ? ((int64_t)(k >> 2) * out + o) * 4 + (k & 3) : (int64_t)k * out + o;
}

// NL_/DIN_/DINT_/DOUT_ fix the MLP shape at compile time (0 = read it from the arguments).  The usual
// shapes (128 -> 128 [-> 128] -> 32|64) are instantiated: with constant trip counts the weight fetch is
// 72 plain loads and the kernel is a few hundred instructions, which matters because a decode step is
// bound by this kernel's dependent-issue latency, not by its throughput.
template <int NL_, int DIN_, int DINT_, int DOUT_, int ROWS>
__global__ __launch_bounds__(kEncThreads) void encode_pack_kernel(const EncArgs a) {
    constexpr int kRows = ROWS;
    __shared__ __align__(16) float s_act[2][kRows][kMaxDim];
    __shared__ float s_part[kSeg][kRows][kMaxDim];
    // Workgroups go to the 8 XCDs round-robin in linear launch order.  When the grid divides evenly, renumber them so
    // that each XCD owns whole heads: the tiles of a head then share one L2 and its weights leave HBM once, not once
    // per tile.
    int bx = blockIdx.x, by = blockIdx.y;
    {
        const int n = gridDim.x * gridDim.y;
        if (n % 8 == 0 && gridDim.x > 1) {
            const int lin = blockIdx.x + gridDim.x * blockIdx.y;
            const int v = (lin % 8) * (n / 8) + lin / 8;
            bx = v % gridDim.x;
            by = v / gridDim.x;
        }
    }
    const bool second = by >= a.side[0].n_heads;
    const EncSide &sd = a.side[second ? 1 : 0];
    const int head = second ? by - a.side[0].n_heads : by;
    const int tile = bx, tid = threadIdx.x;
    const void *__restrict__ x = sd.x;
    const int x_dtype = sd.x_dtype;
    const int64_t x_sb = sd.x_sb, x_sh = sd.x_sh, x_st = sd.x_st;
    const int n_heads = sd.n_heads, T = a.T, arith = a.arith;
    const int n_layers = NL_ ? NL_ : a.n_layers, d_in = DIN_ ? DIN_ : a.d_in, d_int = DINT_ ? DINT_ : a.d_int,
              d_out = DOUT_ ? DOUT_ : a.d_out;
    const float *__restrict__ weights = sd.weights;
    const int64_t per_head = a.per_head;
    uint32_t *__restrict__ codes = sd.codes;
    const int64_t c_sb = sd.c_sb, c_sh = sd.c_sh;
    const int pos0 = sd.pos0;
    const int32_t *__restrict__ pos_dev = sd.pos_dev;
    float *__restrict__ logits = sd.logits;
    const int in_head = head / (n_heads / sd.x_heads);
    const int n_rows = a.B * T;  // < 2^31, validated on the host
    const int row0 = tile * kRows;

    // ---- every weight this thread will need, for all layers, is requested before anything else: the
    // (o, seg) of a layer with `out` outputs is (tid % out, tid / out) for the first out*kSeg threads.
    // Layers wider than 128 outputs do not fit one (o, seg) per thread and stream their weights instead.
    const float *wl[3];
    int l_in[3], l_out[3];
    {
        const float *w = weights + head * per_head;
        for (int l = 0; l < 3; ++l) {
            l_in[l] = (l == 0) ? d_in : d_int;
            l_out[l] = (l == n_layers - 1) ? d_out : d_int;
            wl[l] = w;
            if (l < n_layers) w += (int64_t)l_in[l] * l_out[l] + l_out[l];
        }
    }
    // the inputs are requested first and parked in registers: memory returns loads in order, and the first layer then
    // needs only them and its own weights, not the whole weight prefetch
    constexpr int kXIter = (kRows * kMaxDim + kEncThreads - 1) / kEncThreads;
    float xs[kXIter];
    const EncRope &rp = a.rope;
    float xpair[kXIter];  // rope: the other element of the rotation pair
#pragma unroll
    for (int it = 0; it < kXIter; ++it) {
        const int i = tid + it * kEncThreads;
        xs[it] = 0.f;
        xpair[it] = 0.f;
        if (i < kRows * d_in) {
            const int r = i / d_in, e = i % d_in;
            const int row = row0 + r;
            if (row < n_rows) {
                const int b = row / T, t = row % T;
                int64_t at = t;
                if (sd.x_at_pos) at = max(pos_dev ? pos_dev[b] + sd.pos_bias : pos0, 0);  // an empty sequence hashes row 0, written nowhere
                xs[it] = ha_load_elem(x, b * x_sb + in_head * x_sh + at * x_st + e, x_dtype);
                if (rp.inv_freq || rp.cos_tab) xpair[it] = ha_load_elem(x, b * x_sb + in_head * x_sh + t * x_st + (e ^ 64), x_dtype);
            }
        }
    }
    if (rp.inv_freq || rp.cos_tab) {
        // rotate-half RoPE of the row this thread element belongs to (T = 1, d_in = 128): the angle in fp32, the table
        // rounded to the element type as transformers builds it, the result rounded as the cache stores it.  The first
        // code head of a KV head writes the key and copies the value row; every query head writes its query.
        const bool writes_kv = !second && head % (n_heads / sd.x_heads) == 0;
#pragma unroll
        for (int it = 0; it < kXIter; ++it) {
            const int i = tid + it * kEncThreads;
            if (i >= kRows * d_in) continue;
            const int r = i / d_in, e = i % d_in, b = row0 + r;
            if (b >= n_rows) continue;
            const int p = rp.pos_dev ? rp.pos_dev[b] : rp.pos;
            float y;
            if (rp.cos_tab) {
                const float c = ha_load_elem(rp.cos_tab, b * rp.cs_sb + e, x_dtype), sn = ha_load_elem(rp.sin_tab, b * rp.cs_sb + e, x_dtype);
                const float direct = ha_round_to(__fmul_rn(xs[it], c), x_dtype), crossed = ha_round_to(__fmul_rn(xpair[it], sn), x_dtype);
                y = ha_round_to(__fadd_rn(direct, e < 64 ? -crossed : crossed), x_dtype);
            } else {
                const float ang = (float)p * rp.inv_freq[e & 63];
                const float c = ha_round_to(cosf(ang), x_dtype), sn = ha_round_to(sinf(ang), x_dtype);
                y = ha_round_to(e < 64 ? xs[it] * c - xpair[it] * sn : xs[it] * c + xpair[it] * sn, x_dtype);
            }
            xs[it] = y;
            if (second) {
                ha_store_elem(rp.q_out, ((int64_t)b * n_heads + head) * HA_HEAD_DIM + e, y, x_dtype);
            } else if (writes_kv && p >= 0 && p < rp.cache_len) {
                const int64_t dst = b * rp.kv_sb + (int64_t)in_head * rp.kv_sh + (int64_t)p * rp.kv_ss + e;
                ha_store_elem(rp.k_cache, dst, y, x_dtype);
                ha_store_elem(rp.v_cache, dst, ha_load_elem(rp.v_src, b * rp.v_sb + (int64_t)in_head * HA_HEAD_DIM + e, x_dtype), x_dtype);
            }
        }
    }
    float wreg[3][kMaxPerSeg];
#pragma unroll
    for (int l = 0; l < 3; ++l) {
        const bool fits = l < n_layers && l_out[l] * kSeg <= kEncThreads && l_in[l] / kSeg <= kMaxPerSeg;
        const bool active = fits && tid < l_out[l] * kSeg;
        const int out = l < n_layers ? l_out[l] : 1, per = l < n_layers ? l_in[l] / kSeg : 0;
        const int o = tid % out, seg = tid / out;
        if ((l_in[l] & 15) == 0) {
            // inputs in groups of four (ha_usa_weight_index): the 64 lanes of a wave, consecutive outputs of one
            // segment, fetch 1 KiB of consecutive memory per request - a quarter of the requests of a dword walk
            const float4 *w4 = reinterpret_cast<const float4 *>(wl[l]) + (int64_t)(seg * per / 4) * out + o;
#pragma unroll
            for (int i4 = 0; i4 < kMaxPerSeg / 4; ++i4) {
                const float4 v = (active && 4 * i4 < per) ? w4[(int64_t)i4 * out] : float4{0.f, 0.f, 0.f, 0.f};
                wreg[l][4 * i4 + 0] = v.x;
                wreg[l][4 * i4 + 1] = v.y;
                wreg[l][4 * i4 + 2] = v.z;
                wreg[l][4 * i4 + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int i = 0; i < kMaxPerSeg; ++i) wreg[l][i] = (active && i < per) ? wl[l][(int64_t)(seg * per + i) * out + o] : 0.f;
        }
    }
#pragma unroll
    for (int it = 0; it < kXIter; ++it) {
        const int i = tid + it * kEncThreads;
        if (i < kRows * d_in) s_act[0][i / d_in][i % d_in] = arith == HA_ARITH_BF16 ? ha_round_bf16(xs[it]) : xs[it];
    }
    __syncthreads();

    int cur = 0;
#pragma unroll
    for (int l = 0; l < 3; ++l) {
        if (l >= n_layers) break;
        const int in = l_in[l], out = l_out[l];
        const int per = in / kSeg;
        const float *Wt = wl[l], *bias = wl[l] + (int64_t)in * out;
        const bool fits = out * kSeg <= kEncThreads && per <= kMaxPerSeg;

        if (fits) {
            if (tid < out * kSeg) {
                const int o = tid % out, seg = tid / out;
                float p[kRows];
#pragma unroll
                for (int r = 0; r < kRows; ++r) p[r] = 0.f;
                if ((per & 3) == 0) {  // 128-bit LDS reads of four consecutive inputs
#pragma unroll
                    for (int i = 0; i < kMaxPerSeg; i += 4) {
                        if (i < per) {
#pragma unroll
                            for (int r = 0; r < kRows; ++r) {
                                const float4 xv = *reinterpret_cast<const float4 *>(&s_act[cur][r][seg * per + i]);
                                p[r] = fmaf(xv.x, wreg[l][i], p[r]);
                                p[r] = fmaf(xv.y, wreg[l][i + 1], p[r]);
                                p[r] = fmaf(xv.z, wreg[l][i + 2], p[r]);
                                p[r] = fmaf(xv.w, wreg[l][i + 3], p[r]);
                            }
                        }
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < kMaxPerSeg; ++i) {
                        if (i < per) {
#pragma unroll
                            for (int r = 0; r < kRows; ++r) p[r] = fmaf(s_act[cur][r][seg * per + i], wreg[l][i], p[r]);
                        }
                    }
                }
#pragma unroll
                for (int r = 0; r < kRows; ++r) s_part[seg][r][o] = p[r];
            }
        } else {
            for (int t2 = tid; t2 < out * kSeg; t2 += kEncThreads) {
                const int o = t2 % out, seg = t2 / out;
                float p[kRows];
#pragma unroll
                for (int r = 0; r < kRows; ++r) p[r] = 0.f;
                for (int i = 0; i < per; ++i) {
                    const float wv = Wt[weight_index(in, out, seg * per + i, o)];
#pragma unroll
                    for (int r = 0; r < kRows; ++r) p[r] = fmaf(s_act[cur][r][seg * per + i], wv, p[r]);
                }
#pragma unroll
                for (int r = 0; r < kRows; ++r) s_part[seg][r][o] = p[r];
            }
        }
        __syncthreads();
        for (int t2 = tid; t2 < out * kRows; t2 += kEncThreads) {
            const int o = t2 % out, r = t2 / out;
            float a = bias[o];
#pragma unroll
            for (int sgm = 0; sgm < kSeg; ++sgm) a += s_part[sgm][r][o];
            if (arith == HA_ARITH_BF16) a = ha_round_bf16(a);
            if (l + 1 < n_layers) {
                a = a / (1.0f + expf(-a));
                if (arith == HA_ARITH_BF16) a = ha_round_bf16(a);
            }
            s_act[cur ^ 1][r][o] = a;
        }
        __syncthreads();
        cur ^= 1;
    }

    // sign bits -> words.  Wave w packs output dims [64w, 64w+64): ballot low half = word 2w, high half = word 2w+1.
    const int W = d_out / 32;
    const int wave = tid >> 6, lane = tid & 63;
    for (int r = 0; r < kRows; ++r) {
        const int row = row0 + r;
        if (row >= n_rows) break;  // uniform
        const int b = row / T, t = row % T;
        const bool bit = tid < d_out && s_act[cur][r][tid] > 0.0f;
        const uint64_t bal = __ballot(bit);
        if (logits && tid < d_out) logits[(((int64_t)b * n_heads + head) * T + t) * d_out + tid] = s_act[cur][r][tid];
        const int64_t pos = (int64_t)(pos_dev ? pos_dev[b] + sd.pos_bias : pos0) + t;
        uint32_t *c = codes + b * c_sb + head * c_sh + pos * W;
        const bool inside = pos >= 0 && (sd.pos_cap == 0 || pos < sd.pos_cap);
        if (lane == 0 && wave * 2 < W && inside) c[wave * 2] = (uint32_t)bal;
        if (lane == 32 && wave * 2 + 1 < W && inside) c[wave * 2 + 1] = (uint32_t)(bal >> 32);
    }
}

int validate_encode(const void *x, int B, int x_heads, int n_heads, int T, const void *weights, int n_layers, int head_dim,
                    int int_dim, int final_dim, const uint32_t *codes, int64_t c_sb, int64_t c_sh, int pos0,
                    const int32_t *pos_dev) {
    HA_REQUIRE(x && weights && codes, HA_ERR_NULL_POINTER, "x/weights/codes is NULL");
    HA_REQUIRE(B > 0 && x_heads > 0 && n_heads > 0 && T > 0, HA_ERR_BAD_SHAPE, "B, x_heads, n_heads, T must be positive");
    HA_REQUIRE(n_heads <= 65535, HA_ERR_BAD_SHAPE, "n_heads is limited to 65535");
    HA_REQUIRE(n_heads % x_heads == 0, HA_ERR_BAD_SHAPE, "n_heads=%d not a multiple of x_heads=%d", n_heads, x_heads);
    HA_REQUIRE(n_layers >= 1 && n_layers <= 3, HA_ERR_BAD_SHAPE, "n_layers=%d, must be 1..3", n_layers);
    HA_REQUIRE(head_dim > 0 && head_dim <= kMaxDim && int_dim > 0 && int_dim <= kMaxDim && head_dim % kSeg == 0 && int_dim % kSeg == 0,
               HA_ERR_BAD_SHAPE, "head_dim and int_dim must be multiples of %d in 1..%d", kSeg, kMaxDim);
    HA_REQUIRE(final_dim == 32 || final_dim == 64, HA_ERR_BAD_SHAPE, "final_dim=%d, must be 32 or 64", final_dim);
    HA_REQUIRE(pos0 >= 0, HA_ERR_BAD_SHAPE, "pos0 must be non-negative");
    HA_REQUIRE(c_sh >= 0 && c_sb >= 0, HA_ERR_BAD_SHAPE, "negative code stride");
    {
        // positions given by the host are checked against the tokens a (sequence, head) row of the code buffer spans (from
        // its strides, as launch_encode derives pos_cap); only positions read from device memory are left to the kernel
        const int64_t span = n_heads > 1 ? c_sh : (B > 1 ? c_sb : 0), cap = span > 0 ? span / (final_dim / 32) : 0;
        HA_REQUIRE(pos_dev || cap == 0 || (int64_t)pos0 + T <= cap, HA_ERR_BAD_SHAPE,
                   "positions %d..%lld lie beyond the %lld tokens a code row spans", pos0, (long long)pos0 + T - 1, (long long)cap);
    }
    HA_REQUIRE(ha_aligned(codes, 4) && ha_aligned(weights, 16), HA_ERR_MISALIGNED, "codes must be 4-byte, weights 16-byte aligned");
    return HA_OK;
}

// Rows per workgroup: a decode step's launch is bound by the latency of one workgroup, and fewer rows mean less work on
// that path (three layers, back to back: 7.6 us with four rows, 5.0 us with one at 4 sequences); but every workgroup
// fetches its head's weights, so the grid is kept within 1.5 workgroups per CU (640 workgroups of one row at 16
// sequences: 9.2 us against 7.1 us for 320 of two).  Bulk encodes keep four rows.
int launch_encode(const EncArgs &a_in, int64_t n_rows, int heads, hipStream_t s) {
    EncArgs a = a_in;
    // capacity of a code row from its strides (rows of [B, heads, S_cap, W] are c_sh = S_cap * W words apart)
    const int W = a.d_out / 32;
    for (int i = 0; i < 2; ++i) {
        const int64_t span = a.side[i].n_heads > 1 ? a.side[i].c_sh : (a.B > 1 ? a.side[i].c_sb : 0);
        a.side[i].pos_cap = span > 0 ? span / W : 0;
    }
    int rows = kMaxRows;
    for (int r = 1; r < kMaxRows; r *= 2)
        if (((n_rows + r - 1) / r) * heads <= 384) {
            rows = r;
            break;
        }
    const dim3 grid((unsigned)((n_rows + rows - 1) / rows), (unsigned)heads);
#define HA_ENC_ROWS(NL_, DIN_, DINT_, DOUT_)                                                                                \
    do {                                                                                                                    \
        if (rows == 1) hipLaunchKernelGGL((encode_pack_kernel<NL_, DIN_, DINT_, DOUT_, 1>), grid, dim3(kEncThreads), 0, s, a);      \
        else if (rows == 2) hipLaunchKernelGGL((encode_pack_kernel<NL_, DIN_, DINT_, DOUT_, 2>), grid, dim3(kEncThreads), 0, s, a); \
        else hipLaunchKernelGGL((encode_pack_kernel<NL_, DIN_, DINT_, DOUT_, kMaxRows>), grid, dim3(kEncThreads), 0, s, a);         \
        HA_CHECK_LAUNCH("encode_pack_kernel");                                                                              \
        return HA_OK;                                                                                                       \
    } while (0)
#define HA_ENC_CASE(NL_, DOUT_) \
    if (a.n_layers == NL_ && a.d_in == 128 && (NL_ == 1 || a.d_int == 128) && a.d_out == DOUT_) HA_ENC_ROWS(NL_, 128, 128, DOUT_)
    HA_ENC_CASE(3, 32);
    HA_ENC_CASE(3, 64);
    HA_ENC_CASE(2, 32);
    HA_ENC_CASE(2, 64);
    HA_ENC_CASE(1, 32);
    HA_ENC_CASE(1, 64);
#undef HA_ENC_CASE
    HA_ENC_ROWS(0, 0, 0, 0);
#undef HA_ENC_ROWS
}

}  // namespace

extern "C" {

int64_t ha_usa_packed_floats(int n_layers, int head_dim, int int_dim, int final_dim) {
    if (n_layers < 1 || n_layers > 3 || head_dim <= 0 || int_dim <= 0 || final_dim <= 0) return 0;
    int64_t n = 0;
    for (int l = 0; l < n_layers; ++l) {
        const int64_t in = (l == 0) ? head_dim : int_dim, out = (l == n_layers - 1) ? final_dim : int_dim;
        n += in * out + out;
    }
    return n;
}

int ha_encode_pack(const void *x, int x_dtype, int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_t, int B, int x_heads,
                   int n_heads, int T, const float *weights, int n_layers, int head_dim, int int_dim, int final_dim, int arith,
                   uint32_t *codes, int64_t c_stride_b, int64_t c_stride_h, int pos0, const int32_t *pos_dev, float *logits,
                   void *stream) {
    int st = validate_encode(x, B, x_heads, n_heads, T, weights, n_layers, head_dim, int_dim, final_dim, codes, c_stride_b,
                             c_stride_h, pos0, pos_dev);
    if (st) return st;
    HA_REQUIRE(x_dtype == HA_F32 || x_dtype == HA_BF16 || x_dtype == HA_F16, HA_ERR_BAD_DTYPE, "x_dtype %d", x_dtype);
    HA_REQUIRE(arith == HA_ARITH_F32 || arith == HA_ARITH_BF16, HA_ERR_BAD_DTYPE, "arith %d", arith);
    HA_REQUIRE((int64_t)B * T < 2147483647LL - kMaxRows, HA_ERR_BAD_SHAPE, "too many rows for one launch");
    if ((st = ha_require_device())) return st;
    EncArgs a = {};
    a.side[0] = EncSide{x, x_dtype, x_stride_b, x_stride_h, x_stride_t, x_heads, n_heads, weights, codes, c_stride_b, c_stride_h,
                        pos0, pos_dev, logits};
    a.side[1] = a.side[0];
    a.side[1].n_heads = 0;
    a.B = B; a.T = T; a.n_layers = n_layers; a.d_in = head_dim; a.d_int = int_dim; a.d_out = final_dim; a.arith = arith;
    a.per_head = ha_usa_packed_floats(n_layers, head_dim, int_dim, final_dim);
    return launch_encode(a, (int64_t)B * T, n_heads, (hipStream_t)stream);
}

int ha_encode_step(const void *k_new, int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_t, const void *q, int64_t q_stride_b,
                   int64_t q_stride_h, int x_dtype, int B, int Hkv, int Hc, int H, int T_new, const float *weights_k,
                   const float *weights_q, int n_layers, int head_dim, int int_dim, int final_dim, int arith, uint32_t *kcodes,
                   int64_t kc_stride_b, int64_t kc_stride_h, int pos0, const int32_t *pos_dev, uint32_t *qcodes, void *stream) {
    int st = validate_encode(k_new, B, Hkv, Hc, T_new, weights_k, n_layers, head_dim, int_dim, final_dim, kcodes, kc_stride_b,
                             kc_stride_h, pos0, pos_dev);
    if (st) return st;
    HA_REQUIRE(q && weights_q && qcodes, HA_ERR_NULL_POINTER, "q/weights_q/qcodes is NULL");
    HA_REQUIRE(H > 0 && H + Hc <= 65535, HA_ERR_BAD_SHAPE, "H must be positive and H + Hc <= 65535");
    HA_REQUIRE(T_new == 1, HA_ERR_BAD_SHAPE, "ha_encode_step encodes one new key per sequence (T_new=%d)", T_new);
    HA_REQUIRE(x_dtype == HA_F32 || x_dtype == HA_BF16 || x_dtype == HA_F16, HA_ERR_BAD_DTYPE, "x_dtype %d", x_dtype);
    HA_REQUIRE(arith == HA_ARITH_F32 || arith == HA_ARITH_BF16, HA_ERR_BAD_DTYPE, "arith %d", arith);
    if ((st = ha_require_device())) return st;
    const int W = final_dim / 32;
    EncArgs a = {};
    a.side[0] = EncSide{k_new, x_dtype, k_stride_b, k_stride_h, k_stride_t, Hkv, Hc, weights_k, kcodes, kc_stride_b, kc_stride_h,
                        pos0, pos_dev, nullptr};
    a.side[1] = EncSide{q, x_dtype, q_stride_b, q_stride_h, (int64_t)head_dim, H, H, weights_q, qcodes, (int64_t)H * W, (int64_t)W,
                        0, nullptr, nullptr};
    a.B = B; a.T = 1; a.n_layers = n_layers; a.d_in = head_dim; a.d_int = int_dim; a.d_out = final_dim; a.arith = arith;
    a.per_head = ha_usa_packed_floats(n_layers, head_dim, int_dim, final_dim);
    return launch_encode(a, B, Hc + H, (hipStream_t)stream);
}

int ha_encode_step_cached(const void *k_cache, int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_s, const void *q,
                          int64_t q_stride_b, int64_t q_stride_h, int x_dtype, int B, int Hkv, int Hc, int H,
                          const int32_t *seq_lens, const float *weights_k, const float *weights_q, int n_layers, int head_dim,
                          int int_dim, int final_dim, int arith, uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h,
                          uint32_t *qcodes, void *stream) {
    int st = validate_encode(k_cache, B, Hkv, Hc, 1, weights_k, n_layers, head_dim, int_dim, final_dim, kcodes, kc_stride_b,
                             kc_stride_h, 0, seq_lens);
    if (st) return st;
    HA_REQUIRE(q && weights_q && qcodes && seq_lens, HA_ERR_NULL_POINTER, "q/weights_q/qcodes/seq_lens is NULL");
    HA_REQUIRE(H > 0 && H + Hc <= 65535, HA_ERR_BAD_SHAPE, "H must be positive and H + Hc <= 65535");
    HA_REQUIRE(k_stride_s >= head_dim, HA_ERR_BAD_SHAPE, "cache rows overlap: k_stride_s=%lld < head_dim=%d", (long long)k_stride_s,
               head_dim);
    HA_REQUIRE(x_dtype == HA_F32 || x_dtype == HA_BF16 || x_dtype == HA_F16, HA_ERR_BAD_DTYPE, "x_dtype %d", x_dtype);
    HA_REQUIRE(arith == HA_ARITH_F32 || arith == HA_ARITH_BF16, HA_ERR_BAD_DTYPE, "arith %d", arith);
    if ((st = ha_require_device())) return st;
    const int W = final_dim / 32;
    EncArgs a = {};
    a.side[0] = EncSide{k_cache, x_dtype, k_stride_b, k_stride_h, k_stride_s, Hkv, Hc, weights_k, kcodes, kc_stride_b, kc_stride_h,
                        0, seq_lens, nullptr, -1, 1};
    a.side[1] = EncSide{q, x_dtype, q_stride_b, q_stride_h, (int64_t)head_dim, H, H, weights_q, qcodes, (int64_t)H * W, (int64_t)W,
                        0, nullptr, nullptr, 0, 0};
    a.B = B; a.T = 1; a.n_layers = n_layers; a.d_in = head_dim; a.d_int = int_dim; a.d_out = final_dim; a.arith = arith;
    a.per_head = ha_usa_packed_floats(n_layers, head_dim, int_dim, final_dim);
    return launch_encode(a, B, Hc + H, (hipStream_t)stream);
}

static int rope_encode_step_impl(const void *qkv, int64_t qkv_stride_b, int x_dtype, int B, int H, int Hkv, int Hc, int pos,
                        const int32_t *pos_dev, const float *inv_freq, const void *cos_tab, const void *sin_tab, int64_t cs_sb,
                        void *q_out, void *k_cache, void *v_cache,
                        int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, int64_t cache_len, const float *weights_k,
                        const float *weights_q, int n_layers, int head_dim, int int_dim, int final_dim, int arith, uint32_t *kcodes,
                        int64_t kc_stride_b, int64_t kc_stride_h, uint32_t *qcodes, void *stream) {
    HA_REQUIRE(qkv && (inv_freq || (cos_tab && sin_tab)) && q_out && k_cache && v_cache, HA_ERR_NULL_POINTER,
               "qkv / rotation (inv_freq, or cos and sin) / q_out / k_cache / v_cache is NULL");
    HA_REQUIRE(cs_sb >= 0 && (!cos_tab || (ha_aligned(cos_tab, 2) && ha_aligned(sin_tab, 2))), HA_ERR_BAD_SHAPE, "bad cos/sin table stride or alignment");
    HA_REQUIRE(H > 0 && Hkv > 0 && Hc > 0, HA_ERR_BAD_SHAPE, "H, Hkv, Hc must be positive");
    int st = validate_encode(qkv, B, Hkv, Hc, 1, weights_k, n_layers, head_dim, int_dim, final_dim, kcodes, kc_stride_b, kc_stride_h,
                             pos_dev ? 0 : pos, pos_dev);
    if (st) return st;
    HA_REQUIRE(weights_q && qcodes, HA_ERR_NULL_POINTER, "weights_q/qcodes is NULL");
    HA_REQUIRE(head_dim == HA_HEAD_DIM, HA_ERR_BAD_SHAPE, "the rotary front end needs 128-wide heads");
    HA_REQUIRE(H + Hc <= 65535, HA_ERR_BAD_SHAPE, "H + Hc <= 65535");
    HA_REQUIRE(x_dtype == HA_F32 || x_dtype == HA_BF16 || x_dtype == HA_F16, HA_ERR_BAD_DTYPE, "x_dtype %d", x_dtype);
    HA_REQUIRE(arith == HA_ARITH_F32 || arith == HA_ARITH_BF16, HA_ERR_BAD_DTYPE, "arith %d", arith);
    HA_REQUIRE(qkv_stride_b >= (int64_t)(H + 2 * Hkv) * HA_HEAD_DIM, HA_ERR_BAD_SHAPE, "qkv row stride shorter than (H + 2 Hkv) * 128");
    HA_REQUIRE(cache_len > 0 && (pos_dev || (pos >= 0 && pos < cache_len)), HA_ERR_BAD_SHAPE, "position %d outside the cache of %lld tokens",
               pos, (long long)cache_len);
    HA_REQUIRE(kv_stride_s >= HA_HEAD_DIM && kv_stride_h > 0 && kv_stride_b > 0, HA_ERR_BAD_SHAPE, "cache strides smaller than a row");
    if ((st = ha_require_device())) return st;
    const int W = final_dim / 32;
    const int64_t eb = x_dtype == HA_F32 ? 4 : 2;
    EncArgs a = {};
    // raw rows of the fused projection: queries at column 0, keys behind the H query heads, values behind the keys
    a.side[0] = EncSide{(const char *)qkv + (int64_t)H * HA_HEAD_DIM * eb, x_dtype, qkv_stride_b, (int64_t)HA_HEAD_DIM, (int64_t)HA_HEAD_DIM, Hkv, Hc,
                        weights_k, kcodes, kc_stride_b, kc_stride_h, pos, pos_dev, nullptr};
    a.side[1] = EncSide{qkv, x_dtype, qkv_stride_b, (int64_t)HA_HEAD_DIM, (int64_t)HA_HEAD_DIM, H, H, weights_q, qcodes, (int64_t)H * W,
                        (int64_t)W, 0, nullptr, nullptr};
    a.B = B; a.T = 1; a.n_layers = n_layers; a.d_in = head_dim; a.d_int = int_dim; a.d_out = final_dim; a.arith = arith;
    a.per_head = ha_usa_packed_floats(n_layers, head_dim, int_dim, final_dim);
    a.rope = EncRope{inv_freq, cos_tab, sin_tab, cs_sb, (const char *)qkv + (int64_t)(H + Hkv) * HA_HEAD_DIM * eb, qkv_stride_b, q_out, k_cache,
                     v_cache, kv_stride_b, kv_stride_h, kv_stride_s, pos, pos_dev, cache_len};
    return launch_encode(a, B, Hc + H, (hipStream_t)stream);
}

int ha_rope_encode_step(const void *qkv, int64_t qkv_stride_b, int x_dtype, int B, int H, int Hkv, int Hc, int pos,
                        const int32_t *pos_dev, const float *inv_freq, void *q_out, void *k_cache, void *v_cache,
                        int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, int64_t cache_len, const float *weights_k,
                        const float *weights_q, int n_layers, int head_dim, int int_dim, int final_dim, int arith, uint32_t *kcodes,
                        int64_t kc_stride_b, int64_t kc_stride_h, uint32_t *qcodes, void *stream) {
    HA_REQUIRE(inv_freq, HA_ERR_NULL_POINTER, "inv_freq is NULL");
    return rope_encode_step_impl(qkv, qkv_stride_b, x_dtype, B, H, Hkv, Hc, pos, pos_dev, inv_freq, nullptr, nullptr, 0, q_out, k_cache, v_cache,
                                 kv_stride_b, kv_stride_h, kv_stride_s, cache_len, weights_k, weights_q, n_layers, head_dim, int_dim, final_dim,
                                 arith, kcodes, kc_stride_b, kc_stride_h, qcodes, stream);
}

int ha_rope_encode_step_cos_sin(const void *qkv, int64_t qkv_stride_b, int x_dtype, int B, int H, int Hkv, int Hc, int pos,
                                const int32_t *pos_dev, const void *cos, const void *sin, int64_t cos_sin_stride_b, void *q_out,
                                void *k_cache, void *v_cache, int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                                int64_t cache_len, const float *weights_k, const float *weights_q, int n_layers, int head_dim, int int_dim,
                                int final_dim, int arith, uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, uint32_t *qcodes,
                                void *stream) {
    HA_REQUIRE(cos && sin, HA_ERR_NULL_POINTER, "cos/sin is NULL");
    return rope_encode_step_impl(qkv, qkv_stride_b, x_dtype, B, H, Hkv, Hc, pos, pos_dev, nullptr, cos, sin, cos_sin_stride_b, q_out, k_cache,
                                 v_cache, kv_stride_b, kv_stride_h, kv_stride_s, cache_len, weights_k, weights_q, n_layers, head_dim, int_dim,
                                 final_dim, arith, kcodes, kc_stride_b, kc_stride_h, qcodes, stream);
}

}  // extern "C"
