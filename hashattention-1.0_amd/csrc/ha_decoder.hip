// The two elementwise steps of a decoder layer that sit right against the attention step, each as one launch:
//   ha_rope_append  rotate-half RoPE of the new token's q and k, k and v written into the caches in place
//   ha_swiglu       silu(gate) * up of the feed-forward block
//   ha_linear_skinny  y = x W^T (+ residual) for a handful of rows (one token per sequence): streams W once
// The first two are a few hundred KB of traffic: latency-bound, one element pair / element per thread.
#include "ha_common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// y[m, n] = sum_k x[m, k] W[n, k] (+ res[m, n]), bf16 in, fp32 accumulate, bf16 out, M <= 16 (with a residual the product is
// rounded to bf16 before the addition, as a Linear followed by `x + h` rounds it: efficiency/model.py:190-191).  HBM-bound on W
// (2 N K bytes, read once).  One workgroup owns 16 consecutive output columns n; its NWAVE waves split K.  A wave
// feeds v_mfma_f32_16x16x32_bf16 with A = the 16 rows of W (lane: row l % 16, 8 consecutive k at 8 (l / 16)) and
// B = x^T padded to 16 columns, so a wave load brings 64 contiguous bytes of each of the 16 rows and two consecutive
// loads complete every 128-byte line.  Loads of the next four k-steps are in flight while the current four are
// multiplied (4 KiB of W per wave, 64 KiB per CU with two workgroups resident).  The matrix unit is idle most of
// the time at these shapes: it is there to keep the VALU out of the way of the loads.
// ------------------------------------------------------------------------------------------------
// Row-streaming form of the same product for M <= 8 and K <= 16384 (every projection of a decode step).
// A workgroup owns RB consecutive rows of W; its NWAVE waves cut K into slices of XCH chunks of 512 elements, and a
// wave keeps its slice of x (M x XCH x 16 bytes per lane) in registers for the whole workgroup.  A wave load is then
// one contiguous KiB of one row of W, the waves of a workgroup together read whole rows front to back, and the next
// R rows are in flight while R rows are multiplied (a third stage in flight cost occupancy and was slower) (v_dot2c_f32_bf16: two MACs per lane and instruction, no
// unpacking).  The R x MM per-lane sums are folded with a reduce-scatter inside each quad (two DPP stages, the
// value count halving at each) and two row rotations, so a 16-lane row ends with each sum once; rows of lanes and
// waves meet in LDS.
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float dot8(const uint4 &a, const uint4 &b, float c) {
    c = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.x), __builtin_bit_cast(bf16x2, b.x), c, false);
    c = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.y), __builtin_bit_cast(bf16x2, b.y), c, false);
    c = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.z), __builtin_bit_cast(bf16x2, b.z), c, false);
    c = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.w), __builtin_bit_cast(bf16x2, b.w), c, false);
    return c;
}
// A guarded 128-bit load as a load under the execution mask.  Written as `ok ? *p : zero` with `zero` a variable, the
// compiler selects between two addresses (global memory and the private copy of `zero`) and loads through a generic
// pointer: flat loads, which also occupy the LDS path and its counter.
__device__ __forceinline__ uint4 load16_or_zero(const void *p, bool ok) {
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (ok) v = *reinterpret_cast<const uint4 *>(p);
    return v;
}
// the same for weights: read once per launch, so with the non-temporal hint (x and the norm weight stay in L2)
__device__ __forceinline__ uint4 stream16_or_zero(const void *p, bool ok) {
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (ok) v = ha_load16_stream(reinterpret_cast<const uint4 *>(p));
    return v;
}
typedef float f32x2 __attribute__((ext_vector_type(2)));
// two floats rounded to bf16 (nearest even, v_cvt_pk_bf16_f32) in one word: `lo` in the low half
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
}
template <int CTRL> __device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

// FUSE bit 0: RMSNorm of x in front, x <- bf16(bf16(x * rsqrt(mean x^2 + eps)) * norm_w): the two roundings of the RMSNorm
// modules this replaces (transformers' LlamaRMSNorm, and efficiency/model.py:314-319 of the reference's harness: the
// normalised row is cast to the input type before it meets the weight).  Every workgroup holds all of x, so it norms it itself.  FUSE bit 1: SwiGLU behind (W = [gate rows; up rows],
// N = 2 F): a workgroup owns RB / 2 gate rows and the RB / 2 up rows of the same columns and writes
// bf16(bf16(silu(bf16 gate)) * bf16 up) to out [M, F], the roundings of a separate activation launch.
template <int NWAVE, int XCH, int R, int MM, int FUSE>
__global__ __launch_bounds__(NWAVE * 64) void gemv_rows_kernel(const uint16_t *__restrict__ x, int64_t x_sm,
                                                               const uint16_t *__restrict__ w, int64_t w_sn,
                                                               const uint16_t *__restrict__ res, int64_t res_sm,
                                                               uint16_t *__restrict__ out, int64_t out_sm, int M, int N, int K, int RB,
                                                               const uint16_t *__restrict__ norm_w, float eps) {
    constexpr int NV = R * MM;       // sums per lane and row group: 8 or 16
    constexpr int NP = NWAVE * 4;    // partials per sum: one per 16-lane row of every wave
    constexpr bool kNorm = FUSE & 1, kGlu = FUSE & 2;
    extern __shared__ float s_part[];  // [RB * MM][NP]
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int half = RB / 2, F = N / 2;  // SwiGLU: rows [0, half) of a block are gate rows, the rest the up rows of the same columns
    // The workgroup walks row blocks blockIdx.x, blockIdx.x + gridDim.x, ...: its slice of x (and the norm) is set up
    // once, and the first rows of the next block are requested while the sums of the current one are written out.
    const int nblk = kGlu ? (F + half - 1) / half : (N + RB - 1) / RB;
    // row of W behind local row r of the block that starts at column n0, or -1
    auto w_row = [&](int n0, int r) {
        if constexpr (kGlu) {
            const int c = n0 + (r < half ? r : r - half);
            return c < F ? (r < half ? c : F + c) : -1;
        } else {
            return (r < RB && n0 + r < N) ? n0 + r : -1;
        }
    };
    const int kbase = wave * XCH * 512 + lane * 8;  // first element of this lane's 16 bytes in chunk 0 of its slice

    uint4 xr[XCH][MM];
#pragma unroll
    for (int c = 0; c < XCH; ++c)
#pragma unroll
        for (int m = 0; m < MM; ++m) {
            const int k = kbase + c * 512;
            xr[c][m] = load16_or_zero(x + (int64_t)m * x_sm + k, m < M && k < K);
        }

    uint4 wc[R][XCH], wn[R][XCH];
    auto fetch = [&](int n0, int r0, uint4 (&wv)[R][XCH]) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int c = 0; c < XCH; ++c) {
                const int k = kbase + c * 512;
                const int n = w_row(n0, r0 + r);
                wv[r][c] = stream16_or_zero(w + (int64_t)n * w_sn + k, n >= 0 && k < K);
            }
    };
    int blk = blockIdx.x;
    int n0 = blk * (kGlu ? half : RB);
    fetch(n0, 0, wc);  // the first weight rows are requested before the norm is worked out
    if constexpr (kNorm) {
        uint4 gw[XCH];
#pragma unroll
        for (int c = 0; c < XCH; ++c) {
            const int k = kbase + c * 512;
            gw[c] = load16_or_zero(norm_w + k, k < K);
        }
        float ss[MM];
#pragma unroll
        for (int m = 0; m < MM; ++m) {
            float a = 0.f;
#pragma unroll
            for (int c = 0; c < XCH; ++c) {
                const uint32_t *p = reinterpret_cast<const uint32_t *>(&xr[c][m]);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float lo = __uint_as_float(p[i] << 16), hi = __uint_as_float(p[i] & 0xffff0000u);
                    a = fmaf(lo, lo, fmaf(hi, hi, a));
                }
            }
#pragma unroll
            for (int o = 32; o >= 1; o >>= 1) a += __shfl_xor(a, o);
            ss[m] = a;
        }
        if (lane == 0)
#pragma unroll
            for (int m = 0; m < MM; ++m) s_part[wave * MM + m] = ss[m];
        __syncthreads();
        float rstd[MM];
#pragma unroll
        for (int m = 0; m < MM; ++m) {
            float a = 0.f;
            for (int wv = 0; wv < NWAVE; ++wv) a += s_part[wv * MM + m];
            rstd[m] = rsqrtf(a / (float)K + eps);
        }
        __syncthreads();  // s_part is written again by the main loop
#pragma unroll
        for (int c = 0; c < XCH; ++c) {
            const uint32_t *g = reinterpret_cast<const uint32_t *>(&gw[c]);
#pragma unroll
            for (int m = 0; m < MM; ++m) {
                uint32_t *p = reinterpret_cast<uint32_t *>(&xr[c][m]);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // both roundings with the packed hardware conversion (round to nearest even): every instruction here is
                    // on the path of every workgroup before its first product
                    const uint32_t n = pack_bf16x2(__uint_as_float(p[i] << 16) * rstd[m], __uint_as_float(p[i] & 0xffff0000u) * rstd[m]);
                    p[i] = pack_bf16x2(__uint_as_float(n << 16) * __uint_as_float(g[i] << 16),
                                       __uint_as_float(n & 0xffff0000u) * __uint_as_float(g[i] & 0xffff0000u));
                }
            }
        }
    }
    auto total = [&](int r, int m) {
        const float *pp = s_part + (r * MM + m) * NP;
        float y = 0.f;
#pragma unroll 8
        for (int p = 0; p < NP; ++p) y += pp[p];
        return y;
    };
    while (true) {
        const int nrows = kGlu ? RB : min(RB, N - n0);
        const int blk_next = blk + gridDim.x;
        const int n0_next = blk_next * (kGlu ? half : RB);
        for (int r0 = 0; r0 < nrows; r0 += R) {
            if (r0 + R < nrows) fetch(n0, r0 + R, wn);
            else if (blk_next < nblk) fetch(n0_next, 0, wn);
            float v[NV];
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int m = 0; m < MM; ++m) {
                    float a = 0.f;
#pragma unroll
                    for (int c = 0; c < XCH; ++c) a = dot8(wc[r][c], xr[c][m], a);
                    v[r * MM + m] = a;
                }
            // reduce-scatter inside the quad: after stage 0 a lane holds the pair sums of the values with index bit 0
            // equal to its lane bit 0, after stage 1 the quad sums of the values i with i % 4 == lane % 4
            float u[NV / 2], t[NV / 4];
            const bool b0 = lane & 1, b1 = lane & 2;
#pragma unroll
            for (int j = 0; j < NV / 2; ++j) {
                const float keep = b0 ? v[2 * j + 1] : v[2 * j], send = b0 ? v[2 * j] : v[2 * j + 1];
                u[j] = keep + dpp_f<0xB1>(send);  // quad_perm [1,0,3,2]
            }
#pragma unroll
            for (int j = 0; j < NV / 4; ++j) {
                const float keep = b1 ? u[2 * j + 1] : u[2 * j], send = b1 ? u[2 * j] : u[2 * j + 1];
                t[j] = keep + dpp_f<0x4E>(send);  // quad_perm [2,3,0,1]
            }
            // the four quads of a 16-lane row: rotations by 4 and 8 keep lane % 4
#pragma unroll
            for (int j = 0; j < NV / 4; ++j) {
                t[j] += dpp_f<0x124>(t[j]);  // row_ror:4
                t[j] += dpp_f<0x128>(t[j]);  // row_ror:8
            }
            if ((lane & 12) == 0) {  // lanes 0..3 of each row: value i = 4 j + lane % 4 of this row group
                const int p = wave * 4 + (lane >> 4), q = lane & 3;
#pragma unroll
                for (int j = 0; j < NV / 4; ++j) {
                    const int i = 4 * j + q, r = i / MM, m = i % MM;
                    if (r0 + r < RB) s_part[((r0 + r) * MM + m) * NP + p] = t[j];
                }
            }
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int c = 0; c < XCH; ++c) wc[r][c] = wn[r][c];
        }
        __syncthreads();
        if constexpr (kGlu) {
            const int ncols = min(half, F - n0);
            for (int o = tid; o < ncols * M; o += NWAVE * 64) {
                const int m = o / ncols, r = o % ncols;
                const float g = ha_round_bf16(total(r, m)), u = ha_round_bf16(total(r + half, m));
                const float y = ha_round_bf16(g / (1.0f + __expf(-g))) * u;
                out[(int64_t)m * out_sm + n0 + r] = (uint16_t)ha_f32_to_bf16_bits(y);
            }
        } else {
            for (int o = tid; o < nrows * M; o += NWAVE * 64) {
                const int m = o / nrows, r = o % nrows;  // consecutive threads write consecutive columns of y
                float y = total(r, m);
                if (res) y = ha_round_bf16(y) + __uint_as_float((uint32_t)res[(int64_t)m * res_sm + n0 + r] << 16);  // the Linear's rounding, then the addition's
                out[(int64_t)m * out_sm + n0 + r] = (uint16_t)ha_f32_to_bf16_bits(y);
            }
        }
        if (blk_next >= nblk) break;
        blk = blk_next;
        n0 = n0_next;
        __syncthreads();  // the sums of this block are read: the next one may overwrite them
    }
}

template <int NWAVE>
__global__ __launch_bounds__(NWAVE * 64) void skinny_linear_kernel(const uint16_t *__restrict__ x, int64_t x_sm,
                                                                   const uint16_t *__restrict__ w, int64_t w_sn,
                                                                   const uint16_t *__restrict__ res, int64_t res_sm,
                                                                   uint16_t *__restrict__ out, int64_t out_sm, int M, int N, int K) {
    constexpr int PF = 4;
    __shared__ float s_c[NWAVE][16][17];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int n = min(n0 + r, N - 1);
    const int steps = K / 32;                                   // k-steps of 32
    const int per = ((steps + NWAVE - 1) / NWAVE + PF - 1) / PF * PF;  // per wave, whole groups of PF
    const int s_beg = wave * per, s_end = min(s_beg + per, steps);
    const uint4 *wp = reinterpret_cast<const uint4 *>(w + (int64_t)n * w_sn) + g;
    const uint4 *xp = reinterpret_cast<const uint4 *>(x + (int64_t)min(r, M - 1) * x_sm) + g;
    const bool x_ok = r < M;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    uint4 wc[PF], xc[PF], wn[PF], xn[PF];
    auto fetch = [&](int s0, uint4 (&wv)[PF], uint4 (&xv)[PF]) {
#pragma unroll
        for (int i = 0; i < PF; ++i) {
            const bool ok = s0 + i < s_end;
            wv[i] = stream16_or_zero(wp + (int64_t)(s0 + i) * 4, ok);
            xv[i] = load16_or_zero(xp + (int64_t)(s0 + i) * 4, ok && x_ok);
        }
    };
    if (s_beg < s_end) fetch(s_beg, wc, xc);
    for (int s0 = s_beg; s0 < s_end; s0 += PF) {
        if (s0 + PF < s_end) fetch(s0 + PF, wn, xn);
#pragma unroll
        for (int i = 0; i < PF; ++i)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wc[i]), __builtin_bit_cast(bf16x8, xc[i]), acc, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < PF; ++i) {
            wc[i] = wn[i];
            xc[i] = xn[i];
        }
    }
    // acc[i] = C[row 4 g + i (the column n0 + 4 g + i of y)][col r (the row m of y)]
#pragma unroll
    for (int i = 0; i < 4; ++i) s_c[wave][4 * g + i][r] = acc[i];
    __syncthreads();
    for (int t = tid; t < 16 * M; t += NWAVE * 64) {
        const int m = t >> 4, nl = t & 15;
        if (n0 + nl >= N) continue;
        float y = 0.f;
#pragma unroll
        for (int wv = 0; wv < NWAVE; ++wv) y += s_c[wv][nl][m];
        if (res) y = ha_round_bf16(y) + __uint_as_float((uint32_t)res[(int64_t)m * res_sm + n0 + nl] << 16);  // the Linear's rounding, then the addition's
        out[(int64_t)m * out_sm + n0 + nl] = (uint16_t)ha_f32_to_bf16_bits(y);
    }
}

// grid (H + 2 Hkv, B), 64 threads: thread i owns the pair (i, i + 64) of one head vector.
__global__ __launch_bounds__(64) void rope_append_kernel(const void *__restrict__ qkv, int64_t qkv_sb, int dtype, int H, int Hkv, int pos,
                                                         const int32_t *__restrict__ pos_dev, const float *__restrict__ inv_freq,
                                                         void *__restrict__ q_out, void *__restrict__ k_cache,
                                                         void *__restrict__ v_cache, int64_t kv_sb, int64_t kv_sh, int64_t kv_ss,
                                                         int64_t cache_len) {
    const int head = blockIdx.x, b = blockIdx.y, i = threadIdx.x;
    const int p = pos_dev ? pos_dev[b] : pos;
    const bool inside = p >= 0 && p < cache_len;  // a device-side position beyond the cache writes no key or value
    const int64_t src = b * qkv_sb + (int64_t)head * HA_HEAD_DIM;
    const float x0 = ha_load_elem(qkv, src + i, dtype), x1 = ha_load_elem(qkv, src + i + 64, dtype);
    if (head >= H + Hkv) {  // value: copied as it is
        if (!inside) return;
        const int64_t dst = b * kv_sb + (int64_t)(head - H - Hkv) * kv_sh + (int64_t)p * kv_ss;
        ha_store_elem(v_cache, dst + i, x0, dtype);
        ha_store_elem(v_cache, dst + i + 64, x1, dtype);
        return;
    }
    // the angle in fp32, the table rounded to the model dtype: as transformers' rotary embedding builds it
    const float ang = (float)p * inv_freq[i];
    const float c = ha_round_to(cosf(ang), dtype), s = ha_round_to(sinf(ang), dtype);
    const float y0 = x0 * c - x1 * s, y1 = x1 * c + x0 * s;
    if (head < H) {
        const int64_t dst = ((int64_t)b * H + head) * HA_HEAD_DIM;
        ha_store_elem(q_out, dst + i, y0, dtype);
        ha_store_elem(q_out, dst + i + 64, y1, dtype);
    } else if (inside) {
        const int64_t dst = b * kv_sb + (int64_t)(head - H) * kv_sh + (int64_t)p * kv_ss;
        ha_store_elem(k_cache, dst + i, y0, dtype);
        ha_store_elem(k_cache, dst + i + 64, y1, dtype);
    }
}

__global__ __launch_bounds__(256) void swiglu_kernel(const void *__restrict__ gate_up, int64_t gu_sb, int dtype, int F,
                                                     void *__restrict__ out) {
    const int b = blockIdx.y, i = blockIdx.x * 256 + threadIdx.x;
    if (i >= F) return;
    const float g = ha_load_elem(gate_up, b * gu_sb + i, dtype), u = ha_load_elem(gate_up, b * gu_sb + F + i, dtype);
    ha_store_elem(out, (int64_t)b * F + i, ha_round_to(g / (1.0f + __expf(-g)), dtype) * u, dtype);
}

// One workgroup per row: y = round(round(x * rsqrt(mean x^2 + eps)) * w), both roundings to the element type - the RMSNorm
// modules of transformers (LlamaRMSNorm: the normalised row is cast back to the input type before it meets the weight) and of
// the reference's harness (efficiency/model.py:314-319).  VEC: 16-bit elements, rows of whole 16-byte pieces.
template <bool VEC>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const void *__restrict__ x, int64_t x_sm, const void *__restrict__ w, int dtype,
                                                      int K, float eps, void *__restrict__ y, int64_t y_sm) {
    __shared__ float s_sum[4];
    const int m = blockIdx.x, tid = threadIdx.x;
    const char *xr = (const char *)x + (int64_t)m * x_sm * (dtype == HA_F32 ? 4 : 2);
    char *yr = (char *)y + (int64_t)m * y_sm * (dtype == HA_F32 ? 4 : 2);
    auto widen = [&](uint32_t bits16) {
        return dtype == HA_BF16 ? __uint_as_float(bits16 << 16) : __half2float(__ushort_as_half((unsigned short)bits16));
    };
    auto narrow = [&](float f) {
        return dtype == HA_BF16 ? ha_f32_to_bf16_bits(f) : (uint32_t)__half_as_ushort(__float2half(f));
    };
    // VEC: the row and the weight are requested together and stay in registers between the two passes (rows of up to 8192
    // elements: one memory round trip for the whole launch); what lies beyond is read again
    constexpr int kHold = 4;
    [[maybe_unused]] uint4 xv[kHold], gv[kHold];
    float a = 0.f;
    if constexpr (VEC) {
#pragma unroll
        for (int i = 0; i < kHold; ++i) {
            const int k = (tid + i * 256) * 8;
            xv[i] = gv[i] = make_uint4(0u, 0u, 0u, 0u);
            if (k < K) {
                xv[i] = *reinterpret_cast<const uint4 *>(xr + k * 2);
                gv[i] = *reinterpret_cast<const uint4 *>((const char *)w + k * 2);
            }
        }
        auto squares = [&](const uint4 &v) {
            const uint32_t p[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float lo = widen(p[i] & 0xffffu), hi = widen(p[i] >> 16);
                a = fmaf(lo, lo, fmaf(hi, hi, a));
            }
        };
#pragma unroll
        for (int i = 0; i < kHold; ++i) squares(xv[i]);
        for (int k = (tid + kHold * 256) * 8; k < K; k += 256 * 8) squares(*reinterpret_cast<const uint4 *>(xr + k * 2));
    } else {
        for (int k = tid; k < K; k += 256) {
            const float v = ha_load_elem(xr, k, dtype);
            a = fmaf(v, v, a);
        }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) a += __shfl_xor(a, o);
    if ((tid & 63) == 0) s_sum[tid >> 6] = a;
    __syncthreads();
    const float rstd = rsqrtf((s_sum[0] + s_sum[1] + s_sum[2] + s_sum[3]) / (float)K + eps);
    if constexpr (VEC) {
        auto scaled = [&](const uint4 &v, const uint4 &g) {
            const uint32_t p[4] = {v.x, v.y, v.z, v.w}, q[4] = {g.x, g.y, g.z, g.w};
            uint32_t r[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float lo = ha_round_to(widen(p[i] & 0xffffu) * rstd, dtype) * widen(q[i] & 0xffffu);
                const float hi = ha_round_to(widen(p[i] >> 16) * rstd, dtype) * widen(q[i] >> 16);
                r[i] = narrow(lo) | (narrow(hi) << 16);
            }
            return make_uint4(r[0], r[1], r[2], r[3]);
        };
#pragma unroll
        for (int i = 0; i < kHold; ++i) {
            const int k = (tid + i * 256) * 8;
            if (k < K) *reinterpret_cast<uint4 *>(yr + k * 2) = scaled(xv[i], gv[i]);
        }
        for (int k = (tid + kHold * 256) * 8; k < K; k += 256 * 8)
            *reinterpret_cast<uint4 *>(yr + k * 2) =
                scaled(*reinterpret_cast<const uint4 *>(xr + k * 2), *reinterpret_cast<const uint4 *>((const char *)w + k * 2));
    } else {
        for (int k = tid; k < K; k += 256)
            ha_store_elem(yr, k, ha_round_to(ha_load_elem(xr, k, dtype) * rstd, dtype) * ha_load_elem(w, k, dtype), dtype);
    }
}

}  // namespace

extern "C" {

int ha_rmsnorm(const void *x, int64_t x_stride_m, const void *weight, int dtype, int M, int K, float eps, void *out, int64_t out_stride_m,
               void *stream) {
    HA_REQUIRE(x && weight && out, HA_ERR_NULL_POINTER, "x/weight/out is NULL");
    HA_REQUIRE(dtype == HA_F32 || dtype == HA_BF16 || dtype == HA_F16, HA_ERR_BAD_DTYPE, "unknown dtype %d", dtype);
    HA_REQUIRE(M > 0 && K > 0 && x_stride_m >= K && out_stride_m >= K && eps >= 0.f, HA_ERR_BAD_SHAPE, "bad rmsnorm shape");
    int st = ha_require_device();
    if (st) return st;
    const bool vec = dtype != HA_F32 && K % 8 == 0 && x_stride_m % 8 == 0 && out_stride_m % 8 == 0 && ha_aligned(x, 16) &&
                     ha_aligned(weight, 16) && ha_aligned(out, 16);
    if (vec)
        hipLaunchKernelGGL(rmsnorm_kernel<true>, dim3(M), dim3(256), 0, (hipStream_t)stream, x, x_stride_m, weight, dtype, K, eps, out,
                           out_stride_m);
    else
        hipLaunchKernelGGL(rmsnorm_kernel<false>, dim3(M), dim3(256), 0, (hipStream_t)stream, x, x_stride_m, weight, dtype, K, eps, out,
                           out_stride_m);
    HA_CHECK_LAUNCH("rmsnorm_kernel");
    return HA_OK;
}

int ha_rope_append(const void *qkv, int64_t qkv_stride_b, int dtype, int B, int H, int Hkv, int pos, const int32_t *pos_dev,
                   const float *inv_freq, void *q_out, void *k_cache, void *v_cache, int64_t kv_stride_b, int64_t kv_stride_h,
                   int64_t kv_stride_s, int64_t cache_len, void *stream) {
    HA_REQUIRE(qkv && inv_freq && q_out && k_cache && v_cache, HA_ERR_NULL_POINTER, "qkv/inv_freq/q_out/k_cache/v_cache is NULL");
    HA_REQUIRE(dtype == HA_F32 || dtype == HA_BF16 || dtype == HA_F16, HA_ERR_BAD_DTYPE, "unknown dtype %d", dtype);
    HA_REQUIRE(B > 0 && H > 0 && Hkv > 0 && B <= 65535, HA_ERR_BAD_SHAPE, "B, H, Hkv must be positive (B <= 65535)");
    HA_REQUIRE(qkv_stride_b >= (int64_t)(H + 2 * Hkv) * HA_HEAD_DIM, HA_ERR_BAD_SHAPE, "qkv row stride shorter than (H + 2 Hkv) * 128");
    HA_REQUIRE(cache_len > 0 && (pos_dev || (pos >= 0 && pos < cache_len)), HA_ERR_BAD_SHAPE, "position %d outside the cache of %lld tokens",
               pos, (long long)cache_len);
    HA_REQUIRE(kv_stride_s >= HA_HEAD_DIM && kv_stride_h > 0 && kv_stride_b > 0, HA_ERR_BAD_SHAPE, "cache strides smaller than a row");
    int st = ha_require_device();
    if (st) return st;
    hipLaunchKernelGGL(rope_append_kernel, dim3(H + 2 * Hkv, B), dim3(64), 0, (hipStream_t)stream, qkv, qkv_stride_b, dtype, H, Hkv, pos,
                       pos_dev, inv_freq, q_out, k_cache, v_cache, kv_stride_b, kv_stride_h, kv_stride_s, cache_len);
    HA_CHECK_LAUNCH("rope_append_kernel");
    return HA_OK;
}

int ha_swiglu(const void *gate_up, int64_t gate_up_stride_b, int dtype, int B, int F, void *out, void *stream) {
    HA_REQUIRE(gate_up && out, HA_ERR_NULL_POINTER, "gate_up/out is NULL");
    HA_REQUIRE(dtype == HA_F32 || dtype == HA_BF16 || dtype == HA_F16, HA_ERR_BAD_DTYPE, "unknown dtype %d", dtype);
    HA_REQUIRE(B > 0 && F > 0 && B <= 65535 && gate_up_stride_b >= 2 * (int64_t)F, HA_ERR_BAD_SHAPE, "bad swiglu shape");
    int st = ha_require_device();
    if (st) return st;
    hipLaunchKernelGGL(swiglu_kernel, dim3((F + 255) / 256, B), dim3(256), 0, (hipStream_t)stream, gate_up, gate_up_stride_b, dtype, F, out);
    HA_CHECK_LAUNCH("swiglu_kernel");
    return HA_OK;
}

}  // extern "C"

static int linear_skinny_impl(const void *x, int64_t x_stride_m, const void *w, int64_t w_stride_n, const void *residual,
                              int64_t residual_stride_m, const void *norm_weight, float eps, int act, void *out, int64_t out_stride_m,
                              int M, int N, int K, void *stream) {
    HA_REQUIRE(x && w && out, HA_ERR_NULL_POINTER, "x/w/out is NULL");
    HA_REQUIRE(M >= 1 && M <= 16 && N >= 1 && K >= 32 && K % 32 == 0, HA_ERR_BAD_SHAPE, "need 1 <= M <= 16, N >= 1, K a multiple of 32");
    HA_REQUIRE(act == HA_ACT_NONE || act == HA_ACT_SWIGLU, HA_ERR_BAD_SHAPE, "unknown activation %d", act);
    const int n_out = act == HA_ACT_SWIGLU ? N / 2 : N;
    HA_REQUIRE(act != HA_ACT_SWIGLU || (N % 2 == 0 && !residual), HA_ERR_BAD_SHAPE, "SwiGLU needs an even number of weight rows and no residual");
    HA_REQUIRE(x_stride_m >= K && w_stride_n >= K && out_stride_m >= n_out && (!residual || residual_stride_m >= N), HA_ERR_BAD_SHAPE,
               "strides smaller than the rows they span");
    HA_REQUIRE(ha_aligned(x, 16) && ha_aligned(w, 16) && x_stride_m % 8 == 0 && w_stride_n % 8 == 0, HA_ERR_MISALIGNED,
               "x and W rows must be 16-byte aligned");
    const bool fused = norm_weight || act != HA_ACT_NONE;
    HA_REQUIRE(!fused || (M <= 8 && K <= 16384), HA_ERR_BAD_SHAPE, "the fused norm / activation forms need M <= 8 and K <= 16384");
    HA_REQUIRE(!norm_weight || (ha_aligned(norm_weight, 16) && eps >= 0.f), HA_ERR_MISALIGNED, "norm weight must be 16-byte aligned, eps >= 0");
    int st = ha_require_device();
    if (st) return st;
    const uint16_t *xp = (const uint16_t *)x, *wp = (const uint16_t *)w, *rp = (const uint16_t *)residual;
    const uint16_t *gp = (const uint16_t *)norm_weight;
    uint16_t *op = (uint16_t *)out;
    hipStream_t s = (hipStream_t)stream;
    if (M <= 8 && K <= 16384) {
        // rows per workgroup, measured at M = 4.  Plain product: 8 rows for K <= 4096 (QKV 11.6 us against 14.2 with 16
        // rows, output projection 9.6 against 10.3, gate/up 41.1 against 43.6), 16 for the vocabulary projection (174.8
        // us against 178.3 with 8 and 182.1 with 64) and for longer rows (down projection 24.8 us against 26.0 with 8);
        // counts that are not multiples of 8 were always slower.  With the norm in front every workgroup repeats the
        // norm of x, so fewer, larger workgroups win (whole decoder step 6.3 ms against 6.8 ms with 8 rows everywhere).
        const int chunks = (K + 511) / 512;
        const int fuse = (norm_weight ? 1 : 0) | (act == HA_ACT_SWIGLU ? 2 : 0);
        int RB = (fuse & 1) ? ((int64_t)N >= 64 * 1024 ? 64 : (int64_t)N >= 32 * 512 ? 32 : 16) : (chunks <= 8 && (int64_t)N < 64 * 1024) ? 8 : 16;
        {
            // A grid of a few blocks per CU is quantised: workgroups go round the 256 CUs, the launch lasts as long as the CU
            // with the most rows, and a CU holds two of these workgroups (one of the 1024-thread ones).  When the usual row
            // count gives more blocks than are resident at once but not many more (a second, partly filled round), take the row
            // count (a multiple of 8) that leaves the busiest CU the fewest rows, and among equals the one that gives a CU its
            // two workgroups (one), then the fewest.  Gate/up 28672 x 4096 at M = 4: 32 rows make 896 blocks, 4 on some CUs =
            // 128 rows; 56 rows make 512, 2 x 56 everywhere: 49.1 -> 44.2 us launched alone (47.4 with 112 rows, 54.3 with
            // 48), 45.3 -> 43.7 us inside the decoder step (whose 5.6 ms do not show the 50 us: 713 / 713 against 715 / 703 tokens/s on one box).  Grids that fit one round keep the usual count: QKV 6144 x 4096
            // (384 blocks of 16 rows) was 1.5 us faster alone with 24 rows (one block per CU) and 0.9 us slower inside the step.
            constexpr int kCUs = 256;
            const int64_t units = act == HA_ACT_SWIGLU ? N / 2 : N;     // rows that a block's RB (RB / 2 gate rows) stand for
            const int per_block = act == HA_ACT_SWIGLU ? RB / 2 : RB;
            const int64_t usual = (units + per_block - 1) / per_block;
            if (usual > 2 * kCUs && usual <= 4 * kCUs) {
                const int MMx = M <= 4 ? 4 : 8, NWx = chunks <= 8 ? 8 : 16;
                const int rb_max = min(128, 4096 / (MMx * NWx));           // the partial sums of a block fit 64 KB of LDS
                const int want = NWx == 8 ? 2 : 1;
                int64_t best_rows = -1;
                int best_rank = 0;
                for (int rb = 8; rb <= rb_max; rb += 8) {
                    const int pb = act == HA_ACT_SWIGLU ? rb / 2 : rb;
                    const int64_t blocks = (units + pb - 1) / pb, per_cu = (blocks + kCUs - 1) / kCUs, rows = per_cu * rb;
                    const int rank = per_cu == want ? 0 : per_cu == 3 - want ? 1 : (int)per_cu;
                    if (best_rows < 0 || rows < best_rows || (rows == best_rows && rank < best_rank)) {
                        best_rows = rows;
                        best_rank = rank;
                        RB = rb;
                    }
                }
            }
        }
#ifdef HASHATTN_TUNING_ENV
        if (const char *e = getenv("HA_GEMV_RB")) RB = atoi(e);
#endif
        const int nblk = act == HA_ACT_SWIGLU ? (N / 2 + RB / 2 - 1) / (RB / 2) : (N + RB - 1) / RB;
        // one workgroup per row block: the kernel can walk several blocks per workgroup, but a grid cut down to the
        // resident workgroups measured no better (gate/up 43.3 - 48.1 us against 42.2; whole decoder step unchanged)
        const dim3 g2(nblk);
#define HA_GEMV_F(NW_, XCH_, R_, MM_, F_)                                                                                     \
    hipLaunchKernelGGL((gemv_rows_kernel<NW_, XCH_, R_, MM_, F_>), g2, dim3(NW_ * 64), (size_t)RB * MM_ * NW_ * 4 * sizeof(float), s, \
                       xp, x_stride_m, wp, w_stride_n, rp, residual_stride_m, op, out_stride_m, M, N, K, RB, gp, eps)
#define HA_GEMV(NW_, XCH_, R_, MM_)                                  \
    do {                                                             \
        if (fuse == 0) HA_GEMV_F(NW_, XCH_, R_, MM_, 0);             \
        else if (fuse == 1) HA_GEMV_F(NW_, XCH_, R_, MM_, 1);        \
        else if (fuse == 2) HA_GEMV_F(NW_, XCH_, R_, MM_, 2);        \
        else HA_GEMV_F(NW_, XCH_, R_, MM_, 3);                       \
    } while (0)
        if (chunks <= 8) {
            if (M <= 4) HA_GEMV(8, 1, 4, 4);
            else HA_GEMV(8, 1, 2, 8);
        } else if (chunks <= 16) {
            if (M <= 4) HA_GEMV(16, 1, 4, 4);
            else HA_GEMV(16, 1, 2, 8);
        } else {
            if (M <= 4) HA_GEMV(16, 2, 2, 4);
            else HA_GEMV(16, 2, 1, 8);
        }
#undef HA_GEMV
#undef HA_GEMV_F
        HA_CHECK_LAUNCH("gemv_rows_kernel");
        return HA_OK;
    }
    const dim3 grid((N + 15) / 16);
    // few output columns: split K eight ways so that the grid still covers the CUs with enough loads in flight
    if ((int64_t)N * 4 < 16 * 4096)
        hipLaunchKernelGGL(skinny_linear_kernel<8>, grid, dim3(512), 0, (hipStream_t)stream, (const uint16_t *)x, x_stride_m,
                           (const uint16_t *)w, w_stride_n, (const uint16_t *)residual, residual_stride_m, (uint16_t *)out, out_stride_m,
                           M, N, K);
    else
        hipLaunchKernelGGL(skinny_linear_kernel<4>, grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t *)x, x_stride_m,
                           (const uint16_t *)w, w_stride_n, (const uint16_t *)residual, residual_stride_m, (uint16_t *)out, out_stride_m,
                           M, N, K);
    HA_CHECK_LAUNCH("skinny_linear_kernel");
    return HA_OK;
}

extern "C" {

int ha_linear_skinny(const void *x, int64_t x_stride_m, const void *w, int64_t w_stride_n, const void *residual,
                     int64_t residual_stride_m, void *out, int64_t out_stride_m, int M, int N, int K, void *stream) {
    return linear_skinny_impl(x, x_stride_m, w, w_stride_n, residual, residual_stride_m, nullptr, 0.f, HA_ACT_NONE, out, out_stride_m, M, N,
                              K, stream);
}

int ha_linear_skinny_fused(const void *x, int64_t x_stride_m, const void *w, int64_t w_stride_n, const void *residual,
                           int64_t residual_stride_m, const void *norm_weight, float eps, int act, void *out, int64_t out_stride_m,
                           int M, int N, int K, void *stream) {
    return linear_skinny_impl(x, x_stride_m, w, w_stride_n, residual, residual_stride_m, norm_weight, eps, act, out, out_stride_m, M, N, K,
                              stream);
}

}  // extern "C"
