// Bulk (prefill) hash-MLP encode for fp32 hash modules on the gfx950 matrix cores.
//
// The same chain of GEMMs as ha_encode_mfma.hip, Y^T = W . X^T per MLP head, in fp32 throughout:
// v_mfma_f32_32x32x2_f32 multiplies a 32-output x 2-input block of W by 2 inputs x 32 tokens and keeps the
// 32 x 32 result in fp32.  Lane (t = lane % 32, half = lane / 32) supplies, for every k-step, ONE input value
// of token t (operand B) and one weight of output row lane % 32 (operand A); which of the two inputs of the
// step a lane supplies is its half.
//
// Chaining without shuffles.  After a layer, lane (t, half) holds for output block ob the 16 outputs
// o = 32 ob + 8 q + 4 half + i (register r = 4 q + i).  A dot product does not care about the order of its
// terms, so k-step s = 16 ob + r of the next layer simply takes "register r of block ob" from both halves:
// half 0 supplies feature 32 ob + 8 q + i, half 1 feature 32 ob + 8 q + 4 + i, and the next layer's weights
// are stored in LDS in exactly that order.  The first layer reads its 64 inputs per lane as one contiguous
// piece of the row (half 0: features 0..63, half 1: 64..127; k-step s takes features s and 64 + s).
//
// The two hidden layers' weights live in LDS (64 KiB each, four k-steps per 128-bit read); the final layer
// (32 or 64 outputs, a ninth or a fifth of the work) takes its A operand straight from the blob in global
// memory, which stays in the L1/L2 - so one workgroup of 512 threads per CU holds at most 128 KiB of LDS.
// A wave owns 32 tokens: 64 + 64 registers of activations, 32 of accumulators (two output blocks in flight, so
// that consecutive MFMAs never depend on each other), and the second wave of a SIMD runs its SiLU while the
// first one's MFMAs occupy the matrix pipe.
//
// Arithmetic: fp32 inputs (bf16/fp16 rows are widened exactly), fp32 weights, fp32 accumulate in the matrix
// core's own order, SiLU as y * rcp(1 + exp2(-y log2 e)) with the hardware exp2 and reciprocal (1 ulp each).
// The summation order differs from ha_encode_pack's fixed order, so a sign bit may differ from that kernel's
// where the logit is within rounding of zero (|logit| of a few 1e-6).
#include "ha_common.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kFThreads = 512;
constexpr int kFWaves = kFThreads / HA_WAVE;
constexpr int kFTokPerWave = 32;
constexpr int kFTile = kFWaves * kFTokPerWave;  // 256 tokens per workgroup tile
constexpr int kFDim = 128;
constexpr int kFKSteps = kFDim / 2;             // 64 k-steps of two inputs
constexpr int kFLayerBytes = kFDim * kFDim * 4;  // one hidden layer in LDS

// First feature of the four consecutive ones that k-steps 4 ks4 .. 4 ks4 + 3 take from a lane of this half.
// They are consecutive and aligned at four, i.e. one 16-byte group of the blob's [in / 4][out][4] layout.
__device__ __forceinline__ int feature_group(int ks4, int half, bool from_rows) {
    return from_rows ? ks4 + 16 * half : 8 * (ks4 >> 2) + 2 * (ks4 & 3) + half;
}

// Copy one 128 -> 128 layer from the blob into A-operand order: [ob][ks4][lane] float4.
__device__ __forceinline__ void fill_layer(float4 *dst, const float *w, bool from_rows, int tid) {
    for (int c = tid; c < 4 * 16 * 64; c += kFThreads) {
        const int lane = c & 63, ks4 = (c >> 6) & 15, ob = c >> 10;
        const int o = 32 * ob + (lane & 31), half = lane >> 5;
        dst[c] = *reinterpret_cast<const float4 *>(w + ((int64_t)feature_group(ks4, half, from_rows) * kFDim + o) * 4);
    }
}

__device__ __forceinline__ float silu_f32(float y) {
    const float t = __builtin_amdgcn_exp2f(y * -1.4426950408889634f);
    return y * __builtin_amdgcn_rcpf(1.0f + t);
}

__device__ __forceinline__ void init_bias(f32x16 &acc, const float *bias, int ob, int half) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float4 bv = *reinterpret_cast<const float4 *>(bias + 32 * ob + 8 * q + 4 * half);
        acc[4 * q + 0] = bv.x;
        acc[4 * q + 1] = bv.y;
        acc[4 * q + 2] = bv.z;
        acc[4 * q + 3] = bv.w;
    }
}

// Two output blocks (ob0, ob0 + 1) of a layer whose weights are in LDS.
__device__ __forceinline__ void block_pair_lds(const float4 *Wp, const float *bias, const float (&Bin)[kFKSteps], int ob0, int lane,
                                               f32x16 &acc0, f32x16 &acc1) {
    init_bias(acc0, bias, ob0, lane >> 5);
    init_bias(acc1, bias, ob0 + 1, lane >> 5);
    const float4 *p0 = Wp + (ob0 * 16) * 64 + lane;
    const float4 *p1 = p0 + 16 * 64;
    float4 a0 = p0[0], a1 = p1[0];
#pragma unroll
    for (int ks4 = 0; ks4 < 16; ++ks4) {
        const float4 c0 = a0, c1 = a1;
        if (ks4 + 1 < 16) {
            a0 = p0[(ks4 + 1) * 64];
            a1 = p1[(ks4 + 1) * 64];
        }
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(c0.x, Bin[4 * ks4 + 0], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(c1.x, Bin[4 * ks4 + 0], acc1, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(c0.y, Bin[4 * ks4 + 1], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(c1.y, Bin[4 * ks4 + 1], acc1, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(c0.z, Bin[4 * ks4 + 2], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(c1.z, Bin[4 * ks4 + 2], acc1, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(c0.w, Bin[4 * ks4 + 3], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(c1.w, Bin[4 * ks4 + 3], acc1, 0, 0, 0);
    }
}

// hidden layer 128 -> 128 with SiLU: Bout is the next layer's operand set
__device__ __forceinline__ void hidden_layer_f32(const float4 *Wp, const float *bias, const float (&Bin)[kFKSteps],
                                                 float (&Bout)[kFKSteps], int lane) {
#pragma unroll
    for (int ob0 = 0; ob0 < 4; ob0 += 2) {
        f32x16 acc0, acc1;
        block_pair_lds(Wp, bias, Bin, ob0, lane, acc0, acc1);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            Bout[16 * ob0 + r] = silu_f32(acc0[r]);
            Bout[16 * (ob0 + 1) + r] = silu_f32(acc1[r]);
        }
    }
}

// One output block of the final layer, A operand from the blob in global memory.  `from_rows`: the layer reads the
// input rows (a one-layer MLP), else the activations of a hidden layer.
template <int D>
__device__ __forceinline__ void final_block(const float *w, const float *bias, const float (&Bin)[kFKSteps], int ob, int lane,
                                            bool from_rows, f32x16 &acc) {
    const int half = lane >> 5, o = 32 * ob + (lane & 31);
    init_bias(acc, bias, ob, half);
    f32x16 acc_b;  // second chain: even / odd groups of k-steps, summed at the end
#pragma unroll
    for (int r = 0; r < 16; ++r) acc_b[r] = 0.f;
#pragma unroll
    for (int ks4 = 0; ks4 < 16; ks4 += 2) {
        const float4 a = *reinterpret_cast<const float4 *>(w + ((int64_t)feature_group(ks4, half, from_rows) * D + o) * 4);
        const float4 b = *reinterpret_cast<const float4 *>(w + ((int64_t)feature_group(ks4 + 1, half, from_rows) * D + o) * 4);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, Bin[4 * ks4 + 0], acc, 0, 0, 0);
        acc_b = __builtin_amdgcn_mfma_f32_32x32x2f32(b.x, Bin[4 * ks4 + 4], acc_b, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, Bin[4 * ks4 + 1], acc, 0, 0, 0);
        acc_b = __builtin_amdgcn_mfma_f32_32x32x2f32(b.y, Bin[4 * ks4 + 5], acc_b, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, Bin[4 * ks4 + 2], acc, 0, 0, 0);
        acc_b = __builtin_amdgcn_mfma_f32_32x32x2f32(b.z, Bin[4 * ks4 + 6], acc_b, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, Bin[4 * ks4 + 3], acc, 0, 0, 0);
        acc_b = __builtin_amdgcn_mfma_f32_32x32x2f32(b.w, Bin[4 * ks4 + 7], acc_b, 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] += acc_b[r];
}

template <typename E> struct RowLoad;
template <> struct RowLoad<ElemF32> {
    __device__ static __forceinline__ void load64(const void *row, int half, float (&f)[kFKSteps]) {
        const float4 *p = reinterpret_cast<const float4 *>(row) + 16 * half;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float4 v = p[i];
            f[4 * i] = v.x, f[4 * i + 1] = v.y, f[4 * i + 2] = v.z, f[4 * i + 3] = v.w;
        }
    }
};
template <> struct RowLoad<ElemBF16> {
    __device__ static __forceinline__ void load64(const void *row, int half, float (&f)[kFKSteps]) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float g[8];
            Elem<ElemBF16>::unpack(Elem<ElemBF16>::load8(row, 8 * half + i), g);
#pragma unroll
            for (int j = 0; j < 8; ++j) f[8 * i + j] = g[j];
        }
    }
};
template <> struct RowLoad<ElemF16> {
    __device__ static __forceinline__ void load64(const void *row, int half, float (&f)[kFKSteps]) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float g[8];
            Elem<ElemF16>::unpack(Elem<ElemF16>::load8(row, 8 * half + i), g);
#pragma unroll
            for (int j = 0; j < 8; ++j) f[8 * i + j] = g[j];
        }
    }
};

// grid (workgroups per sequence, n_heads, B).  NL layers, final width D (32 or 64), rows of element type E.
template <int NL, int D, typename E>
__global__ __launch_bounds__(kFThreads) void encode_mfma_f32_kernel(const void *__restrict__ x, int64_t x_sb, int64_t x_sh, int64_t x_st,
                                                                    int x_heads, int n_heads, int T, int tiles_per_wg,
                                                                    const float *__restrict__ wblob, int64_t per_head,
                                                                    uint32_t *__restrict__ codes, int64_t c_sb, int64_t c_sh,
                                                                    int64_t c_cap, int pos0, const int32_t *__restrict__ pos_dev) {
    extern __shared__ float4 smem_f32[];
    constexpr int NOBF = D / 32;
    constexpr int W = D / 32;
    constexpr int kLayerFloats = kFDim * kFDim + kFDim;  // weights + bias of a hidden layer in the blob

    const int head = blockIdx.y, b = blockIdx.z, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int in_head = head / (n_heads / x_heads);
    const float *wh = wblob + head * per_head;
    float4 *wp[NL > 1 ? NL - 1 : 1];
#pragma unroll
    for (int l = 0; l < NL - 1; ++l) {
        wp[l] = smem_f32 + l * (kFLayerBytes / 16);
        fill_layer(wp[l], wh + (int64_t)l * kLayerFloats, l == 0, tid);
    }
    if constexpr (NL > 1) __syncthreads();
    const float *w_final = wh + (int64_t)(NL - 1) * kLayerFloats;
    const float *b_final = w_final + kFDim * D;

    const int half = lane >> 5, tl = lane & 31;
    const char *xb = reinterpret_cast<const char *>(x) + (b * x_sb + in_head * x_sh) * Elem<E>::bytes;
    const int64_t pos = pos_dev ? pos_dev[b] : pos0;
    uint32_t *cb = codes + b * c_sb + head * c_sh;

    for (int it = 0; it < tiles_per_wg; ++it) {
        const int64_t t0 = ((int64_t)blockIdx.x * tiles_per_wg + it) * kFTile + wave * kFTokPerWave;
        if (t0 >= T) break;  // uniform per wave; no workgroup barrier below this point
        int64_t t = t0 + tl;
        const bool live = t < T;
        if (!live) t = T - 1;

        float Ba[kFKSteps], Bb[kFKSteps];
        RowLoad<E>::load64(xb + t * x_st * Elem<E>::bytes, half, Ba);
        if constexpr (NL >= 2) hidden_layer_f32(wp[0], wh + kFDim * kFDim, Ba, Bb, lane);
        if constexpr (NL >= 3) hidden_layer_f32(wp[1], wh + kLayerFloats + kFDim * kFDim, Bb, Ba, lane);

#pragma unroll
        for (int ob = 0; ob < NOBF; ++ob) {
            f32x16 acc;
            if constexpr (NL == 2) final_block<D>(w_final, b_final, Bb, ob, lane, false, acc);
            else final_block<D>(w_final, b_final, Ba, ob, lane, NL == 1, acc);
            uint32_t part = 0;
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int i = 0; i < 4; ++i) part |= (acc[4 * q + i] > 0.0f ? 1u : 0u) << (8 * q + 4 * half + i);
            const uint32_t word = part | (uint32_t)__shfl_xor((int)part, 32);
            const int64_t p = pos + t0 + tl;
            if (half == 0 && live && p >= 0 && p < c_cap) cb[p * W + ob] = word;
        }
    }
}

template <int NL, int D, typename E>
int launch_f32(dim3 grid, hipStream_t s, const void *x, int64_t x_sb, int64_t x_sh, int64_t x_st, int x_heads, int n_heads, int T,
               int tiles_per_wg, const float *w, int64_t per_head, uint32_t *codes, int64_t c_sb, int64_t c_sh, int64_t c_cap, int pos0,
               const int32_t *pos_dev) {
    constexpr int lds = (NL - 1) * kFLayerBytes;
    auto kern = encode_mfma_f32_kernel<NL, D, E>;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) HA_FAIL(HA_ERR_HIP, "hipFuncSetAttribute(%d bytes LDS): %s", lds, hipGetErrorString(e));
    }
    hipLaunchKernelGGL(kern, grid, dim3(kFThreads), lds, s, x, x_sb, x_sh, x_st, x_heads, n_heads, T, tiles_per_wg, w, per_head, codes,
                       c_sb, c_sh, c_cap, pos0, pos_dev);
    HA_CHECK_LAUNCH("encode_mfma_f32_kernel");
    return HA_OK;
}

}  // namespace

extern "C" int ha_encode_pack_prefill_f32(const void *x, int x_dtype, int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_t, int B,
                                          int x_heads, int n_heads, int T, const float *weights, int n_layers, int head_dim,
                                          int int_dim, int final_dim, uint32_t *codes, int64_t c_stride_b, int64_t c_stride_h,
                                          int pos0, const int32_t *pos_dev, void *stream) {
    HA_REQUIRE(x && weights && codes, HA_ERR_NULL_POINTER, "x/weights/codes is NULL");
    HA_REQUIRE(x_dtype == HA_F32 || x_dtype == HA_BF16 || x_dtype == HA_F16, HA_ERR_BAD_DTYPE, "x_dtype=%d", x_dtype);
    HA_REQUIRE(B > 0 && x_heads > 0 && n_heads > 0 && T > 0 && B <= 65535 && n_heads <= 65535, HA_ERR_BAD_SHAPE,
               "B, x_heads, n_heads, T must be positive (B, n_heads <= 65535)");
    HA_REQUIRE(n_heads % x_heads == 0, HA_ERR_BAD_SHAPE, "n_heads=%d not a multiple of x_heads=%d", n_heads, x_heads);
    HA_REQUIRE(n_layers >= 1 && n_layers <= 3, HA_ERR_BAD_SHAPE, "n_layers=%d, must be 1..3", n_layers);
    HA_REQUIRE(head_dim == kFDim && int_dim == kFDim, HA_ERR_BAD_SHAPE, "the MFMA encoder needs head_dim == int_dim == 128");
    HA_REQUIRE(final_dim == 32 || final_dim == 64, HA_ERR_BAD_SHAPE, "final_dim=%d, must be 32 or 64", final_dim);
    HA_REQUIRE(pos0 >= 0 && c_stride_b >= 0 && c_stride_h >= 0, HA_ERR_BAD_SHAPE, "negative position or stride");
    const int eb = ha_dtype_bytes(x_dtype);
    HA_REQUIRE(ha_aligned(x, 16) && (x_stride_b * eb) % 16 == 0 && (x_stride_h * eb) % 16 == 0 && (x_stride_t * eb) % 16 == 0 &&
                   x_stride_t >= kFDim,
               HA_ERR_MISALIGNED, "x rows must be 16-byte aligned rows of 128");
    HA_REQUIRE(ha_aligned(weights, 16) && ha_aligned(codes, 4), HA_ERR_MISALIGNED, "weights/codes misaligned");
    const int W = final_dim / 32;
    // tokens a (sequence, head) row of the code buffer spans, from its strides (a row nobody follows: unbounded)
    const int64_t c_cap = c_stride_h > 0 ? c_stride_h / W : (c_stride_b > 0 ? c_stride_b / W : INT64_MAX);
    HA_REQUIRE(pos_dev || (int64_t)pos0 + T <= c_cap, HA_ERR_BAD_SHAPE, "pos0 + T = %lld exceeds the %lld tokens of a code row",
               (long long)pos0 + T, (long long)c_cap);
    int st = ha_require_device();
    if (st) return st;

    const int64_t per_head = ha_usa_packed_floats(n_layers, head_dim, int_dim, final_dim);
    HA_REQUIRE(per_head % 4 == 0, HA_ERR_MISALIGNED, "blob of one head is not a multiple of 16 bytes");
    const int tiles = (T + kFTile - 1) / kFTile;
    // one workgroup per CU holds the hidden layers in LDS: several tiles each so that the 128 KiB fill amortises, as long
    // as the grid still covers the 256 CUs a few times
    int tiles_per_wg = 1;
    while (tiles_per_wg < 16 && (int64_t)B * n_heads * ((tiles + 2 * tiles_per_wg - 1) / (2 * tiles_per_wg)) >= 1024) tiles_per_wg *= 2;
    const dim3 grid((tiles + tiles_per_wg - 1) / tiles_per_wg, n_heads, B);
    hipStream_t s = (hipStream_t)stream;
#define HA_F32_CASE(NL_, D_, E_)                                                                                                   \
    return launch_f32<NL_, D_, E_>(grid, s, x, x_stride_b, x_stride_h, x_stride_t, x_heads, n_heads, T, tiles_per_wg, weights,     \
                                   per_head, codes, c_stride_b, c_stride_h, c_cap, pos0, pos_dev)
#define HA_F32_DTYPE(NL_, D_)                                    \
    do {                                                         \
        if (n_layers == NL_ && final_dim == D_) {                \
            if (x_dtype == HA_F32) HA_F32_CASE(NL_, D_, ElemF32); \
            if (x_dtype == HA_BF16) HA_F32_CASE(NL_, D_, ElemBF16); \
            HA_F32_CASE(NL_, D_, ElemF16);                       \
        }                                                        \
    } while (0)
    HA_F32_DTYPE(3, 32);
    HA_F32_DTYPE(3, 64);
    HA_F32_DTYPE(2, 32);
    HA_F32_DTYPE(2, 64);
    HA_F32_DTYPE(1, 32);
    HA_F32_DTYPE(1, 64);
#undef HA_F32_DTYPE
#undef HA_F32_CASE
    HA_FAIL(HA_ERR_BAD_SHAPE, "unsupported MLP shape");
}
