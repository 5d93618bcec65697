// The two elementwise steps of a decoder layer that sit right against the attention step, each as one launch:
//   ha_rope_append  rotate-half RoPE of the new token's q and k, k and v written into the caches in place
//   ha_swiglu       silu(gate) * up of the feed-forward block
// Both are a few hundred KB of traffic: latency-bound, one element pair / element per thread.
#include "ha_common.h"

namespace {

__device__ __forceinline__ void store_elem(void *p, int64_t i, float x, int dtype) {
    if (dtype == HA_F32) reinterpret_cast<float *>(p)[i] = x;
    else if (dtype == HA_BF16) reinterpret_cast<uint16_t *>(p)[i] = (uint16_t)ha_f32_to_bf16_bits(x);
    else reinterpret_cast<__half *>(p)[i] = __float2half(x);
}
__device__ __forceinline__ float round_to(float x, int dtype) {
    if (dtype == HA_F32) return x;
    if (dtype == HA_BF16) return ha_round_bf16(x);
    return __half2float(__float2half(x));
}

// grid (H + 2 Hkv, B), 64 threads: thread i owns the pair (i, i + 64) of one head vector.
__global__ __launch_bounds__(64) void rope_append_kernel(const void *__restrict__ qkv, int64_t qkv_sb, int dtype, int H, int Hkv, int pos,
                                                         const int32_t *__restrict__ pos_dev, const float *__restrict__ inv_freq,
                                                         void *__restrict__ q_out, void *__restrict__ k_cache,
                                                         void *__restrict__ v_cache, int64_t kv_sb, int64_t kv_sh, int64_t kv_ss) {
    const int head = blockIdx.x, b = blockIdx.y, i = threadIdx.x;
    const int p = pos_dev ? pos_dev[b] : pos;
    const int64_t src = b * qkv_sb + (int64_t)head * HA_HEAD_DIM;
    const float x0 = ha_load_elem(qkv, src + i, dtype), x1 = ha_load_elem(qkv, src + i + 64, dtype);
    if (head >= H + Hkv) {  // value: copied as it is
        const int64_t dst = b * kv_sb + (int64_t)(head - H - Hkv) * kv_sh + (int64_t)p * kv_ss;
        store_elem(v_cache, dst + i, x0, dtype);
        store_elem(v_cache, dst + i + 64, x1, dtype);
        return;
    }
    // the angle in fp32, the table rounded to the model dtype: as transformers' rotary embedding builds it
    const float ang = (float)p * inv_freq[i];
    const float c = round_to(cosf(ang), dtype), s = round_to(sinf(ang), dtype);
    const float y0 = x0 * c - x1 * s, y1 = x1 * c + x0 * s;
    if (head < H) {
        const int64_t dst = ((int64_t)b * H + head) * HA_HEAD_DIM;
        store_elem(q_out, dst + i, y0, dtype);
        store_elem(q_out, dst + i + 64, y1, dtype);
    } else {
        const int64_t dst = b * kv_sb + (int64_t)(head - H) * kv_sh + (int64_t)p * kv_ss;
        store_elem(k_cache, dst + i, y0, dtype);
        store_elem(k_cache, dst + i + 64, y1, dtype);
    }
}

__global__ __launch_bounds__(256) void swiglu_kernel(const void *__restrict__ gate_up, int64_t gu_sb, int dtype, int F,
                                                     void *__restrict__ out) {
    const int b = blockIdx.y, i = blockIdx.x * 256 + threadIdx.x;
    if (i >= F) return;
    const float g = ha_load_elem(gate_up, b * gu_sb + i, dtype), u = ha_load_elem(gate_up, b * gu_sb + F + i, dtype);
    store_elem(out, (int64_t)b * F + i, round_to(g / (1.0f + __expf(-g)), dtype) * u, dtype);
}

}  // namespace

extern "C" {

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
                       pos_dev, inv_freq, q_out, k_cache, v_cache, kv_stride_b, kv_stride_h, kv_stride_s);
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
