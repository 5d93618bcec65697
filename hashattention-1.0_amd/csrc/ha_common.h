// Shared host/device helpers of the gfx950 HashAttention kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>

#include "hashattn.h"

#define HA_WAVE 64
#define HA_HEAD_DIM 128

// ---- host: error reporting -------------------------------------------------------------------
void ha_set_error(const char *fmt, ...);

#define HA_FAIL(code, ...)          \
    do {                            \
        ha_set_error(__VA_ARGS__);  \
        return (code);              \
    } while (0)

#define HA_REQUIRE(cond, code, ...) \
    do {                            \
        if (!(cond)) HA_FAIL(code, __VA_ARGS__); \
    } while (0)

// Validation is complete before this runs; it reports a missing GPU as a status, never aborts.
int ha_require_device(void);

#define HA_CHECK_LAUNCH(name)                                                              \
    do {                                                                                   \
        hipError_t e_ = hipGetLastError();                                                 \
        if (e_ != hipSuccess) HA_FAIL(HA_ERR_HIP, "%s: %s", name, hipGetErrorString(e_));  \
    } while (0)

static inline bool ha_aligned(const void *p, size_t a) { return ((uintptr_t)p % a) == 0; }
static inline int ha_dtype_bytes(int dt) { return dt == HA_F32 ? 4 : 2; }

// ---- device: element loads --------------------------------------------------------------------
#ifdef __HIPCC__

__device__ __forceinline__ float ha_bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float ha_bf16_hi(uint32_t u) { return __uint_as_float(u & 0xFFFF0000u); }

// round-to-nearest-even fp32 -> bf16 bits (NaN kept quiet)
__device__ __forceinline__ uint32_t ha_f32_to_bf16_bits(float f) {
    uint32_t x = __float_as_uint(f);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (x >> 16) | 0x40u;
    return (x + 0x7FFFu + ((x >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ float ha_round_bf16(float f) { return __uint_as_float(ha_f32_to_bf16_bits(f) << 16); }

// Row element types.  A "slice" is the 8 consecutive head-dim elements one lane owns
// (16 lanes x 8 = 128); Loader<T>::load8 fetches it with 128-bit loads.
// A 128-bit load of data that is read once (K/V rows of a decode step, weights of a projection): the non-temporal
// hint keeps such lines from displacing what the launch reads repeatedly (codes, windows, the activations) in L2.
// Measured on the gather of the sparse attend kernel at B = 16, 64K tokens: 94 -> 87 us.
__device__ __forceinline__ uint4 ha_load16_stream(const uint4 *p) {
    typedef unsigned int ha_u32x4 __attribute__((ext_vector_type(4)));
    const ha_u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const ha_u32x4 *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

struct ElemF32 {};
struct ElemBF16 {};
struct ElemF16 {};

template <typename E> struct Raw8;
template <> struct Raw8<ElemF32> { uint4 a, b; };
template <> struct Raw8<ElemBF16> { uint4 a; };
template <> struct Raw8<ElemF16> { uint4 a; };

template <typename E> struct Elem;
template <> struct Elem<ElemF32> {
    static constexpr int bytes = 4;
    __device__ static __forceinline__ Raw8<ElemF32> load8(const void *row, int slice) {
        const uint4 *p = reinterpret_cast<const uint4 *>(row) + slice * 2;
        Raw8<ElemF32> r;
        r.a = p[0];
        r.b = p[1];
        return r;
    }
    __device__ static __forceinline__ Raw8<ElemF32> load8s(const void *row, int slice) {
        const uint4 *p = reinterpret_cast<const uint4 *>(row) + slice * 2;
        Raw8<ElemF32> r;
        r.a = ha_load16_stream(p);
        r.b = ha_load16_stream(p + 1);
        return r;
    }
    __device__ static __forceinline__ void unpack(const Raw8<ElemF32> &r, float (&f)[8]) {
        f[0] = __uint_as_float(r.a.x); f[1] = __uint_as_float(r.a.y); f[2] = __uint_as_float(r.a.z); f[3] = __uint_as_float(r.a.w);
        f[4] = __uint_as_float(r.b.x); f[5] = __uint_as_float(r.b.y); f[6] = __uint_as_float(r.b.z); f[7] = __uint_as_float(r.b.w);
    }
    // sum over the slice of a[i] * b[i]
    __device__ static __forceinline__ float dot8(const Raw8<ElemF32> &a, const Raw8<ElemF32> &b) {
        float fa[8], fb[8], d = 0.f;
        unpack(a, fa);
        unpack(b, fb);
#pragma unroll
        for (int i = 0; i < 8; ++i) d = fmaf(fa[i], fb[i], d);
        return d;
    }
    __device__ static __forceinline__ void store1(void *row, int i, float x) { reinterpret_cast<float *>(row)[i] = x; }
};
template <> struct Elem<ElemBF16> {
    static constexpr int bytes = 2;
    __device__ static __forceinline__ Raw8<ElemBF16> load8(const void *row, int slice) {
        Raw8<ElemBF16> r;
        r.a = reinterpret_cast<const uint4 *>(row)[slice];
        return r;
    }
    __device__ static __forceinline__ Raw8<ElemBF16> load8s(const void *row, int slice) {
        Raw8<ElemBF16> r;
        r.a = ha_load16_stream(reinterpret_cast<const uint4 *>(row) + slice);
        return r;
    }
    __device__ static __forceinline__ void unpack(const Raw8<ElemBF16> &r, float (&f)[8]) {
        f[0] = ha_bf16_lo(r.a.x); f[1] = ha_bf16_hi(r.a.x); f[2] = ha_bf16_lo(r.a.y); f[3] = ha_bf16_hi(r.a.y);
        f[4] = ha_bf16_lo(r.a.z); f[5] = ha_bf16_hi(r.a.z); f[6] = ha_bf16_lo(r.a.w); f[7] = ha_bf16_hi(r.a.w);
    }
    // sum over the slice of a[i] * b[i]: two elements per instruction (v_dot2c_f32_bf16), products and sums in fp32, nothing
    // unpacked
    __device__ static __forceinline__ float dot8(const Raw8<ElemBF16> &a, const Raw8<ElemBF16> &b) {
        typedef __bf16 ha_bf16x2 __attribute__((ext_vector_type(2)));
        float d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(ha_bf16x2, a.a.x), __builtin_bit_cast(ha_bf16x2, b.a.x), 0.f, false);
        d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(ha_bf16x2, a.a.y), __builtin_bit_cast(ha_bf16x2, b.a.y), d, false);
        d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(ha_bf16x2, a.a.z), __builtin_bit_cast(ha_bf16x2, b.a.z), d, false);
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(ha_bf16x2, a.a.w), __builtin_bit_cast(ha_bf16x2, b.a.w), d, false);
    }
    __device__ static __forceinline__ void store1(void *row, int i, float x) {
        reinterpret_cast<uint16_t *>(row)[i] = (uint16_t)ha_f32_to_bf16_bits(x);
    }
};
template <> struct Elem<ElemF16> {
    static constexpr int bytes = 2;
    __device__ static __forceinline__ Raw8<ElemF16> load8(const void *row, int slice) {
        Raw8<ElemF16> r;
        r.a = reinterpret_cast<const uint4 *>(row)[slice];
        return r;
    }
    __device__ static __forceinline__ Raw8<ElemF16> load8s(const void *row, int slice) {
        Raw8<ElemF16> r;
        r.a = ha_load16_stream(reinterpret_cast<const uint4 *>(row) + slice);
        return r;
    }
    __device__ static __forceinline__ void unpack(const Raw8<ElemF16> &r, float (&f)[8]) {
        const uint32_t w[4] = {r.a.x, r.a.y, r.a.z, r.a.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __half2float(__ushort_as_half((unsigned short)(w[i] & 0xFFFFu)));
            f[2 * i + 1] = __half2float(__ushort_as_half((unsigned short)(w[i] >> 16)));
        }
    }
    // sum over the slice of a[i] * b[i]: two elements per instruction (v_dot2c_f32_f16)
    __device__ static __forceinline__ float dot8(const Raw8<ElemF16> &a, const Raw8<ElemF16> &b) {
        typedef _Float16 ha_f16x2 __attribute__((ext_vector_type(2)));
        float d = __builtin_amdgcn_fdot2(__builtin_bit_cast(ha_f16x2, a.a.x), __builtin_bit_cast(ha_f16x2, b.a.x), 0.f, false);
        d = __builtin_amdgcn_fdot2(__builtin_bit_cast(ha_f16x2, a.a.y), __builtin_bit_cast(ha_f16x2, b.a.y), d, false);
        d = __builtin_amdgcn_fdot2(__builtin_bit_cast(ha_f16x2, a.a.z), __builtin_bit_cast(ha_f16x2, b.a.z), d, false);
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(ha_f16x2, a.a.w), __builtin_bit_cast(ha_f16x2, b.a.w), d, false);
    }
    __device__ static __forceinline__ void store1(void *row, int i, float x) {
        reinterpret_cast<__half *>(row)[i] = __float2half_rn(x);
    }
};

// single element load to float (scalar paths: q vectors, encode inputs)
__device__ __forceinline__ float ha_load_elem(const void *p, int64_t i, int dtype) {
    if (dtype == HA_F32) return reinterpret_cast<const float *>(p)[i];
    if (dtype == HA_BF16) return __uint_as_float((uint32_t) reinterpret_cast<const uint16_t *>(p)[i] << 16);
    return __half2float(reinterpret_cast<const __half *>(p)[i]);
}

// single element store from float, and the value such a store leaves behind
__device__ __forceinline__ void ha_store_elem(void *p, int64_t i, float x, int dtype) {
    if (dtype == HA_F32) reinterpret_cast<float *>(p)[i] = x;
    else if (dtype == HA_BF16) reinterpret_cast<uint16_t *>(p)[i] = (uint16_t)ha_f32_to_bf16_bits(x);
    else reinterpret_cast<__half *>(p)[i] = __float2half(x);
}
__device__ __forceinline__ float ha_round_to(float x, int dtype) {
    if (dtype == HA_F32) return x;
    if (dtype == HA_BF16) return ha_round_bf16(x);
    return __half2float(__float2half(x));
}

#endif  // __HIPCC__
