// Shared device/host helpers for the gfx950 kernels of liboptimus_mi355x.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/optimus_mi355x.h"

#define OM_WAVE 64

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;

static inline hipStream_t om_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

static inline int om_launch_status() {
    return hipGetLastError() == hipSuccess ? OM_OK : OM_ERR_LAUNCH;
}

static inline bool om_aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// bf16 <-> fp32 on raw bits; round-to-nearest-even, NaN kept quiet (what at::BFloat16 does).
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) {
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

// Element traits for the row movers: a 16-byte vector of T and fp32 views of it.
template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int VEC = 4;
    __device__ static __forceinline__ void unpack(const u32x4 &v, float *f) {
        for (int i = 0; i < 4; i++) f[i] = __uint_as_float(v[i]);
    }
    __device__ static __forceinline__ u32x4 pack(const float *f) {
        u32x4 v;
        for (int i = 0; i < 4; i++) v[i] = __float_as_uint(f[i]);
        return v;
    }
    __device__ static __forceinline__ float load(const float *p) { return *p; }
    __device__ static __forceinline__ void store(float *p, float f) { *p = f; }
};
template <> struct Elem<uint16_t> {  // bf16 as raw bits
    static constexpr int VEC = 8;
    __device__ static __forceinline__ void unpack(const u32x4 &v, float *f) {
        for (int i = 0; i < 4; i++) {
            f[2 * i] = __uint_as_float(v[i] << 16);
            f[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
        }
    }
    __device__ static __forceinline__ u32x4 pack(const float *f) {
        u32x4 v;
        for (int i = 0; i < 4; i++)
            v[i] = static_cast<uint32_t>(f32_to_bf16_bits(f[2 * i])) |
                   (static_cast<uint32_t>(f32_to_bf16_bits(f[2 * i + 1])) << 16);
        return v;
    }
    __device__ static __forceinline__ float load(const uint16_t *p) { return bf16_bits_to_f32(*p); }
    __device__ static __forceinline__ void store(uint16_t *p, float f) { *p = f32_to_bf16_bits(f); }
};

// Wave-wide reductions over 64 lanes (xor butterfly: every lane ends with the result).
__device__ __forceinline__ float wave_sum(float v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ int wave_sum_i(int v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
