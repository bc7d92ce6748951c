// Shared device-side helpers for the gfx950 attention kernels: storage-type conversions,
// vector types for MFMA operands, wavefront (64 lanes) reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hipattn.h"

namespace hipattn {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;

// ---- storage tags ---------------------------------------------------------------------
struct F32Tag {
    using storage = float;
    static constexpr hipattn_dtype dtype = HIPATTN_F32;
};
struct F16Tag {
    using storage = uint16_t;
    static constexpr hipattn_dtype dtype = HIPATTN_F16;
};
struct BF16Tag {
    using storage = uint16_t;
    static constexpr hipattn_dtype dtype = HIPATTN_BF16;
};

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }

// round to nearest even; NaN stays quiet NaN
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
    uint32_t x = __float_as_uint(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
    x += 0x7fffu + ((x >> 16) & 1u);
    return (uint16_t)(x >> 16);
}

__device__ __forceinline__ float f16_bits_to_float(uint16_t h) {
    half_t v = __builtin_bit_cast(half_t, h);
    return (float)v;
}

// v_cvt_f16_f32: round to nearest even, subnormals kept, overflow to inf
__device__ __forceinline__ uint16_t float_to_f16_bits(float f) {
    half_t v = (half_t)f;
    return __builtin_bit_cast(uint16_t, v);
}

template <typename Tag>
__device__ __forceinline__ float load_as_float(const void* base, int64_t idx);
template <>
__device__ __forceinline__ float load_as_float<F32Tag>(const void* base, int64_t idx) {
    return ((const float*)base)[idx];
}
template <>
__device__ __forceinline__ float load_as_float<F16Tag>(const void* base, int64_t idx) {
    return f16_bits_to_float(((const uint16_t*)base)[idx]);
}
template <>
__device__ __forceinline__ float load_as_float<BF16Tag>(const void* base, int64_t idx) {
    return bf16_bits_to_float(((const uint16_t*)base)[idx]);
}

template <typename Tag>
__device__ __forceinline__ void store_from_float(void* base, int64_t idx, float v);
template <>
__device__ __forceinline__ void store_from_float<F32Tag>(void* base, int64_t idx, float v) {
    ((float*)base)[idx] = v;
}
template <>
__device__ __forceinline__ void store_from_float<F16Tag>(void* base, int64_t idx, float v) {
    ((uint16_t*)base)[idx] = float_to_f16_bits(v);
}
template <>
__device__ __forceinline__ void store_from_float<BF16Tag>(void* base, int64_t idx, float v) {
    ((uint16_t*)base)[idx] = float_to_bf16_bits(v);
}

// dtype-erased scalar access for the shape-generic kernels
__device__ __forceinline__ float load_scalar(const void* base, int64_t idx, int dtype) {
    switch (dtype) {
        case HIPATTN_F32: return ((const float*)base)[idx];
        case HIPATTN_F16: return f16_bits_to_float(((const uint16_t*)base)[idx]);
        default: return bf16_bits_to_float(((const uint16_t*)base)[idx]);
    }
}
__device__ __forceinline__ void store_scalar(void* base, int64_t idx, int dtype, float v) {
    switch (dtype) {
        case HIPATTN_F32: ((float*)base)[idx] = v; break;
        case HIPATTN_F16: ((uint16_t*)base)[idx] = float_to_f16_bits(v); break;
        default: ((uint16_t*)base)[idx] = float_to_bf16_bits(v); break;
    }
}

__host__ __device__ __forceinline__ int dtype_bytes(int dtype) {
    return dtype == HIPATTN_F32 ? 4 : (dtype == HIPATTN_U8 ? 1 : 2);
}

__host__ __device__ __forceinline__ int64_t cache_row_bytes(int cache_dtype, int head_dim) {
    switch (cache_dtype) {
        case HIPATTN_F32: return 4 * (int64_t)head_dim;
        case HIPATTN_F16:
        case HIPATTN_BF16: return 2 * (int64_t)head_dim;
        default: return (int64_t)head_dim + 8;
    }
}

// one element of a cache row, dequantised
__device__ __forceinline__ float load_cache_elem(const uint8_t* row, int d, int cache_dtype) {
    switch (cache_dtype) {
        case HIPATTN_F32: return ((const float*)row)[d];
        case HIPATTN_F16: return f16_bits_to_float(((const uint16_t*)row)[d]);
        case HIPATTN_BF16: return bf16_bits_to_float(((const uint16_t*)row)[d]);
        default: {
            float scale = ((const float*)row)[0];
            float zp = ((const float*)row)[1];
            return ((float)row[8 + d] - zp) * scale;
        }
    }
}

// ---- wavefront reductions (64 lanes) -----------------------------------------------------
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}
__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fminf(v, __shfl_xor(v, off, kWave));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

}  // namespace hipattn
