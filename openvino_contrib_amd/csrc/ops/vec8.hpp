// Eight consecutive elements of an f32 / f16 / bf16 tensor as floats: the unit the element-wise and
// normalisation kernels of libhipops.so load and store (16 bytes of a 16-bit type per lane).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_common.hpp"

namespace hipops {

using namespace hipattn;

// ---- eight consecutive elements as floats ---------------------------------------------------
struct Float8 {
    float v[8];
};

__device__ __forceinline__ Float8 load8(const void* base, int64_t idx, int dtype) {
    Float8 r;
    if (dtype == HIPATTN_F32) {
        const float4_t a = *(const float4_t*)((const float*)base + idx);
        const float4_t b = *(const float4_t*)((const float*)base + idx + 4);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            r.v[i] = a[i];
            r.v[4 + i] = b[i];
        }
    } else {
        const uint4_t raw = *(const uint4_t*)((const uint16_t*)base + idx);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint16_t lo = (uint16_t)(raw[i] & 0xffffu), hi = (uint16_t)(raw[i] >> 16);
            if (dtype == HIPATTN_F16) {
                r.v[2 * i] = f16_bits_to_float(lo);
                r.v[2 * i + 1] = f16_bits_to_float(hi);
            } else {
                r.v[2 * i] = bf16_bits_to_float(lo);
                r.v[2 * i + 1] = bf16_bits_to_float(hi);
            }
        }
    }
    return r;
}

// rounds to nearest even with the hardware's packed conversions
__device__ __forceinline__ void store8(void* base, int64_t idx, int dtype, const Float8& r) {
    typedef float float2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    if (dtype == HIPATTN_F32) {
        float4_t a, b;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            a[i] = r.v[i];
            b[i] = r.v[4 + i];
        }
        *(float4_t*)((float*)base + idx) = a;
        *(float4_t*)((float*)base + idx + 4) = b;
    } else {
        uint4_t raw;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float2_t pair = {r.v[2 * i], r.v[2 * i + 1]};
            if (dtype == HIPATTN_F16)
                raw[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, half2_t));
            else
                raw[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2_t));
        }
        *(uint4_t*)((uint16_t*)base + idx) = raw;
    }
}

}  // namespace hipops
