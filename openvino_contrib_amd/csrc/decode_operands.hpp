// Operand helpers of the single-token matrix-core kernels (paged_decode.hip, paged_scores.hip): the MFMA
// 16x16x32 wrappers per operand type, query fragments, and u8 -> fp16 operands.
#pragma once
#include "device_common.hpp"

namespace hipattn {

// the low (high) halves of a and b side by side, a's first: one v_perm_b32 each
__device__ __forceinline__ uint32_t pack_lo(uint32_t a, uint32_t b) { return __builtin_amdgcn_perm(b, a, 0x05040100u); }
__device__ __forceinline__ uint32_t pack_hi(uint32_t a, uint32_t b) { return __builtin_amdgcn_perm(b, a, 0x07060302u); }

// The largest of the values that lanes l, l ^ 16, l ^ 32 and l ^ 48 hold, in the vector ALU: v_permlane16_swap
// (the odd rows of sixteen lanes of the first operand change places with the even rows of the second) and
// v_permlane32_swap (the same for the two halves of the wavefront) on two copies of the value leave every
// lane with both partners' values; through LDS (ds_bpermute) each step is a round trip that the softmax of
// every block would wait for.
__device__ __forceinline__ float max_over_rows(float x) {
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    const float y = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(y), __float_as_uint(y), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

__device__ __forceinline__ half8_t as_half8(uint4_t v) { return __builtin_bit_cast(half8_t, v); }

// Element type of the MFMA operands: fp16 for fp16 and u8 caches, bf16 for bf16 caches.
template <bool kBf16>
struct Op16;
template <>
struct Op16<false> {
    using vec8 = half8_t;
    static __device__ __forceinline__ vec8 from_bits(uint4_t v) { return __builtin_bit_cast(vec8, v); }
    static __device__ __forceinline__ float4_t mma(vec8 a, vec8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ void set(vec8& v, int i, float x) { v[i] = (half_t)x; }
    static __device__ __forceinline__ float get(const vec8& v, int i) { return (float)v[i]; }
};
template <>
struct Op16<true> {
    using vec8 = bf16x8_t;
    static __device__ __forceinline__ vec8 from_bits(uint4_t v) { return __builtin_bit_cast(vec8, v); }
    static __device__ __forceinline__ float4_t mma(vec8 a, vec8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ void set(vec8& v, int i, float x) { v[i] = (__bf16)x; }
    static __device__ __forceinline__ float get(const vec8& v, int i) { return (float)v[i]; }
};

// 8 consecutive query elements in the operand type (same type: the bits; otherwise converted:
// bf16 -> fp16 is exact inside the fp16 range, fp16 -> bf16 rounds to 8 bits)
template <bool kBf16>
__device__ __forceinline__ typename Op16<kBf16>::vec8 load_q8(const void* q, int64_t elem, int q_dtype) {
    using O = Op16<kBf16>;
    const uint4_t raw = *(const uint4_t*)((const uint16_t*)q + elem);
    if (q_dtype == (kBf16 ? HIPATTN_BF16 : HIPATTN_F16)) return O::from_bits(raw);
    typename O::vec8 r;
#pragma unroll
    for (int w = 0; w < 4; w++) {
        float lo, hi;
        if constexpr (kBf16) {  // fp16 queries
            lo = f16_bits_to_float((uint16_t)(raw[w] & 0xffffu));
            hi = f16_bits_to_float((uint16_t)(raw[w] >> 16));
        } else {  // bf16 queries
            lo = __uint_as_float(raw[w] << 16);
            hi = __uint_as_float(raw[w] & 0xffff0000u);
        }
        O::set(r, 2 * w, lo);
        O::set(r, 2 * w + 1, hi);
    }
    return r;
}

// u8 -> fp16 operands.  0x6400 | byte is the fp16 number 1024 + byte, exactly.  The operands keep
// that bias: it adds 1024 * sum(q) to a score and 1024 * sum(p') to an output, which are folded
// into the zero-point terms the kernel subtracts anyway (the products are exact in fp32 and the
// sums stay far inside its 24 bits), so the bias costs no instruction.
constexpr float kByteBias = 1024.0f;
// two bytes of one word (selector bytes 0..3 = its bytes, 4 = the bias byte 0x64)
__device__ __forceinline__ uint32_t bytes_to_biased_half2(uint32_t src, uint32_t sel) {
    return __builtin_amdgcn_perm(0x64646464u, src, sel);
}
// one byte of each of two words (selector bytes 0..3 pick from lo_src, 4..7 from hi_src, 0x0c yields 0x00)
__device__ __forceinline__ uint32_t bytes_to_biased_half2(uint32_t lo_src, uint32_t hi_src, uint32_t sel) {
    return __builtin_amdgcn_perm(hi_src, lo_src, sel) | 0x64006400u;
}

}  // namespace hipattn
