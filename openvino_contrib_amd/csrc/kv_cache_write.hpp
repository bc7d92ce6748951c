// Device side of the KV-cache block writer, shared by the stand-alone writer kernel and the
// paged-attention prologue kernel (which also plans the decode schedule in the same launch).
#pragma once

#include <type_traits>

#include "device_common.hpp"
#include "kernels.hpp"

namespace hipattn {

// Largest s in [0, n) with prefix[s] <= x; requires prefix[0] <= x.  64-ary search: every round
// is one vector load and one ballot, so a batch of 4096 sequences needs two rounds.
__device__ __forceinline__ int locate_sequence(const int32_t* __restrict__ prefix, int n, int x, int lane) {
    int lo = 0, hi = n;
    while (hi - lo > 1) {
        const int step = (hi - lo + 63) / 64;
        const int idx = lo + lane * step;
        const bool ok = idx < hi && prefix[idx] <= x;
        const int k = __builtin_popcountll(__builtin_amdgcn_ballot_w64(ok)) - 1;  // prefix is monotone
        lo = lo + k * step;
        hi = min(hi, lo + step);
    }
    return lo;
}

// Where token t goes: physical block and position inside it; false when it has no valid target
// (padding tokens outside every sequence, positions beyond the sequence's block table, block
// numbers outside the pool).  A chain of dependent loads, done once per wavefront.
__device__ __forceinline__ bool kv_write_slot(const KvWriteParams& p, int t, int lane, int& pb, int& pos) {
    if (t >= p.num_tokens) return false;
    if (t < p.subsequence_begins[0] || t >= p.subsequence_begins[p.num_seqs]) return false;
    const int s = locate_sequence(p.subsequence_begins, p.num_seqs, t, lane);
    pos = p.past_lens[s] + (t - p.subsequence_begins[s]);
    if (pos < 0) return false;
    const int lb = pos / p.block_size;
    const int tb0 = p.block_indices_begins[s];
    if (lb >= p.block_indices_begins[s + 1] - tb0) return false;
    pb = p.block_indices[tb0 + lb];
    return pb >= 0 && pb < p.num_blocks;
}

__device__ __forceinline__ float bits16_to_float(uint32_t bits, int dtype) {
    return dtype == HIPATTN_F16 ? f16_bits_to_float((uint16_t)bits) : bf16_bits_to_float((uint16_t)bits);
}
__device__ __forceinline__ uint32_t float_to_bits16(float x, int dtype) {
    return dtype == HIPATTN_F16 ? float_to_f16_bits(x) : float_to_bf16_bits(x);
}

// Minimum (maximum) of a value over each group of sixteen consecutive lanes, every lane getting the result.
template <bool kMax>
__device__ __forceinline__ float row16_reduce(float x) {
    const auto pick = [](float a, float b) { return kMax ? fmaxf(a, b) : fminf(a, b); };
    const auto dpp = [](float v, auto ctrl) {
        return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), decltype(ctrl)::value, 0xf, 0xf, false));
    };
    x = pick(x, dpp(x, std::integral_constant<int, 0xB1>{}));   // quad_perm [1, 0, 3, 2]
    x = pick(x, dpp(x, std::integral_constant<int, 0x4E>{}));   // quad_perm [2, 3, 0, 1]
    x = pick(x, dpp(x, std::integral_constant<int, 0x141>{}));  // row_half_mirror
    x = pick(x, dpp(x, std::integral_constant<int, 0x140>{}));  // row_mirror
    return x;
}

// Eight consecutive elements (d0 .. d0 + 7) of a new 128-element row, given as the 16 bytes `raw` of
// the kv type, go into the cache row at `row`, converted or quantised.  Sixteen consecutive lanes
// (a 16-lane group) hold one row between them; the u8 quantiser's minimum and maximum are reduced
// over that group, so every lane of the group must call this together (`active` false: take part
// in the reduction, store nothing).  The arithmetic is that of the element-wise path below, value
// for value (the quantiser's minimum and maximum do not depend on the order of the reduction).
__device__ __forceinline__ void kv_store_row8(const KvWriteParams& p, uint4_t raw, uint8_t* row, int d0, bool active,
                                              int lane) {
    if (p.cache_dtype == p.kv_dtype) {
        if (active) *(uint4_t*)(row + d0 * 2) = raw;
        return;
    }
    float x[8];
#pragma unroll
    for (int i = 0; i < 8; i++) x[i] = bits16_to_float((raw[i >> 1] >> ((i & 1) * 16)) & 0xffffu, p.kv_dtype);
    if (p.cache_dtype == HIPATTN_U8) {
        float mn = x[0], mx = x[0];
#pragma unroll
        for (int i = 1; i < 8; i++) {
            mn = fminf(mn, x[i]);
            mx = fmaxf(mx, x[i]);
        }
        // over the 16 lanes of the row, in the vector ALU (DPP: lane ^ 1, lane ^ 2, then the mirror image inside
        // eight and inside sixteen lanes, which by then holds the other half's result)
        mn = row16_reduce<false>(mn);
        mx = row16_reduce<true>(mx);
        float scale = (mx - mn) / 255.0f;
        if (scale == 0.0f) scale = 0.0001f;
        const float zp = -mn / scale + 0.0f;  // -0 becomes +0
        const float inv = 1.0f / scale;
        uint32_t q[8];
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = (uint32_t)fminf(fmaxf(rintf(fmaf(x[i], inv, zp)), 0.0f), 255.0f);
        uint2_t packed;
        packed[0] = q[0] | (q[1] << 8) | (q[2] << 16) | (q[3] << 24);
        packed[1] = q[4] | (q[5] << 8) | (q[6] << 16) | (q[7] << 24);
        if (active) {
            *(uint2_t*)(row + 8 + d0) = packed;
            if ((lane & 15) == 0) *(float2*)row = make_float2(scale, zp);
        }
    } else {  // the other 16-bit type
        uint4_t out;
#pragma unroll
        for (int i = 0; i < 4; i++)
            out[i] = float_to_bits16(x[2 * i], p.cache_dtype) | (float_to_bits16(x[2 * i + 1], p.cache_dtype) << 16);
        if (active) *(uint4_t*)(row + d0 * 2) = out;
    }
}

// Head size 128 with 16-bit new rows (p.vector_rows): the wavefront takes four kv heads of one
// token, which lie side by side in k_new / v_new, with one 16-byte load per lane for K and one for
// V -- 16 lanes and 8 elements each to a head -- and writes the cache rows with 16-byte (16-bit
// caches) or 8-byte (u8) stores.
__device__ __forceinline__ void kv_cache_write_rows128(const KvWriteParams& p, int64_t wv, int lane) {
    const int chunks = (p.num_heads_kv + 3) >> 2;
    const int t = (int)(wv / chunks);
    const int h = (int)(wv % chunks) * 4 + (lane >> 4);
    const int d0 = (lane & 15) * 8;
    int pb = 0, pos = 0;
    if (!kv_write_slot(p, t, lane, pb, pos)) return;  // wavefront-uniform
    const bool active = h < p.num_heads_kv;
    const int hh = active ? h : 0;  // idle lanes follow head 0 and store nothing
    const int64_t src_off = ((int64_t)t * p.num_heads_kv + hh) * 128 + d0;
    const uint4_t kraw = *(const uint4_t*)((const uint16_t*)p.k_new + src_off);
    const uint4_t vraw = *(const uint4_t*)((const uint16_t*)p.v_new + src_off);
    const int64_t rb = cache_row_bytes(p.cache_dtype, 128);
    const int64_t row_off = (((int64_t)pb * p.num_heads_kv + hh) * p.block_size + pos % p.block_size) * rb;
    kv_store_row8(p, kraw, p.key_cache + row_off, d0, active, lane);
    kv_store_row8(p, vraw, p.value_cache + row_off, d0, active, lane);
}

// The K row and the V row of ONE (token, kv head) pair, head size 128, 16-bit new rows, written by
// one wavefront that already knows the slot: lanes 0-15 take the K row, lanes 16-31 the V row.
// This is what a decode wavefront does for the sequence whose last cache block it is about to read.
__device__ __forceinline__ void kv_cache_write_pair128(const KvWriteParams& p, int t, int h, int pb, int pos, int lane) {
    const int which = lane >> 4;  // 0: K, 1: V, 2 and 3: idle
    const bool active = which < 2;
    const int d0 = (lane & 15) * 8;
    const int64_t src_off = ((int64_t)t * p.num_heads_kv + h) * 128 + d0;
    const uint16_t* src = (const uint16_t*)((which & 1) ? p.v_new : p.k_new);
    const uint4_t raw = *(const uint4_t*)(src + src_off);
    const int64_t rb = cache_row_bytes(p.cache_dtype, 128);
    const int64_t row_off = (((int64_t)pb * p.num_heads_kv + h) * p.block_size + pos % p.block_size) * rb;
    kv_store_row8(p, raw, ((which & 1) ? p.value_cache : p.key_cache) + row_off, d0, active, lane);
}

// Wavefront `wv` of the writer: the K rows and the V rows of one token for p.heads_per_wave kv
// heads, element by element: any head size, any pair of types.  The token's slot is looked up once
// per wavefront.
template <int kMaxPerLane>
__device__ __forceinline__ void kv_cache_write_wave(const KvWriteParams& p, int64_t wv, int lane) {
    if (p.vector_rows) {
        kv_cache_write_rows128(p, wv, lane);
        return;
    }
    const int hpw = p.heads_per_wave;
    const int groups = (p.num_heads_kv + hpw - 1) / hpw;
    const int t = (int)(wv / groups);
    const int h_begin = (int)(wv % groups) * hpw, h_end = min(h_begin + hpw, p.num_heads_kv);
    int pb = 0, pos = 0;
    if (!kv_write_slot(p, t, lane, pb, pos)) return;

    const int D = p.head_dim;
    const int64_t rb = cache_row_bytes(p.cache_dtype, D);
    for (int h = h_begin; h < h_end; h++) {
        const int64_t row_off = (((int64_t)pb * p.num_heads_kv + h) * p.block_size + pos % p.block_size) * rb;
        const int64_t src_off = ((int64_t)t * p.num_heads_kv + h) * D;

#pragma unroll
        for (int which = 0; which < 2; which++) {
            const void* src = which ? p.v_new : p.k_new;
            uint8_t* row = (which ? p.value_cache : p.key_cache) + row_off;
            float x[kMaxPerLane];
            float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
#pragma unroll
            for (int i = 0; i < kMaxPerLane; i++) {
                int d = lane + i * 64;
                if (d < D) {
                    x[i] = load_scalar(src, src_off + d, p.kv_dtype);
                    mn = fminf(mn, x[i]);
                    mx = fmaxf(mx, x[i]);
                } else {
                    x[i] = 0.0f;
                }
            }
            if (p.cache_dtype == HIPATTN_U8) {
                mn = wave_min(mn);
                mx = wave_max(mx);
                float scale = (mx - mn) / 255.0f;
                if (scale == 0.0f) scale = 0.0001f;
                const float zp = -mn / scale + 0.0f;  // -0 becomes +0
                const float inv = 1.0f / scale;
                if (lane == 0) {
                    ((float*)row)[0] = scale;
                    ((float*)row)[1] = zp;
                }
#pragma unroll
                for (int i = 0; i < kMaxPerLane; i++) {
                    int d = lane + i * 64;
                    if (d < D) {
                        float q = rintf(fmaf(x[i], inv, zp));
                        q = fminf(fmaxf(q, 0.0f), 255.0f);
                        row[8 + d] = (uint8_t)q;
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < kMaxPerLane; i++) {
                    int d = lane + i * 64;
                    if (d < D) store_scalar(row, d, p.cache_dtype, x[i]);
                }
            }
        }
    }
}

}  // namespace hipattn
