// Device side of the KV-cache block writer, shared by the stand-alone writer kernel and the
// paged-attention prologue kernel (which also plans the decode schedule in the same launch).
#pragma once

#include "device_common.hpp"
#include "kernels.hpp"

namespace hipattn {

// sequence that owns token t: largest s with subsequence_begins[s] <= t
__device__ __forceinline__ int find_sequence(const int32_t* __restrict__ begins, int num_seqs, int t) {
    int lo = 0, hi = num_seqs;  // invariant: begins[lo] <= t < begins[hi]
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if (begins[mid] <= t)
            lo = mid;
        else
            hi = mid;
    }
    return lo;
}

// Wavefront `wv` of the writer: the K rows and the V rows of one token for p.heads_per_wave kv
// heads.  The token's slot (sequence by binary search, position, block table entry: a chain of
// dependent loads) is looked up once per wavefront.
template <int kMaxPerLane>
__device__ __forceinline__ void kv_cache_write_wave(const KvWriteParams& p, int64_t wv, int lane) {
    const int hpw = p.heads_per_wave;
    const int groups = (p.num_heads_kv + hpw - 1) / hpw;
    const int t = (int)(wv / groups);
    const int h_begin = (int)(wv % groups) * hpw, h_end = min(h_begin + hpw, p.num_heads_kv);
    if (t >= p.num_tokens) return;
    // tokens outside every sequence (padding after the last subsequence) are ignored
    if (t < p.subsequence_begins[0] || t >= p.subsequence_begins[p.num_seqs]) return;
    const int s = find_sequence(p.subsequence_begins, p.num_seqs, t);
    const int pos = p.past_lens[s] + (t - p.subsequence_begins[s]);
    if (pos < 0) return;
    const int lb = pos / p.block_size;
    const int tb0 = p.block_indices_begins[s];
    if (lb >= p.block_indices_begins[s + 1] - tb0) return;
    const int pb = p.block_indices[tb0 + lb];
    if (pb < 0 || pb >= p.num_blocks) return;

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
