// Device-side KV-cache block writer: scatters the new key/value rows of a batch into the
// paged caches, converting or quantising on the way.  HBM-bound byte moving: one wavefront
// per (token, kv head) -- per token for large batches --, contiguous rows, no staging.
//
// Nearest reference analogue: the row scatter of src/kernels/scatter_nd_update.cu:19-34,
// 36-79 (which first copies the whole input, scatter_nd_update.cu:170-171; this writer
// touches only the new rows) and the whole-state copies of
// src/cuda_variable_state.hpp:135-160.  Out-of-range targets are skipped as in
// tests/unit/kernels/scatter_update.cpp:59-86.
#include "kv_cache_write.hpp"

namespace hipattn {

template <int kMaxPerLane>
__global__ __launch_bounds__(256) void kv_cache_write_kernel(KvWriteParams p) {
    kv_cache_write_wave<kMaxPerLane>(p, (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6), threadIdx.x & 63);
}

hipError_t launch_kv_cache_write(const KvWriteParams& params, hipStream_t stream) {
    if (params.num_tokens == 0 || params.num_seqs == 0) return hipSuccess;
    KvWriteParams p = params;
    dim3 grid((unsigned)((kv_write_wavefronts(p) + 3) / 4));
    if (p.head_dim <= 128)
        hipLaunchKernelGGL(kv_cache_write_kernel<2>, grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(kv_cache_write_kernel<8>, grid, dim3(256), 0, stream, p);
    return hipGetLastError();
}

// ---- cache rotation ---------------------------------------------------------------------------
// One wavefront per (listed block, token, kv head): the row's pairs (i, i + D/2) over the lanes, turned in fp32
// and stored in the cache's type; a u8 row is quantised again from the minimum and maximum of the turned
// values, with the writer's arithmetic.  Rare (a cache-eviction policy asks for it now and then), so plain.
// No counterpart in the reference.
__global__ __launch_bounds__(256) void rotate_key_cache_kernel(KeyRotationParams p) {
    const int lane = threadIdx.x & 63;
    const int64_t wv = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t rows = (int64_t)p.num_rotated * p.block_size * p.num_heads_kv;
    if (wv >= rows) return;
    const int h = (int)(wv % p.num_heads_kv), t = (int)((wv / p.num_heads_kv) % p.block_size);
    const int b = (int)(wv / ((int64_t)p.num_heads_kv * p.block_size));
    const int pb = p.rotated_block_indices[b];
    if (pb < 0 || pb >= p.num_blocks) return;  // names no block
    const int delta = p.rotation_deltas[(int64_t)b * p.deltas_per_block + (p.deltas_per_block == 1 ? 0 : t)];
    if (delta < 0 || delta >= p.lut_rows) return;  // no row of the table: the token stays as it is
    const int D = p.head_dim, half = D / 2;
    uint8_t* const row = p.key_cache + (((int64_t)pb * p.num_heads_kv + h) * p.block_size + t) * cache_row_bytes(p.cache_dtype, D);
    constexpr int kMaxPairs = 4;  // head sizes up to 512
    float y0[kMaxPairs], y1[kMaxPairs];
    float mn = INFINITY, mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < kMaxPairs; u++) {
        const int i = lane + 64 * u;
        y0[u] = y1[u] = 0.0f;
        if (i < half) {
            const float x0 = load_cache_elem(row, i, p.cache_dtype), x1 = load_cache_elem(row, i + half, p.cache_dtype);
            const float cs = load_scalar(p.trig_lut, (int64_t)delta * D + i, p.lut_dtype);
            const float sn = load_scalar(p.trig_lut, (int64_t)delta * D + half + i, p.lut_dtype);
            const float t0 = x1 * sn, t1 = x1 * cs;
            y0[u] = __builtin_fmaf(x0, cs, -t0);
            y1[u] = __builtin_fmaf(x0, sn, t1);
            mn = fminf(mn, fminf(y0[u], y1[u]));
            mx = fmaxf(mx, fmaxf(y0[u], y1[u]));
        }
    }
    float scale = 0.0f, zp = 0.0f, inv = 0.0f;
    if (p.cache_dtype == HIPATTN_U8) {
        mn = wave_min(mn);  // (every load of the row has returned: the values above depend on them)
        mx = wave_max(mx);
        scale = (mx - mn) / 255.0f;
        if (scale == 0.0f) scale = 0.0001f;
        zp = -mn / scale + 0.0f;
        inv = 1.0f / scale;
        if (lane == 0) *(float2*)row = make_float2(scale, zp);
    }
#pragma unroll
    for (int u = 0; u < kMaxPairs; u++) {
        const int i = lane + 64 * u;
        if (i >= half) continue;
        switch (p.cache_dtype) {
            case HIPATTN_F32:
                ((float*)row)[i] = y0[u];
                ((float*)row)[i + half] = y1[u];
                break;
            case HIPATTN_F16:
            case HIPATTN_BF16:
                ((uint16_t*)row)[i] = (uint16_t)float_to_bits16(y0[u], p.cache_dtype);
                ((uint16_t*)row)[i + half] = (uint16_t)float_to_bits16(y1[u], p.cache_dtype);
                break;
            default:
                row[8 + i] = (uint8_t)fminf(fmaxf(rintf(fmaf(y0[u], inv, zp)), 0.0f), 255.0f);
                row[8 + i + half] = (uint8_t)fminf(fmaxf(rintf(fmaf(y1[u], inv, zp)), 0.0f), 255.0f);
        }
    }
}

hipError_t launch_rotate_key_cache(const KeyRotationParams& p, hipStream_t stream) {
    const int64_t rows = (int64_t)p.num_rotated * p.block_size * p.num_heads_kv;
    if (rows == 0) return hipSuccess;
    if ((rows + 3) / 4 > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(rotate_key_cache_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, p);
    return hipGetLastError();
}

}  // namespace hipattn
