// Shape-generic attention kernels: fp32 VALU arithmetic, one wavefront per (query row, head),
// keys streamed in tiles of 64 with an online softmax.  These cover every dtype, head size
// (<= 512) and block size the ABI accepts, serve the small f32 correctness configuration,
// and are the on-device cross-check of the MFMA paths.  They are not tuned.
//
// Replaces the reference's decomposed chain MatMul -> Multiply -> Select/Add -> Softmax ->
// MatMul (src/ops/matmul.cpp:185-227, src/ops/softmax.cpp:178-193, src/ops/select.cpp:50-91).
#include "device_common.hpp"
#include "kernels.hpp"

namespace hipattn {

constexpr int kGenericMaxD = 512;
constexpr int kGenericSlots = kGenericMaxD / 64;
constexpr int kWavesPerBlock = 4;

// No additive term on the scores.
struct NoBias {
    __device__ __forceinline__ float operator()(int) const { return 0.0f; }
};

// ALiBi: slope * (key position - query position).
struct DistanceBias {
    float slope;
    int pos;
    __device__ __forceinline__ float operator()(int j) const { return slope * (float)(j - pos); }
};

// One row of an attention mask: element j at row + j * stride (stride 0: broadcast over the keys).
// Boolean masks (u8, nonzero = the key takes part) become 0 / -inf; float masks are added to the
// scaled scores, as ScaledDotProductAttention specifies.
struct MaskRow {
    const uint8_t* row;
    int64_t stride;  // elements
    int dtype;       // HIPATTN_F32 / F16 / BF16, or HIPATTN_U8 for boolean
    __device__ __forceinline__ float operator()(int j) const {
        if (dtype == HIPATTN_U8) return row[j * stride] ? 0.0f : -INFINITY;
        return load_scalar(row, j * stride, dtype);
    }
};

// Attend one query row to keys [j0, j1).  q_lds holds the row in fp32; KV yields row
// pointers and says which keys exist (a key in a block outside the cache has probability zero);
// bias(j) is added to the scaled score of key j.  Every lane of the wavefront must call this; the
// result for head-dim slot d = lane + 64 * i is returned in o[i], already normalised.  A row that
// can attend nothing (empty range, every key masked with -inf) yields zeros.
// sink: -INFINITY, or a logit that joins the row's softmax without a value row (the denominator grows by exp(sink)).
template <typename KV, typename Bias>
__device__ __forceinline__ void attend_row_wave(const float* q_lds, const KV& kv, const Bias& bias, int j0, int j1, int D,
                                                float scale, float (&o)[kGenericSlots], float sink = -INFINITY) {
    const int lane = threadIdx.x & 63;
    float m = -INFINITY, l = 0.0f;
#pragma unroll
    for (int i = 0; i < kGenericSlots; i++) o[i] = 0.0f;
    const float c = scale * kLog2e;
    for (int base = j0; base < j1; base += 64) {
        const int j = base + lane;
        float s = -INFINITY;
        if (j < j1 && kv.exists(j)) {
            const uint8_t* krow = kv.k_row(j);
            float acc = 0.0f;
            for (int d = 0; d < D; d++) acc = fmaf(q_lds[d], load_cache_elem(krow, d, kv.dtype), acc);
            s = fmaf(acc, c, bias(j) * kLog2e);
        }
        const float m_new = fmaxf(m, wave_max(s));
        if (m_new == -INFINITY) continue;  // nothing attended so far (wave-uniform)
        const float alpha = fast_exp2(m - m_new);  // exp2(-inf) = 0 on the first tile
        const float pj = (s != -INFINITY) ? fast_exp2(s - m_new) : 0.0f;
        l = l * alpha + wave_sum(pj);
        m = m_new;
#pragma unroll
        for (int i = 0; i < kGenericSlots; i++) o[i] *= alpha;
        const int n = min(64, j1 - base);
        for (int jj = 0; jj < n; jj++) {
            const float pb = __shfl(pj, jj, 64);
            if (pb == 0.0f) continue;  // (wave-uniform) masked keys may be unreadable or hold anything
            const uint8_t* vrow = kv.v_row(base + jj);
#pragma unroll
            for (int i = 0; i < kGenericSlots; i++) {
                const int d = lane + 64 * i;
                if (d < D) o[i] = fmaf(pb, load_cache_elem(vrow, d, kv.dtype), o[i]);
            }
        }
    }
    if (l > 0.0f && sink != -INFINITY) l += fast_exp2(sink * kLog2e - m);
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
    for (int i = 0; i < kGenericSlots; i++) o[i] *= inv;
}

struct DenseKV {
    const uint8_t* k;
    const uint8_t* v;
    int64_t row_bytes;
    int dtype;
    __device__ __forceinline__ bool exists(int) const { return true; }
    __device__ __forceinline__ const uint8_t* k_row(int j) const { return k + j * row_bytes; }
    __device__ __forceinline__ const uint8_t* v_row(int j) const { return v + j * row_bytes; }
};

struct PagedKV {
    const uint8_t* k;
    const uint8_t* v;
    const int32_t* blocks;  // this sequence's slice of block_indices
    int64_t row_bytes;
    int64_t block_stride;   // bytes between physical blocks
    int64_t head_off;       // byte offset of this kv head inside a block
    int block_size;
    int dtype;
    int num_blocks;
    // a block id outside the cache: its keys are skipped (probability zero), as the decode kernel does
    __device__ __forceinline__ bool exists(int j) const {
        const int pb = blocks[j / block_size];
        return pb >= 0 && pb < num_blocks;
    }
    __device__ __forceinline__ int64_t off(int j) const {
        return (int64_t)blocks[j / block_size] * block_stride + head_off + (int64_t)(j % block_size) * row_bytes;
    }
    __device__ __forceinline__ const uint8_t* k_row(int j) const { return k + off(j); }
    __device__ __forceinline__ const uint8_t* v_row(int j) const { return v + off(j); }
};

__global__ __launch_bounds__(64 * kWavesPerBlock) void sdpa_generic_kernel(SdpaParams p) {
    __shared__ float q_lds[kWavesPerBlock][kGenericMaxD];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t rows = (int64_t)p.batch * p.num_heads_q * p.len_q;
    const int64_t r = (int64_t)blockIdx.x * kWavesPerBlock + wave;
    if (r >= rows) return;  // whole wavefront leaves together; no block-wide barrier below
    const int D = p.head_dim;
    const int i = (int)(r % p.len_q);
    const int h = (int)((r / p.len_q) % p.num_heads_q);
    const int b = (int)(r / ((int64_t)p.len_q * p.num_heads_q));
    const int G = p.num_heads_q / p.num_heads_kv;
    for (int d = lane; d < D; d += 64) q_lds[wave][d] = load_scalar(p.q, r * D + d, p.dtype);
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0);  // LDS writes of this wavefront visible to all its lanes
    const int64_t rb = cache_row_bytes(p.dtype, D);
    const int64_t kv_off = ((int64_t)b * p.num_heads_kv + h / G) * p.len_kv * rb;
    DenseKV kv{(const uint8_t*)p.k + kv_off, (const uint8_t*)p.v + kv_off, rb, p.dtype};
    const int j1 = p.causal ? min(i + 1, p.len_kv) : p.len_kv;
    float o[kGenericSlots];
    if (p.mask && !p.causal) {  // (the operator ignores attention_mask when causal is set)
        const int64_t moff = (int64_t)b * p.mask_stride[0] + (int64_t)h * p.mask_stride[1] + (int64_t)i * p.mask_stride[2];
        const MaskRow bias{(const uint8_t*)p.mask + moff * (p.mask_dtype == HIPATTN_U8 ? 1 : dtype_bytes(p.mask_dtype)),
                           p.mask_stride[3], p.mask_dtype};
        attend_row_wave(q_lds[wave], kv, bias, 0, j1, D, p.scale, o);
    } else {
        attend_row_wave(q_lds[wave], kv, NoBias{}, 0, j1, D, p.scale, o);
    }
#pragma unroll
    for (int s = 0; s < kGenericSlots; s++) {
        const int d = lane + 64 * s;
        if (d < D) store_scalar(p.out, r * D + d, p.dtype, o[s]);
    }
}

__device__ __forceinline__ int find_sequence_of_token(const int32_t* __restrict__ begins, int num_seqs, int t) {
    int lo = 0, hi = num_seqs;
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if (begins[mid] <= t)
            lo = mid;
        else
            hi = mid;
    }
    return lo;
}

__global__ __launch_bounds__(64 * kWavesPerBlock) void paged_generic_kernel(PagedParams p) {
    __shared__ float q_lds[kWavesPerBlock][kGenericMaxD];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t rows = (int64_t)p.num_tokens * p.num_heads_q;
    const int64_t r = (int64_t)blockIdx.x * kWavesPerBlock + wave;
    if (r >= rows) return;
    const int t = (int)(r / p.num_heads_q);
    const int h = (int)(r % p.num_heads_q);
    if (t < p.subsequence_begins[0] || t >= p.subsequence_begins[p.num_seqs]) return;
    const int s = find_sequence_of_token(p.subsequence_begins, p.num_seqs, t);
    const int pos = p.past_lens[s] + (t - p.subsequence_begins[s]);
    const int D = p.head_dim;
    const int G = p.num_heads_q / p.num_heads_kv;
    for (int d = lane; d < D; d += 64) q_lds[wave][d] = load_scalar(p.q, r * D + d, p.q_dtype);
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0);
    const int64_t rb = cache_row_bytes(p.cache_dtype, D);
    PagedKV kv{p.key_cache,
               p.value_cache,
               p.block_indices + p.block_indices_begins[s],
               rb,
               (int64_t)p.num_heads_kv * p.block_size * rb,
               (int64_t)(h / G) * p.block_size * rb,
               p.block_size,
               p.cache_dtype,
               p.num_blocks};
    // never read beyond the sequence's block table
    const int table_tokens = (p.block_indices_begins[s + 1] - p.block_indices_begins[s]) * p.block_size;
    const int j1 = min(pos + 1, table_tokens);
    int j0 = 0;
    if (p.sliding_window > 0 && pos - p.sliding_window + 1 > 0) j0 = pos - p.sliding_window + 1;
    float o[kGenericSlots];
    const float sink = p.sinks ? p.sinks[h] : -INFINITY;
    if (p.alibi_slopes)
        attend_row_wave(q_lds[wave], kv, DistanceBias{p.alibi_slopes[h], pos}, j0, j1, D, p.scale, o, sink);
    else
        attend_row_wave(q_lds[wave], kv, NoBias{}, j0, j1, D, p.scale, o, sink);
#pragma unroll
    for (int sl = 0; sl < kGenericSlots; sl++) {
        const int d = lane + 64 * sl;
        if (d < D) store_scalar(p.out, r * D + d, p.out_dtype, o[sl]);
    }
}

hipError_t launch_sdpa_generic(const SdpaParams& p, hipStream_t stream) {
    const int64_t rows = (int64_t)p.batch * p.num_heads_q * p.len_q;
    if (rows == 0) return hipSuccess;
    const int64_t blocks = (rows + kWavesPerBlock - 1) / kWavesPerBlock;
    hipLaunchKernelGGL(sdpa_generic_kernel, dim3((unsigned)blocks), dim3(64 * kWavesPerBlock), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_paged_generic(const PagedParams& p, hipStream_t stream) {
    const int64_t rows = (int64_t)p.num_tokens * p.num_heads_q;
    if (rows == 0 || p.num_seqs == 0) return hipSuccess;
    const int64_t blocks = (rows + kWavesPerBlock - 1) / kWavesPerBlock;
    hipLaunchKernelGGL(paged_generic_kernel, dim3((unsigned)blocks), dim3(64 * kWavesPerBlock), 0, stream, p);
    return hipGetLastError();
}

__global__ void fill_bytes_kernel(uint8_t* dst, uint8_t value, size_t bytes) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < bytes; i += stride) dst[i] = value;
}

// out[i] = a[i] + b[i]; the floating types add in fp32 and round once, i32 wraps
__global__ void add_kernel(const void* a, const void* b, void* out, int64_t n, int dtype) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        if (dtype < 0)
            ((int32_t*)out)[i] = (int32_t)((uint32_t)((const int32_t*)a)[i] + (uint32_t)((const int32_t*)b)[i]);
        else
            store_scalar(out, i, dtype, load_scalar(a, i, dtype) + load_scalar(b, i, dtype));
    }
}

hipError_t launch_add(const void* a, const void* b, void* out, int64_t n, int dtype, hipStream_t stream) {
    if (n == 0) return hipSuccess;
    int64_t blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(add_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, a, b, out, n, dtype);
    return hipGetLastError();
}

hipError_t launch_fill_bytes(void* dst, int value, size_t bytes, hipStream_t stream) {
    if (bytes == 0) return hipSuccess;
    size_t blocks = (bytes + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(fill_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (uint8_t*)dst, (uint8_t)value,
                       bytes);
    return hipGetLastError();
}

}  // namespace hipattn
