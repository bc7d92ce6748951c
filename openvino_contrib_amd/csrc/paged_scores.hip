// The second output of PagedAttentionExtension: per key position of every sequence, the attention
// probability it received, summed over the query heads and over the sequence's last
// `score_aggregation_window` query tokens (all of its new tokens when no window is given) -- what a
// cache-eviction policy ranks tokens by.  Shape-generic fp32 VALU kernels in the style of the
// generic attention kernels, run after the cache holds the step's new keys; not tuned.
//
//   paged_lse_kernel     one wavefront per (query token, head): log-sum-exp of its scaled scores
//   paged_scores_kernel  one wavefront per (sequence, 64 keys): every lane owns a key and adds up
//                        exp(score - lse) over the heads and the window's tokens, in a fixed order
//                        (the result does not depend on the launch shape)
#include "device_common.hpp"
#include "kernels.hpp"

namespace hipattn {

namespace {

constexpr int kMaxD = 512;
constexpr int kWaves = 4;

struct SeqView {
    int begin, end;      // tokens of the sequence in the batch
    int past;            // cache length before this step
    int first_scored;    // first token whose probabilities are aggregated
    int table_tokens;    // tokens the sequence's block table can hold
    const int32_t* blocks;
};

__device__ __forceinline__ SeqView seq_view(const ScoresParams& p, int s) {
    SeqView v;
    v.begin = p.subsequence_begins[s];
    v.end = p.subsequence_begins[s + 1];
    v.past = p.past_lens[s];
    int w = v.end - v.begin;
    if (p.score_window != nullptr) w = max(0, min(w, p.score_window[s]));
    v.first_scored = v.end - w;
    v.table_tokens = (p.block_indices_begins[s + 1] - p.block_indices_begins[s]) * p.block_size;
    v.blocks = p.block_indices + p.block_indices_begins[s];
    return v;
}

// keys a query at cache position `pos` attends: (pos - window, pos], clipped to the block table
__device__ __forceinline__ void key_range(const ScoresParams& p, const SeqView& v, int pos, int& j0, int& j1) {
    j1 = min(pos + 1, v.table_tokens);
    j0 = (p.sliding_window > 0 && pos - p.sliding_window + 1 > 0) ? pos - p.sliding_window + 1 : 0;
}

__device__ __forceinline__ const uint8_t* key_row(const ScoresParams& p, const SeqView& v, int j, int kvh, int64_t rb) {
    const int pb = v.blocks[j / p.block_size];
    if (pb < 0 || pb >= p.num_blocks) return nullptr;  // a block outside the cache: probability zero
    return p.key_cache + ((int64_t)pb * p.num_heads_kv + kvh) * p.block_size * rb + (int64_t)(j % p.block_size) * rb;
}

__device__ __forceinline__ int sequence_of(const int32_t* __restrict__ begins, int num_seqs, int t) {
    int lo = 0, hi = num_seqs;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (begins[mid] <= t)
            lo = mid;
        else
            hi = mid;
    }
    return lo;
}

}  // namespace

__global__ __launch_bounds__(64 * kWaves) void paged_lse_kernel(ScoresParams p) {
    __shared__ float q_lds[kWaves][kMaxD];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * kWaves + wave;
    if (r >= (int64_t)p.num_tokens * p.num_heads_q) return;
    const int t = (int)(r / p.num_heads_q), h = (int)(r % p.num_heads_q);
    if (t < p.subsequence_begins[0] || t >= p.subsequence_begins[p.num_seqs]) return;
    const int s = sequence_of(p.subsequence_begins, p.num_seqs, t);
    const SeqView v = seq_view(p, s);
    if (t < v.first_scored) return;  // not aggregated: its log-sum-exp is never read
    const int D = p.head_dim;
    for (int d = lane; d < D; d += 64) q_lds[wave][d] = load_scalar(p.q, r * D + d, p.q_dtype);
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0);
    const int64_t rb = cache_row_bytes(p.cache_dtype, D);
    const int kvh = h / (p.num_heads_q / p.num_heads_kv);
    int j0, j1;
    key_range(p, v, v.past + (t - v.begin), j0, j1);
    const float c = p.scale * kLog2e;
    float m = -INFINITY, l = 0.0f;
    for (int base = j0; base < j1; base += 64) {
        const int j = base + lane;
        float sc = -INFINITY;
        if (j < j1) {
            if (const uint8_t* krow = key_row(p, v, j, kvh, rb)) {
                float acc = 0.0f;
                for (int d = 0; d < D; d++) acc = fmaf(q_lds[wave][d], load_cache_elem(krow, d, p.cache_dtype), acc);
                sc = acc * c;
            }
        }
        const float m_new = fmaxf(m, wave_max(sc));
        if (m_new == -INFINITY) continue;
        l = l * fast_exp2(m - m_new) + wave_sum(sc != -INFINITY ? fast_exp2(sc - m_new) : 0.0f);
        m = m_new;
    }
    if (lane == 0) p.lse[r] = l > 0.0f ? m + __builtin_amdgcn_logf(l) : INFINITY;  // v_log_f32 is log2; +inf: every probability 0
}

__global__ __launch_bounds__(64 * kWaves) void paged_scores_kernel(ScoresParams p) {
    __shared__ float q_lds[kWaves][kMaxD];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int s = blockIdx.y;
    const SeqView v = seq_view(p, s);
    const int ctx = v.past + (v.end - v.begin);
    const int base = (blockIdx.x * kWaves + wave) * 64;
    if (base >= ctx) return;  // wave-uniform
    // where this sequence's scores start: the context lengths of the sequences ahead of it
    int64_t ahead = 0;
    for (int i = lane; i < s; i += 64) ahead += p.past_lens[i] + (p.subsequence_begins[i + 1] - p.subsequence_begins[i]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ahead += __shfl_xor(ahead, off, 64);
    const int j = base + lane;
    const int D = p.head_dim;
    const int G = p.num_heads_q / p.num_heads_kv;
    const int64_t rb = cache_row_bytes(p.cache_dtype, D);
    const float c = p.scale * kLog2e;
    float total = 0.0f;
    for (int kvh = 0; kvh < p.num_heads_kv; kvh++) {
        const uint8_t* krow = (j < ctx && j < v.table_tokens) ? key_row(p, v, j, kvh, rb) : nullptr;
        for (int t = v.first_scored; t < v.end; t++) {
            int j0, j1;
            key_range(p, v, v.past + (t - v.begin), j0, j1);
            if (base >= j1 || base + 64 <= j0) continue;  // wave-uniform: no key of this tile is attended
            const bool mine = krow != nullptr && j >= j0 && j < j1;
            for (int g = 0; g < G; g++) {
                const int h = kvh * G + g;
                const int64_t r = (int64_t)t * p.num_heads_q + h;
                __builtin_amdgcn_wave_barrier();  // the previous row has been read by every lane
                for (int d = lane; d < D; d += 64) q_lds[wave][d] = load_scalar(p.q, r * D + d, p.q_dtype);
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_s_waitcnt(0);
                if (mine) {
                    float acc = 0.0f;
                    for (int d = 0; d < D; d++) acc = fmaf(q_lds[wave][d], load_cache_elem(krow, d, p.cache_dtype), acc);
                    total += fast_exp2(acc * c - p.lse[r]);
                }
            }
        }
    }
    if (j < ctx && ahead + j < p.scores_capacity) p.scores[ahead + j] = total;
}

hipError_t launch_paged_scores(const ScoresParams& p, hipStream_t stream) {
    const int64_t rows = (int64_t)p.num_tokens * p.num_heads_q;
    if (rows == 0 || p.num_seqs == 0 || p.max_context_len == 0) return hipSuccess;
    hipLaunchKernelGGL(paged_lse_kernel, dim3((unsigned)((rows + kWaves - 1) / kWaves)), dim3(64 * kWaves), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int tiles = (p.max_context_len + 64 * kWaves - 1) / (64 * kWaves);
    hipLaunchKernelGGL(paged_scores_kernel, dim3((unsigned)tiles, (unsigned)p.num_seqs), dim3(64 * kWaves), 0, stream, p);
    return hipGetLastError();
}

}  // namespace hipattn
