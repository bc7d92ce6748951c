// The second output of PagedAttentionExtension: per key position of every sequence, the attention
// probability it received, summed over the query heads and over the sequence's last
// `score_aggregation_window` query tokens (all of its new tokens when no window is given) -- what a
// cache-eviction policy ranks tokens by.  fp32 VALU kernels, run after the cache holds the step's
// new keys, in two passes over the K rows:
//
//   paged_lse_*_kernel     log-sum-exp of every aggregated (query token, head)'s scaled scores
//   paged_scores_*_kernel  one wavefront per (sequence, 64 keys): every lane owns a key and adds up
//                          exp(score - lse) over the heads and the window's tokens, in a fixed order
//                          (the result does not depend on the launch shape)
//
// "fast": head sizes up to 128, key rows in registers, one read of a row per pass and kv head;
// the plain pair covers every other shape the ABI accepts.
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

static hipError_t launch_paged_scores_generic(const ScoresParams& p, hipStream_t stream);

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

// ---- head sizes up to 128 in multiples of 8, GQA groups up to 16: a lane holds its key's row in
// registers as floats (16-byte loads), the query rows of one (token, kv head) wait in LDS
// pre-multiplied by scale * log2(e), and every key row is read once per pass and kv head.  The
// loops run over a compile-time head size kD >= head_dim without branches (loads beyond the row
// are redirected to its start and their values dropped; the staged queries are zero there), so
// that the loads of a row are all in flight together.
constexpr int kFastG = 8;

template <int kD>
__device__ __forceinline__ void load_key_row(const uint8_t* row, int D, int dtype, float (&kf)[kD]) {
    if (dtype == HIPATTN_F32) {
#pragma unroll
        for (int c = 0; c < kD / 4; c++) {
            const bool in = c * 4 < D;
            const float4_t v = ((const float4_t*)row)[in ? c : 0];
#pragma unroll
            for (int i = 0; i < 4; i++) kf[c * 4 + i] = in ? v[i] : 0.0f;
        }
    } else if (dtype == HIPATTN_U8) {
        const float scale = ((const float*)row)[0], zp = ((const float*)row)[1];
#pragma unroll
        for (int c = 0; c < kD / 8; c++) {
            const bool in = c * 8 < D;
            const uint2_t v = ((const uint2_t*)(row + 8))[in ? c : 0];
#pragma unroll
            for (int i = 0; i < 8; i++) kf[c * 8 + i] = in ? ((float)((v[i >> 2] >> (8 * (i & 3))) & 0xffu) - zp) * scale : 0.0f;
        }
    } else {
#pragma unroll
        for (int c = 0; c < kD / 8; c++) {
            const bool in = c * 8 < D;
            const uint4_t v = ((const uint4_t*)row)[in ? c : 0];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const uint32_t w = v[i >> 1];
                // bf16: the bits are the upper half of the float; f16: v_cvt_f32_f16
                const float x = dtype == HIPATTN_F16 ? f16_bits_to_float((uint16_t)(w >> (16 * (i & 1))))
                                                     : __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
                kf[c * 8 + i] = in ? x : 0.0f;
            }
        }
    }
}

template <int kD>
__device__ __forceinline__ float dot_row(const float* q, const float (&kf)[kD]) {
    float acc = 0.0f;
#pragma unroll
    for (int c = 0; c < kD / 4; c++) {
        const float4_t qv = ((const float4_t*)q)[c];
#pragma unroll
        for (int i = 0; i < 4; i++) acc = fmaf(qv[i], kf[c * 4 + i], acc);
    }
    return acc;
}

// the G query rows of (token t, kv head kvh) into an LDS slot of G rows of kD floats, times c, zero beyond head_dim
template <int kD>
__device__ __forceinline__ void stage_queries(const ScoresParams& p, float* slot, int t, int kvh, int G, float c, int lane, int lanes) {
    const int D = p.head_dim;
    for (int i = lane; i < G * kD; i += lanes) {
        const int g = i / kD, d = i % kD;
        slot[i] = d < D ? c * load_scalar(p.q, ((int64_t)t * p.num_heads_q + kvh * G + g) * D + d, p.q_dtype) : 0.0f;
    }
}

// one workgroup per (query token, kv head): its four wavefronts share the key tiles and combine
// their running (max, sum) of the G heads through LDS
template <int kD>
__global__ __launch_bounds__(64 * kWaves) void paged_lse_fast_kernel(ScoresParams p) {
    __shared__ __attribute__((aligned(16))) float q_lds[kFastG * kD];
    __shared__ float part[kWaves][kFastG][2];
    __shared__ float ml[kFastG][64 * kWaves][2];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int t = blockIdx.x / p.num_heads_kv, kvh = blockIdx.x % p.num_heads_kv;
    if (t < p.subsequence_begins[0] || t >= p.subsequence_begins[p.num_seqs]) return;
    const int s = sequence_of(p.subsequence_begins, p.num_seqs, t);
    const SeqView v = seq_view(p, s);
    if (t < v.first_scored) return;  // the whole workgroup leaves together
    const int D = p.head_dim, G = p.num_heads_q / p.num_heads_kv;
    const int64_t rb = cache_row_bytes(p.cache_dtype, D);
    stage_queries<kD>(p, q_lds, t, kvh, G, p.scale * kLog2e, threadIdx.x, 64 * kWaves);
    __syncthreads();
    int j0, j1;
    key_range(p, v, v.past + (t - v.begin), j0, j1);
    // a lane's running (max, sum) per head live in LDS: indexing them by a runtime head number in
    // registers would send them to scratch memory
    for (int g = 0; g < G; g++) ml[g][threadIdx.x][0] = -INFINITY, ml[g][threadIdx.x][1] = 0.0f;
    float kf[kD];
    for (int base = j0 + wave * 64; base < j1; base += 64 * kWaves) {
        const int j = base + lane;
        const uint8_t* krow = j < j1 ? key_row(p, v, j, kvh, rb) : nullptr;
        if (krow == nullptr) continue;
        load_key_row<kD>(krow, D, p.cache_dtype, kf);
#pragma unroll 1
        for (int g = 0; g < G; g++) {
            const float sc = dot_row<kD>(q_lds + g * kD, kf);
            const float m_old = ml[g][threadIdx.x][0];
            const float m_new = fmaxf(m_old, sc);
            ml[g][threadIdx.x][1] = ml[g][threadIdx.x][1] * fast_exp2(m_old - m_new) + fast_exp2(sc - m_new);
            ml[g][threadIdx.x][0] = m_new;
        }
    }
#pragma unroll 1
    for (int g = 0; g < G; g++) {
        const float mg = ml[g][threadIdx.x][0];
        const float mw = wave_max(mg);
        const float lw = wave_sum(mg == -INFINITY ? 0.0f : ml[g][threadIdx.x][1] * fast_exp2(mg - mw));
        if (lane == 0) part[wave][g][0] = mw, part[wave][g][1] = lw;
    }
    __syncthreads();
    if (threadIdx.x < G) {
        const int g = threadIdx.x;
        float mm = -INFINITY, ll = 0.0f;
        for (int w = 0; w < kWaves; w++) mm = fmaxf(mm, part[w][g][0]);
        for (int w = 0; w < kWaves; w++)
            if (part[w][g][0] != -INFINITY) ll += part[w][g][1] * fast_exp2(part[w][g][0] - mm);
        // v_log_f32 is log2; +inf when nothing is attended: every probability then comes out 0
        p.lse[(int64_t)t * p.num_heads_q + kvh * G + g] = ll > 0.0f ? mm + __builtin_amdgcn_logf(ll) : INFINITY;
    }
}

// one wavefront per (sequence, 64 keys): a lane's key against every kv head's G heads of every aggregated token
template <int kD>
__global__ __launch_bounds__(64 * kWaves) void paged_scores_fast_kernel(ScoresParams p) {
    __shared__ __attribute__((aligned(16))) float q_lds[kWaves][kFastG * kD];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int s = blockIdx.y;
    const SeqView v = seq_view(p, s);
    const int ctx = v.past + (v.end - v.begin);
    const int base = (blockIdx.x * kWaves + wave) * 64;
    if (base >= ctx) return;  // wave-uniform
    int64_t ahead = 0;
    for (int i = lane; i < s; i += 64) ahead += p.past_lens[i] + (p.subsequence_begins[i + 1] - p.subsequence_begins[i]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ahead += __shfl_xor(ahead, off, 64);
    const int j = base + lane;
    const int D = p.head_dim, G = p.num_heads_q / p.num_heads_kv;
    const int64_t rb = cache_row_bytes(p.cache_dtype, D);
    const float c = p.scale * kLog2e;
    float total = 0.0f;
    float kf[kD];
    for (int kvh = 0; kvh < p.num_heads_kv; kvh++) {
        const uint8_t* krow = (j < ctx && j < v.table_tokens) ? key_row(p, v, j, kvh, rb) : nullptr;
        if (krow != nullptr) load_key_row<kD>(krow, D, p.cache_dtype, kf);
        for (int t = v.first_scored; t < v.end; t++) {
            int j0, j1;
            key_range(p, v, v.past + (t - v.begin), j0, j1);
            if (base >= j1 || base + 64 <= j0) continue;  // wave-uniform: no key of this tile is attended
            __builtin_amdgcn_wave_barrier();  // the rows staged before have been read by every lane
            stage_queries<kD>(p, q_lds[wave], t, kvh, G, c, lane, 64);
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_s_waitcnt(0);
            if (krow != nullptr && j >= j0 && j < j1) {
#pragma unroll 1
                for (int g = 0; g < G; g++)
                    total += fast_exp2(dot_row<kD>(q_lds[wave] + g * kD, kf) - p.lse[(int64_t)t * p.num_heads_q + kvh * G + g]);
            }
        }
    }
    if (j < ctx && ahead + j < p.scores_capacity) p.scores[ahead + j] = total;
}

template <int kD>
static hipError_t launch_fast(const ScoresParams& p, hipStream_t stream) {
    const int64_t groups = (int64_t)p.num_tokens * p.num_heads_kv;
    if (groups > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(paged_lse_fast_kernel<kD>, dim3((unsigned)groups), dim3(64 * kWaves), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int tiles = (p.max_context_len + 64 * kWaves - 1) / (64 * kWaves);
    hipLaunchKernelGGL(paged_scores_fast_kernel<kD>, dim3((unsigned)tiles, (unsigned)p.num_seqs), dim3(64 * kWaves), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_paged_scores(const ScoresParams& p, hipStream_t stream) {
    if ((int64_t)p.num_tokens * p.num_heads_q == 0 || p.num_seqs == 0 || p.max_context_len == 0) return hipSuccess;
    const int G = p.num_heads_q / p.num_heads_kv;
    const bool fast = p.head_dim <= 128 && p.head_dim % 8 == 0 && G <= kFastG && ((uintptr_t)p.key_cache % 16) == 0;
    if (fast) return p.head_dim <= 64 ? launch_fast<64>(p, stream) : launch_fast<128>(p, stream);
    return launch_paged_scores_generic(p, stream);
}

static hipError_t launch_paged_scores_generic(const ScoresParams& p, hipStream_t stream) {
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
