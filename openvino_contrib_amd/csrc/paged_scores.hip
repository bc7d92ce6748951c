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
//
// Head sizes 64 and 128 with 16-bit queries on fp16 / bf16 / u8 caches (blocks of 16 tokens or more, up to
// 16 query heads per kv head, or more in equal groups of 8 to 16) take the matrix cores instead, when the caller's workspace has room
// for the raw scores: the K rows are read ONCE,
//
//   paged_scores_mma_kernel      one wavefront per (aggregated token, kv head, 512 keys): S^T = K Q^T on
//                                v_mfma_f32_16x16x32 as in the decode kernel, the scaled scores (log2
//                                domain) stored to the workspace, a (max, sum) per head and wavefront
//   paged_scores_lse_kernel      the wavefronts' (max, sum) of a (token, head) combined to its log-sum-exp
//   paged_scores_sum_kernel      a lane per key: exp2(score - lse) added up over heads and tokens in a
//                                fixed order
#include "decode_operands.hpp"
#include "device_common.hpp"
#include "kernels.hpp"

#include <algorithm>
#include <cstdlib>
#include <type_traits>

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


// ---- matrix cores: raw scores to the workspace, one read of the K rows ---------------------------
namespace {

constexpr int kMmaUnit = 32;         // keys a wavefront works through at a time (two tiles of 16)
constexpr int kMmaChunkUnits = 8;   // units per wavefront
constexpr int kMmaWaves = 4;         // wavefronts (items) per workgroup
constexpr size_t kMmaRawCap = size_t(256) << 20;  // largest raw-score area the size query asks a caller for

__host__ __device__ inline int mma_units_bound(int max_context_len) { return (max_context_len + kMmaUnit - 1) / kMmaUnit + 1; }
__host__ __device__ inline int mma_chunks(int max_context_len) { return (mma_units_bound(max_context_len) + kMmaChunkUnits - 1) / kMmaChunkUnits; }
__host__ __device__ inline int mma_stride(int max_context_len) { return mma_units_bound(max_context_len) * kMmaUnit; }

// More than 16 query heads per kv head: in equal groups of 8 to 16, each group an item of its own that reads the
// kv head's rows again (0: no such split).
__host__ __device__ inline int mma_kv_share(int heads_q, int heads_kv) {
    const int G = heads_q / heads_kv;
    if (G <= 16) return 1;
    for (int share = 2; share <= G; share++) {
        if (G % share != 0 || G / share > 16) continue;
        return G / share >= 8 ? share : 0;
    }
    return 0;
}

// The keys an aggregated token's scores cover, and whether it has any.
struct MmaRow {
    int s, j0, j1;
    bool scored;
};
__device__ __forceinline__ MmaRow mma_row(const ScoresParams& p, int t, SeqView& v) {
    MmaRow r;
    r.scored = false;
    r.s = 0;
    r.j0 = r.j1 = 0;
    // a decode batch has token t in sequence t: tried first, one round of loads instead of a search
    const int guess = min(t, p.num_seqs - 1);
    if (p.subsequence_begins[guess] <= t && t < p.subsequence_begins[guess + 1]) {
        r.s = guess;
    } else {
        if (t < p.subsequence_begins[0] || t >= p.subsequence_begins[p.num_seqs]) return r;
        r.s = sequence_of(p.subsequence_begins, p.num_seqs, t);
    }
    v = seq_view(p, r.s);
    if (t < v.first_scored) return r;
    key_range(p, v, v.past + (t - v.begin), r.j0, r.j1);
    r.j1 = min(r.j1, p.max_context_len);  // (the raw area is sized by the caller's bound)
    r.scored = r.j0 < r.j1;
    return r;
}

template <bool kU8, int kHD>
struct KeyRegs {
    using Piece = typename std::conditional<kU8, uint2_t, uint4_t>::type;
    Piece k[2][kHD / 32];  // [tile][k-step]: K[tile*16 + (lane & 15)][(i*4 + kg)*8 .. +8]
    float2 sz[kU8 ? 8 : 1];  // u8: (scale, zero-point) of token tile*16 + kg*4 + r at [tile*4 + r]
    int ok;                // bit t: tile t lies in a block of the cache and holds an attended key
};

}  // namespace

template <bool kU8, bool kBf16, int kHD>
__global__ __launch_bounds__(64 * kMmaWaves) void paged_scores_mma_kernel(ScoresParams p) {
    using O = Op16<kBf16>;
    const int lane = threadIdx.x & 63, n16 = lane & 15, kg = lane >> 4;
    const int chunks = mma_chunks(p.max_context_len);
    const int share = mma_kv_share(p.num_heads_q, p.num_heads_kv);  // (1 unless a kv head has more than 16 query heads)
    const int heads = p.num_heads_kv * share;                        // items per (token, chunk): head groups
    const int G = p.num_heads_q / heads;
    const int shift = __builtin_ctz(p.block_size);
    constexpr int kRow = kU8 ? kHD + 8 : 2 * kHD;
    const float c = p.scale * kLog2e;
    // Items are (token, chunk, kv head), kv heads side by side, four to a workgroup; an item beyond its sequence's
    // end leaves at once.  (A workgroup per item, wavefronts walking the item list in steps of the grid, 4, 8 or 16
    // units per item: all within 5 % of each other on 64 decode rows of 512..8,192 keys, 0.17-0.18 ms.)
    const int64_t items = (int64_t)heads * p.num_tokens * chunks;
    const int64_t item = (int64_t)blockIdx.x * kMmaWaves + __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    if (item >= items) return;
    // kvh: the head group (query heads kvh * G ...), whose K rows are those of kv head kvh / share
    const int kvh = (int)(item % heads), chunk = (int)((item / heads) % chunks), t = (int)(item / ((int64_t)heads * chunks));
    SeqView v;
    MmaRow row = mma_row(p, t, v);
    if (!row.scored) return;
    // (wave-uniform values the loop is steered by, kept in scalar registers: as loaded values in vector registers
    // they would make every iteration wait for all outstanding loads)
    row.j0 = __builtin_amdgcn_readfirstlane(row.j0);
    row.j1 = __builtin_amdgcn_readfirstlane(row.j1);
    const int u_first = row.j0 / kMmaUnit + chunk * kMmaChunkUnits;
    const int u_end = min((row.j1 + kMmaUnit - 1) / kMmaUnit, u_first + kMmaChunkUnits);
    if (u_first >= u_end) return;

    // Q^T operand: k-step i of lane (head n16, kg) holds Q[head][(i*4 + kg)*8 .. +8], so that the four lanes of a
    // key row read 64 contiguous bytes of it per load instruction; heads beyond the group are zero
    typename O::vec8 qf[kHD / 32];
    float sumq = 0.0f;
#pragma unroll
    for (int i = 0; i < kHD / 32; i++) {
        if (n16 < G) {
            qf[i] = load_q8<kBf16>(p.q, ((int64_t)t * p.num_heads_q + kvh * G + n16) * kHD + (i * 4 + kg) * 8, p.q_dtype);
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) O::set(qf[i], e, 0.0f);
        }
        if constexpr (kU8) {
#pragma unroll
            for (int e = 0; e < 8; e++) sumq += O::get(qf[i], e);
        }
    }
    if constexpr (kU8) {
        sumq += __shfl_xor(sumq, 16, 64);
        sumq += __shfl_xor(sumq, 32, 64);
    }

    // the blocks of the chunk's 32 tiles, one per lane, fetched ahead of everything: no table load sits between a
    // unit and its rows
    int my_pb = -1;
    {
        const int tok = (u_first * 2 + lane) * 16;  // the first key of tile `lane` of the chunk
        if (lane < 2 * kMmaChunkUnits && tok < row.j1 && tok + 16 > row.j0) my_pb = v.blocks[tok >> shift];
    }
    // No branch around the loads (the wait counts the compiler inserts stay exact only in straight-line code, and
    // an inexact one waits for the unit that was just requested as well): a tile without a block of its own
    // reads block 0 and is masked out of the scores.
    auto fetch = [&](int u, KeyRegs<kU8, kHD>& r) __attribute__((always_inline)) {
        r.ok = 0;
#pragma unroll
        for (int tl = 0; tl < 2; tl++) {
            const int tok = u * kMmaUnit + tl * 16;  // the tile's first key
            const int pb = __builtin_amdgcn_readlane(my_pb, (u - u_first) * 2 + tl);  // (-1: no attended key in the tile)
            const bool ok = pb >= 0 && pb < p.num_blocks;
            r.ok |= ok ? 1 << tl : 0;
            const uint8_t* const base = p.key_cache + (((int64_t)(ok ? pb : 0) * p.num_heads_kv + kvh / share) * p.block_size + (tok & (p.block_size - 1))) * kRow;
#pragma unroll
            for (int i = 0; i < kHD / 32; i++) {
                if constexpr (kU8)
                    r.k[tl][i] = *(const uint2_t*)(base + n16 * kRow + 8 + (i * 4 + kg) * 8);
                else
                    r.k[tl][i] = *(const uint4_t*)(base + n16 * kRow + (i * 4 + kg) * 16);
            }
            if constexpr (kU8) {
#pragma unroll
                for (int q = 0; q < 4; q++) r.sz[tl * 4 + q] = *(const float2*)(base + (kg * 4 + q) * kRow);
            }
        }
    };

    float m = -INFINITY, l = 0.0f;  // of this lane's keys, for head n16
    float* const raw_row = p.raw + ((int64_t)t * p.num_heads_q + kvh * G + n16) * p.raw_stride;
    auto process = [&](int u, const KeyRegs<kU8, kHD>& r) __attribute__((always_inline)) {
        float x[8];
        float mloc = -INFINITY;
#pragma unroll
        for (int tl = 0; tl < 2; tl++) {
            float4_t sc = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < kHD / 32; i++) {
                typename O::vec8 a;
                if constexpr (!kU8) {
                    a = O::from_bits(r.k[tl][i]);
                } else {
                    // bytes as fp16 numbers 1024 + byte, then exactly byte - 128: small operands keep the
                    // cancellation against the zero-point term small
                    uint4_t w;
                    w[0] = bytes_to_biased_half2(r.k[tl][i][0], 0x04010400u);
                    w[1] = bytes_to_biased_half2(r.k[tl][i][0], 0x04030402u);
                    w[2] = bytes_to_biased_half2(r.k[tl][i][1], 0x04010400u);
                    w[3] = bytes_to_biased_half2(r.k[tl][i][1], 0x04030402u);
                    a = O::from_bits(w);
                    if constexpr (!kBf16) a = a - (half_t)1152.0f;
                }
                sc = O::mma(a, qf[i], sc);
            }
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int tok = u * kMmaUnit + tl * 16 + kg * 4 + q;
                float val = sc[q];
                if constexpr (kU8) val = r.sz[tl * 4 + q].x * (val - (r.sz[tl * 4 + q].y - 128.0f) * sumq);
                val = (((r.ok >> tl) & 1) && tok >= row.j0 && tok < row.j1) ? val * c : -INFINITY;
                x[tl * 4 + q] = val;
                mloc = fmaxf(mloc, val);
            }
            // (every key of the row's units gets a value, -inf where it takes no part: the sum kernel reads them all)
            if (n16 < G) *(float4_t*)(raw_row + u * kMmaUnit + tl * 16 + kg * 4) = (float4_t){x[tl * 4], x[tl * 4 + 1], x[tl * 4 + 2], x[tl * 4 + 3]};
        }
        const float m_new = fmaxf(m, mloc);
        if (m_new != -INFINITY) {
            float add = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; j++) add += fast_exp2(x[j] - m_new);
            l = l * fast_exp2(m - m_new) + add;
            m = m_new;
        }
    };

    // two register stages: unit u + 1 is in flight while unit u is worked on
    // (the last unit is requested once more rather than branching round the request)
    KeyRegs<kU8, kHD> ra, rb;
    fetch(u_first, ra);
    int u = u_first;
    while (u < u_end) {
        fetch(min(u + 1, u_end - 1), rb);
        process(u, ra);
        if (u + 1 >= u_end) break;
        fetch(min(u + 2, u_end - 1), ra);
        process(u + 1, rb);
        u += 2;
    }

    // the four lanes of a head
    float m_all = fmaxf(m, __shfl_xor(m, 16, 64));
    m_all = fmaxf(m_all, __shfl_xor(m_all, 32, 64));
    float part = (m == -INFINITY) ? 0.0f : l * fast_exp2(m - m_all);
    part += __shfl_xor(part, 16, 64);
    part += __shfl_xor(part, 32, 64);
    if (kg == 0 && n16 < G) p.part[((int64_t)t * p.num_heads_q + kvh * G + n16) * chunks + chunk] = make_float2(m_all, part);
}

// one lane per (token, head): the log-sum-exp from the wavefronts' (max, sum)
__global__ __launch_bounds__(256) void paged_scores_lse_kernel(ScoresParams p) {
    const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (r >= (int64_t)p.num_tokens * p.num_heads_q) return;
    const int t = (int)(r / p.num_heads_q);
    SeqView v;
    const MmaRow row = mma_row(p, t, v);
    if (!row.scored) {
        p.lse[r] = INFINITY;  // nothing attended (or not aggregated: never read)
        return;
    }
    const int chunks = mma_chunks(p.max_context_len);
    const int units = (row.j1 + kMmaUnit - 1) / kMmaUnit - row.j0 / kMmaUnit;
    const int used = (units + kMmaChunkUnits - 1) / kMmaChunkUnits;
    float m = -INFINITY, l = 0.0f;
    for (int ch = 0; ch < used; ch++) {
        const float2 ml = p.part[r * chunks + ch];
        const float m_new = fmaxf(m, ml.x);
        if (m_new == -INFINITY) continue;
        l = l * fast_exp2(m - m_new) + ml.y * fast_exp2(ml.x - m_new);
        m = m_new;
    }
    p.lse[r] = l > 0.0f ? m + __builtin_amdgcn_logf(l) : INFINITY;
}

// one lane per key of a sequence: the probabilities it received, heads and tokens in a fixed order
__global__ __launch_bounds__(256) void paged_scores_sum_kernel(ScoresParams p) {
    const int lane = threadIdx.x & 63;
    const int s = blockIdx.y;
    const SeqView v = seq_view(p, s);
    const int ctx = v.past + (v.end - v.begin);
    const int base = blockIdx.x * 256 + (threadIdx.x & ~63);
    if (base >= ctx) return;  // wave-uniform
    int64_t ahead = 0;
    for (int i = lane; i < s; i += 64) ahead += p.past_lens[i] + (p.subsequence_begins[i + 1] - p.subsequence_begins[i]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ahead += __shfl_xor(ahead, off, 64);
    const int j = base + lane;
    float total = 0.0f;
    for (int t = v.first_scored; t < v.end; t++) {
        int j0, j1;
        key_range(p, v, v.past + (t - v.begin), j0, j1);
        j1 = min(j1, p.max_context_len);
        if (base >= j1 || base + 64 <= j0) continue;  // wave-uniform: no key of this wavefront is attended
        if (j < j0 || j >= j1) continue;
        const float* raw = p.raw + (int64_t)t * p.num_heads_q * p.raw_stride + j;
        const float* lse = p.lse + (int64_t)t * p.num_heads_q;
        for (int h = 0; h < p.num_heads_q; h++) total += fast_exp2(raw[(int64_t)h * p.raw_stride] - lse[h]);
    }
    if (j < ctx && ahead + j < p.scores_capacity) p.scores[ahead + j] = total;
}

static bool mma_shape(int q_dtype, int cache_dtype, int head_dim, int block_size, int heads_q, int heads_kv) {
    if (!(head_dim == 64 || head_dim == 128)) return false;
    if (block_size < 16 || (block_size & (block_size - 1))) return false;
    if (mma_kv_share(heads_q, heads_kv) == 0) return false;
    if (!(q_dtype == HIPATTN_F16 || q_dtype == HIPATTN_BF16)) return false;
    // fp16 queries on a bf16 cache would be rounded to eight bits for the product: the fp32 kernels keep them
    if (cache_dtype == HIPATTN_BF16) return q_dtype == HIPATTN_BF16;
    return cache_dtype == HIPATTN_F16 || cache_dtype == HIPATTN_U8;
}

size_t paged_scores_workspace(int q_dtype, int cache_dtype, int head_dim, int block_size, int heads_q, int heads_kv, int num_tokens,
                              int64_t max_context_len, size_t* lse_bytes, size_t* part_bytes) {
    const size_t rows = (size_t)num_tokens * heads_q;
    const size_t lse = (rows * sizeof(float) + 255) / 256 * 256;
    if (lse_bytes) *lse_bytes = lse;
    if (part_bytes) *part_bytes = 0;
    if (!mma_shape(q_dtype, cache_dtype, head_dim, block_size, heads_q, heads_kv) || max_context_len <= 0 || max_context_len > (1 << 28))
        return rows * sizeof(float);
    const size_t raw = rows * (size_t)mma_stride((int)max_context_len) * sizeof(float);
    if (raw > kMmaRawCap) return rows * sizeof(float);
    const size_t part = (rows * (size_t)mma_chunks((int)max_context_len) * sizeof(float2) + 255) / 256 * 256;
    if (part_bytes) *part_bytes = part;
    return lse + part + raw;
}

template <bool kU8, bool kBf16>
static hipError_t launch_mma(const ScoresParams& p, hipStream_t stream) {
    const int64_t items = (int64_t)p.num_tokens * mma_chunks(p.max_context_len) * p.num_heads_kv * mma_kv_share(p.num_heads_q, p.num_heads_kv);
    if ((items + kMmaWaves - 1) / kMmaWaves > 0x7fffffffLL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)((items + kMmaWaves - 1) / kMmaWaves));
    if (p.head_dim == 128)
        hipLaunchKernelGGL((paged_scores_mma_kernel<kU8, kBf16, 128>), grid, dim3(64 * kMmaWaves), 0, stream, p);
    else
        hipLaunchKernelGGL((paged_scores_mma_kernel<kU8, kBf16, 64>), grid, dim3(64 * kMmaWaves), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int64_t rows = (int64_t)p.num_tokens * p.num_heads_q;
    hipLaunchKernelGGL(paged_scores_lse_kernel, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, stream, p);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(paged_scores_sum_kernel, dim3((unsigned)((p.max_context_len + 255) / 256), (unsigned)p.num_seqs), dim3(256), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_paged_scores(const ScoresParams& p, hipStream_t stream) {
    if ((int64_t)p.num_tokens * p.num_heads_q == 0 || p.num_seqs == 0 || p.max_context_len == 0) return hipSuccess;
    if (p.raw != nullptr && mma_shape(p.q_dtype, p.cache_dtype, p.head_dim, p.block_size, p.num_heads_q, p.num_heads_kv) &&
        ((uintptr_t)p.key_cache % 16) == 0 && ((uintptr_t)p.q % 16) == 0) {
        if (p.cache_dtype == HIPATTN_U8) return launch_mma<true, false>(p, stream);
        if (p.cache_dtype == HIPATTN_BF16) return launch_mma<false, true>(p, stream);
        return launch_mma<false, false>(p, stream);
    }
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
