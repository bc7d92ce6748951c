// Split-context paged-attention decode for gfx950 (one new token per sequence).
//
// Work decomposition: grid (chunk, kv head, sequence).  A workgroup of four wavefronts owns
// `chunk_tokens` consecutive cache positions of one kv head of one sequence and serves the
// whole GQA group (all query heads sharing that kv head, up to 16) so that every KV byte is
// read from HBM exactly once.  Wavefront w walks the chunk's 32-token blocks w, w+4, ...;
// per block it reads the block-table entry, streams the 8 KiB (fp16) or 4352 B (u8) of K and
// of V for this head straight from global memory into MFMA operand registers, and keeps an
// online softmax.  Partial (max, sum, output) triples are merged across the four wavefronts
// in LDS and, when the context spans several chunks, across chunks by paged_merge_kernel
// (a log-sum-exp reduction).
//
// MFMA use (v_mfma_f32_16x16x32_f16).  Scores are computed transposed, S^T = K Q^T, with the
// 16 tokens of a tile on the M side and the (padded) 16 query heads on the N side; the
// accumulator layout then gives each lane four consecutive tokens of one head, which is
// exactly the B-operand layout the second product O^T = V^T P^T needs, so P never moves
// between lanes.  The contraction index of an MFMA can be permuted freely as long as both
// operands use the same permutation; that freedom is used to make every global load a
// contiguous 16-byte (fp16) or 8-byte (u8) piece of a cache row:
//   K operand: lane (tok = lane & 15, kg = lane >> 4) holds K[tok][kg*32 + i*8 .. +8], i = 0..3
//   V operand: lane (c = lane & 15, kg) loads V[tok(kg,j)][c*8 .. +8] for its 8 tokens j and
//              transposes the 8x8 patch in registers; MFMA e then yields O[:, c*8 + e].
// u8 caches are dequantised in registers: bytes become exact fp16 integers, the per-token
// scale is folded into the score / probability and the zero-point into a rank-one
// correction (q.(k - zp) s = s (q.k) - s zp sum(q)).
//
// No counterpart in the reference: its decode path copies the whole contiguous KV state
// three times per token (src/cuda_variable_state.hpp:135-160, src/ops/read_value.cpp:65-71,
// src/ops/assign.cpp:52-54) and materialises the scores in HBM (src/ops/matmul.cpp:204-226,
// src/ops/softmax.cpp:184-192).
#include <algorithm>

#include "device_common.hpp"
#include "kernels.hpp"

namespace hipattn {

constexpr int kD = 128;           // head size of the fast path
constexpr int kBS = 32;           // cache block size of the fast path
constexpr int kDecodeWaves = 4;
constexpr int kDecodeThreads = 64 * kDecodeWaves;

struct DecodeRange {
    int valid;        // sequence is a decode sequence with something to attend
    int token;        // row of q / out
    int ctx;          // attended positions end (exclusive)
    int j0;           // attended positions begin
    int first_block;  // logical block holding j0
    int end_block;    // one past the logical block holding ctx - 1
};

// Range of cache positions a decode sequence attends; shared by the decode and merge kernels.
__device__ __forceinline__ DecodeRange decode_range(const PagedParams& p, int s) {
    DecodeRange r;
    const int t0 = p.subsequence_begins[s];
    r.valid = (p.subsequence_begins[s + 1] - t0 == 1);
    r.token = t0;
    const int table_tokens = (p.block_indices_begins[s + 1] - p.block_indices_begins[s]) * p.block_size;
    r.ctx = min(p.past_lens[s] + 1, table_tokens);
    r.j0 = 0;
    if (p.sliding_window > 0 && r.ctx - p.sliding_window > 0) r.j0 = r.ctx - p.sliding_window;
    if (r.ctx <= 0) r.valid = 0;
    r.first_block = r.j0 / p.block_size;
    r.end_block = (r.ctx + p.block_size - 1) / p.block_size;
    return r;
}

__device__ __forceinline__ uint32_t pack_lo(uint32_t a, uint32_t b) { return (a & 0xffffu) | (b << 16); }
__device__ __forceinline__ uint32_t pack_hi(uint32_t a, uint32_t b) { return (a >> 16) | (b & 0xffff0000u); }

__device__ __forceinline__ half8_t as_half8(uint4_t v) { return __builtin_bit_cast(half8_t, v); }

// 8 consecutive query elements as fp16 (bf16 queries are widened exactly)
__device__ __forceinline__ half8_t load_q8(const void* q, int64_t elem, int q_dtype) {
    if (q_dtype == HIPATTN_F16) {
        return as_half8(*(const uint4_t*)((const uint16_t*)q + elem));
    }
    const uint4_t raw = *(const uint4_t*)((const uint16_t*)q + elem);
    half8_t r;
#pragma unroll
    for (int w = 0; w < 4; w++) {
        r[2 * w] = (half_t)__uint_as_float(raw[w] << 16);
        r[2 * w + 1] = (half_t)__uint_as_float(raw[w] & 0xffff0000u);
    }
    return r;
}

// four bytes of `w` selected pairwise -> two exact fp16 integers (0..255)
__device__ __forceinline__ uint32_t bytes_to_half2(uint32_t lo_src, uint32_t hi_src, uint32_t sel) {
    // v_perm_b32: selector bytes 0..3 pick from lo_src, 4..7 from hi_src, 0x0c yields 0x00
    uint32_t x = __builtin_amdgcn_perm(hi_src, lo_src, sel) | 0x64006400u;  // 1024 + byte, twice
    half2_t h = __builtin_bit_cast(half2_t, x) - (half2_t){(half_t)1024.0f, (half_t)1024.0f};
    return __builtin_bit_cast(uint32_t, h);
}

template <bool kU8>
struct BlockRegs;

template <>
struct BlockRegs<false> {
    uint4_t k[2][4];  // [tile][k-step]: K[tile*16 + (lane&15)][kg*32 + i*8 .. +8]
    uint4_t v[8];     // [j = tile*4 + r]: V[tile*16 + kg*4 + r][(lane&15)*8 .. +8]
};

template <>
struct BlockRegs<true> {
    uint2_t k[2][4];  // 8 bytes each
    uint2_t v[8];
    float2 ksz[8];    // (scale, zp) of K for token j = tile*4 + r of this lane
    float2 vsz[8];
};

template <bool kU8>
__device__ __forceinline__ void load_block(BlockRegs<kU8>& b, const uint8_t* kbase, const uint8_t* vbase, int n16,
                                           int kg) {
    if constexpr (!kU8) {
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                b.k[t][i] = *(const uint4_t*)(kbase + (t * 16 + n16) * 256 + kg * 64 + i * 16);
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                b.v[t * 4 + r] = *(const uint4_t*)(vbase + (t * 16 + kg * 4 + r) * 256 + n16 * 16);
    } else {
        constexpr int kRow = kD + 8;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                b.k[t][i] = *(const uint2_t*)(kbase + (t * 16 + n16) * kRow + 8 + kg * 32 + i * 8);
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int tok = t * 16 + kg * 4 + r;
                b.v[t * 4 + r] = *(const uint2_t*)(vbase + tok * kRow + 8 + n16 * 8);
                b.ksz[t * 4 + r] = *(const float2*)(kbase + tok * kRow);
                b.vsz[t * 4 + r] = *(const float2*)(vbase + tok * kRow);
            }
    }
}

struct WaveState {
    float m;          // running max of the scaled scores (log2 domain), per head (lane & 15)
    float l;          // this lane's share of the running sum
    float corr;       // u8 only: this lane's share of sum_j p'_j zp_j
    float4_t acc[8];  // acc[e][r] = O[head][(kg*4 + r)*8 + e]
};

template <bool kU8>
__device__ __forceinline__ void process_block(WaveState& st, BlockRegs<kU8>& b, const half8_t (&qf)[4], float sumq,
                                              float c, int tok_base, int j0, int ctx, int kg) {
    // ---- S^T = K Q^T : two tiles of 16 tokens x 16 heads
    float4_t s[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        s[t] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            half8_t a;
            if constexpr (!kU8) {
                a = as_half8(b.k[t][i]);
            } else {
                uint4_t w;
                w[0] = bytes_to_half2(b.k[t][i][0], 0u, 0x0c010c00u);
                w[1] = bytes_to_half2(b.k[t][i][0], 0u, 0x0c030c02u);
                w[2] = bytes_to_half2(b.k[t][i][1], 0u, 0x0c010c00u);
                w[3] = bytes_to_half2(b.k[t][i][1], 0u, 0x0c030c02u);
                a = as_half8(w);
            }
            s[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qf[i], s[t], 0, 0, 0);
        }
    }
    // ---- mask, scale, online softmax.  Lane holds tokens tok_base + t*16 + kg*4 + r.
    float sv[8];
    float mloc = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int j = t * 4 + r;
            const int tok = tok_base + t * 16 + kg * 4 + r;
            float x = s[t][r];
            if constexpr (kU8) x = b.ksz[j].x * (x - b.ksz[j].y * sumq);
            x = (tok >= j0 && tok < ctx) ? x * c : -INFINITY;
            sv[j] = x;
            mloc = fmaxf(mloc, x);
        }
    mloc = fmaxf(mloc, __shfl_xor(mloc, 16, 64));
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
    const float m_new = fmaxf(st.m, mloc);  // finite: every processed block holds an attended token
    const float alpha = fast_exp2(st.m - m_new);
    st.m = m_new;
    // Rows outside the attended range may hold anything (never-written cache memory): their
    // probability is exactly zero, and fp16 V rows are cleared so that 0 * NaN cannot occur.
    const bool partial = (tok_base < j0) || (tok_base + kBS > ctx);  // wavefront-uniform
    if (partial) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int tok = tok_base + (j >> 2) * 16 + kg * 4 + (j & 3);
            if (!(tok >= j0 && tok < ctx)) {
                if constexpr (kU8) {
                    b.vsz[j] = make_float2(0.0f, 0.0f);
                } else {
                    b.v[j] = (uint4_t){0u, 0u, 0u, 0u};
                }
            }
        }
    }
    half8_t pf;
    float lsum = 0.0f, csum = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        float pj = fast_exp2(sv[j] - m_new);
        lsum += pj;
        if constexpr (kU8) {
            pj *= b.vsz[j].x;
            const half_t ph = (half_t)pj;
            csum = fmaf((float)ph, b.vsz[j].y, csum);
            pf[j] = ph;
        } else {
            pf[j] = (half_t)pj;
        }
    }
    st.l = st.l * alpha + lsum;
    if constexpr (kU8) st.corr = st.corr * alpha + csum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {
#pragma unroll
        for (int e = 0; e < 8; e++) st.acc[e] *= alpha;
    }
    // ---- O^T += V^T P^T : transpose the lane's 8 tokens x 8 head-dim patch in registers
#pragma unroll
    for (int e = 0; e < 8; e++) {
        uint4_t w;
        if constexpr (!kU8) {
#pragma unroll
            for (int jp = 0; jp < 4; jp++) {
                const uint32_t lo = b.v[2 * jp][e >> 1], hi = b.v[2 * jp + 1][e >> 1];
                w[jp] = (e & 1) ? pack_hi(lo, hi) : pack_lo(lo, hi);
            }
        } else {
            const uint32_t sel = 0x0c000c00u | ((4u + (e & 3)) << 16) | (uint32_t)(e & 3);
#pragma unroll
            for (int jp = 0; jp < 4; jp++)
                w[jp] = bytes_to_half2(b.v[2 * jp][e >> 2], b.v[2 * jp + 1][e >> 2], sel);
        }
        st.acc[e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(w), pf, st.acc[e], 0, 0, 0);
    }
}

template <bool kU8>
__global__ __launch_bounds__(kDecodeThreads) void paged_decode_kernel(PagedParams p) {
    __shared__ float o_lds[kDecodeWaves][16][kD + 4];
    __shared__ float ml_lds[kDecodeWaves][2][16];

    const int chunk = blockIdx.x, h = blockIdx.y, s = blockIdx.z;
    const DecodeRange rg = decode_range(p, s);
    if (!rg.valid) return;
    const int blocks_per_chunk = p.chunk_tokens / kBS;
    const int b_begin = rg.first_block + chunk * blocks_per_chunk;
    if (b_begin >= rg.end_block) return;
    const int b_end = min(b_begin + blocks_per_chunk, rg.end_block);
    const int n_chunks = (rg.end_block - rg.first_block + blocks_per_chunk - 1) / blocks_per_chunk;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, n16 = lane & 15, kg = lane >> 4;
    const int G = p.num_heads_q / p.num_heads_kv;
    const float c = p.scale * kLog2e;

    // Q^T operand: lane (head n16, kg) holds Q[head][kg*32 + i*8 .. +8]; padding heads are zero
    half8_t qf[4];
    float sumq = 0.0f;
    {
        const int64_t qrow = ((int64_t)rg.token * p.num_heads_q + (int64_t)h * G + n16) * kD;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if (n16 < G) {
                qf[i] = load_q8(p.q, qrow + kg * 32 + i * 8, p.q_dtype);
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) qf[i][e] = (half_t)0.0f;
            }
            if constexpr (kU8) {
#pragma unroll
                for (int e = 0; e < 8; e++) sumq += (float)qf[i][e];
            }
        }
        if constexpr (kU8) {
            sumq += __shfl_xor(sumq, 16, 64);
            sumq += __shfl_xor(sumq, 32, 64);
        }
    }

    WaveState st;
    st.m = -INFINITY;
    st.l = 0.0f;
    st.corr = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; e++) st.acc[e] = (float4_t){0.f, 0.f, 0.f, 0.f};

    const int32_t* table = p.block_indices + p.block_indices_begins[s];
    constexpr int64_t kRowBytes = kU8 ? (kD + 8) : (2 * kD);
    const int64_t block_stride = (int64_t)p.num_heads_kv * kBS * kRowBytes;
    const int64_t head_off = (int64_t)h * kBS * kRowBytes;

    auto block_ptrs = [&](int lb, const uint8_t*& kb, const uint8_t*& vb) -> bool {
        const int pb = table[lb];
        if (pb < 0 || pb >= p.num_blocks) return false;  // never read outside the cache
        const int64_t off = (int64_t)pb * block_stride + head_off;
        kb = p.key_cache + off;
        vb = p.value_cache + off;
        return true;
    };

    // two register stages: the loads of block i+4 are in flight while block i is consumed
    BlockRegs<kU8> ra, rb;
    const uint8_t *kb = nullptr, *vb = nullptr;
    int lb = b_begin + wave;
    bool va = false, vb_ok = false;
    if (lb < b_end) {
        va = block_ptrs(lb, kb, vb);
        if (va) load_block<kU8>(ra, kb, vb, n16, kg);
    }
    while (lb < b_end) {
        const int lb_next = lb + kDecodeWaves;
        vb_ok = false;
        if (lb_next < b_end) {
            vb_ok = block_ptrs(lb_next, kb, vb);
            if (vb_ok) load_block<kU8>(rb, kb, vb, n16, kg);
        }
        if (va) process_block<kU8>(st, ra, qf, sumq, c, lb * kBS, rg.j0, rg.ctx, kg);
        if (lb_next >= b_end) break;
        const int lb_next2 = lb_next + kDecodeWaves;
        va = false;
        if (lb_next2 < b_end) {
            va = block_ptrs(lb_next2, kb, vb);
            if (va) load_block<kU8>(ra, kb, vb, n16, kg);
        }
        if (vb_ok) process_block<kU8>(st, rb, qf, sumq, c, lb_next * kBS, rg.j0, rg.ctx, kg);
        lb = lb_next2;
    }

    // ---- merge the four wavefronts through LDS
    float l = st.l, corr = st.corr;
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if constexpr (kU8) {
        corr += __shfl_xor(corr, 16, 64);
        corr += __shfl_xor(corr, 32, 64);
    }
    if (kg == 0) {
        ml_lds[wave][0][n16] = st.m;
        ml_lds[wave][1][n16] = l;
    }
#pragma unroll
    for (int e = 0; e < 8; e++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            float v = st.acc[e][r];
            if constexpr (kU8) v -= corr;
            o_lds[wave][n16][(kg * 4 + r) * 8 + e] = v;
        }
    __syncthreads();

    // thread -> (head g, 8 consecutive head-dim slots)
    for (int item = tid; item < G * (kD / 8); item += kDecodeThreads) {
        const int g = item / (kD / 8), d0 = (item % (kD / 8)) * 8;
        float mt = -INFINITY;
#pragma unroll
        for (int w = 0; w < kDecodeWaves; w++) mt = fmaxf(mt, ml_lds[w][0][g]);
        float lt = 0.0f;
        float o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < kDecodeWaves; w++) {
            const float mw = ml_lds[w][0][g];
            const float f = (mw == -INFINITY) ? 0.0f : fast_exp2(mw - mt);
            lt += f * ml_lds[w][1][g];
#pragma unroll
            for (int e = 0; e < 8; e++) o[e] += f * o_lds[w][g][d0 + e];
        }
        const int hq = h * G + g;
        if (n_chunks == 1) {
            const float inv = lt > 0.0f ? 1.0f / lt : 0.0f;
            const int64_t orow = ((int64_t)rg.token * p.num_heads_q + hq) * kD + d0;
#pragma unroll
            for (int e = 0; e < 8; e++) store_scalar(p.out, orow + e, p.out_dtype, o[e] * inv);
        } else {
            const int64_t slot = ((int64_t)s * p.num_heads_q + hq) * p.max_chunks + chunk;
            float* po = p.part_out + slot * kD + d0;
            *(float4*)(po) = make_float4(o[0], o[1], o[2], o[3]);
            *(float4*)(po + 4) = make_float4(o[4], o[5], o[6], o[7]);
            if (d0 == 0) {
                p.part_ml[slot * 2] = mt;
                p.part_ml[slot * 2 + 1] = lt;
            }
        }
    }
}

// Log-sum-exp reduction of the per-chunk partials of one (sequence, query head).
__global__ __launch_bounds__(kD) void paged_merge_kernel(PagedParams p) {
    const int hq = blockIdx.x, s = blockIdx.y;
    const DecodeRange rg = decode_range(p, s);
    if (!rg.valid) return;
    const int blocks_per_chunk = p.chunk_tokens / kBS;
    int n_chunks = (rg.end_block - rg.first_block + blocks_per_chunk - 1) / blocks_per_chunk;
    if (n_chunks <= 1) return;  // the decode kernel already wrote the final row
    if (n_chunks > p.max_chunks) n_chunks = p.max_chunks;  // caller understated max_context_len: stay in bounds
    const int d = threadIdx.x;
    const int64_t slot0 = ((int64_t)s * p.num_heads_q + hq) * p.max_chunks;
    float mt = -INFINITY;
    for (int ch = 0; ch < n_chunks; ch++) mt = fmaxf(mt, p.part_ml[(slot0 + ch) * 2]);
    float lt = 0.0f, o = 0.0f;
    for (int ch = 0; ch < n_chunks; ch++) {
        const float f = fast_exp2(p.part_ml[(slot0 + ch) * 2] - mt);
        lt += f * p.part_ml[(slot0 + ch) * 2 + 1];
        o += f * p.part_out[(slot0 + ch) * kD + d];
    }
    const float inv = lt > 0.0f ? 1.0f / lt : 0.0f;
    store_scalar(p.out, ((int64_t)rg.token * p.num_heads_q + hq) * kD + d, p.out_dtype, o * inv);
}

hipError_t launch_paged_decode(const PagedParams& p, hipStream_t stream, const KernelProbe& probe) {
    dim3 grid(p.max_chunks, p.num_heads_kv, p.num_seqs);
    if (probe.before) (void)hipEventRecord(probe.before, stream);
    if (p.cache_dtype == HIPATTN_U8)
        hipLaunchKernelGGL(paged_decode_kernel<true>, grid, dim3(kDecodeThreads), 0, stream, p);
    else
        hipLaunchKernelGGL(paged_decode_kernel<false>, grid, dim3(kDecodeThreads), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (probe.after) (void)hipEventRecord(probe.after, stream);
    if (e != hipSuccess) return e;
    if (p.max_chunks > 1) {
        hipLaunchKernelGGL(paged_merge_kernel, dim3(p.num_heads_q, p.num_seqs), dim3(kD), 0, stream, p);
        e = hipGetLastError();
    }
    return e;
}

// ---- host side of the fast path ---------------------------------------------------------

bool paged_fast_supported(const PagedParams& p) {
    const int G = p.num_heads_q / p.num_heads_kv;
    return p.head_dim == kD && p.block_size == kBS && G <= 16 &&
           (p.q_dtype == HIPATTN_F16 || p.q_dtype == HIPATTN_BF16) &&
           (p.cache_dtype == HIPATTN_F16 || p.cache_dtype == HIPATTN_U8);
}

// Largest number of 32-token blocks a decode sequence can attend.
static int max_decode_blocks(const PagedParams& p) {
    int blocks = (p.max_context_len + kBS - 1) / kBS;
    if (p.sliding_window > 0) blocks = std::min(blocks, (p.sliding_window + kBS - 1) / kBS + 1);
    return std::max(blocks, 1);
}

// Tokens per split: enough workgroups to fill 256 CUs several times over while keeping the
// partial-result traffic (520 B per query head and split) small against the KV bytes read.
static int choose_chunk_tokens(const PagedParams& p) {
    if (p.chunk_tokens > 0) return std::max(kBS, (p.chunk_tokens / kBS) * kBS);
    const int64_t total_blocks = (int64_t)p.num_seqs * p.num_heads_kv * max_decode_blocks(p);
    const int min_chunk = (p.cache_dtype == HIPATTN_U8) ? 1024 : 512;
    int chunk = 4096;
    while (chunk > min_chunk && total_blocks * kBS / chunk < 4096) chunk >>= 1;
    while (chunk > 128 && total_blocks * kBS / chunk < 512) chunk >>= 1;
    return chunk;
}

static size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

size_t paged_fast_workspace_bytes(const PagedParams& p) {
    const int chunk = choose_chunk_tokens(p);
    const int max_chunks = (max_decode_blocks(p) * kBS + chunk - 1) / chunk;
    size_t bytes = align_up(((size_t)p.num_seqs + 1) * sizeof(int32_t), 256);
    if (max_chunks > 1) {
        const size_t slots = (size_t)p.num_seqs * p.num_heads_q * max_chunks;
        bytes += align_up(slots * kD * sizeof(float), 256) + align_up(slots * 2 * sizeof(float), 256);
    }
    return bytes;
}

void paged_fast_plan(PagedParams& p, void* workspace) {
    p.chunk_tokens = choose_chunk_tokens(p);
    p.max_chunks = (max_decode_blocks(p) * kBS + p.chunk_tokens - 1) / p.chunk_tokens;
    uint8_t* w = (uint8_t*)workspace;
    p.tile_prefix = (int32_t*)w;
    w += align_up(((size_t)p.num_seqs + 1) * sizeof(int32_t), 256);
    p.part_out = nullptr;
    p.part_ml = nullptr;
    if (p.max_chunks > 1) {
        const size_t slots = (size_t)p.num_seqs * p.num_heads_q * p.max_chunks;
        p.part_out = (float*)w;
        w += align_up(slots * kD * sizeof(float), 256);
        p.part_ml = (float*)w;
    }
    // query tiles of multi-token sequences: each has >= 2 tokens and wastes at most one tile
    const int multi = std::min(p.num_seqs, p.num_tokens / 2);
    p.max_q_tiles = p.num_tokens / 128 + multi;
}

hipError_t launch_paged_fast(const PagedParams& p, hipStream_t stream, const KernelProbe& probe) {
    hipError_t e = launch_paged_decode(p, stream, probe);
    if (e != hipSuccess) return e;
    if (p.max_q_tiles > 0) {
        if (p.cache_dtype == HIPATTN_U8) {
            PagedParams g = p;
            g.generic_skip_single = 1;
            e = launch_paged_generic(g, stream);
        } else {
            e = launch_paged_prefill(p, stream);
        }
    }
    return e;
}

}  // namespace hipattn
