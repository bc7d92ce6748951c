// Paged-attention decode for gfx950 (sequences with exactly one new token), scheduled
// stream-K style over the whole batch.
//
// Work decomposition.  The unit of work is 32 tokens of the cache of one kv head of one sequence
// -- one cache block of 32 tokens, two of 16, or a 32-token part of a larger one ("block-head": at head size 128, 8 KiB of K plus
// 8 KiB of V in fp16, 2 x 4352 B in u8).  All
// block-heads of the batch are laid out on one line, ordered (sequence, kv head, block), and
// the line is cut into `num_waves` equal pieces; wavefront w owns piece w.  The kernel is
// launched with exactly as many single-wavefront workgroups as fit on the device at once, so
// every wavefront streams the same number of bytes and they all finish together: no tail, no
// per-chunk launch cost, no dependence on how the contexts happen to be distributed.  A piece
// that covers a whole (sequence, kv head) segment writes the final output rows; otherwise the
// wavefront leaves a partial (running max, sum, unnormalised output) per query head in the
// workspace and paged_merge_kernel combines the pieces of a segment with a log-sum-exp
// reduction.  The
// per-sequence block counts and their prefix sum come from the plan workgroup of the prologue
// kernel, which reads past_lens / subsequence_begins on the device: the host never sees the
// lengths.  The same launch performs the operator's KV-cache write.
//
// One wavefront serves the whole GQA group (all query heads sharing the kv head, up to 16),
// so every KV byte is read from HBM exactly once.  Per block it streams K and V straight from
// global memory into MFMA operand registers (two register stages: the next block's loads are
// in flight while the current block is consumed) and keeps an online softmax.
//
// MFMA use (v_mfma_f32_16x16x32_f16; _bf16 for bf16 caches).  Scores are computed transposed, S^T = K Q^T, with the
// 16 tokens of a tile on the M side and the (padded) 16 query heads on the N side; the
// accumulator layout then gives each lane four consecutive tokens of one head, which is
// exactly the B-operand layout the second product O^T = V^T P^T needs, so P never moves
// between lanes.  The contraction index of an MFMA can be permuted freely as long as both
// operands use the same permutation; that freedom is used to make every global load a
// contiguous 16-byte (fp16, bf16) or 8-byte (u8) piece of a cache row:
//   K operand: lane (tok = lane & 15, kg = lane >> 4) holds K[tok][kg*32 + i*8 .. +8], i = 0..3
//   V operand: lane (c = lane & 15, kg) loads V[tok(kg,j)][c*8 .. +8] for its 8 tokens j and
//              transposes the 8x8 patch in registers; MFMA e then yields O[:, c*8 + e].
// u8 caches are dequantised in registers: bytes become exact fp16 integers, the per-token
// scale is folded into the score / probability and the zero-point into a rank-one
// correction (q.(k - zp) s = s (q.k) - s zp sum(q)).
//
// Shapes.  The kernel is a template over the head size it is built for (128 or 64: a lane's K
// piece count and the number of MFMAs per tile follow), the cache block size (32, 16, or 0: a larger power of two read from the call) and whether
// the call's head size may be smaller than the built one (any multiple of 8: rows are then
// head_dim elements apart at run time and the query columns that do not exist are zeros).  The
// figures and layouts above are those of head size 128.
//
// Mixed batches (decode sequences and multi-token chunks in one call).  The chunks go to the flash
// kernel over the block table, which is bound by the matrix cores; the decode sequences are bound
// by HBM.  Each of the two kernels needs whole compute units (registers, LDS), so they cannot
// share one, but they can share the chip: the decode kernel is then launched with eight
// wavefronts to a workgroup -- a workgroup owns a compute unit -- directly behind the prologue,
// and the flash kernel on a side stream that waits for the prologue too and takes the other
// compute units (and every one the decode workgroups give back).  How many compute units the
// decode part keeps is decided by the plan on the device, in proportion to the work of the two
// parts (cache bytes to stream against key tiles to multiply), so that both end together;
// workgroups beyond that number leave at once.  The caller's stream waits for the side stream
// before the call returns, so to the caller the call is still one piece of work in stream order.
//
// No counterpart in the reference: its decode path copies the whole contiguous KV state
// three times per token (src/cuda_variable_state.hpp:135-160, src/ops/read_value.cpp:65-71,
// src/ops/assign.cpp:52-54) and materialises the scores in HBM (src/ops/matmul.cpp:204-226,
// src/ops/softmax.cpp:184-192).
#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <type_traits>

#include "decode_operands.hpp"
#include "device_common.hpp"
#include "kernels.hpp"
#include "kv_cache_write.hpp"

namespace hipattn {

constexpr int kD = 128;   // head size of the benchmark configurations (the kernels also take 64 and, padded, any multiple of 8 below: templates kHD, kPad)
constexpr int kBS = 32;   // their cache block size (also 16: template kBlk)
constexpr int kUnit = 32; // tokens a wavefront works through at a time: one block of 32, or two of 16

struct alignas(32) DecodeRange {
    int write_pos;    // cache position of the row's own new token when it has a slot in the table, else -1
    int token;        // row of q / out
    int ctx;          // attended positions end (exclusive)
    int j0;           // attended positions begin
    int new_begin;    // cache position of the first token its sequence contributes to this batch (past_lens)
    int nb;           // number of 32-token units attended (0 when not valid)
    int table_begin;  // offset of the sequence's block table in block_indices
    int empty_row;    // a single-token row with nothing to attend: its output row is zeros
};
static_assert(sizeof(DecodeRange) == 32, "one 32-byte record per sequence");

// Sequence that owns token t: the last s with subsequence_begins[s] <= t.
__device__ __forceinline__ int sequence_of_token(const PagedParams& p, int t) {
    int lo = 0, hi = p.num_seqs;  // begins[lo] <= t < begins[hi]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (p.subsequence_begins[mid] <= t)
            lo = mid;
        else
            hi = mid;
    }
    return lo;
}

// Range of cache positions a single-token row attends.  Computed once per call by the plan and
// stored per record (seq_info), so that the decode and merge kernels fetch it with one load.
//
// Records are per sequence when the batch may hold multi-token sequences (max_q_tiles > 0: those go
// to the chunked-prefill kernel and only sequences of exactly one token are decode rows).  A batch
// with as many tokens as sequences is planned per TOKEN instead (max_q_tiles == 0, no prefill
// launch): record i is token i, whichever sequence it belongs to, so a batch that only looks like
// a decode step -- an empty sequence beside a two-token one -- still gets every row right; its
// extra tokens are simply decode rows with their own context length.
__device__ __forceinline__ DecodeRange decode_range(const PagedParams& p, int i) {
    DecodeRange r;
    int s = i, pos_in_seq = 0;
    bool single = true;
    // everything a row of an ordinary decode batch needs is fetched at once, on the guess that row i is
    // sequence i (one level of memory latency instead of two); a guess that fails is redone below
    // (rows beyond the last sequence exist only when rows are tokens: the guess is then made on the last sequence)
    const int ig = min(i, p.num_seqs - 1);
    const int b0 = p.subsequence_begins[ig], b1 = p.subsequence_begins[ig + 1];
    int tb0 = p.block_indices_begins[ig], tb1 = p.block_indices_begins[ig + 1], past = p.past_lens[ig];
    if (p.max_q_tiles == 0) {
        if (!(ig == i && b0 == i && b1 == i + 1)) {
            s = sequence_of_token(p, i);
            tb0 = p.block_indices_begins[s];
            tb1 = p.block_indices_begins[s + 1];
            past = p.past_lens[s];
        }
        pos_in_seq = i - p.subsequence_begins[s];
        r.token = i;
        // a token outside every sequence (padding in front of the first or behind the last): no row at all
        single = i >= p.subsequence_begins[0] && i < p.subsequence_begins[p.num_seqs];
    } else {
        r.token = b0;
        single = (b1 - b0 == 1);
    }
    const int table_tokens = (tb1 - tb0) * p.block_size;
    r.ctx = min(past + pos_in_seq + 1, table_tokens);
    r.j0 = 0;
    if (p.sliding_window > 0 && r.ctx - p.sliding_window > 0) r.j0 = r.ctx - p.sliding_window;
    const bool valid = single && r.ctx > 0;
    r.write_pos = (single && past + pos_in_seq < table_tokens) ? past + pos_in_seq : -1;
    r.empty_row = single && r.ctx <= 0;
    r.new_begin = past;
    r.nb = valid ? (r.ctx + kUnit - 1) / kUnit - r.j0 / kUnit : 0;  // in units of 32 tokens
    r.table_begin = tb0;
    return r;
}

#ifndef HIPATTN_U8_STAGES
#define HIPATTN_U8_STAGES 2
#endif

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
    // (scale, zp) of one token: lane (i = lane & 15, kg) holds those of the K row (i < 8) or V row
    // (i >= 8) of token j = i & 7 of its 16-lane row, i.e. of token (j >> 2) * 16 + kg * 4 + (j & 3);
    // the lanes of the row read them with a DPP row broadcast.  (Loading all eight pairs of K and
    // of V into every lane costs sixteen load instructions and 32 registers per block.)
    float2 sz;
};

// A bf16 block turned into fp16 operands in its registers (fp16 queries on a bf16 cache: rounding the queries to
// bf16's eight bits instead costs the decode rows their 2e-3).  bf16 -> fp16 is exact inside fp16's range; beyond it
// the conversion (towards zero) stops at the largest finite fp16 number.
__device__ __forceinline__ uint32_t bf16x2_to_f16x2(uint32_t w) {
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(__uint_as_float(w << 16), __uint_as_float(w & 0xffff0000u)));
}
__device__ __forceinline__ void bf16_block_to_f16(BlockRegs<false>& b) {
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int e = 0; e < 4; e++) b.k[t][i][e] = bf16x2_to_f16x2(b.k[t][i][e]);
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) b.v[j][e] = bf16x2_to_f16x2(b.v[j][e]);
}

// value of lane kLane of the caller's 16-lane row (v_mov_b32 row_newbcast, folded into the consumer where possible)
template <int kLane>
__device__ __forceinline__ float row_broadcast(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x150 + kLane, 0xf, 0xf, false));
}

// kb[t] / vb[t]: the first row of the unit's 16-token tile t in the key / value cache (one block of
// 32 tokens: kb[1] is sixteen rows behind kb[0]; blocks of 16: two blocks).  Head size kHD: a K row
// is read in kHD / 32 pieces per lane, a V row by the kHD / 8 lanes that have a piece of it.
template <bool kU8, int kHD = kD, int kBlk = kBS>
__device__ __forceinline__ void load_block(BlockRegs<kU8>& b, const uint8_t* const (&kb)[2], const uint8_t* const (&vb)[2],
                                           int n16, int kg) {
    if constexpr (!kU8) {
        constexpr int kRow = 2 * kHD;
        // (with blocks of 32 both tiles are addressed from the block's first row: one base register)
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < kHD / 32; i++)
                b.k[t][i] = kBlk == 32 ? *(const uint4_t*)(kb[0] + (t * 16 + n16) * kRow + kg * (kHD / 2) + i * 16)
                                       : *(const uint4_t*)(kb[t] + n16 * kRow + kg * (kHD / 2) + i * 16);
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                if (kHD == 128 || n16 * 8 < kHD)
                    b.v[t * 4 + r] = kBlk == 32 ? *(const uint4_t*)(vb[0] + (t * 16 + kg * 4 + r) * kRow + n16 * 16)
                                                : *(const uint4_t*)(vb[t] + (kg * 4 + r) * kRow + n16 * 16);
                else
                    b.v[t * 4 + r] = (uint4_t){0u, 0u, 0u, 0u};
            }
    } else {
        constexpr int kRow = kHD + 8;
        // a lane's K bytes are kHD / 4 consecutive ones of a row, in pieces of eight; its V bytes the
        // eight of its columns, when the head has them
        const bool v_cols = kHD == 128 || n16 * 8 < kHD;
        if constexpr (kBlk == 32) {  // both tiles from the block's first row
            const uint8_t* const kbase = kb[0];
            const uint8_t* const vbase = vb[0];
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int i = 0; i < kHD / 32; i++)
                    b.k[t][i] = *(const uint2_t*)(kbase + (t * 16 + n16) * kRow + 8 + kg * (kHD / 4) + i * 8);
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int tok = t * 16 + kg * 4 + r;
                    if (v_cols)
                        b.v[t * 4 + r] = *(const uint2_t*)(vbase + tok * kRow + 8 + n16 * 8);
                    else
                        b.v[t * 4 + r] = (uint2_t){0u, 0u};
                }
            {
                const int j = n16 & 7, tok = (j >> 2) * 16 + kg * 4 + (j & 3);
                b.sz = *(const float2*)((n16 < 8 ? kbase : vbase) + tok * kRow);
            }
        } else {  // a block per tile
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int i = 0; i < kHD / 32; i++)
                    b.k[t][i] = *(const uint2_t*)(kb[t] + n16 * kRow + 8 + kg * (kHD / 4) + i * 8);
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    if (v_cols)
                        b.v[t * 4 + r] = *(const uint2_t*)(vb[t] + (kg * 4 + r) * kRow + 8 + n16 * 8);
                    else
                        b.v[t * 4 + r] = (uint2_t){0u, 0u};
                }
            {
                const int j = n16 & 7, row = kg * 4 + (j & 3);
                // One of four tile bases per lane, put together arithmetically: a per-lane index into
                // (or a select among the elements of) the arrays would move them to scratch memory.
                const uintptr_t k0 = (uintptr_t)kb[0], k1 = (uintptr_t)kb[1], v0 = (uintptr_t)vb[0], v1 = (uintptr_t)vb[1];
                const uintptr_t second = (uintptr_t)(j >> 2), value = (uintptr_t)(n16 >> 3);
                const uintptr_t in_k = k0 + second * (k1 - k0), in_v = v0 + second * (v1 - v0);
                b.sz = *(const float2*)(in_k + value * (in_v - in_k) + (uintptr_t)(row * kRow));
            }
        }
    }
}

// The same for a head size below kHD: rows are `row` bytes apart; koff[i] is this lane's offset of K
// piece i inside a tile -- a piece past the end of the row is pointed at the row's first piece, which
// is valid memory and meets zeros in the query operand -- and the lanes whose V columns do not exist
// (v_ok false) get zeros.  voff: the lane's offset of its first V row's piece.  u8 rows: the payload
// behind eight bytes of scale and zero-point, pieces of eight bytes.
template <bool kU8, int kHD, int kBlk>
__device__ __forceinline__ void load_block_padded(BlockRegs<kU8>& b, const uint8_t* const (&kb)[2], const uint8_t* const (&vb)[2],
                                                  int row, const int (&koff)[kHD / 32], int voff, bool v_ok, int n16, int kg) {
    using Piece = typename std::conditional<kU8, uint2_t, uint4_t>::type;
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const uint8_t* const kt = kBlk == 32 ? kb[0] + t * 16 * row : kb[t];
#pragma unroll
        for (int i = 0; i < kHD / 32; i++) b.k[t][i] = *(const Piece*)(kt + koff[i]);
    }
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const uint8_t* const vt = kBlk == 32 ? vb[0] + t * 16 * row : vb[t];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            Piece piece = {};
            if (v_ok) piece = *(const Piece*)(vt + voff + r * row);
            b.v[t * 4 + r] = piece;
        }
    }
    if constexpr (kU8) {
        const int j = n16 & 7, at = (kg * 4 + (j & 3)) * row;
        if constexpr (kBlk == 32) {
            b.sz = *(const float2*)((n16 < 8 ? kb[0] : vb[0]) + (j >> 2) * 16 * row + at);
        } else {  // (one of four tile bases per lane, put together arithmetically: see load_block)
            const uintptr_t k0 = (uintptr_t)kb[0], k1 = (uintptr_t)kb[1], v0 = (uintptr_t)vb[0], v1 = (uintptr_t)vb[1];
            const uintptr_t second = (uintptr_t)(j >> 2), value = (uintptr_t)(n16 >> 3);
            const uintptr_t in_k = k0 + second * (k1 - k0), in_v = v0 + second * (v1 - v0);
            b.sz = *(const float2*)(in_k + value * (in_v - in_k) + (uintptr_t)at);
        }
    }
}

struct WaveState {
    float m;          // running max of the scaled scores (log2 domain), per head (lane & 15)
    float l;          // this lane's share of the running sum
    float corr;       // u8 only: this lane's share of sum_j p'_j zp_j
    float4_t acc[8];  // acc[e][r] = O[head][(kg*4 + r)*8 + e]
};

// kTileMask (blocks of 16): `tiles_in` has bit t set when tile t of the unit lies in a block of the
// cache; with blocks of 32 both tiles always do and the argument is ignored.
// kAlibi: slopes holds the ALiBi slopes of the group's query heads (`heads` of them; lane n16 serves head n16),
// and slope * (token - last attended token) joins the scaled score.  The slope is fetched where it is used:
// the loop has no register left to hold it (a constant added to a whole row leaves its softmax alone,
// so the distance may be measured from the row's last attended token instead of its own position).
// A template argument rather than a test of the pointer: the test alone cost the u8 kernel 1.3 %.
template <bool kU8, bool kBf16, int kHD = kD, bool kTileMask = false, bool kAlibi = false>
__device__ __forceinline__ void process_block(WaveState& st, BlockRegs<kU8>& b, const typename Op16<kBf16>::vec8 (&qf)[4], float sumq,
                                              float c, int tok_base, int j0, int ctx, int kg, int tiles_in = 3,
                                              const float* slopes = nullptr, int heads = 0) {
    const int tiles = kTileMask ? tiles_in : 3;
    // ---- S^T = K Q^T : two tiles of 16 tokens x 16 heads
    float4_t s[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        s[t] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < kHD / 32; i++) {
            typename Op16<kBf16>::vec8 a;
            if constexpr (!kU8) {
                a = Op16<kBf16>::from_bits(b.k[t][i]);
            } else {
                uint4_t w;
                w[0] = bytes_to_biased_half2(b.k[t][i][0], 0x04010400u);
                w[1] = bytes_to_biased_half2(b.k[t][i][0], 0x04030402u);
                w[2] = bytes_to_biased_half2(b.k[t][i][1], 0x04010400u);
                w[3] = bytes_to_biased_half2(b.k[t][i][1], 0x04030402u);
                a = Op16<kBf16>::from_bits(w);
            }
            s[t] = Op16<kBf16>::mma(a, qf[i], s[t]);
        }
    }
    // ---- mask, scale, online softmax.  Lane holds tokens tok_base + t*16 + kg*4 + r.
    float sv[8];
    float mloc = -INFINITY;
    // u8: this lane's token's scale, zero-point plus byte bias, and their product (see BlockRegs)
    float sz_scale = 0.0f, sz_zero = 0.0f, sz_prod = 0.0f;
    const bool partial = (tok_base < j0) || (tok_base + kUnit > ctx) || tiles != 3;  // wavefront-uniform
    if constexpr (kU8) {
        sz_scale = b.sz.x;
        sz_zero = b.sz.y + kByteBias;
        if (partial) {
            // Rows outside the attended range may hold anything (never-written cache memory): their
            // probability is exactly zero, and their scale and zero-point are cleared so that
            // 0 * NaN cannot occur.
            const int j = ((int)threadIdx.x & 7), tok = tok_base + (j >> 2) * 16 + kg * 4 + (j & 3);
            if (!(tok >= j0 && tok < ctx && ((tiles >> (j >> 2)) & 1))) sz_scale = sz_zero = 0.0f;
        }
        sz_prod = sz_scale * sz_zero;
    }
    auto dequant_score = [&](auto jc, float x) {
        constexpr int j = decltype(jc)::value;
        return fmaf(row_broadcast<j>(sz_scale), x, -(row_broadcast<j>(sz_prod) * sumq));
    };
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int j = t * 4 + r;
            const int tok = tok_base + t * 16 + kg * 4 + r;
            float x = s[t][r];
            if constexpr (kU8) {
                switch (j) {
                    case 0: x = dequant_score(std::integral_constant<int, 0>{}, x); break;
                    case 1: x = dequant_score(std::integral_constant<int, 1>{}, x); break;
                    case 2: x = dequant_score(std::integral_constant<int, 2>{}, x); break;
                    case 3: x = dequant_score(std::integral_constant<int, 3>{}, x); break;
                    case 4: x = dequant_score(std::integral_constant<int, 4>{}, x); break;
                    case 5: x = dequant_score(std::integral_constant<int, 5>{}, x); break;
                    case 6: x = dequant_score(std::integral_constant<int, 6>{}, x); break;
                    default: x = dequant_score(std::integral_constant<int, 7>{}, x); break;
                }
            }
            x = (tok >= j0 && tok < ctx && ((tiles >> t) & 1)) ? x * c : -INFINITY;
            sv[j] = x;
            if constexpr (!kAlibi) mloc = fmaxf(mloc, x);
        }
    if constexpr (kAlibi) {
        const int n16 = (int)threadIdx.x & 15;
        const float slope = *(const volatile float*)(slopes + (n16 < heads ? n16 : 0)) * kLog2e;
        const float first = (float)(tok_base + kg * 4 - (ctx - 1));
#pragma unroll
        for (int j = 0; j < 8; j++) {
            sv[j] = fmaf(slope, first + (float)((j >> 2) * 16 + (j & 3)), sv[j]);
            mloc = fmaxf(mloc, sv[j]);
        }
    }
    mloc = max_over_rows(mloc);
    const float m_new = fmaxf(st.m, mloc);  // finite: every processed block holds an attended token
    const float alpha = fast_exp2(st.m - m_new);
    st.m = m_new;
    // Rows outside the attended range may hold anything (never-written cache memory): their
    // probability is exactly zero, and fp16 V rows are cleared so that 0 * NaN cannot occur.
    if constexpr (!kU8) {
        if (partial) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int tok = tok_base + (j >> 2) * 16 + kg * 4 + (j & 3);
                if (!(tok >= j0 && tok < ctx && ((tiles >> (j >> 2)) & 1))) b.v[j] = (uint4_t){0u, 0u, 0u, 0u};
            }
        }
    }
    typename Op16<kBf16>::vec8 pf;
    float lsum = 0.0f, csum = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        float pj = fast_exp2(sv[j] - m_new);
        lsum += pj;
        if constexpr (kU8) {
            float vs, vz;  // scale and zero-point (plus bias) of V's token j: lanes 8 + j of the row
            switch (j) {
                case 0: vs = row_broadcast<8>(sz_scale); vz = row_broadcast<8>(sz_zero); break;
                case 1: vs = row_broadcast<9>(sz_scale); vz = row_broadcast<9>(sz_zero); break;
                case 2: vs = row_broadcast<10>(sz_scale); vz = row_broadcast<10>(sz_zero); break;
                case 3: vs = row_broadcast<11>(sz_scale); vz = row_broadcast<11>(sz_zero); break;
                case 4: vs = row_broadcast<12>(sz_scale); vz = row_broadcast<12>(sz_zero); break;
                case 5: vs = row_broadcast<13>(sz_scale); vz = row_broadcast<13>(sz_zero); break;
                case 6: vs = row_broadcast<14>(sz_scale); vz = row_broadcast<14>(sz_zero); break;
                default: vs = row_broadcast<15>(sz_scale); vz = row_broadcast<15>(sz_zero); break;
            }
            pj *= vs;
            Op16<kBf16>::set(pf, j, pj);
            csum = fmaf(Op16<kBf16>::get(pf, j), vz, csum);
        } else {
            Op16<kBf16>::set(pf, j, pj);
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
                w[jp] = bytes_to_biased_half2(b.v[2 * jp][e >> 2], b.v[2 * jp + 1][e >> 2], sel);
        }
        st.acc[e] = Op16<kBf16>::mma(Op16<kBf16>::from_bits(w), pf, st.acc[e]);
    }
}


// Length of one (sequence, kv head) segment on the work line: its blocks plus `switch_cost`
// units that stand for the time a wavefront loses when it starts on a new segment (dependent
// loads of the sequence's lengths, its block table and the queries).  Cutting the line into
// equal pieces then equalises time, not just bytes.
__device__ __forceinline__ int line_units(int nb, int switch_cost) { return nb > 0 ? nb + switch_cost : 0; }

__device__ __forceinline__ void zero_output_row(const PagedParams& p, int token) {
    const int64_t n = (int64_t)p.num_heads_q * p.head_dim, o0 = (int64_t)token * n;
    for (int64_t e = 0; e < n; e++) {
        if (p.out_dtype == HIPATTN_F32)
            ((float*)p.out)[o0 + e] = 0.0f;
        else
            ((uint16_t*)p.out)[o0 + e] = 0;
    }
}

// ---- plan ----------------------------------------------------------------------------------
// Exclusive prefix sums over the sequences of (a) attended blocks of decode sequences and
// (b) 128-row query tiles of multi-token sequences.  One workgroup; sequences are split evenly
// over the threads.
__device__ __forceinline__ void plan_block(const PagedParams& p) {
    __shared__ int wave_blk[4];
    __shared__ int wave_tile[4];
    __shared__ float wave_keys[4];
    const int tid = threadIdx.x;
    if (tid < 64) p.dyn_counter[tid] = 0;  // tickets for the dynamic pieces of this call, one counter per group
    const int per = (p.num_rows + 255) / 256;
    const int s0 = min(tid * per, p.num_rows), s1 = min(s0 + per, p.num_rows);
    int blk = 0, tile = 0;
    float key_tiles = 0.0f;  // 64-key tiles the flash kernel works through, summed over 128-row query tiles
    for (int s = s0; s < s1; s++) {
        // (rows are sequences whenever the lengths matter here: max_q_tiles > 0)
        const int qlen = p.max_q_tiles > 0 ? p.subsequence_begins[s + 1] - p.subsequence_begins[s] : 1;
        blk += line_units(decode_range(p, s).nb, p.switch_cost);
        tile += (qlen > 1 && p.max_q_tiles > 0) ? (qlen + 127) / 128 : 0;
        if (p.overlap && qlen > 1) {
            const int past = p.past_lens[s];
            for (int r0 = 0; r0 < qlen; r0 += 128) {
                int keys = past + min(qlen, r0 + 128);
                if (p.sliding_window > 0) keys = min(keys, p.sliding_window + 128);
                key_tiles += (float)((keys + 63) >> 6);
            }
        }
    }
    // Exclusive prefix sums over the 256 threads: a scan inside each wavefront (six shuffle steps),
    // then the totals of the wavefronts ahead.  (One thread adding up 256 values in LDS took about as
    // long as the rest of the launch.)
    const int lane = tid & 63, wv = tid >> 6;
    int scan_blk = blk, scan_tile = tile;
    float scan_keys = key_tiles;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int ub = __shfl_up(scan_blk, d, 64), ut = __shfl_up(scan_tile, d, 64);
        const float uk = __shfl_up(scan_keys, d, 64);
        if (lane >= d) {
            scan_blk += ub;
            scan_tile += ut;
            scan_keys += uk;
        }
    }
    if (lane == 63) {
        wave_blk[wv] = scan_blk;
        wave_tile[wv] = scan_tile;
        wave_keys[wv] = scan_keys;
    }
    __syncthreads();
    int ahead_blk = 0, ahead_tile = 0, total_blk = 0;
    float total_keys = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; w++) {
        ahead_blk += w < wv ? wave_blk[w] : 0;
        ahead_tile += w < wv ? wave_tile[w] : 0;
        total_blk += wave_blk[w];
        total_keys += wave_keys[w];
    }
    if (tid == 0 && p.overlap) {
        // Compute-unit time of the two parts, in microseconds, as measured with both running:
        // a compute unit of the decode kernel streams about 33 GB/s of fp16 cache (u8: 24 GB/s),
        // one of the flash kernel does a 128-row x 64-key tile of one head in about 1.1 us
        // (u8 caches, dequantised on the way: 1.4 us).  Each part gets compute units in
        // proportion to its work, so that both end together.
        const bool u8 = p.cache_dtype == HIPATTN_U8;
        const float decode_us = (float)total_blk * p.num_heads_kv * (u8 ? 8704.0f / 24000.0f : 16384.0f / 33000.0f) * p.overlap_share;
        const float prefill_us = total_keys * p.num_heads_q * (u8 ? 1.4f : 1.1f);
        const int cus = p.num_waves >> 3;
        int mine = (int)ceilf(cus * decode_us / fmaxf(decode_us + prefill_us, 1.0f));
        mine = max(1, min(mine, cus));
        p.plan_waves[0] = mine * 8;
    }
    blk = ahead_blk + scan_blk - blk;
    tile = ahead_tile + scan_tile - tile;
    for (int s = s0; s < s1; s++) {
        const int qlen = p.max_q_tiles > 0 ? p.subsequence_begins[s + 1] - p.subsequence_begins[s] : 1;
        p.blk_prefix[s] = blk;
        p.tile_prefix[s] = tile;
        const DecodeRange rg = decode_range(p, s);
        ((DecodeRange*)p.seq_info)[s] = rg;
        if (rg.empty_row) zero_output_row(p, rg.token);  // (rare: an empty block table) nothing will visit this row
        blk += line_units(rg.nb, p.switch_cost);
        tile += (qlen > 1 && p.max_q_tiles > 0) ? (qlen + 127) / 128 : 0;
    }
    if (s1 == p.num_rows && s0 < p.num_rows) {
        p.blk_prefix[p.num_rows] = blk;
        p.tile_prefix[p.num_rows] = tile;
    }
}

// One launch for step 1 of the operator and the schedule: workgroups [0, write_blocks) scatter
// the new K/V rows into the caches (four wavefronts of the writer each), workgroup write_blocks
// plans.  The plan reads lengths only, never the cache, so the two parts do not interact.
__global__ __launch_bounds__(256) void paged_prologue_kernel(KvWriteParams wp, PagedParams p, int write_blocks) {
    if ((int)blockIdx.x < write_blocks) {
        const int64_t wv = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
        if (wp.head_dim <= 128)  // (elements of a row per lane: two up to head size 128, four up to 256)
            kv_cache_write_wave<2>(wp, wv, threadIdx.x & 63);
        else
            kv_cache_write_wave<4>(wp, wv, threadIdx.x & 63);
    } else {
        plan_block(p);
    }
}

// How the work line [0, total) is cut into pieces.  Pieces 0 .. W-1 are the static ones, one per
// wavefront, and share the first three quarters of the line equally; pieces W .. W+P-1 share the
// last quarter and are handed out on demand (an atomic counter), so wavefronts that run faster
// -- older ones win the arbitration for the memory pipeline, some XCDs see more bandwidth --
// take more of them and all wavefronts finish together.
struct Line {
    int64_t total, t_static, t_dyn;
    int W, P;
    __device__ __forceinline__ Line(int64_t total_, int W_, int P_) : total(total_), W(W_), P(P_) {
        t_dyn = P_ > 0 ? total_ / 4 : 0;
        t_static = total_ - t_dyn;
    }
    // first line unit of piece id (id may be W + P: the end of the line)
    __device__ __forceinline__ int64_t begin(int id) const {
        if (id <= W) return (int64_t)id * t_static / W;
        return t_static + (int64_t)(id - W) * t_dyn / P;
    }
    // the (non-empty) piece that holds line unit pos, 0 <= pos < total
    __device__ __forceinline__ int piece_at(int64_t pos) const {
        if (pos < t_static) return (int)(((pos + 1) * W - 1) / t_static);
        return W + (int)(((pos - t_static + 1) * P - 1) / t_dyn);
    }
};

// eight consecutive output elements, one 16-byte store for the 16-bit types
__device__ __forceinline__ void store_out8(void* out, int64_t elem, int dtype, const float (&o)[8]) {
    if (dtype == HIPATTN_F32) {
        float* po = (float*)out + elem;
        *(float4*)(po) = make_float4(o[0], o[1], o[2], o[3]);
        *(float4*)(po + 4) = make_float4(o[4], o[5], o[6], o[7]);
        return;
    }
    uint4_t w;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t lo = dtype == HIPATTN_F16 ? float_to_f16_bits(o[2 * i]) : float_to_bf16_bits(o[2 * i]);
        const uint32_t hi = dtype == HIPATTN_F16 ? float_to_f16_bits(o[2 * i + 1]) : float_to_bf16_bits(o[2 * i + 1]);
        w[i] = lo | (hi << 16);
    }
    *(uint4_t*)((uint16_t*)out + elem) = w;
}

// Log-sum-exp reduction of the partials that pieces id_first..id_last left for query head g of
// segment (s, h), done by one wavefront.  Pieces are taken 64 at a time: lane i fetches the
// (max, sum) pair of piece i, the weights come out of two wavefront reductions, and the output
// rows are then accumulated with independent loads (lane l owns head-dim 2l and 2l + 1).
__device__ __forceinline__ void merge_segment_head(const PagedParams& p, const Line& line, int s, int h, int g,
                                                   int token, int id_first, int id_last, int lane) {
    const int Hkv = p.num_heads_kv, G = p.num_heads_q / p.num_heads_kv, D = p.head_dim;
    // lane l owns head-dim 2l, 2l + 1 and, at head size 256, 128 + 2l, 129 + 2l
    float m_run = -INFINITY, l_run = 0.0f, ox[2] = {0.0f, 0.0f}, oy[2] = {0.0f, 0.0f};
    for (int id0 = id_first; id0 <= id_last; id0 += 64) {
        const int id = id0 + lane;
        const bool have = id <= id_last && line.begin(id) < line.begin(id + 1);  // skip empty pieces
        const int64_t slot = (int64_t)id + (int64_t)s * Hkv + h;
        float mw = -INFINITY, lw = 0.0f;
        if (have) {
            const float2 ml = *(const float2*)(p.part_ml + (slot * G + g) * 2);
            mw = ml.x;
            lw = ml.y;
        }
        const float m_new = fmaxf(m_run, wave_max(mw));
        const float rescale = (m_run == -INFINITY) ? 0.0f : fast_exp2(m_run - m_new);
        const float f = (mw == -INFINITY) ? 0.0f : fast_exp2(mw - m_new);
        l_run = l_run * rescale + wave_sum(f * lw);
#pragma unroll
        for (int c = 0; c < 2; c++) {
            ox[c] *= rescale;
            oy[c] *= rescale;
        }
        m_run = m_new;
        const uint64_t live = __builtin_amdgcn_ballot_w64(have);
        const int n = min(64, id_last - id0 + 1);
        for (int i = 0; i < n; i++) {
            if (!((live >> i) & 1)) continue;
            const float fi = __shfl(f, i, 64);
            const int64_t sl = (int64_t)(id0 + i) + (int64_t)s * Hkv + h;
#pragma unroll
            for (int c = 0; c < 2; c++) {
                const int d = 128 * c + 2 * lane;
                if (d < D) {
                    const float2 v = *(const float2*)(p.part_out + (sl * G + g) * D + d);
                    ox[c] = fmaf(fi, v.x, ox[c]);
                    oy[c] = fmaf(fi, v.y, oy[c]);
                }
            }
        }
    }
    // (the attention sink of the head, when there is one: a logit in the denominator without a value row)
    if (p.sinks != nullptr && l_run > 0.0f) l_run += fast_exp2(p.sinks[h * G + g] * kLog2e - m_run);
    const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
#pragma unroll
    for (int c = 0; c < 2; c++) {
        const int d = 128 * c + 2 * lane;
        if (d >= D) continue;
        const int64_t o = ((int64_t)token * p.num_heads_q + (int64_t)h * G + g) * D + d;
        if (p.out_dtype == HIPATTN_F32) {
            *(float2*)((float*)p.out + o) = make_float2(ox[c] * inv, oy[c] * inv);
        } else {
            const uint32_t lo = p.out_dtype == HIPATTN_F16 ? float_to_f16_bits(ox[c] * inv) : float_to_bf16_bits(ox[c] * inv);
            const uint32_t hi = p.out_dtype == HIPATTN_F16 ? float_to_f16_bits(oy[c] * inv) : float_to_bf16_bits(oy[c] * inv);
            *(uint32_t*)((uint16_t*)p.out + o) = lo | (hi << 16);
        }
    }
}

// ---- partial results that another wavefront of the same launch reads ------------------------
// The compute units of the device sit behind eight L2 caches that are not kept coherent for
// ordinary accesses.  Partials, and the flags that announce them, therefore go through agent-scope
// relaxed atomic accesses (write-through stores, loads that do not take a stale line): no fence,
// which would write back and invalidate whole L2 caches while the kernel streams through them.
// Order is kept by hand: a producer waits for its stores (s_waitcnt vmcnt(0)) before it raises
// the flag, a consumer reads the partial only after it has seen the flag.
//
// Layout of such a partial (fused_merge; the merge kernel's partials keep theirs): the wavefront that
// combines has the lane layout of the one that produced, so a lane's 32 accumulator values and its
// head's (max, sum) travel as seventeen pairs of floats, pair j of active lane a (a = kg * G + head,
// 4 G of them) at pair index j * 4 G + a of the slot.  One store instruction then writes 4 G x 8
// contiguous bytes -- whole cache lines from four query heads per kv head on -- which matters because a
// write-through store of part of a line is a read-modify-write at the memory (4-byte stores, sixteen
// lines per instruction, cost configuration 3's kernel 20 us).
constexpr int kPartPairs = 17;  // per active lane: 16 pairs of outputs, then (max, sum)
__device__ __forceinline__ void agent_store2(float* p, float x, float y) {
    const unsigned long long v = (unsigned long long)__float_as_uint(x) | ((unsigned long long)__float_as_uint(y) << 32);
    __hip_atomic_store((unsigned long long*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void agent_load2(const float* p, float& x, float& y) {
    const unsigned long long v = __hip_atomic_load((const unsigned long long*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    x = __uint_as_float((uint32_t)v);
    y = __uint_as_float((uint32_t)(v >> 32));
}
__device__ __forceinline__ void stores_done() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// The wavefront that holds the LAST units of a segment which other pieces worked on too combines
// the partials of all of them (its own among them, left in the workspace like the others) when its
// own piece is done: a piece meets such a segment only as the first of its run, so it has at most
// one to combine, and the pieces it waits for have lower numbers, i.e. were dispatched before it.
// Lane (head n16, kg) owns head-dim (kg*4 + r)*8 + e of its head, as in the accumulators.
// Waiting is bounded (kMergeSpinLimit polls of about a microsecond each): a flag that never comes --
// which a consistent plan cannot produce -- leaves the rows unwritten instead of a hung wavefront.
constexpr int kMergeSpinLimit = 1 << 22;
struct MergeArgs {
    float* part_out;
    float* part_ml;
    uint64_t* part_flag;
    unsigned long long merge_tag;
    void* out;
    int out_dtype, num_heads_q, num_heads_kv, head_dim;
    const float* sinks;
};
template <int kHD, bool kPad>
__device__ __forceinline__ void merge_in_kernel(const MergeArgs& p, const Line& line, int s, int h, int token,
                                                int id_first, int id_last, int lane) {
    const int Hkv = p.num_heads_kv, G = p.num_heads_q / p.num_heads_kv;
    const int head_dim = kPad ? p.head_dim : kHD;
    const int n16 = lane & 15, kg = lane >> 4;
    // flags of the other pieces: lane i polls piece id_first + i (64 at a time)
    for (int id0 = id_first; id0 < id_last; id0 += 64) {
        const int id = id0 + lane;
        const bool have = id < id_last && line.begin(id) < line.begin(id + 1);  // (empty pieces leave nothing)
        unsigned long long* flag = (unsigned long long*)p.part_flag + ((int64_t)id + (int64_t)s * Hkv + h);
        bool ready = !have;
        for (int spin = 0; spin < kMergeSpinLimit; spin++) {
            if (!ready) ready = __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == p.merge_tag;
            if (__builtin_amdgcn_ballot_w64(!ready) == 0) break;
            __builtin_amdgcn_s_sleep(2);
        }
        if (__builtin_amdgcn_ballot_w64(!ready) != 0) return;
        // taken: a replay of a captured call comes with the same tag and must not see this flag again
        if (have) __hip_atomic_store(flag, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    float m_run = -INFINITY, l_run = 0.0f;
    float4_t acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = (float4_t){0.f, 0.f, 0.f, 0.f};
    const bool mine = n16 < G;
    // two pieces at a time, every load of the two issued before the first is used: the merge is a chain
    // of memory round trips at the very end of the kernel, and four at a time make the register allocator spill
    for (int id0 = id_first; id0 <= id_last; id0 += 2) {
        float mw[2], lw[2];
        float4_t part[2][8];
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int id = id0 + u;
            mw[u] = -INFINITY;
            lw[u] = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; e++) part[u][e] = (float4_t){0.f, 0.f, 0.f, 0.f};
            if (mine && id <= id_last && line.begin(id) < line.begin(id + 1)) {
                const int64_t slot = (int64_t)id + (int64_t)s * Hkv + h;
                const float* rec = p.part_out + (slot * kPartPairs * 4 * G + (kg * G + n16)) * 2;
#pragma unroll
                for (int r = 0; r < 4; r++)
#pragma unroll
                    for (int e2 = 0; e2 < 4; e2++) {
                        float x, y;
                        agent_load2(rec + (r * 4 + e2) * 8 * G, x, y);
                        part[u][2 * e2][r] = x;
                        part[u][2 * e2 + 1][r] = y;
                    }
                agent_load2(rec + 16 * 8 * G, mw[u], lw[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const float m_new = fmaxf(m_run, mw[u]);
            const float rescale = (m_run == -INFINITY) ? 0.0f : fast_exp2(m_run - m_new);
            const float f = (mw[u] == -INFINITY) ? 0.0f : fast_exp2(mw[u] - m_new);
            l_run = l_run * rescale + f * lw[u];
#pragma unroll
            for (int e = 0; e < 8; e++) acc[e] = acc[e] * rescale + part[u][e] * f;
            m_run = m_new;
        }
    }
    if (!mine) return;
    if (p.sinks != nullptr && l_run > 0.0f) l_run += fast_exp2(p.sinks[h * G + n16] * kLog2e - m_run);
    const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int d0 = (kg * 4 + r) * 8;
        if ((kPad || kHD < 128) && d0 >= head_dim) continue;
        float o[8];
#pragma unroll
        for (int e = 0; e < 8; e++) o[e] = acc[e][r] * inv;
        store_out8(p.out, ((int64_t)token * p.num_heads_q + h * G + n16) * head_dim + d0, p.out_dtype, o);
    }
}

// Pure decode batches of up to kSelfPlanMaxRows rows need no prologue launch: every wavefront works
// out the schedule for itself (one record per row into LDS, lane-parallel, and a wavefront scan for
// the prefix sums), which is shorter than the chain of dependent global loads through a plan another
// kernel left behind, and the wavefront that is about to read the last cache block of a (row, kv
// head) first writes that row's new K and V rows into it -- the operator's cache write, done by
// the only wavefront that needs its result during this call.  Wavefront 0 leaves the plan in the
// workspace for the merge kernel.
constexpr int kSelfPlanMaxRows = 256;

// kWaves wavefronts to a workgroup.  1 is the ordinary launch.  With 8 a workgroup owns a compute
// unit's whole register file: `gridDim.x` workgroups then keep exactly that many compute units and
// leave the others free for a kernel that runs beside this one.
// kHD, kBlk: head size (128 or 64) and cache block size (32, 16, or 0: a larger power of two); the self-planning form and the
// eight-wavefront form exist for head size 128 only (the eight-wavefront form also for 16-bit caches at the
// head sizes between 64 and 128, kPad), the self-planning form on blocks of 32 or 16 only.
// kPad: the call's head size (p.head_dim, a multiple of 8) may be smaller than kHD: the missing columns of
// Q are zeros and those of V are not read.
template <bool kU8, bool kBf16, int kWaves, bool kSelfPlan = false, int kHD = kD, int kBlk = kBS, bool kPad = false, bool kAlibi = false, bool kHalfFromBf16 = false>
__global__ __launch_bounds__(64 * kWaves) __attribute__((amdgpu_waves_per_eu(2, 2))) void paged_decode_kernel(PagedParams p, KvWriteParams wp, int do_write) {
    // kHalfFromBf16: the cache holds bf16, the operands are fp16 (fp16 queries): blocks are converted as they arrive
    static_assert(!kHalfFromBf16 || (!kU8 && !kBf16 && kWaves == 1 && !kSelfPlan && kHD == 128 && !kPad && !kAlibi), "bf16 blocks as fp16 operands: the ordinary launch at head size 128 only");
    static_assert(!kAlibi || (kWaves == 1 && !kSelfPlan), "the distance bias (p.alibi_slopes) exists in the ordinary launch only");
    // The merge inside the kernel (p.fused_merge) is built into the u8 instantiations only: the 16-bit ones use
    // every register in their loop, and with that code behind the loop the allocator spilled 29 of them.
    constexpr bool kFusedBuilt = kU8;
    static_assert(!(kU8 && kBf16), "u8 caches are dequantised to fp16 operands");
    static_assert(!kPad || (!kSelfPlan && (kWaves == 1 || (kHD == 128 && !kU8))), "padded head sizes: no self-planning form; eight wavefronts for 16-bit caches in the head-128 build");
    static_assert(kHD == 128 || (!kSelfPlan && kWaves == 1), "head size 64 has the ordinary launch only");
    static_assert((kHD == 64 || kHD == 128) && (kBlk == 16 || kBlk == 32 || kBlk == 0), "head size 64 or 128, blocks of 16, 32 or more");
    // kBlk == 0: any larger power of two (p.block_size); a block then holds several units, one after the other
    static_assert(kBlk != 0 || !kSelfPlan, "larger blocks: no self-planning form");
    constexpr int kEntries = kBlk == 16 ? 2 : 1;  // block-table entries per unit
    constexpr int kTileBlk = kBlk == 16 ? 16 : 32;  // how a unit's two tiles lie: a block each, or sixteen rows apart
    const int blk = kBlk ? kBlk : p.block_size;
    const int sub_mask = kBlk ? 0 : (p.block_size >> 5) - 1;  // kBlk == 0: unit u is part (u & sub_mask) of its block
    static_assert(!kSelfPlan || kWaves == 1, "a wavefront that plans for itself is a workgroup of its own");
    const int w = kWaves == 1 ? blockIdx.x : blockIdx.x * kWaves + (threadIdx.x >> 6);
    const int lane = kWaves == 1 ? threadIdx.x : (threadIdx.x & 63), n16 = lane & 15, kg = lane >> 4;
    const int Hkv = p.num_heads_kv, G = p.num_heads_q / p.num_heads_kv;
    const float c = p.scale * kLog2e;
    __shared__ DecodeRange plan_rec[kSelfPlan ? kSelfPlanMaxRows : 1];
    __shared__ int plan_prefix[kSelfPlan ? kSelfPlanMaxRows + 1 : 1];
    if constexpr (kSelfPlan) {
        int carry = 0;
        for (int base = 0; base < p.num_rows; base += 64) {
            const int i = base + lane;
            DecodeRange rg;
            int units = 0;
            if (i < p.num_rows) {
                rg = decode_range(p, i);
                units = line_units(rg.nb, p.switch_cost);
                plan_rec[i] = rg;
            }
            int scan = units;  // inclusive scan over the wavefront
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int up = __shfl_up(scan, d, 64);
                if (lane >= d) scan += up;
            }
            if (i < p.num_rows) {
                plan_prefix[i] = carry + scan - units;
                if (w == 0) {  // for the merge kernel
                    ((DecodeRange*)p.seq_info)[i] = rg;
                    p.blk_prefix[i] = carry + scan - units;
                    if (rg.empty_row) zero_output_row(p, rg.token);
                }
            }
            carry += __shfl(scan, 63, 64);
        }
        if (lane == 0) {
            plan_prefix[p.num_rows] = carry;
            if (w == 0) p.blk_prefix[p.num_rows] = carry;
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the records are in LDS (the wavefront is the whole workgroup)
        __builtin_amdgcn_wave_barrier();
    }
    auto prefix_at = [&](int i) -> int {
        if constexpr (kSelfPlan)
            return plan_prefix[i];
        else
            return p.blk_prefix[i];
    };
    const int64_t total = (int64_t)prefix_at(p.num_rows) * Hkv;
    if (total <= 0) return;
    // eight to a workgroup: the plan has chosen how many of the launched wavefronts work
    const int num_waves = kWaves == 1 ? p.num_waves : p.plan_waves[0];
    if (w >= num_waves) return;
    const Line line(total, num_waves, p.dyn_pieces);

    constexpr int64_t kRowBytesBuilt = kU8 ? (kHD + 8) : (2 * kHD);
    const int head_dim = kPad ? p.head_dim : kHD;                       // (a constant unless kPad)
    const int64_t kRowBytes = kPad ? (kU8 ? p.head_dim + 8 : 2 * p.head_dim) : kRowBytesBuilt;
    const int64_t block_stride = (int64_t)(Hkv / p.kv_share) * blk * kRowBytes;  // (kv_share: see PagedParams)
    // kPad: this lane's K piece offsets, V offset and whether its V columns exist
    int koff[kHD / 32];
    int voff = 0;
    bool v_ok = true;
    if constexpr (kPad) {
#pragma unroll
        for (int i = 0; i < kHD / 32; i++) {
            const int first = kg * (kHD / 4) + i * 8;  // first of the piece's eight columns
            koff[i] = n16 * (int)kRowBytes + (kU8 ? 8 + (first < head_dim ? first : 0) : (first < head_dim ? first * 2 : 0));
        }
        voff = kg * 4 * (int)kRowBytes + (kU8 ? 8 + n16 * 8 : n16 * 16);
        v_ok = n16 * 8 < head_dim;
    }

    // The static piece first, then dynamic pieces for as long as there are any.  The ticket for
    // the next dynamic piece is drawn before the current piece is worked on, so its latency is hidden.
    // Tickets come from one counter per group of wavefronts (a single counter would serialise
    // thousands of same-address atomics); group g owns the dynamic pieces g, g + groups, ...
    // A group mixes wavefronts of every XCD and of both dispatch halves (w / 8 mod groups).
    const int group = (w >> 3) % p.dyn_groups;
    int piece = w;
    int merge_seg = -1;  // (fused_merge) the segment this piece has to combine, as sequence * kv heads + kv head
    for (;;) {
    int ticket_lane0 = 0;
    if (p.dyn_pieces > 0 && lane == 0) ticket_lane0 = atomicAdd(p.dyn_counter + group, 1);
    int64_t L = line.begin(piece);
    const int64_t L_end = line.begin(piece + 1);
    int s = 0;
    if (L < L_end) {
        if constexpr (kSelfPlan) {  // the last row whose prefix is <= L / Hkv (the prefix is monotone)
            const int x = (int)(L / Hkv);
            int cnt = 0;
            for (int base = 0; base < p.num_rows; base += 64) {
                const int i = base + lane;
                cnt += __builtin_popcountll(__builtin_amdgcn_ballot_w64(i < p.num_rows && plan_prefix[i] <= x));
            }
            s = max(cnt - 1, 0);
        } else {
            s = locate_sequence(p.blk_prefix, p.num_rows, (int)(L / Hkv), lane);
        }
    }

    while (L < L_end) {
        while (s + 1 < p.num_rows && (int64_t)prefix_at(s + 1) * Hkv <= L) s++;  // next row with blocks
        DecodeRange rg;
        if constexpr (kSelfPlan)
            rg = plan_rec[s];
        else
            rg = ((const DecodeRange*)p.seq_info)[s];
        const int nb = rg.nb;
        if (nb <= 0) break;  // cannot happen for a consistent plan; never loop forever
        const int seglen = nb + p.switch_cost;
        const int64_t seq_L0 = (int64_t)prefix_at(s) * Hkv;
        const int h = (int)((L - seq_L0) / seglen);
        const int64_t seg_B0 = seq_L0 + (int64_t)h * seglen + p.switch_cost;  // line position of the segment's block 0
        const int64_t seg_L1 = seg_B0 + nb;                        // end of the segment
        const int64_t from = max(L, seg_B0), to = min(L_end, seg_L1);
        if (from >= to) {  // the piece ends inside the switch-cost units: no block of this segment is ours
            L = to;
            continue;
        }
        const int b_rel = (int)(from - seg_B0);
        const int n = (int)(to - from);  // blocks of this segment in this piece
        const bool whole = (n == nb);
        L = from;
        // the segment ends here and began in an earlier piece: this piece combines it when it is done
        // (one scalar carried through the loop; the rest is worked out again then)
        if constexpr (kFusedBuilt) {
            if (p.fused_merge && !whole && b_rel + n == nb) merge_seg = s * Hkv + h;
        }
        const int lb0 = rg.j0 / kUnit + b_rel;          // first unit of 32 tokens
        // (kBlk == 0: the table is indexed by the block of the absolute unit, lb0 + ... >> log2(units per block))
        const int32_t* table = p.block_indices + rg.table_begin + (kBlk ? lb0 * kEntries : 0);
        // table entries from there on that hold attended tokens (the row's table may end with them)
        const int entries = (rg.ctx + blk - 1) / blk - (kBlk ? lb0 * kEntries : 0);
        const int h_kv = p.kv_share == 1 ? h : h / p.kv_share;  // the kv head whose rows this segment reads
        const int64_t head_off = (int64_t)h_kv * blk * kRowBytes;
        const int sub_shift = kBlk ? 0 : __builtin_ctz(p.block_size >> 5);

        if constexpr (kSelfPlan) {
            // The new tokens of this call whose cache rows this piece is about to read go into the cache
            // first: the row's own token (in the segment's last block) and, when its sequence
            // contributes several tokens to the batch, the tokens ahead of it.  The same wavefront
            // stores and then loads, and the stores are waited for below; a token that several rows
            // attend is written by each of their wavefronts with the same bytes.
            if (do_write && rg.write_pos >= 0) {
                const int q_lo = max(rg.new_begin, lb0 * kUnit), q_hi = min(rg.write_pos, (lb0 + n) * kUnit - 1);
                for (int q = q_lo; q <= q_hi; q++) {  // (wave-uniform; one pass for a decode row)
                    const int pb_new = p.block_indices[rg.table_begin + q / blk];
                    if (pb_new >= 0 && pb_new < p.num_blocks)
                        kv_cache_write_pair128(wp, rg.token - (rg.write_pos - q), h_kv, pb_new, q, lane);
                }
                if (q_lo <= q_hi) __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the rows have reached the cache
            }
        }
        // Q^T operand: lane (head n16, kg) holds Q[head][kg * kHD/4 + i*8 .. +8]; padding heads are zero
        typename Op16<kBf16>::vec8 qf[4];
        float sumq = 0.0f;
        {
            const int64_t qrow = ((int64_t)rg.token * p.num_heads_q + (int64_t)h * G + n16) * head_dim;
#pragma unroll
            for (int i = 0; i < kHD / 32; i++) {
                if (n16 < G && (!kPad || kg * (kHD / 4) + i * 8 < head_dim)) {
                    qf[i] = load_q8<kBf16>(p.q, qrow + kg * (kHD / 4) + i * 8, p.q_dtype);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; e++) Op16<kBf16>::set(qf[i], e, 0.0f);
                }
                if constexpr (kU8) {
#pragma unroll
                    for (int e = 0; e < 8; e++) sumq += Op16<kBf16>::get(qf[i], e);
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
        const float* const slopes = kAlibi ? p.alibi_slopes + h * G : nullptr;  // ALiBi, this group's heads

        // units in groups of 64 table entries: one vector load fetches the group's block-table entries
        constexpr int kGroup = 64 / kEntries;
        for (int g0 = 0; g0 < n; g0 += kGroup) {
            const int gn = min(kGroup, n - g0);
            const int my_entry = kBlk ? g0 * kEntries + lane : (lb0 + g0 + lane) >> sub_shift;
            const int my_pb = (lane < gn * kEntries && my_entry < entries) ? table[my_entry] : -1;
            // which tiles of unit i were issued (0: none, the unit is skipped); never reads outside the cache
            auto issue = [&](BlockRegs<kU8>& regs, int i) -> int {
                if constexpr (kEntries == 1) {
                    const int pb = __builtin_amdgcn_readlane(my_pb, i);
                    if (pb < 0 || pb >= p.num_blocks) return 0;
                    int64_t off = (int64_t)pb * block_stride + head_off;
                    if constexpr (kBlk == 0) off += (int64_t)((lb0 + g0 + i) & sub_mask) * (kUnit * kRowBytes);
                    const uint8_t* const kb[2] = {p.key_cache + off, p.key_cache + off + 16 * kRowBytes};
                    const uint8_t* const vb[2] = {p.value_cache + off, p.value_cache + off + 16 * kRowBytes};
                    if constexpr (kPad)
                        load_block_padded<kU8, kHD, kTileBlk>(regs, kb, vb, (int)kRowBytes, koff, voff, v_ok, n16, kg);
                    else
                        load_block<kU8, kHD, kTileBlk>(regs, kb, vb, n16, kg);
                    return 3;
                } else {
                    const int pb0 = __builtin_amdgcn_readlane(my_pb, 2 * i), pb1 = __builtin_amdgcn_readlane(my_pb, 2 * i + 1);
                    // A tile counts only if it holds an attended token: a unit whose one valid block lies wholly
                    // ahead of the window (or behind the context) is skipped like a unit without blocks, so that
                    // every processed unit has a finite score.
                    const int tok0 = (lb0 + g0 + i) * kUnit;
                    const int ok = (pb0 >= 0 && pb0 < p.num_blocks && tok0 + 16 > rg.j0 && tok0 < rg.ctx ? 1 : 0) |
                                   (pb1 >= 0 && pb1 < p.num_blocks && tok0 + 32 > rg.j0 && tok0 + 16 < rg.ctx ? 2 : 0);
                    if (ok == 0) return 0;
                    // a tile without a block is read from the other tile's block: valid memory, and masked
                    const int64_t off0 = (int64_t)((ok & 1) ? pb0 : pb1) * block_stride + head_off;
                    const int64_t off1 = (int64_t)((ok & 2) ? pb1 : pb0) * block_stride + head_off;
                    const uint8_t* const kb[2] = {p.key_cache + off0, p.key_cache + off1};
                    const uint8_t* const vb[2] = {p.value_cache + off0, p.value_cache + off1};
                    if constexpr (kPad)
                        load_block_padded<kU8, kHD, kTileBlk>(regs, kb, vb, (int)kRowBytes, koff, voff, v_ok, n16, kg);
                    else
                        load_block<kU8, kHD, kTileBlk>(regs, kb, vb, n16, kg);
                    return ok;
                }
            };
            if constexpr (!kU8) {
                // two register stages: block i+1 is in flight while block i is consumed
                BlockRegs<kU8> ra, rb;
                int ok_a = issue(ra, 0), ok_b = 0;
                int i = 0;
                while (i < gn) {
                    ok_b = (i + 1 < gn) ? issue(rb, i + 1) : 0;
                    if constexpr (kHalfFromBf16) bf16_block_to_f16(ra);
                    if (ok_a) process_block<kU8, kBf16, kHD, kEntries != 1, kAlibi>(st, ra, qf, sumq, c, (lb0 + g0 + i) * kUnit, rg.j0, rg.ctx, kg, ok_a, slopes, G);
                    if (i + 1 >= gn) break;
                    ok_a = (i + 2 < gn) ? issue(ra, i + 2) : 0;
                    if constexpr (kHalfFromBf16) bf16_block_to_f16(rb);
                    if (ok_b) process_block<kU8, kBf16, kHD, kEntries != 1, kAlibi>(st, rb, qf, sumq, c, (lb0 + g0 + i + 1) * kUnit, rg.j0, rg.ctx, kg, ok_b, slopes, G);
                    i += 2;
                }
            } else {
                // kStages register stages: blocks i+1 .. i+kStages-1 are in flight while block i is
                // consumed.  (Measured on the 128-sequence u8 workload: two stages 452 us, three 455 us,
                // four spill registers and fall to 629 us.)
                constexpr int kStages = HIPATTN_U8_STAGES;
                BlockRegs<kU8> regs[kStages];
                int ok[kStages];
#pragma unroll
                for (int u = 0; u < kStages - 1; u++) ok[u] = (u < gn) ? issue(regs[u], u) : 0;
                for (int i = 0; i < gn; i += kStages) {
#pragma unroll
                    for (int u = 0; u < kStages; u++) {
                        const int idx = i + u;
                        if (idx >= gn) break;
                        constexpr int kLast = kStages - 1;
                        ok[(u + kLast) % kStages] =
                            (idx + kLast < gn) ? issue(regs[(u + kLast) % kStages], idx + kLast) : 0;
                        if (ok[u]) process_block<kU8, kBf16, kHD, kEntries != 1, kAlibi>(st, regs[u], qf, sumq, c, (lb0 + g0 + idx) * kUnit, rg.j0, rg.ctx, kg, ok[u], slopes, G);
                    }
                }
            }
        }

        // ---- this wavefront's result for the segment
        float l = st.l, corr = st.corr;
        l += __shfl_xor(l, 16, 64);
        l += __shfl_xor(l, 32, 64);
        if constexpr (kU8) {
            corr += __shfl_xor(corr, 16, 64);
            corr += __shfl_xor(corr, 32, 64);
        }
        const int64_t slot = (int64_t)piece + (int64_t)s * Hkv + h;  // unique per (piece, segment)
        if (n16 < G) {
            if (whole && p.sinks != nullptr && l > 0.0f) l += fast_exp2(p.sinks[h * G + n16] * kLog2e - st.m);
            const float inv = whole ? (l > 0.0f ? 1.0f / l : 0.0f) : 1.0f;
            // acc[e][r] is head-dim (kg*4 + r)*8 + e: eight consecutive outputs per r
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float o[8];
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    float v = st.acc[e][r];
                    if constexpr (kU8) v -= corr;
                    o[e] = v * inv;
                }
                const int d0 = (kg * 4 + r) * 8;
                // (rows of the accumulator beyond the head size hold nothing; a fused partial carries them all the same)
                if ((kPad || kHD < 128) && d0 >= head_dim && (whole || !(kFusedBuilt && p.fused_merge))) continue;
                if (whole) {
                    store_out8(p.out, ((int64_t)rg.token * p.num_heads_q + h * G + n16) * head_dim + d0, p.out_dtype, o);
                } else if (kFusedBuilt && p.fused_merge) {
                    float* rec = p.part_out + (slot * kPartPairs * 4 * G + (kg * G + n16)) * 2;
#pragma unroll
                    for (int e2 = 0; e2 < 4; e2++) agent_store2(rec + (r * 4 + e2) * 8 * G, o[2 * e2], o[2 * e2 + 1]);
                } else {
                    float* po = p.part_out + (slot * G + n16) * head_dim + d0;
                    *(float4*)(po) = make_float4(o[0], o[1], o[2], o[3]);
                    *(float4*)(po + 4) = make_float4(o[4], o[5], o[6], o[7]);
                }
            }
            if (kFusedBuilt && !whole && p.fused_merge) {
                agent_store2(p.part_out + (slot * kPartPairs * 4 * G + (kg * G + n16)) * 2 + 16 * 8 * G, st.m, l);
            } else if (!whole && kg == 0) {
                p.part_ml[(slot * G + n16) * 2] = st.m;
                p.part_ml[(slot * G + n16) * 2 + 1] = l;
            }
        }
        if (kFusedBuilt && p.fused_merge && !whole && b_rel + n < nb) {
            // a partial another wavefront will combine: announced once the stores above have completed
            // (no load is in flight at the end of a segment, so the wait is for these stores alone)
            stores_done();
            if (lane == 0)
                __hip_atomic_store((unsigned long long*)p.part_flag + slot, p.merge_tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        L += n;
    }
    if (kFusedBuilt && merge_seg >= 0) {
        stores_done();  // this wavefront's own partial of that segment
        const int ms = merge_seg / Hkv, mh = merge_seg - ms * Hkv;
        DecodeRange mr;
        if constexpr (kSelfPlan)
            mr = plan_rec[ms];
        else
            mr = ((const DecodeRange*)p.seq_info)[ms];
        const int64_t first_unit = (int64_t)prefix_at(ms) * Hkv + (int64_t)mh * (mr.nb + p.switch_cost) + p.switch_cost;
        const MergeArgs ma = {p.part_out, p.part_ml, p.part_flag, p.merge_tag, p.out, p.out_dtype, p.num_heads_q, p.num_heads_kv, p.head_dim, p.sinks};
        merge_in_kernel<kHD, kPad>(ma, line, ms, mh, mr.token, line.piece_at(first_unit), piece, lane);
        merge_seg = -1;
    }
    if (p.dyn_pieces <= 0) break;
    const int next = group + __shfl(ticket_lane0, 0, 64) * p.dyn_groups;
    if (next >= p.dyn_pieces) break;  // this group's share of the line is used up (every wavefront gets here)
    piece = num_waves + next;
    }
}

// ---- head size 256 ------------------------------------------------------------------------------
// The same schedule, products and lane layouts, with the head dimension worked through in two
// halves of 128 columns so that the registers hold: a unit of 32 tokens arrives as four
// half-stages of 32 registers -- K columns 0..127, K columns 128..255, V columns 0..127, V columns
// 128..255 -- the scores are the sum of the two K halves' products, the probabilities go into two
// sets of output accumulators, and while one half-stage is consumed the next is in flight.  A
// wavefront therefore has half as many bytes in flight as the head-128 kernel, and twice as many
// wavefronts are launched (eight per compute unit).
struct HalfRegs {
    uint4_t x[8];  // K: [tile * 4 + piece]; V: [tile * 4 + row]
};

// row: bytes from one cache row to the next (512, or 2 * head_dim for a smaller head).  koff[i]: this
// lane's offset of K piece i of the half inside a tile (a piece past the end of the row is pointed at
// the row's first piece: valid memory that meets zeros in the query operand).
template <int kBlk>
__device__ __forceinline__ void load_k_half(HalfRegs& b, const uint8_t* const (&kb)[2], int row, const int (&koff)[4]) {
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const uint8_t* const kt = kBlk == 32 ? kb[0] + t * 16 * row : kb[t];
#pragma unroll
        for (int i = 0; i < 4; i++) b.x[t * 4 + i] = *(const uint4_t*)(kt + koff[i]);
    }
}

// voff: this lane's offset of its first V row's piece of the half; v_ok: its columns exist.
template <int kBlk>
__device__ __forceinline__ void load_v_half(HalfRegs& b, const uint8_t* const (&vb)[2], int row, int voff, bool v_ok) {
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const uint8_t* const vt = kBlk == 32 ? vb[0] + t * 16 * row : vb[t];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            uint4_t piece = {0u, 0u, 0u, 0u};
            if (v_ok) piece = *(const uint4_t*)(vt + voff + r * row);
            b.x[t * 4 + r] = piece;
        }
    }
}

struct WaveState256 {
    float m, l;
    float corr;  // u8 only: this lane's share of sum_j p'_j (zp_j + bias)
    float4_t acc[2][8];  // acc[half][e][r] = O[head][128 * half + (kg*4 + r)*8 + e]
};

template <bool kBf16>
__device__ __forceinline__ void scores_half(float4_t (&s)[2], const HalfRegs& k, const typename Op16<kBf16>::vec8 (&q)[4]) {
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int i = 0; i < 4; i++) s[t] = Op16<kBf16>::mma(Op16<kBf16>::from_bits(k.x[t * 4 + i]), q[i], s[t]);
}

// Mask, scale and online softmax of a unit's scores (lane: tokens tok_base + t*16 + kg*4 + r); the
// accumulators are rescaled when a row's maximum moved.  Returns the probabilities as the B operand.
template <bool kBf16>
__device__ __forceinline__ typename Op16<kBf16>::vec8 softmax_unit(WaveState256& st, const float4_t (&s)[2], float c, int tok_base,
                                                                  int j0, int ctx, int kg, int tiles) {
    float sv[8];
    float mloc = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int tok = tok_base + t * 16 + kg * 4 + r;
            const float x = (tok >= j0 && tok < ctx && ((tiles >> t) & 1)) ? s[t][r] * c : -INFINITY;
            sv[t * 4 + r] = x;
            mloc = fmaxf(mloc, x);
        }
    mloc = max_over_rows(mloc);
    const float m_new = fmaxf(st.m, mloc);
    // (-inf only while nothing has been attended yet and this unit's blocks both lie outside the cache:
    // everything stays at zero then; exp2(-inf - -inf) would be NaN)
    const float m_use = m_new == -INFINITY ? 0.0f : m_new;
    const float alpha = fast_exp2(st.m - m_use);
    st.m = m_new;
    typename Op16<kBf16>::vec8 pf;
    float lsum = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float pj = fast_exp2(sv[j] - m_use);
        lsum += pj;
        Op16<kBf16>::set(pf, j, pj);
    }
    st.l = st.l * alpha + lsum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int e = 0; e < 8; e++) st.acc[h][e] *= alpha;
    }
    return pf;
}

// O^T += V^T P^T for one half of the columns.  Rows outside the attended range may hold anything
// (never-written cache memory): their probability is exactly zero and they are cleared, so that
// 0 * NaN cannot occur.
template <bool kBf16>
__device__ __forceinline__ void pv_half(float4_t (&acc)[8], HalfRegs& v, typename Op16<kBf16>::vec8 pf, bool partial, int tok_base,
                                        int j0, int ctx, int kg, int tiles) {
    if (partial) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int tok = tok_base + (j >> 2) * 16 + kg * 4 + (j & 3);
            if (!(tok >= j0 && tok < ctx && ((tiles >> (j >> 2)) & 1))) v.x[j] = (uint4_t){0u, 0u, 0u, 0u};
        }
    }
#pragma unroll
    for (int e = 0; e < 8; e++) {
        uint4_t w;
#pragma unroll
        for (int jp = 0; jp < 4; jp++) {
            const uint32_t lo = v.x[2 * jp][e >> 1], hi = v.x[2 * jp + 1][e >> 1];
            w[jp] = (e & 1) ? pack_hi(lo, hi) : pack_lo(lo, hi);
        }
        acc[e] = Op16<kBf16>::mma(Op16<kBf16>::from_bits(w), pf, acc[e]);
    }
}

// ---- the same for u8 caches: a half-stage is 32 tokens x 128 bytes (16 registers), so K (both halves, plus
// the tokens' scales and zero-points) and V (both halves) are the two stages that alternate, and a
// wavefront has as many bytes in flight as with a 16-bit cache.
struct HalfRegs8 {
    uint2_t x[8];  // K: [tile * 4 + piece]; V: [tile * 4 + row]
};

template <int kBlk>
__device__ __forceinline__ void load_k_half8(HalfRegs8& b, const uint8_t* const (&kb)[2], int row, const int (&koff)[4]) {
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const uint8_t* const kt = kBlk == 32 ? kb[0] + t * 16 * row : kb[t];
#pragma unroll
        for (int i = 0; i < 4; i++) b.x[t * 4 + i] = *(const uint2_t*)(kt + koff[i]);
    }
}

template <int kBlk>
__device__ __forceinline__ void load_v_half8(HalfRegs8& b, const uint8_t* const (&vb)[2], int row, int voff, bool v_ok) {
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const uint8_t* const vt = kBlk == 32 ? vb[0] + t * 16 * row : vb[t];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            uint2_t piece = {0u, 0u};
            if (v_ok) piece = *(const uint2_t*)(vt + voff + r * row);
            b.x[t * 4 + r] = piece;
        }
    }
}

// (scale, zp) of one token per lane, laid out as in BlockRegs<true>
template <int kBlk>
__device__ __forceinline__ float2 load_scale_zp(const uint8_t* const (&kb)[2], const uint8_t* const (&vb)[2], int row, int n16, int kg) {
    const int j = n16 & 7, at = (kg * 4 + (j & 3)) * row;
    if constexpr (kBlk == 32) {
        return *(const float2*)((n16 < 8 ? kb[0] : vb[0]) + (j >> 2) * 16 * row + at);
    } else {  // (one of four tile bases per lane, put together arithmetically: see load_block)
        const uintptr_t k0 = (uintptr_t)kb[0], k1 = (uintptr_t)kb[1], v0 = (uintptr_t)vb[0], v1 = (uintptr_t)vb[1];
        const uintptr_t second = (uintptr_t)(j >> 2), value = (uintptr_t)(n16 >> 3);
        const uintptr_t in_k = k0 + second * (k1 - k0), in_v = v0 + second * (v1 - v0);
        return *(const float2*)(in_k + value * (in_v - in_k) + (uintptr_t)at);
    }
}

__device__ __forceinline__ void scores_half8(float4_t (&s)[2], const HalfRegs8& k, const Op16<false>::vec8 (&q)[4]) {
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint4_t w;
            w[0] = bytes_to_biased_half2(k.x[t * 4 + i][0], 0x04010400u);
            w[1] = bytes_to_biased_half2(k.x[t * 4 + i][0], 0x04030402u);
            w[2] = bytes_to_biased_half2(k.x[t * 4 + i][1], 0x04010400u);
            w[3] = bytes_to_biased_half2(k.x[t * 4 + i][1], 0x04030402u);
            s[t] = Op16<false>::mma(Op16<false>::from_bits(w), q[i], s[t]);
        }
}

// softmax_unit for byte scores: the tokens' scales and zero-points turn them into scores, the
// probabilities leave multiplied by V's scales, and st.corr collects sum_j p'_j (zp_j + bias).
__device__ __forceinline__ Op16<false>::vec8 softmax_unit8(WaveState256& st, const float4_t (&s)[2], float2 sz, float sumq, float c,
                                                          int tok_base, int j0, int ctx, int kg, int tiles, bool partial) {
    float sz_scale = sz.x, sz_zero = sz.y + kByteBias;
    if (partial) {  // rows outside the attended range may hold anything: their scale and zero-point are cleared
        const int j = ((int)threadIdx.x & 7), tok = tok_base + (j >> 2) * 16 + kg * 4 + (j & 3);
        if (!(tok >= j0 && tok < ctx && ((tiles >> (j >> 2)) & 1))) sz_scale = sz_zero = 0.0f;
    }
    const float sz_prod = sz_scale * sz_zero;
    float ks[8], kp[8], vs[8], vz[8];
    ks[0] = row_broadcast<0>(sz_scale); kp[0] = row_broadcast<0>(sz_prod); vs[0] = row_broadcast<8>(sz_scale); vz[0] = row_broadcast<8>(sz_zero);
    ks[1] = row_broadcast<1>(sz_scale); kp[1] = row_broadcast<1>(sz_prod); vs[1] = row_broadcast<9>(sz_scale); vz[1] = row_broadcast<9>(sz_zero);
    ks[2] = row_broadcast<2>(sz_scale); kp[2] = row_broadcast<2>(sz_prod); vs[2] = row_broadcast<10>(sz_scale); vz[2] = row_broadcast<10>(sz_zero);
    ks[3] = row_broadcast<3>(sz_scale); kp[3] = row_broadcast<3>(sz_prod); vs[3] = row_broadcast<11>(sz_scale); vz[3] = row_broadcast<11>(sz_zero);
    ks[4] = row_broadcast<4>(sz_scale); kp[4] = row_broadcast<4>(sz_prod); vs[4] = row_broadcast<12>(sz_scale); vz[4] = row_broadcast<12>(sz_zero);
    ks[5] = row_broadcast<5>(sz_scale); kp[5] = row_broadcast<5>(sz_prod); vs[5] = row_broadcast<13>(sz_scale); vz[5] = row_broadcast<13>(sz_zero);
    ks[6] = row_broadcast<6>(sz_scale); kp[6] = row_broadcast<6>(sz_prod); vs[6] = row_broadcast<14>(sz_scale); vz[6] = row_broadcast<14>(sz_zero);
    ks[7] = row_broadcast<7>(sz_scale); kp[7] = row_broadcast<7>(sz_prod); vs[7] = row_broadcast<15>(sz_scale); vz[7] = row_broadcast<15>(sz_zero);
    float sv[8];
    float mloc = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int j = t * 4 + r, tok = tok_base + t * 16 + kg * 4 + r;
            const float x = fmaf(ks[j], s[t][r], -(kp[j] * sumq));
            sv[j] = (tok >= j0 && tok < ctx && ((tiles >> t) & 1)) ? x * c : -INFINITY;
            mloc = fmaxf(mloc, sv[j]);
        }
    mloc = max_over_rows(mloc);
    const float m_new = fmaxf(st.m, mloc);
    const float m_use = m_new == -INFINITY ? 0.0f : m_new;  // (see softmax_unit)
    const float alpha = fast_exp2(st.m - m_use);
    st.m = m_new;
    Op16<false>::vec8 pf;
    float lsum = 0.0f, csum = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        float pj = fast_exp2(sv[j] - m_use);
        lsum += pj;
        pj *= vs[j];
        Op16<false>::set(pf, j, pj);
        csum = fmaf(Op16<false>::get(pf, j), vz[j], csum);
    }
    st.l = st.l * alpha + lsum;
    st.corr = st.corr * alpha + csum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int e = 0; e < 8; e++) st.acc[h][e] *= alpha;
    }
    return pf;
}

// O^T += V^T P^T for one half of the columns, V as biased bytes (every byte is a finite number, and
// the probabilities of rows outside the attended range are exactly zero)
__device__ __forceinline__ void pv_half8(float4_t (&acc)[8], const HalfRegs8& v, Op16<false>::vec8 pf) {
#pragma unroll
    for (int e = 0; e < 8; e++) {
        uint4_t w;
        const uint32_t sel = 0x0c000c00u | ((4u + (e & 3)) << 16) | (uint32_t)(e & 3);
#pragma unroll
        for (int jp = 0; jp < 4; jp++) w[jp] = bytes_to_biased_half2(v.x[2 * jp][e >> 2], v.x[2 * jp + 1][e >> 2], sel);
        acc[e] = Op16<false>::mma(Op16<false>::from_bits(w), pf, acc[e]);
    }
}

// kPad: the call's head size (p.head_dim, a multiple of 8 above 128) may be smaller than 256.
// kU8: a u8 cache (fp16 operands).
template <bool kBf16, int kBlk, bool kPad, bool kU8 = false>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2, 2))) void paged_decode256_kernel(PagedParams p) {
    static_assert(!(kU8 && kBf16), "u8 caches are dequantised to fp16 operands");
    // kBlk: 16, 32, or 0 for any larger power of two (p.block_size: a block then holds several units)
    constexpr int kEntries = kBlk == 16 ? 2 : 1;
    constexpr int kTileBlk = kBlk == 16 ? 16 : 32;
    const int blk = kBlk ? kBlk : p.block_size;
    const int sub_mask = kBlk ? 0 : (p.block_size >> 5) - 1;
    const int sub_shift = kBlk ? 0 : __builtin_ctz(p.block_size >> 5);
    const int w = blockIdx.x, lane = threadIdx.x, n16 = lane & 15, kg = lane >> 4;
    const int kHD = kPad ? p.head_dim : 256;  // (a constant unless kPad)
    const int kRowBytes = kU8 ? kHD + 8 : 2 * kHD;
    // this lane's piece offsets inside a tile, per half, and whether its V columns exist
    int koff[2][4], voff[2];
    bool v_ok[2];
#pragma unroll
    for (int half = 0; half < 2; half++) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int first = half * 128 + kg * 32 + i * 8;  // first of the piece's eight columns
            koff[half][i] = n16 * kRowBytes + (kU8 ? 8 + (first < kHD ? first : 0) : (first < kHD ? first * 2 : 0));
        }
        voff[half] = kg * 4 * kRowBytes + (kU8 ? 8 + half * 128 + n16 * 8 : half * 256 + n16 * 16);
        v_ok[half] = half * 128 + n16 * 8 < kHD;
    }
    const int Hkv = p.num_heads_kv, G = p.num_heads_q / p.num_heads_kv;
    const float c = p.scale * kLog2e;
    const int64_t total = (int64_t)p.blk_prefix[p.num_rows] * Hkv;
    if (total <= 0 || w >= p.num_waves) return;
    const Line line(total, p.num_waves, 0);
    const int64_t block_stride = (int64_t)(Hkv / p.kv_share) * blk * kRowBytes;
    int64_t L = line.begin(w);
    const int64_t L_end = line.begin(w + 1);
    if (L >= L_end) return;
    int s = locate_sequence(p.blk_prefix, p.num_rows, (int)(L / Hkv), lane);
    while (L < L_end) {
        while (s + 1 < p.num_rows && (int64_t)p.blk_prefix[s + 1] * Hkv <= L) s++;  // next row with units
        const DecodeRange rg = ((const DecodeRange*)p.seq_info)[s];
        const int nb = rg.nb;
        if (nb <= 0) break;  // cannot happen for a consistent plan; never loop forever
        const int seglen = nb + p.switch_cost;
        const int64_t seq_L0 = (int64_t)p.blk_prefix[s] * Hkv;
        const int h = (int)((L - seq_L0) / seglen);
        const int64_t seg_B0 = seq_L0 + (int64_t)h * seglen + p.switch_cost;
        const int64_t seg_L1 = seg_B0 + nb;
        const int64_t from = max(L, seg_B0), to = min(L_end, seg_L1);
        if (from >= to) {
            L = to;
            continue;
        }
        const int b_rel = (int)(from - seg_B0);
        const int n = (int)(to - from);
        const bool whole = (n == nb);
        L = from;
        const int lb0 = rg.j0 / kUnit + b_rel;
        const int32_t* table = p.block_indices + rg.table_begin + (kBlk ? lb0 * kEntries : 0);
        const int entries = (rg.ctx + blk - 1) / blk - (kBlk ? lb0 * kEntries : 0);
        const int64_t head_off = (int64_t)(p.kv_share == 1 ? h : h / p.kv_share) * blk * kRowBytes;

        // Q^T operand in two halves: lane (head n16, kg) holds Q[head][128*half + kg*32 + i*8 .. +8]
        typename Op16<kBf16>::vec8 qf[2][4];
        float sumq = 0.0f;  // u8: the sum of the head's query elements (see process_block)
        {
            const int64_t qrow = ((int64_t)rg.token * p.num_heads_q + (int64_t)h * G + n16) * kHD;
#pragma unroll
            for (int half = 0; half < 2; half++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    if (n16 < G && half * 128 + kg * 32 + i * 8 < kHD) {
                        qf[half][i] = load_q8<kBf16>(p.q, qrow + half * 128 + kg * 32 + i * 8, p.q_dtype);
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; e++) Op16<kBf16>::set(qf[half][i], e, 0.0f);
                    }
                    if constexpr (kU8) {
#pragma unroll
                        for (int e = 0; e < 8; e++) sumq += Op16<kBf16>::get(qf[half][i], e);
                    }
                }
            if constexpr (kU8) {
                sumq += __shfl_xor(sumq, 16, 64);
                sumq += __shfl_xor(sumq, 32, 64);
            }
        }
        WaveState256 st;
        st.m = -INFINITY;
        st.l = 0.0f;
        st.corr = 0.0f;
#pragma unroll
        for (int half = 0; half < 2; half++)
#pragma unroll
            for (int e = 0; e < 8; e++) st.acc[half][e] = (float4_t){0.f, 0.f, 0.f, 0.f};

        constexpr int kGroup = 64 / kEntries;
        for (int g0 = 0; g0 < n; g0 += kGroup) {
            const int gn = min(kGroup, n - g0);
            const int my_entry = kBlk ? g0 * kEntries + lane : (lb0 + g0 + lane) >> sub_shift;
            const int my_pb = (lane < gn * kEntries && my_entry < entries) ? table[my_entry] : -1;
            // Bases of the two tiles of unit i, and which of them lie in a block of the cache.  A block id
            // outside the cache is replaced by one inside it, so that the loads need no branch; the mask
            // keeps such a tile out of the scores and clears its V rows.
            auto unit = [&](int i, const uint8_t* (&kb)[2], const uint8_t* (&vb)[2]) -> int {
                if constexpr (kEntries == 1) {
                    const int pb = __builtin_amdgcn_readlane(my_pb, i);
                    const int ok = (pb >= 0 && pb < p.num_blocks) ? 3 : 0;
                    int64_t off = (int64_t)min(max(pb, 0), p.num_blocks - 1) * block_stride + head_off;
                    if constexpr (kBlk == 0) off += (int64_t)((lb0 + g0 + i) & sub_mask) * (kUnit * kRowBytes);
                    kb[0] = p.key_cache + off;
                    kb[1] = kb[0] + 16 * kRowBytes;
                    vb[0] = p.value_cache + off;
                    vb[1] = vb[0] + 16 * kRowBytes;
                    return ok;
                } else {
                    const int pb0 = __builtin_amdgcn_readlane(my_pb, 2 * i), pb1 = __builtin_amdgcn_readlane(my_pb, 2 * i + 1);
                    const int ok = (pb0 >= 0 && pb0 < p.num_blocks ? 1 : 0) | (pb1 >= 0 && pb1 < p.num_blocks ? 2 : 0);
                    const int64_t off0 = (int64_t)min(max(pb0, 0), p.num_blocks - 1) * block_stride + head_off;
                    const int64_t off1 = (int64_t)min(max(pb1, 0), p.num_blocks - 1) * block_stride + head_off;
                    kb[0] = p.key_cache + off0;
                    kb[1] = p.key_cache + off1;
                    vb[0] = p.value_cache + off0;
                    vb[1] = p.value_cache + off1;
                    return ok;
                }
            };
            if constexpr (kU8) {
                // Two stages: K of unit i (both halves, with the scales and zero-points) is there when
                // iteration i begins; V arrives while the scores are worked out, the next unit's K while
                // the outputs are.  No branch in the body, as below.
                HalfRegs8 rk[2], rv[2];
                float2 sz;
                {
                    const uint8_t *kb[2], *vb[2];
                    (void)unit(0, kb, vb);
                    load_k_half8<kTileBlk>(rk[0], kb, kRowBytes, koff[0]);
                    load_k_half8<kTileBlk>(rk[1], kb, kRowBytes, koff[1]);
                    sz = load_scale_zp<kTileBlk>(kb, vb, kRowBytes, n16, kg);
                }
                for (int i = 0; i < gn; i++) {
                    const int tok_base = (lb0 + g0 + i) * kUnit;
                    const uint8_t *kb[2], *vb[2];
                    const int ok = unit(i, kb, vb);
                    const bool partial = (tok_base < rg.j0) || (tok_base + kUnit > rg.ctx) || ok != 3;  // wavefront-uniform
                    float4_t sc[2] = {(float4_t){0.f, 0.f, 0.f, 0.f}, (float4_t){0.f, 0.f, 0.f, 0.f}};
                    load_v_half8<kTileBlk>(rv[0], vb, kRowBytes, voff[0], v_ok[0]);
                    load_v_half8<kTileBlk>(rv[1], vb, kRowBytes, voff[1], v_ok[1]);
                    scores_half8(sc, rk[0], qf[0]);
                    scores_half8(sc, rk[1], qf[1]);
                    const Op16<false>::vec8 pf = softmax_unit8(st, sc, sz, sumq, c, tok_base, rg.j0, rg.ctx, kg, ok, partial);
                    __builtin_amdgcn_sched_barrier(0);
                    {
                        const uint8_t *kbn[2], *vbn[2];
                        (void)unit(min(i + 1, gn - 1), kbn, vbn);
                        load_k_half8<kTileBlk>(rk[0], kbn, kRowBytes, koff[0]);
                        load_k_half8<kTileBlk>(rk[1], kbn, kRowBytes, koff[1]);
                        sz = load_scale_zp<kTileBlk>(kbn, vbn, kRowBytes, n16, kg);
                    }
                    pv_half8(st.acc[0], rv[0], pf);
                    pv_half8(st.acc[1], rv[1], pf);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                // r0 holds the first K half of unit i when iteration i begins (loaded by the iteration before; the
                // last iteration loads its own unit's again rather than branching).  No branch in the body: a
                // unit whose blocks are both outside the cache goes through with every score masked.
                HalfRegs r0, r1;
                {
                    const uint8_t *kb[2], *vb[2];
                    (void)unit(0, kb, vb);
                    load_k_half<kTileBlk>(r0, kb, kRowBytes, koff[0]);
                }
                for (int i = 0; i < gn; i++) {
                    const int tok_base = (lb0 + g0 + i) * kUnit;
                    const uint8_t *kb[2], *vb[2];
                    const int ok = unit(i, kb, vb);  // (scalar work: the bases are not carried from iteration to iteration)
                    const bool partial = (tok_base < rg.j0) || (tok_base + kUnit > rg.ctx) || ok != 3;  // wavefront-uniform
                    float4_t sc[2] = {(float4_t){0.f, 0.f, 0.f, 0.f}, (float4_t){0.f, 0.f, 0.f, 0.f}};
                    // (the scheduling barriers keep each half-stage's loads behind the use of the registers
                    // they overwrite: hoisted to the top of the iteration they would all be live at once)
                    load_k_half<kTileBlk>(r1, kb, kRowBytes, koff[1]);
                    scores_half<kBf16>(sc, r0, qf[0]);
                    __builtin_amdgcn_sched_barrier(0);
                    load_v_half<kTileBlk>(r0, vb, kRowBytes, voff[0], v_ok[0]);
                    scores_half<kBf16>(sc, r1, qf[1]);
                    const typename Op16<kBf16>::vec8 pf = softmax_unit<kBf16>(st, sc, c, tok_base, rg.j0, rg.ctx, kg, ok);
                    __builtin_amdgcn_sched_barrier(0);
                    load_v_half<kTileBlk>(r1, vb, kRowBytes, voff[1], v_ok[1]);
                    pv_half<kBf16>(st.acc[0], r0, pf, partial, tok_base, rg.j0, rg.ctx, kg, ok);
                    __builtin_amdgcn_sched_barrier(0);
                    {
                        const uint8_t *kbn[2], *vbn[2];
                        (void)unit(min(i + 1, gn - 1), kbn, vbn);
                        load_k_half<kTileBlk>(r0, kbn, kRowBytes, koff[0]);
                    }
                    pv_half<kBf16>(st.acc[1], r1, pf, partial, tok_base, rg.j0, rg.ctx, kg, ok);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }

        // ---- this wavefront's result for the segment
        float l = st.l, corr = st.corr;
        l += __shfl_xor(l, 16, 64);
        l += __shfl_xor(l, 32, 64);
        if constexpr (kU8) {
            corr += __shfl_xor(corr, 16, 64);
            corr += __shfl_xor(corr, 32, 64);
        }
        const int64_t slot = (int64_t)w + (int64_t)s * Hkv + h;  // unique per (piece, segment)
        if (n16 < G) {
            if (whole && p.sinks != nullptr && l > 0.0f) l += fast_exp2(p.sinks[h * G + n16] * kLog2e - st.m);
            const float inv = whole ? (l > 0.0f ? 1.0f / l : 0.0f) : 1.0f;
#pragma unroll
            for (int half = 0; half < 2; half++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    float o[8];
#pragma unroll
                    for (int e = 0; e < 8; e++) o[e] = (kU8 ? st.acc[half][e][r] - corr : st.acc[half][e][r]) * inv;
                    const int d0 = half * 128 + (kg * 4 + r) * 8;
                    if (kPad && d0 >= kHD) continue;  // (columns beyond the head size hold nothing)
                    if (whole) {
                        store_out8(p.out, ((int64_t)rg.token * p.num_heads_q + h * G + n16) * kHD + d0, p.out_dtype, o);
                    } else {
                        float* po = p.part_out + (slot * G + n16) * kHD + d0;
                        *(float4*)(po) = make_float4(o[0], o[1], o[2], o[3]);
                        *(float4*)(po + 4) = make_float4(o[4], o[5], o[6], o[7]);
                    }
                }
            if (!whole && kg == 0) {
                p.part_ml[(slot * G + n16) * 2] = st.m;
                p.part_ml[(slot * G + n16) * 2 + 1] = l;
            }
        }
        L += n;
    }
}

// Combines the partials of every (sequence, kv head) segment that more than one piece worked
// on.  A separate launch: the kernel boundary is what makes the partials visible, which is far
// cheaper here than device-scope fences inside the streaming kernel (those write back and
// invalidate whole L2 caches and cost the decode kernel almost half of its bandwidth).
__global__ __launch_bounds__(256) void paged_merge_kernel(PagedParams p) {
    const int Hkv = p.num_heads_kv, G = p.num_heads_q / p.num_heads_kv;
    const int s = blockIdx.x / Hkv, h = blockIdx.x % Hkv;  // one workgroup per segment
    const DecodeRange rg = ((const DecodeRange*)p.seq_info)[s];
    if (rg.nb <= 0) return;
    const int64_t total = (int64_t)p.blk_prefix[p.num_rows] * Hkv;
    if (total <= 0) return;
    const Line line(total, p.overlap ? p.plan_waves[0] : p.num_waves, p.dyn_pieces);
    const int seglen = rg.nb + p.switch_cost;
    const int64_t L0 = (int64_t)p.blk_prefix[s] * Hkv + (int64_t)h * seglen + p.switch_cost, L1 = L0 + rg.nb;
    const int id_first = line.piece_at(L0), id_last = line.piece_at(L1 - 1);
    if (id_first >= id_last) return;  // a single piece covered the segment and wrote the final rows
    for (int g = threadIdx.x >> 6; g < G; g += 4)  // one wavefront per query head of the group
        merge_segment_head(p, line, s, h, g, rg.token, id_first, id_last, threadIdx.x & 63);
}


// Schedule options: process-wide, changed with set_option (hipattn_set_option in the C ABI).  The
// environment variable HIPATTN_<NAME IN CAPITALS> gives an option its initial value; the
// environment is read once, when the first option is looked at, never on the call path.
namespace {
struct Option {
    const char* name;
    const char* env;
    int dflt, lo, hi;
    std::atomic<int> value;
};
Option g_options[] = {
    // 0: one kernel after the other for mixed batches; 1: decode beside the chunks' flash kernel
    {"mixed_overlap", "HIPATTN_MIXED_OVERLAP", 1, 0, 1, {1}},
    // block-times a (sequence, kv head) segment start is charged on the decode work line
    {"decode_switch_cost", "HIPATTN_DECODE_SWITCH_COST", 5, 0, 64, {5}},
    // on-demand pieces per wavefront for the last quarter of the decode work line (0: none)
    {"decode_dyn_pieces_per_wave", "HIPATTN_DECODE_DYN_PIECES_PER_WAVE", 0, 0, 64, {0}},
    // scales the compute units the plan gives the decode part of a mixed batch (100 = as modelled)
    {"mixed_decode_share_percent", "HIPATTN_MIXED_DECODE_SHARE_PERCENT", 100, 10, 1000, {100}},
    // 1: dense SDPA at head sizes below 128 runs the tuned head-128 kernel on rows of fewer columns; 0: the plain kernels
    {"sdpa_padded_rows", "HIPATTN_SDPA_PADDED_ROWS", 1, 0, 1, {1}},
    // 1: the decode kernels that have the code for it (u8 caches) combine the partials of split segments
    // themselves; 0: a merge launch behind every decode kernel
    {"decode_fused_merge", "HIPATTN_DECODE_FUSED_MERGE", 1, 0, 1, {1}},
};
enum { kOptMixedOverlap = 0, kOptSwitchCost, kOptDynPieces, kOptSharePercent, kOptSdpaPadded, kOptFusedMerge };

void init_options_from_environment() {
    static std::once_flag once;
    std::call_once(once, [] {
        for (Option& o : g_options)
            if (const char* e = getenv(o.env)) o.value.store(std::min(std::max(atoi(e), o.lo), o.hi));
    });
}
int option(int which) {
    init_options_from_environment();
    return g_options[which].value.load(std::memory_order_relaxed);
}
}  // namespace

bool sdpa_padded_rows_enabled() { return option(kOptSdpaPadded) != 0; }

bool set_option(const char* name, int value) {
    init_options_from_environment();
    for (Option& o : g_options)
        if (strcmp(o.name, name) == 0) {
            o.value.store(value < 0 ? o.dflt : std::min(std::max(value, o.lo), o.hi));
            return true;
        }
    return false;
}

// ---- host side of the fast path ---------------------------------------------------------

// Every head size up to 256 that is a multiple of 8 with 16-bit and u8 caches, on blocks of 16, 32 or a
// larger power of two.

// fp16 queries on a bf16 cache at head size 128: the ordinary launch with the blocks converted to fp16 operands
// (kHalfFromBf16; no self-planning or eight-wavefront form of it is built, nor one with the distance bias).
static bool half_operands_from_bf16(const PagedParams& p) {
    return p.cache_dtype == HIPATTN_BF16 && p.q_dtype == HIPATTN_F16 && p.head_dim == kD && !p.alibi_slopes;
}

bool paged_fast_supported(const PagedParams& p) {
    const int G = p.num_heads_q / p.num_heads_kv;
    if (G > 16 || !(p.q_dtype == HIPATTN_F16 || p.q_dtype == HIPATTN_BF16)) return false;
    // (head sizes below 64 / between 64 and 128: the head-64 / head-128 kernel with zero columns)
    if (p.block_size < 16 || (p.block_size & (p.block_size - 1)) != 0) return false;  // 16, 32, or a larger power of two
    if (p.alibi_slopes && p.head_dim > 128) return false;  // (the head-256 decode kernel has no distance term: the query-tile kernel takes the batch)
    // (above 128: paged_decode256_kernel)
    return p.head_dim >= 8 && p.head_dim <= 256 && p.head_dim % 8 == 0 &&
           (p.cache_dtype == HIPATTN_F16 || p.cache_dtype == HIPATTN_BF16 || p.cache_dtype == HIPATTN_U8);
}

PagedParams split_kv_heads(const PagedParams& p) {
    const int G = p.num_heads_q / p.num_heads_kv;
    if (G <= 16 || p.kv_share != 1) return p;
    for (int share = 2; share <= G; share++) {
        if (G % share != 0 || G / share > 16) continue;
        if (G / share < 8) break;  // (groups that fill less than half of a 16-row product: the K/V rows would be read too often)
        if ((int64_t)p.num_heads_kv * share > 0x7fff) break;
        PagedParams s = p;
        s.num_heads_kv = p.num_heads_kv * share;
        s.kv_share = share;
        return paged_fast_supported(s) ? s : p;
    }
    return p;  // (a prime number of heads, say: the query-tile kernel keeps the call)
}

// The chunk kernels address K and V by the cache's own kv heads.
static PagedParams with_cache_heads(const PagedParams& p) {
    PagedParams r = p;
    r.num_heads_kv = p.num_heads_kv / p.kv_share;
    r.kv_share = 1;
    return r;
}

// Wavefronts the decode kernel keeps resident: it needs up to 256 registers per lane, i.e. two
// wavefronts per SIMD, eight per compute unit.
static int resident_decode_waves() {
    static thread_local int cached_device = -1, cached_waves = 0;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 2048;
    if (dev != cached_device) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        cached_device = dev;
        cached_waves = cus * 8;
    }
    return cached_waves;
}

// fp16 caches stream best with one wavefront per SIMD (four per compute unit; three measure the
// same); the u8 path has more arithmetic per byte and wants more: six per compute unit measured
// 1.5 % faster than all eight on the 128-sequence u8 configuration, counts that do not divide
// evenly over the compute units 5-10 % slower.
// Upper bound of the 128-row query tiles of the batch's multi-token sequences (the lengths stay
// on the device): each such sequence has at least 2 tokens and wastes at most one tile.
// 0 selects the row-per-token form of the plan, which takes the batch to hold as many rows as
// sequences: only a batch with exactly that many tokens may get it (a single token spread over two
// or more sequences, all but one of them empty, has a bound of 0 by the formula and must not).
static int query_tile_bound(const PagedParams& p) {
    if (p.num_tokens == p.num_seqs && !p.any_lengths) return 0;  // one token per sequence: a pure decode batch
    return std::max(1, p.num_tokens / 128 + std::min(p.num_seqs, p.num_tokens / 2));
}

// Mixed batches run the decode kernel beside the chunks' flash kernel unless the caller fixed the
// number of decode wavefronts or the option mixed_overlap = 0 asks for one kernel after the other.
// Records of the decode plan: one per sequence, or one per token when the batch is planned per token.
static int plan_rows(const PagedParams& p) { return query_tile_bound(p) == 0 ? p.num_tokens : p.num_seqs; }

static bool overlap_wanted(const PagedParams& p) {
    if (query_tile_bound(p) == 0 || p.num_waves > 0 || p.no_side_stream || p.alibi_slopes || half_operands_from_bf16(p)) return false;
    // the eight-wavefront decode kernel: head size 128, and 16-bit caches at the head sizes between 64 and 128
    if (p.head_dim != kD && !(p.head_dim > 64 && p.head_dim < kD && p.cache_dtype != HIPATTN_U8)) return false;
    return option(kOptMixedOverlap) != 0;
}

static int choose_num_waves(const PagedParams& p, bool overlap) {
    if (p.num_waves > 0) return p.num_waves;
    const int resident = resident_decode_waves();
    if (overlap) return resident;  // the most the plan may choose
    // (u8 at head size 64 has the most arithmetic per byte of all: every resident wavefront, 0.59 against
    // 0.48 of HBM peak with six per compute unit on the 128-sequence u8 batch)
    if (p.head_dim > 128) return resident;  // half as many bytes in flight per wavefront: twice the wavefronts
    if (p.cache_dtype == HIPATTN_U8) return p.head_dim <= 64 ? resident : resident / 4 * 3;
    return resident / 2;
}

static size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// On-demand pieces per wavefront for the last quarter of the line.  Off by default: a wavefront
// that starts on a new piece pays a chain of dependent loads (ticket, sequence, block table,
// first block) before it streams again, and on MI355X that costs more than the better balance
// at the end of the kernel wins back.  The option decode_dyn_pieces_per_wave switches it on.
static int choose_dyn_pieces(const PagedParams& p, int num_waves, bool overlap) {
    if (overlap || p.head_dim > 128) return 0;  // (the head-256 kernel has static pieces only)
    return num_waves * option(kOptDynPieces);
}

// Bytes of one slot of unnormalised partial outputs: [G, head_dim] floats for the merge kernel, or the
// fused merge's lane layout (kPartPairs pairs for each of 4 G lanes), whichever is larger.
static size_t part_floats_per_slot(const PagedParams& p) {
    const size_t G = (size_t)(p.num_heads_q / p.num_heads_kv);
    return std::max(G * p.head_dim, (size_t)kPartPairs * 4 * G * 2) * sizeof(float);
}

size_t paged_fast_workspace_bytes(const PagedParams& p) {
    const bool overlap = overlap_wanted(p);
    const int W = choose_num_waves(p, overlap);
    const int G = p.num_heads_q / p.num_heads_kv;
    const size_t rows = (size_t)plan_rows(p);
    const size_t slots = (size_t)W + choose_dyn_pieces(p, W, overlap) + rows * p.num_heads_kv;
    return 512 + 2 * align_up((rows + 1) * sizeof(int32_t), 256) + align_up(rows * 32, 256) +
           align_up(slots * part_floats_per_slot(p), 256) + align_up(slots * G * 2 * sizeof(float), 256) +
           align_up(slots * sizeof(uint64_t), 256);
}

// A value no earlier call of this process used and that memory which was never written is unlikely to hold.
static unsigned long long next_merge_tag() {
    static std::atomic<unsigned long long> counter{0};
    static const unsigned long long base = [] {
        unsigned long long x = 0x9e3779b97f4a7c15ull ^ (unsigned long long)(uintptr_t)&counter;
        x ^= (unsigned long long)std::chrono::steady_clock::now().time_since_epoch().count() * 0xbf58476d1ce4e5b9ull;
        return x | (1ull << 63);
    }();
    return base + (counter.fetch_add(1, std::memory_order_relaxed) << 1) + 1;  // never zero: zero means "taken"
}


void paged_fast_plan(PagedParams& p, void* workspace) {
    const bool overlap = overlap_wanted(p);  // asks whether the caller fixed num_waves: before it is filled in
    p.overlap = overlap ? 1 : 0;
    p.num_waves = choose_num_waves(p, overlap);
    p.switch_cost = option(kOptSwitchCost);
    p.dyn_pieces = choose_dyn_pieces(p, p.num_waves, overlap);
    p.overlap_share = option(kOptSharePercent) / 100.0f;
    p.dyn_groups = std::min(64, std::max(1, p.num_waves / 32));  // every group has at least one wavefront
    const int G = p.num_heads_q / p.num_heads_kv;
    p.max_q_tiles = query_tile_bound(p);
    p.num_rows = plan_rows(p);
    const size_t slots = (size_t)p.num_waves + p.dyn_pieces + (size_t)p.num_rows * p.num_heads_kv;
    uint8_t* w = (uint8_t*)workspace;
    p.dyn_counter = (int32_t*)w;
    w += 256;
    p.plan_waves = (int32_t*)w;
    w += 256;
    p.tile_prefix = (int32_t*)w;
    w += align_up(((size_t)p.num_rows + 1) * sizeof(int32_t), 256);
    p.blk_prefix = (int32_t*)w;
    w += align_up(((size_t)p.num_rows + 1) * sizeof(int32_t), 256);
    p.seq_info = w;
    w += align_up((size_t)p.num_rows * 32, 256);
    p.part_out = (float*)w;
    w += align_up(slots * part_floats_per_slot(p), 256);
    p.part_ml = (float*)w;
    w += align_up(slots * G * 2 * sizeof(float), 256);
    p.part_flag = (uint64_t*)w;
    w += align_up(slots * sizeof(uint64_t), 256);
    // the head-256 kernel and on-demand pieces (whose order of completion is not that of their numbers) keep the merge launch
    // Built into the u8 kernels only (see kFusedBuilt).  Measured, whole steps on one machine: the 128-sequence
    // u8 batch 0.450 ms fused against 0.454 ms with the merge launch.
    p.fused_merge = (option(kOptFusedMerge) != 0 && p.cache_dtype == HIPATTN_U8 && p.dyn_pieces == 0 && p.head_dim <= 128) ? 1 : 0;
    p.merge_tag = next_merge_tag();
}

// ---- scratch of the entry point that allocates nothing (hipattn_paged_attention_noalloc) ------
// A file-scope device array stands in for the caller's workspace: every GPU the library runs on
// holds its own copy until the process ends.  In host code the array's name is not a device
// address; the address on the current device comes from hipGetSymbolAddress, once per device, and
// that pointer is what kernels and host calls get.  Calls that overlap on one GPU share the array
// and race; it keeps the previous call's contents (the plan clears the ticket counters, everything
// else is written before it is read).
constexpr size_t kStaticScratchBytes = HIPATTN_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) uint8_t scratch[kStaticScratchBytes];

hipError_t paged_static_scratch(void** ptr, size_t* bytes) {
    static std::mutex mutex;
    static void* address[64] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> guard(mutex);
    if (!address[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        address[dev] = p;
    }
    *ptr = address[dev];
    *bytes = kStaticScratchBytes;
    return hipSuccess;
}

// A side stream and a fork/join pair of events per (device, caller's stream), made on the first
// mixed batch that stream carries, so that mixed batches on different streams do not wait for each
// other's chunk kernels.  An entry lives until its stream is destroyed through the C ABI
// (release_side_stream) or the process ends; beyond kMaxSideStreams entries further caller streams
// share the device's first entry.  The entry's mutex keeps the record/wait pairs of concurrent
// callers apart.
struct SideStream {
    int device = 0;
    hipStream_t owner = nullptr;
    hipStream_t stream = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
    std::mutex mutex;
};

constexpr int kMaxSideStreams = 32;
static std::mutex g_side_mutex;
static SideStream* g_side[kMaxSideStreams] = {};

static SideStream* side_stream(hipStream_t owner) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> guard(g_side_mutex);
    int free_slot = -1;
    SideStream* shared = nullptr;
    for (int i = 0; i < kMaxSideStreams; i++) {
        SideStream* s = g_side[i];
        if (!s) {
            if (free_slot < 0) free_slot = i;
            continue;
        }
        if (s->device != dev) continue;
        if (s->owner == owner) return s;
        if (!shared) shared = s;
    }
    if (free_slot < 0) return shared;  // table full: share (nullptr if this device has none, the caller reports it)
    SideStream* s = new SideStream;
    s->device = dev;
    s->owner = owner;
    if (hipStreamCreateWithFlags(&s->stream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&s->fork, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&s->join, hipEventDisableTiming) != hipSuccess) {
        if (s->stream) (void)hipStreamDestroy(s->stream);
        if (s->fork) (void)hipEventDestroy(s->fork);
        if (s->join) (void)hipEventDestroy(s->join);
        delete s;
        return nullptr;
    }
    g_side[free_slot] = s;
    return s;
}

// Called before a stream is destroyed: whatever its side stream still runs is waited for, then the
// side stream and its events go.  Streams other callers share through a full table are not owned by
// the stream being destroyed and stay.
void release_side_stream(hipStream_t owner) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return;
    SideStream* s = nullptr;
    {
        std::lock_guard<std::mutex> guard(g_side_mutex);
        for (int i = 0; i < kMaxSideStreams; i++)
            if (g_side[i] && g_side[i]->device == dev && g_side[i]->owner == owner) {
                s = g_side[i];
                g_side[i] = nullptr;
                break;
            }
    }
    if (!s) return;
    {
        std::lock_guard<std::mutex> guard(s->mutex);
        (void)hipStreamSynchronize(s->stream);
        (void)hipStreamDestroy(s->stream);
        (void)hipEventDestroy(s->fork);
        (void)hipEventDestroy(s->join);
    }
    delete s;
}

// The decode kernel for p's cache type, head size and block size (a combination paged_fast_supported
// admits; head sizes other than 128 have the ordinary form only, blocks of more than 32 tokens no self-planning form).
template <bool kU8, bool kBf16, int kWaves, bool kSelfPlan, int kHD, bool kPad>
static void launch_decode_blk(const PagedParams& p, const KvWriteParams& wp, int do_write, dim3 grid, dim3 block, hipStream_t stream) {
    if constexpr (kWaves == 1 && !kSelfPlan && kBf16 && kHD == 128 && !kPad) {
        if (half_operands_from_bf16(p)) {
            if (p.block_size == 32)
                hipLaunchKernelGGL((paged_decode_kernel<false, false, 1, false, 128, 32, false, false, true>), grid, block, 0, stream, p, wp, do_write);
            else if (p.block_size == 16)
                hipLaunchKernelGGL((paged_decode_kernel<false, false, 1, false, 128, 16, false, false, true>), grid, block, 0, stream, p, wp, do_write);
            else
                hipLaunchKernelGGL((paged_decode_kernel<false, false, 1, false, 128, 0, false, false, true>), grid, block, 0, stream, p, wp, do_write);
            return;
        }
    }
    if constexpr (kWaves == 1 && !kSelfPlan) {
        if (p.alibi_slopes) {  // the instantiations with the distance bias
            if (p.block_size == 32)
                hipLaunchKernelGGL((paged_decode_kernel<kU8, kBf16, 1, false, kHD, 32, kPad, true>), grid, block, 0, stream, p, wp, do_write);
            else if (p.block_size == 16)
                hipLaunchKernelGGL((paged_decode_kernel<kU8, kBf16, 1, false, kHD, 16, kPad, true>), grid, block, 0, stream, p, wp, do_write);
            else
                hipLaunchKernelGGL((paged_decode_kernel<kU8, kBf16, 1, false, kHD, 0, kPad, true>), grid, block, 0, stream, p, wp, do_write);
            return;
        }
    }
    if (p.block_size == 32) {
        hipLaunchKernelGGL((paged_decode_kernel<kU8, kBf16, kWaves, kSelfPlan, kHD, 32, kPad>), grid, block, 0, stream, p, wp, do_write);
    } else if (p.block_size == 16) {
        hipLaunchKernelGGL((paged_decode_kernel<kU8, kBf16, kWaves, kSelfPlan, kHD, 16, kPad>), grid, block, 0, stream, p, wp, do_write);
    } else if constexpr (!kSelfPlan) {
        hipLaunchKernelGGL((paged_decode_kernel<kU8, kBf16, kWaves, false, kHD, 0, kPad>), grid, block, 0, stream, p, wp, do_write);
    }
}

template <bool kBf16, bool kPad, bool kU8 = false>
static void launch_decode256_blk(const PagedParams& p, dim3 grid, dim3 block, hipStream_t stream) {
    if (p.block_size == 32)
        hipLaunchKernelGGL((paged_decode256_kernel<kBf16, 32, kPad, kU8>), grid, block, 0, stream, p);
    else if (p.block_size == 16)
        hipLaunchKernelGGL((paged_decode256_kernel<kBf16, 16, kPad, kU8>), grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL((paged_decode256_kernel<kBf16, 0, kPad, kU8>), grid, block, 0, stream, p);
}

template <int kWaves, bool kSelfPlan>
static void launch_decode(const PagedParams& p, const KvWriteParams& wp, int do_write, dim3 grid, dim3 block,
                          hipStream_t stream) {
    const bool bf16 = p.cache_dtype == HIPATTN_BF16, u8 = p.cache_dtype == HIPATTN_U8;
    if (p.head_dim == 128) {
        if (u8)
            launch_decode_blk<true, false, kWaves, kSelfPlan, 128, false>(p, wp, do_write, grid, block, stream);
        else if (bf16)
            launch_decode_blk<false, true, kWaves, kSelfPlan, 128, false>(p, wp, do_write, grid, block, stream);
        else
            launch_decode_blk<false, false, kWaves, kSelfPlan, 128, false>(p, wp, do_write, grid, block, stream);
    } else if constexpr (kWaves == 8) {  // (overlap_wanted: 16-bit caches at head sizes between 64 and 128)
        if (bf16)
            launch_decode_blk<false, true, 8, false, 128, true>(p, wp, do_write, grid, block, stream);
        else
            launch_decode_blk<false, false, 8, false, 128, true>(p, wp, do_write, grid, block, stream);
    } else if constexpr (kWaves == 1 && !kSelfPlan) {
        if (p.head_dim > 128) {
            if (p.head_dim == 256) {
                if (u8) launch_decode256_blk<false, false, true>(p, grid, block, stream);
                else if (bf16) launch_decode256_blk<true, false>(p, grid, block, stream);
                else launch_decode256_blk<false, false>(p, grid, block, stream);
            } else {
                if (u8) launch_decode256_blk<false, true, true>(p, grid, block, stream);
                else if (bf16) launch_decode256_blk<true, true>(p, grid, block, stream);
                else launch_decode256_blk<false, true>(p, grid, block, stream);
            }
        } else if (p.head_dim == 64) {
            if (u8) launch_decode_blk<true, false, 1, false, 64, false>(p, wp, do_write, grid, block, stream);
            else if (bf16) launch_decode_blk<false, true, 1, false, 64, false>(p, wp, do_write, grid, block, stream);
            else launch_decode_blk<false, false, 1, false, 64, false>(p, wp, do_write, grid, block, stream);
        } else if (p.head_dim > 64) {
            if (u8) launch_decode_blk<true, false, 1, false, 128, true>(p, wp, do_write, grid, block, stream);
            else if (bf16) launch_decode_blk<false, true, 1, false, 128, true>(p, wp, do_write, grid, block, stream);
            else launch_decode_blk<false, false, 1, false, 128, true>(p, wp, do_write, grid, block, stream);
        } else {
            if (u8) launch_decode_blk<true, false, 1, false, 64, true>(p, wp, do_write, grid, block, stream);
            else if (bf16) launch_decode_blk<false, true, 1, false, 64, true>(p, wp, do_write, grid, block, stream);
            else launch_decode_blk<false, false, 1, false, 64, true>(p, wp, do_write, grid, block, stream);
        }
    }
}

hipError_t launch_paged_fast(const PagedParams& p, const KvWriteParams* write, hipStream_t stream,
                             const KernelProbe& probe) {
    KvWriteParams wp{};
    int write_blocks = 0;
    if (write) {
        wp = *write;
        if (wp.head_dim > 256) return hipErrorInvalidValue;  // the fast path is head sizes up to 256 only
        write_blocks = (int)((kv_write_wavefronts(wp) + 3) / 4);
    }
    hipError_t e = hipSuccess;
    // A pure decode batch of few rows is one launch less: the decode wavefronts plan for themselves
    // and write the new rows (see kSelfPlanMaxRows).
    const bool self_plan = p.max_q_tiles == 0 && p.num_rows <= kSelfPlanMaxRows && p.dyn_pieces == 0 && p.head_dim == kD &&
                           p.block_size <= 32 && (!write || wp.vector_rows) && !p.alibi_slopes && !half_operands_from_bf16(p);
    if (self_plan) {
        if (probe.before) (void)hipEventRecord(probe.before, stream);
        launch_decode<1, true>(p, wp, write ? 1 : 0, dim3(p.num_waves), dim3(64), stream);
        e = hipGetLastError();
        if (probe.after) (void)hipEventRecord(probe.after, stream);
        if (e != hipSuccess || p.fused_merge) return e;
        hipLaunchKernelGGL(paged_merge_kernel, dim3(p.num_rows * p.num_heads_kv), dim3(256), 0, stream, p);
        return hipGetLastError();
    }
    // prologue: KV-cache write of the new tokens (optional) + plan, one launch
    hipLaunchKernelGGL(paged_prologue_kernel, dim3(write_blocks + 1), dim3(256), 0, stream, wp, p, write_blocks);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    // Shapes without the eight-wavefront decode kernel run the two parts side by side all the same when
    // the decode wavefronts take at most half of every compute unit's registers (and no LDS), so that the
    // chunks' workgroups find room beside them.
    const bool beside = p.max_q_tiles > 0 && !p.overlap && !p.no_side_stream && !p.alibi_slopes && option(kOptMixedOverlap) != 0 &&
                        p.num_waves * 2 <= resident_decode_waves();
    if (p.max_q_tiles > 0 && (p.overlap || beside)) {
        // Mixed batch: the decode sequences stream from HBM on a few compute units while the
        // chunks' flash kernel, on a side stream, has the others; both only need the prologue's
        // results.  The decode kernel stays on the caller's stream, directly behind the prologue,
        // so that it is dispatched first and gets its compute units at once.
        SideStream* side = side_stream(stream);
        if (!side) return hipErrorOutOfMemory;
        std::lock_guard<std::mutex> guard(side->mutex);
        if ((e = hipEventRecord(side->fork, stream)) != hipSuccess) return e;
        if ((e = hipStreamWaitEvent(side->stream, side->fork, 0)) != hipSuccess) return e;
        if (probe.before) (void)hipEventRecord(probe.before, stream);
        if (p.overlap)
            launch_decode<8, false>(p, wp, 0, dim3(p.num_waves / 8), dim3(512), stream);
        else
            launch_decode<1, false>(p, wp, 0, dim3(p.num_waves), dim3(64), stream);
        e = hipGetLastError();
        if (probe.after) (void)hipEventRecord(probe.after, stream);
        const hipError_t e_prefill = launch_paged_prefill(with_cache_heads(p), side->stream);
        if (e == hipSuccess && !p.fused_merge) {
            hipLaunchKernelGGL(paged_merge_kernel, dim3(p.num_rows * p.num_heads_kv), dim3(256), 0, stream, p);
            e = hipGetLastError();
        }
        // always join, also after an error, so the caller's stream never runs ahead of the side stream
        hipError_t e_join = hipEventRecord(side->join, side->stream);
        if (e_join == hipSuccess) e_join = hipStreamWaitEvent(stream, side->join, 0);
        return e != hipSuccess ? e : (e_prefill != hipSuccess ? e_prefill : e_join);
    }
    if (probe.before) (void)hipEventRecord(probe.before, stream);
    launch_decode<1, false>(p, wp, 0, dim3(p.num_waves), dim3(64), stream);
    e = hipGetLastError();
    if (probe.after) (void)hipEventRecord(probe.after, stream);
    if (e != hipSuccess) return e;
    if (!p.fused_merge) {
        hipLaunchKernelGGL(paged_merge_kernel, dim3(p.num_rows * p.num_heads_kv), dim3(256), 0, stream, p);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (p.max_q_tiles > 0) {
        e = launch_paged_prefill(with_cache_heads(p), stream);
    }
    return e;
}

}  // namespace hipattn
