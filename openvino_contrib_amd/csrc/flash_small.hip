// Flash attention on the matrix cores for every 16-bit shape the tuned kernels of flash_prefill.hip
// and paged_decode.hip do not take: head sizes that are multiples of 8 up to 256 (f16 / bf16, causal
// or not, GQA, any attention mask) -- among them head size 64, the shape of the reference's own f16
// test and of the small model families -- dense (v13::ScaledDotProductAttention) and over the block
// table of PagedAttentionExtension (16-bit caches, any power-of-two block size, causal order and
// sliding window of that operator).  The same products and the same register layout as the
// head-size-128 kernel of flash_prefill.hip -- S^T = K Q^T and O^T = V^T P^T on
// v_mfma_f32_32x32x16, the accumulator of the first being the B operand of the second -- in a plain
// structure: four wavefronts per workgroup, 32 query rows each, key tiles of 64 staged through
// registers into a double-buffered, swizzled LDS tile, one workgroup barrier per tile, a
// straightforward online softmax.  Not tuned beyond conflict-free LDS access; it replaces the fp32
// VALU kernels for these shapes.
//
// Replaces the same decomposed chain as flash_prefill.hip (src/ops/matmul.cpp:185-227,
// src/ops/softmax.cpp:178-193, src/ops/select.cpp:50-91 of the reference).
#include <algorithm>

#include "device_common.hpp"
#include "kernels.hpp"

namespace hipattn {

namespace flash_small {

// kDP is the head size the kernel is built for, 64, 128 or 256; the call's head size (w.head_dim, a
// multiple of 8) may be smaller: the missing columns of Q, K and V are zeros in registers and LDS.
// kUsed (head sizes 72..96 in the head-128 build: 96) stops the products at that column: the k-steps and
// output tiles beyond it are not computed.
constexpr int kTileK = 64;                  // keys per tile
constexpr int kWaves = 4;
constexpr int kTileQ = 32 * kWaves;         // query rows per workgroup
template <int kDP>
constexpr int tile_bytes() { return kTileK * kDP * 2; }  // a K or V tile in LDS: rows of kDP / 8 chunks of 16 bytes

template <bool kBf16>
struct Mfma;
template <>
struct Mfma<false> {
    using vec8 = half8_t;
    static __device__ __forceinline__ float16_t mma(vec8 a, vec8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t cvt2(float lo, float hi) {
        typedef float float2_t __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector((float2_t){lo, hi}, half2_t));
    }
    static __device__ __forceinline__ float to_float(uint16_t bits) { return f16_bits_to_float(bits); }
};
template <>
struct Mfma<true> {
    using vec8 = bf16x8_t;
    static __device__ __forceinline__ float16_t mma(vec8 a, vec8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t cvt2(float lo, float hi) {
        typedef float float2_t __attribute__((ext_vector_type(2)));
        typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector((float2_t){lo, hi}, bf16x2_t));
    }
    static __device__ __forceinline__ float to_float(uint16_t bits) { return bf16_bits_to_float(bits); }
};

// both lanes of a pair (l, l + 32) get (value of l, value of l + 32)
__device__ __forceinline__ void pair_values(float x, float& lo, float& hi) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    lo = __uint_as_float(r[0]);
    hi = __uint_as_float(r[1]);
}

// LDS position of the 16-byte chunk c of row r of a tile.  K: sixteen lanes reading one chunk index
// of sixteen consecutive rows (a K fragment) must hit sixteen different 16-byte bank groups: chunk
// c ^ ((r >> 1) & 7) in 128-byte rows, c ^ (r & 15) in 256- and 512-byte rows.  V: the four rows a
// transposing read touches at once must lie in four different quarters of the banks: chunk
// c ^ (4 * ((r >> 1) & 1)) in 128-byte rows, c ^ (4 * (r & 3)) in 256- and 512-byte rows.
template <int kDP>
__device__ __forceinline__ int k_chunk_offset(int r, int c) {
    return kDP == 64 ? r * 128 + ((c ^ ((r >> 1) & 7)) << 4) : r * (kDP * 2) + ((c ^ (r & 15)) << 4);
}
template <int kDP>
__device__ __forceinline__ int v_chunk_offset(int r, int c) {
    return kDP == 64 ? r * 128 + ((c ^ (((r >> 1) & 1) << 2)) << 4) : r * (kDP * 2) + ((c ^ ((r & 3) << 2)) << 4);
}

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef short short8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) uint8_t lds_byte;
typedef __attribute__((address_space(3))) short4_t lds_short4;

// V^T fragment (A operand of O^T = V^T P^T) of k-step ks (16 keys) and head-dim tile dt (32 rows):
// the lane holding head-dim d = dt*32 + n32 gets V[key][d] for keys 16ks + 4hi + {0..3} and
// 16ks + 8 + 4hi + {0..3}: the keys its P^T registers of that k-step belong to.  ds_read_b64_tr_b16
// hands lane i of a 16-lane group element j = what lane 4j + i/4 of the group addressed, at
// 16-bit index i % 4; so lane i addresses row key0 + i/4, head-dim d0 + 4(i % 4).. and receives
// V[key0 + j][d0 + i] (d0 = dt*32 + 16(group & 1), key0 = 16ks + 4(group >> 1)).
template <bool kBf16, int kDP>
__device__ __forceinline__ typename Mfma<kBf16>::vec8 read_v_frag(const lds_byte* v_lds, int lane, int ks, int dt) {
    const int g = lane >> 4, i = lane & 15;
    const int row = 16 * ks + 4 * (g >> 1) + (i >> 2);
    const int d0 = dt * 32 + 16 * (g & 1) + 4 * (i & 3);  // first of this lane's four head-dim elements
    const int c = d0 >> 3, within = (d0 & 7) * 2;
    const lds_byte* p0 = v_lds + v_chunk_offset<kDP>(row, c) + within;
    const lds_byte* p1 = v_lds + v_chunk_offset<kDP>(row + 8, c) + within;
    const short4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)p0);
    const short4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)p1);
    const short8_t a = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
    return __builtin_bit_cast(typename Mfma<kBf16>::vec8, a);
}

// The attention-mask values of one query row for the four consecutive keys key .. key + 3, as
// additions to scores that are exponents to base 2: a floating mask times log2(e), a boolean one 0
// or -inf.  One 4-, 8- or 16-byte load where the keys lie side by side, all four exist and the
// address allows it; element by element otherwise (keys past the end give 0: they are masked anyway).
__device__ __forceinline__ void mask_values4(const uint8_t* row, int64_t key_stride, int dtype, int key, int len_kv, float (&m)[4]) {
    const int esz = dtype == HIPATTN_U8 ? 1 : (dtype == HIPATTN_F32 ? 4 : 2);
    auto value = [&](uint32_t bits) __attribute__((always_inline)) -> float {
        if (dtype == HIPATTN_U8) return bits ? 0.0f : -INFINITY;
        const float x = dtype == HIPATTN_F32 ? __uint_as_float(bits)
                                             : (dtype == HIPATTN_F16 ? f16_bits_to_float((uint16_t)bits) : bf16_bits_to_float((uint16_t)bits));
        return x * kLog2e;
    };
    const uint8_t* at = row + (int64_t)key * key_stride * esz;
    if (key_stride == 1 && key + 3 < len_kv && ((uintptr_t)at & (4 * esz - 1)) == 0) {
        if (esz == 1) {
            const uint32_t w = *(const uint32_t*)at;
#pragma unroll
            for (int e = 0; e < 4; e++) m[e] = value((w >> (8 * e)) & 0xffu);
        } else if (esz == 2) {
            const uint2_t w = *(const uint2_t*)at;
#pragma unroll
            for (int e = 0; e < 4; e++) m[e] = value((w[e >> 1] >> (16 * (e & 1))) & 0xffffu);
        } else {
            const uint4_t w = *(const uint4_t*)at;
#pragma unroll
            for (int e = 0; e < 4; e++) m[e] = value(w[e]);
        }
        return;
    }
#pragma unroll
    for (int e = 0; e < 4; e++) {
        m[e] = 0.0f;
        if (key + e < len_kv) {
            const uint8_t* one = row + (int64_t)(key + e) * key_stride * esz;
            m[e] = value(esz == 1 ? (uint32_t)*one : (esz == 2 ? (uint32_t) * (const uint16_t*)one : *(const uint32_t*)one));
        }
    }
}

// Eight u8 values (words 0, 1) of a cache row with scale and zero-point (words 2, 3) as eight fp16 values.
__device__ __forceinline__ uint4_t dequantised8(uint4_t piece) {
    const float scale = __uint_as_float(piece[2]), bias = -__uint_as_float(piece[3]) * scale;
    uint4_t out;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const uint32_t word = piece[e >> 1] >> (16 * (e & 1));
        out[e] = Mfma<false>::cvt2(fmaf((float)(word & 0xffu), scale, bias), fmaf((float)((word >> 8) & 0xffu), scale, bias));
    }
    return out;
}

// One query tile of one head: what the workgroup reads, where it writes.
struct Work {
    const uint16_t* q;      // row 0 of the tile, this head
    int64_t q_stride;       // elements from one query row to the next
    int q_dtype;            // HIPATTN_F16 / BF16 (converted to the K/V type on load)
    void* out;              // as q
    int64_t out_stride;
    int out_dtype;          // HIPATTN_F16 / BF16 / F32
    int head_dim;           // <= kDP, a multiple of 8
    int rows;               // query rows of the tile that exist (1..128)
    int pos0;               // position of row 0: under `causal` row r attends keys <= pos0 + r * pos_step ...
    int pos_step;           // 1: rows are consecutive tokens; 0: rows are the query heads of one token
    int causal;
    int window;             // ... and, when > 0, keys > that position - window
    int kv_len;
    const uint8_t* k;       // dense: the kv head's rows; paged: the cache at the kv head's offset inside a block
    const uint8_t* v;
    const int32_t* table;   // paged: the sequence's block ids
    int block_shift;        // log2(block size)
    int num_blocks;
    int64_t block_stride;   // bytes from one cache block to the next
    float scale;
    const float* alibi;     // paged: nullptr, or the ALiBi slope of row 0's query head; row r's is alibi[r * alibi_step]
    int alibi_step;         // 0: every row belongs to one head; 1: the rows are consecutive query heads
    const float* sink;      // paged: nullptr, or the attention-sink logit of row 0's query head; row r's is sink[r * alibi_step]
    const uint8_t* mask;    // kMask: the mask row of query row 0 (this batch, this head)
    int64_t mask_row_stride, mask_key_stride;  // in elements
    int mask_dtype;
};

__device__ __forceinline__ uint32_t pack2(int dtype, float lo, float hi) {
    return dtype == HIPATTN_BF16 ? Mfma<true>::cvt2(lo, hi) : Mfma<false>::cvt2(lo, hi);
}

// The workgroup's 128 query rows against the keys they attend.
// kMask: the call carries an attention mask: its values are fetched from global memory ahead of the
// score product of every tile and added behind it.  kPaged: K and V rows are found through w.table.
// kU8 (paged, fp16 products): the cache rows are [scale f32][zero-point f32][head_dim bytes]; a piece
// travels as its eight bytes and the row's scale and zero-point and becomes eight fp16 values
// (byte - zero-point) * scale on its way into LDS.
template <bool kBf16, bool kMask, bool kPaged, int kDP, bool kU8 = false, int kUsed = kDP>
__device__ __forceinline__ void attend(const Work& w, uint8_t (*lds)[2][tile_bytes<kDP>()]) {
    static_assert(!kU8 || (kPaged && !kBf16), "u8 rows exist in paged caches and are multiplied as fp16");
    // kUsed: the columns the products run over (w.head_dim <= kUsed <= kDP, a multiple of 16); the rows in LDS
    // keep the layout of kDP columns
    static_assert(kUsed % 16 == 0 && kUsed <= kDP, "whole k-steps of the score product");
    constexpr int kSteps = kUsed / 16, kOutTiles = (kUsed + 31) / 32;
    using M = Mfma<kBf16>;
    using vec8 = typename M::vec8;
    constexpr int kChunks = kDP / 8;             // 16-byte chunks of a row in LDS
    const int chunks = w.head_dim >> 3;          // ... of which the call's rows fill this many
    const int row_bytes = kU8 ? w.head_dim + 8 : w.head_dim * 2;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int n32 = lane & 31, hi = lane >> 5;
    const int my_row = wave * 32 + n32;          // this lane's query row in the tile (may lie beyond w.rows)
    const int my_pos = w.pos0 + my_row * w.pos_step;
    const bool windowed = kPaged && w.window > 0;

    // key tiles this workgroup visits: up to its last query row under the causal flag, from the
    // first row's window start on
    const int kv_end = w.causal ? min(w.kv_len, w.pos0 + (w.rows - 1) * w.pos_step + 1) : w.kv_len;
    const int tiles = (kv_end + kTileK - 1) / kTileK;
    const int tile0 = windowed ? max(0, w.pos0 - w.window + 1) / kTileK : 0;

    // Q^T fragments (B operand of S^T = K Q^T): lane (n32, hi) holds query row n32, head-dim
    // elements 8 (2i + hi) .. + 7 for k-step i, times scale * log2(e)
    vec8 qf[kSteps];
    {
        const float c = w.scale * kLog2e;
        const int row = min(my_row, w.rows - 1);
        const bool q_bf16 = w.q_dtype == HIPATTN_BF16;
#pragma unroll
        for (int i = 0; i < kSteps; i++) {
            uint4_t raw = {0u, 0u, 0u, 0u};
            if (2 * i + hi < chunks) raw = *(const uint4_t*)(w.q + (int64_t)row * w.q_stride + 8 * (2 * i + hi));
            uint4_t cv;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const uint16_t lo = (uint16_t)(raw[e] & 0xffffu), up = (uint16_t)(raw[e] >> 16);
                cv[e] = q_bf16 ? M::cvt2(bf16_bits_to_float(lo) * c, bf16_bits_to_float(up) * c)
                               : M::cvt2(f16_bits_to_float(lo) * c, f16_bits_to_float(up) * c);
            }
            qf[i] = __builtin_bit_cast(vec8, cv);
        }
    }

    // tile staging: 64 * kChunks 16-byte pieces per K tile and per V tile, kPieces of each per thread
    constexpr int kPieces = kTileK * kChunks / (64 * kWaves);
    // The head-64 build keeps two tiles in flight in registers (kDeep): the loads of tile j + 2 are
    // issued a whole iteration before they are written to LDS; the larger builds have the registers
    // for one.
    constexpr bool kDeep = kDP == 64;
    typedef uint4_t Stage[2 * kPieces];
    Stage stage_a, stage_b;
    // paged: a table entry that names no block of the cache ([0, num_blocks)) stands for keys that take no
    // part.  Their rows are read from a block inside the cache all the same (the loads stay unconditional);
    // which rows of a staged tile they are travels beside the tile: a bit per piece with the registers
    // (bad_a, bad_b), a byte per row with the tile in LDS (row_bad), and the softmax masks those keys.
    uint32_t bad_a = 0, bad_b = 0;
    __shared__ uint8_t row_bad[2][kTileK];
    // paged: the block ids of a tile's rows are looked up one tile ahead of its K/V loads, so that
    // those loads do not wait for the table
    int block_of[kPieces];
    auto lookup = [&](int tile) __attribute__((always_inline)) {
        if constexpr (kPaged) {
#pragma unroll
            for (int s = 0; s < kPieces; s++) {
                const int piece = tid + 64 * kWaves * s, r = piece / kChunks;
                const int key = min(tile * kTileK + r, w.kv_len - 1);
                block_of[s] = w.table[key >> w.block_shift];
            }
        }
    };
    auto fetch = [&](Stage& stage, uint32_t& bad, int tile) __attribute__((always_inline)) {  // (paged: after lookup(tile))
        bad = 0;
#pragma unroll
        for (int s = 0; s < kPieces; s++) {
            const int piece = tid + 64 * kWaves * s, r = piece / kChunks, c = piece % kChunks;
            const int key = min(tile * kTileK + r, w.kv_len - 1);  // rows past the end repeat the last key (masked later)
            int64_t at;
            if constexpr (kPaged) {
                // a block id outside the cache is redirected into it, and its keys are masked
                const int pb = min(max(block_of[s], 0), w.num_blocks - 1);
                if (pb != block_of[s]) bad |= 1u << s;
                at = (int64_t)pb * w.block_stride + (int64_t)(key & ((1 << w.block_shift) - 1)) * row_bytes + (kU8 ? 0 : 16 * c);
            } else {
                at = (int64_t)key * row_bytes + 16 * c;
            }
            stage[s] = stage[kPieces + s] = (uint4_t){0u, 0u, 0u, 0u};
            if (c < chunks) {
                if constexpr (kU8) {
                    const uint2_t kraw = *(const uint2_t*)(w.k + at + 8 + 8 * c), ksz = *(const uint2_t*)(w.k + at);
                    const uint2_t vraw = *(const uint2_t*)(w.v + at + 8 + 8 * c), vsz = *(const uint2_t*)(w.v + at);
                    stage[s] = (uint4_t){kraw[0], kraw[1], ksz[0], ksz[1]};
                    stage[kPieces + s] = (uint4_t){vraw[0], vraw[1], vsz[0], vsz[1]};
                } else {
                    stage[s] = *(const uint4_t*)(w.k + at);
                    stage[kPieces + s] = *(const uint4_t*)(w.v + at);
                }
            }
        }
    };
    auto deposit = [&](const Stage& stage, uint32_t bad, int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < kPieces; s++) {
            const int piece = tid + 64 * kWaves * s, r = piece / kChunks, c = piece % kChunks;
            if constexpr (kPaged) {
                if (c == 0) row_bad[buf][r] = (uint8_t)((bad >> s) & 1u);
            }
            if constexpr (kU8) {
                *(uint4_t*)(lds[buf][0] + k_chunk_offset<kDP>(r, c)) = dequantised8(stage[s]);
                *(uint4_t*)(lds[buf][1] + v_chunk_offset<kDP>(r, c)) = dequantised8(stage[kPieces + s]);
            } else {
                *(uint4_t*)(lds[buf][0] + k_chunk_offset<kDP>(r, c)) = stage[s];
                *(uint4_t*)(lds[buf][1] + v_chunk_offset<kDP>(r, c)) = stage[kPieces + s];
            }
        }
    };

    float16_t o[kOutTiles];
#pragma unroll
    for (int dt = 0; dt < kOutTiles; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[dt][r] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;  // the row's running maximum (both lanes of a pair agree) and this lane's share of the sum

    if (tile0 < tiles) {
        lookup(tile0);
        fetch(stage_a, bad_a, tile0);
        if (tile0 + 1 < tiles) lookup(tile0 + 1);
        deposit(stage_a, bad_a, 0);
        if constexpr (kDeep) {
            if (tile0 + 1 < tiles) {
                fetch(stage_a, bad_a, tile0 + 1);
                if (tile0 + 2 < tiles) lookup(tile0 + 2);
            }
        }
    }
    __syncthreads();
    // One key tile.  kDeep: `next` holds tile j + 1, on its way since the previous iteration, and
    // `ahead` takes the loads of tile j + 2; otherwise `next` takes the loads of tile j + 1 now.
    auto iteration = [&](int j, Stage& next, uint32_t& next_bad, Stage& ahead, uint32_t& ahead_bad) __attribute__((always_inline)) {
        const int buf = (j - tile0) & 1;
        if constexpr (kDeep) {
            if (j + 2 < tiles) {
                fetch(ahead, ahead_bad, j + 2);
                if (j + 3 < tiles) lookup(j + 3);
            }
        } else {
            if (j + 1 < tiles) {
                fetch(next, next_bad, j + 1);  // in flight while this tile is computed
                if (j + 2 < tiles) lookup(j + 2);
            }
        }
        // keys of this tile whose block the table does not name, one bit per key (wave-uniform)
        uint64_t bad_keys = 0;
        if constexpr (kPaged) bad_keys = __builtin_amdgcn_ballot_w64(row_bad[buf][lane] != 0);
        const lds_byte* k_lds = (const lds_byte*)lds[buf][0];
        const lds_byte* v_lds = (const lds_byte*)lds[buf][1];
        const int ts = j * kTileK;

        // the mask values of the wavefront's rows for the 32 keys of half mt of the tile
        auto mask_half = [&](int mt) __attribute__((always_inline)) -> float16_t {
            float16_t add;
            const int row = min(my_row, w.rows - 1);
            const int esz = w.mask_dtype == HIPATTN_U8 ? 1 : (w.mask_dtype == HIPATTN_F32 ? 4 : 2);
            const uint8_t* mrow = w.mask + (int64_t)row * w.mask_row_stride * esz;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                float m4[4];
                mask_values4(mrow, w.mask_key_stride, w.mask_dtype, ts + mt * 32 + 8 * g + 4 * hi, w.kv_len, m4);
#pragma unroll
                for (int e = 0; e < 4; e++) add[4 * g + e] = m4[e];
            }
            return add;
        };
        // (the head-256 build has no registers to hold them across the score product: it fetches them behind it)
        constexpr bool kMaskAhead = kMask && kDP < 256;
        float16_t mask_add[2];
        if constexpr (kMaskAhead) {
#pragma unroll
            for (int mt = 0; mt < 2; mt++) mask_add[mt] = mask_half(mt);
        }
        // scores, transposed: register r of s[mt] is key ts + 32 mt + 8 (r / 4) + 4 hi + r % 4 of query row n32
        float16_t s[2];
#pragma unroll
        for (int mt = 0; mt < 2; mt++) {
#pragma unroll
            for (int r = 0; r < 16; r++) s[mt][r] = 0.0f;
#pragma unroll
            for (int i = 0; i < kSteps; i++) {
                const int row = mt * 32 + n32;
                const vec8 kf = __builtin_bit_cast(vec8, *(const __attribute__((address_space(3))) uint4_t*)(k_lds + k_chunk_offset<kDP>(row, 2 * i + hi)));
                s[mt] = M::mma(kf, qf[i], s[mt]);
            }
        }
        if constexpr (kMaskAhead) {
#pragma unroll
            for (int mt = 0; mt < 2; mt++) s[mt] += mask_add[mt];
        } else if constexpr (kMask) {
            const int row = min(my_row, w.rows - 1);
            const int esz = w.mask_dtype == HIPATTN_U8 ? 1 : (w.mask_dtype == HIPATTN_F32 ? 4 : 2);
            const uint8_t* mrow = w.mask + (int64_t)row * w.mask_row_stride * esz;
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    float m4[4];
                    mask_values4(mrow, w.mask_key_stride, w.mask_dtype, ts + mt * 32 + 8 * g + 4 * hi, w.kv_len, m4);
#pragma unroll
                    for (int e = 0; e < 4; e++) s[mt][4 * g + e] += m4[e];
                }
        }
        // ALiBi: slope * (key - query position) joins the score (an exponent to base 2 here).  The slope is
        // fetched where it is used: held across the loop it would cost the larger builds a spilled register.
        if constexpr (kPaged) {
            if (w.alibi != nullptr) {
                const float slope = *(const volatile float*)(w.alibi + min(my_row, w.rows - 1) * w.alibi_step) * kLog2e;
#pragma unroll
                for (int mt = 0; mt < 2; mt++)
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int key = ts + mt * 32 + 8 * (r >> 2) + 4 * hi + (r & 3);
                        s[mt][r] = fmaf(slope, (float)(key - my_pos), s[mt][r]);
                    }
            }
        }
        // mask: keys past the end, keys after the query under the causal flag, keys that have left
        // the window (the tile holds one for some row of the wavefront when its first key lies
        // before the window of the wavefront's last row)
        const int wave_pos = w.pos0 + wave * 32 * w.pos_step;
        const bool edge = ts + kTileK > w.kv_len || (w.causal && ts + kTileK - 1 > wave_pos) ||
                          (windowed && ts <= wave_pos + 31 * w.pos_step - w.window) || bad_keys != 0;
        if (edge) {
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int in_tile = mt * 32 + 8 * (r >> 2) + 4 * hi + (r & 3), key = ts + in_tile;
                    const bool ok = key < w.kv_len && (!w.causal || key <= my_pos) && (!windowed || key > my_pos - w.window) &&
                                    ((bad_keys >> in_tile) & 1u) == 0;
                    s[mt][r] = ok ? s[mt][r] : -INFINITY;
                }
        }
        // online softmax in the exp2 domain; the row lives in lanes l and l + 32
        float m_tile = -INFINITY;
#pragma unroll
        for (int mt = 0; mt < 2; mt++)
#pragma unroll
            for (int r = 0; r < 16; r++) m_tile = fmaxf(m_tile, s[mt][r]);
        float m_lo, m_hi;
        pair_values(m_tile, m_lo, m_hi);
        const float m_new = fmaxf(m_run, fmaxf(m_lo, m_hi));
        // a row that has met no key yet keeps everything at zero (exp2(-inf - -inf) would be NaN)
        const float m_use = m_new == -INFINITY ? 0.0f : m_new;
        const float alpha = fast_exp2(m_run - m_use);
        vec8 pf[4];
        float sum = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            uint4_t pw;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float p0 = fast_exp2(s[ks >> 1][(ks & 1) * 8 + 2 * e] - m_use);
                const float p1 = fast_exp2(s[ks >> 1][(ks & 1) * 8 + 2 * e + 1] - m_use);
                pw[e] = M::cvt2(p0, p1);
                sum += p0 + p1;
            }
            pf[ks] = __builtin_bit_cast(vec8, pw);
        }
        l_run = l_run * alpha + sum;
        m_run = m_new;
#pragma unroll
        for (int dt = 0; dt < kOutTiles; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[dt][r] *= alpha;
        // O^T += V^T P^T
#pragma unroll
        for (int ks = 0; ks < 4; ks++)
#pragma unroll
            for (int dt = 0; dt < kOutTiles; dt++) o[dt] = M::mma(read_v_frag<kBf16, kDP>(v_lds, lane, ks, dt), pf[ks], o[dt]);

        if (j + 1 < tiles) deposit(next, next_bad, buf ^ 1);  // the other buffer was last read before the previous barrier
        __syncthreads();
    };
    for (int j = tile0; j < tiles; j += 2) {
        iteration(j, stage_a, bad_a, stage_b, bad_b);
        if (j + 1 < tiles) iteration(j + 1, kDeep ? stage_b : stage_a, kDeep ? bad_b : bad_a, kDeep ? stage_a : stage_b, kDeep ? bad_a : bad_b);
    }

    // normalise and store: register r of o[dt] is head-dim 32 dt + 8 (r / 4) + 4 hi + r % 4 of query row n32
    float l_lo, l_hi;
    pair_values(l_run, l_lo, l_hi);
    float l = l_lo + l_hi;
    if constexpr (kPaged) {  // the attention sink of the row's head: a logit in the denominator without a value row
        if (w.sink != nullptr && l > 0.0f) l += fast_exp2(w.sink[min(my_row, w.rows - 1) * w.alibi_step] * kLog2e - m_run);
    }
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    if (my_row < w.rows) {
#pragma unroll
        for (int dt = 0; dt < kOutTiles; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d = dt * 32 + 8 * g + 4 * hi;
                if (d >= w.head_dim) continue;
                const float x0 = o[dt][4 * g] * inv, x1 = o[dt][4 * g + 1] * inv, x2 = o[dt][4 * g + 2] * inv, x3 = o[dt][4 * g + 3] * inv;
                if (kPaged && w.out_dtype == HIPATTN_F32) {
                    *(float4*)((float*)w.out + (int64_t)my_row * w.out_stride + d) = make_float4(x0, x1, x2, x3);
                } else {
                    uint2_t pk;
                    pk[0] = pack2(w.out_dtype, x0, x1);
                    pk[1] = pack2(w.out_dtype, x2, x3);
                    *(uint2_t*)((uint16_t*)w.out + (int64_t)my_row * w.out_stride + d) = pk;
                }
            }
    }
}

// Dense SDPA: one workgroup per (batch, query head, 128-row query tile).  kMask: p.mask rides along
// (ignored under the causal flag).
template <bool kBf16, bool kMask, int kDP, int kUsed>
__device__ __forceinline__ void sdpa_small_tile(const SdpaParams& p, uint8_t (*lds)[2][tile_bytes<kDP>()]) {
    const int q_tiles = (p.len_q + kTileQ - 1) / kTileQ;
    const int qt = blockIdx.x % q_tiles;
    const int h = (blockIdx.x / q_tiles) % p.num_heads_q;
    const int b = blockIdx.x / (q_tiles * p.num_heads_q);
    const int hkv = h / (p.num_heads_q / p.num_heads_kv);
    const int q0 = qt * kTileQ;
    const int D = p.head_dim;
    Work w;
    w.q = (const uint16_t*)p.q + ((int64_t)(b * p.num_heads_q + h) * p.len_q + q0) * D;
    w.q_stride = D;
    w.q_dtype = p.dtype;
    w.out = (uint16_t*)p.out + ((int64_t)(b * p.num_heads_q + h) * p.len_q + q0) * D;
    w.out_stride = D;
    w.out_dtype = p.dtype;
    w.head_dim = D;
    w.rows = min(kTileQ, p.len_q - q0);
    w.pos0 = q0;
    w.pos_step = 1;
    w.causal = p.causal;
    w.window = 0;
    w.kv_len = p.len_kv;
    w.k = (const uint8_t*)p.k + ((int64_t)(b * p.num_heads_kv + hkv) * p.len_kv) * D * 2;
    w.v = (const uint8_t*)p.v + ((int64_t)(b * p.num_heads_kv + hkv) * p.len_kv) * D * 2;
    w.table = nullptr;
    w.block_shift = 0;
    w.num_blocks = 0;
    w.block_stride = 0;
    w.scale = p.scale;
    w.alibi = nullptr;
    w.alibi_step = 0;
    w.sink = nullptr;
    w.mask = nullptr;
    w.mask_row_stride = w.mask_key_stride = 0;
    w.mask_dtype = 0;
    if constexpr (kMask) {
        const int esz = p.mask_dtype == HIPATTN_U8 ? 1 : (p.mask_dtype == HIPATTN_F32 ? 4 : 2);
        w.mask = (const uint8_t*)p.mask +
                 ((int64_t)b * p.mask_stride[0] + (int64_t)h * p.mask_stride[1] + (int64_t)q0 * p.mask_stride[2]) * esz;
        w.mask_row_stride = p.mask_stride[2];
        w.mask_key_stride = p.mask_stride[3];
        w.mask_dtype = p.mask_dtype;
    }
    attend<kBf16, kMask, false, kDP, false, kUsed>(w, lds);
}

// (two workgroups per compute unit also in the head-128 build: at most 256 registers; the head-256
// build needs nearly all 512 and runs one)
template <bool kBf16, int kDP, int kUsed = kDP>
__global__ __launch_bounds__(64 * kWaves) __attribute__((amdgpu_waves_per_eu(2))) void sdpa_flash_small_kernel(SdpaParams p) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[2][2][tile_bytes<kDP>()];  // [buffer][K, V]
    sdpa_small_tile<kBf16, false, kDP, kUsed>(p, lds);
}

// (the mask values of a tile take 32 more registers: no bound on them)
template <bool kBf16, int kDP, int kUsed = kDP>
__global__ __launch_bounds__(64 * kWaves) void sdpa_flash_small_masked_kernel(SdpaParams p) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[2][2][tile_bytes<kDP>()];
    sdpa_small_tile<kBf16, true, kDP, kUsed>(p, lds);
}

// Query tiles of a PagedAttentionExtension batch over the block table (16-bit caches): a sequence
// of n > 1 tokens has ceil(n / 128) tiles per query head; with p.tiles_only a single-token sequence
// has one tile per kv head whose rows are the query heads of the group (without it such sequences
// belong to the decode kernel and have no tile).  The tiles of the batch are numbered by
// p.tile_prefix (written on the device by the plan of the decode path or by paged_tiles_plan_kernel),
// the later -- heavier -- tiles of a sequence first.  One workgroup per (tile, head); the grid is
// an upper bound.
template <bool kBf16, int kDP, bool kU8 = false, int kUsed = kDP>
__global__ __launch_bounds__(64 * kWaves) __attribute__((amdgpu_waves_per_eu(2))) void paged_tiles_kernel(PagedParams p) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[2][2][tile_bytes<kDP>()];
    const int item = blockIdx.x / p.num_heads_q, h = blockIdx.x % p.num_heads_q;
    if (item >= p.tile_prefix[p.num_seqs]) return;
    int lo = 0, hi_s = p.num_seqs;  // the sequence owning the tile: largest s with tile_prefix[s] <= item
    while (hi_s - lo > 1) {
        const int mid = (lo + hi_s) >> 1;
        if (p.tile_prefix[mid] <= item)
            lo = mid;
        else
            hi_s = mid;
    }
    const int s = lo;
    const int tiles_s = p.tile_prefix[s + 1] - p.tile_prefix[s];
    const int qt = tiles_s - 1 - (item - p.tile_prefix[s]);
    const int t0 = p.subsequence_begins[s];
    const int qlen = p.subsequence_begins[s + 1] - t0;
    const int past = p.past_lens[s];
    const int tb0 = p.block_indices_begins[s];
    const int table_len = p.block_indices_begins[s + 1] - tb0;
    const int G = p.num_heads_q / p.num_heads_kv, D = p.head_dim;
    const bool heads_as_rows = qlen == 1;  // (only tiles_only gives such a sequence a tile)
    if (heads_as_rows && h >= p.num_heads_kv) return;
    const int hkv = heads_as_rows ? h : h / G;
    const int64_t row0 = heads_as_rows ? (int64_t)t0 * p.num_heads_q + (int64_t)h * G
                                       : (int64_t)(t0 + qt * kTileQ) * p.num_heads_q + h;
    Work w;
    w.q = (const uint16_t*)p.q + row0 * D;
    w.q_stride = heads_as_rows ? D : (int64_t)p.num_heads_q * D;
    w.q_dtype = p.q_dtype;
    w.out = p.out_dtype == HIPATTN_F32 ? (void*)((float*)p.out + row0 * D) : (void*)((uint16_t*)p.out + row0 * D);
    w.out_stride = w.q_stride;
    w.out_dtype = p.out_dtype;
    w.head_dim = D;
    w.rows = heads_as_rows ? G : min(kTileQ, qlen - qt * kTileQ);
    w.pos0 = past + qt * kTileQ;
    w.pos_step = heads_as_rows ? 0 : 1;
    w.causal = 1;
    w.window = p.sliding_window;
    w.kv_len = min(past + qlen, table_len * p.block_size);
    const int row_bytes = kU8 ? D + 8 : D * 2;
    const int64_t head_off = (int64_t)hkv * p.block_size * row_bytes;
    w.k = p.key_cache + head_off;
    w.v = p.value_cache + head_off;
    w.table = p.block_indices + tb0;
    w.block_shift = __builtin_ctz(p.block_size);
    w.num_blocks = p.num_blocks;
    w.block_stride = (int64_t)p.num_heads_kv * p.block_size * row_bytes;
    w.scale = p.scale;
    w.alibi = p.alibi_slopes ? p.alibi_slopes + (heads_as_rows ? h * G : h) : nullptr;
    w.alibi_step = heads_as_rows ? 1 : 0;
    w.sink = p.sinks ? p.sinks + (heads_as_rows ? h * G : h) : nullptr;
    w.mask = nullptr;
    w.mask_row_stride = w.mask_key_stride = 0;
    w.mask_dtype = 0;
    attend<kBf16, false, true, kDP, kU8, kUsed>(w, lds);
}

// tile_prefix for a batch in which every sequence with tokens goes through paged_tiles_kernel
// (p.tiles_only): exclusive prefix sums of ceil(tokens / 128) over the sequences.  One workgroup.
__global__ __launch_bounds__(256) void paged_tiles_plan_kernel(PagedParams p) {
    __shared__ int wave_total[4];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int per = (p.num_seqs + 255) / 256;
    const int s0 = min(tid * per, p.num_seqs), s1 = min(s0 + per, p.num_seqs);
    int mine = 0;
    for (int s = s0; s < s1; s++) mine += (max(p.subsequence_begins[s + 1] - p.subsequence_begins[s], 0) + kTileQ - 1) / kTileQ;
    int scan = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(scan, d, 64);
        if (lane >= d) scan += up;
    }
    if (lane == 63) wave_total[wv] = scan;
    __syncthreads();
    int tile = scan - mine;
    for (int w = 0; w < wv; w++) tile += wave_total[w];
    for (int s = s0; s < s1; s++) {
        p.tile_prefix[s] = tile;
        tile += (max(p.subsequence_begins[s + 1] - p.subsequence_begins[s], 0) + kTileQ - 1) / kTileQ;
    }
    if (s1 == p.num_seqs && s0 < p.num_seqs) p.tile_prefix[p.num_seqs] = tile;
}

}  // namespace flash_small

static bool aligned16(const void* q) { return ((uintptr_t)q & 15) == 0; }

// 16-bit operands, head sizes that are multiples of 8 up to 256.
bool sdpa_flash_small_supported(const SdpaParams& p) {
    return p.head_dim >= 8 && p.head_dim <= 256 && p.head_dim % 8 == 0 && (p.dtype == HIPATTN_F16 || p.dtype == HIPATTN_BF16) &&
           p.len_kv > 0 && p.len_q > 0 && aligned16(p.q) && aligned16(p.k) && aligned16(p.v) && ((uintptr_t)p.out % 8) == 0;
}

template <bool kMask, int kDP, int kUsed = kDP>
static void launch_sdpa_small(const SdpaParams& p, unsigned groups, hipStream_t stream) {
    const dim3 grid(groups), block(64 * flash_small::kWaves);
    const bool bf16 = p.dtype == HIPATTN_BF16;
    if constexpr (kMask) {
        if (bf16)
            hipLaunchKernelGGL((flash_small::sdpa_flash_small_masked_kernel<true, kDP, kUsed>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((flash_small::sdpa_flash_small_masked_kernel<false, kDP, kUsed>), grid, block, 0, stream, p);
    } else {
        if (bf16)
            hipLaunchKernelGGL((flash_small::sdpa_flash_small_kernel<true, kDP, kUsed>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((flash_small::sdpa_flash_small_kernel<false, kDP, kUsed>), grid, block, 0, stream, p);
    }
}

template <bool kMask>
static void launch_sdpa_small(const SdpaParams& p, unsigned groups, hipStream_t stream) {
    if (p.head_dim <= 64)
        launch_sdpa_small<kMask, 64>(p, groups, stream);
    else if (p.head_dim <= 96)  // (the head-128 build without its last two k-steps and its last output tile)
        launch_sdpa_small<kMask, 128, 96>(p, groups, stream);
    else if (p.head_dim <= 128)
        launch_sdpa_small<kMask, 128>(p, groups, stream);
    else
        launch_sdpa_small<kMask, 256>(p, groups, stream);
}

hipError_t launch_sdpa_flash_small(const SdpaParams& p, hipStream_t stream, const KernelProbe& probe) {
    const int64_t q_tiles = (p.len_q + flash_small::kTileQ - 1) / flash_small::kTileQ;
    const int64_t groups = q_tiles * p.num_heads_q * p.batch;
    if (groups == 0) return hipSuccess;
    if (groups > 0x7fffffffLL) return hipErrorInvalidValue;
    if (probe.before) (void)hipEventRecord(probe.before, stream);
    if (p.mask != nullptr && !p.causal)
        launch_sdpa_small<true>(p, (unsigned)groups, stream);
    else
        launch_sdpa_small<false>(p, (unsigned)groups, stream);
    const hipError_t e = hipGetLastError();
    if (probe.after) (void)hipEventRecord(probe.after, stream);
    return e;
}

static void launch_tiles(const PagedParams& p, unsigned groups, hipStream_t stream) {
    const dim3 grid(groups), block(64 * flash_small::kWaves);
    const bool bf16 = p.cache_dtype == HIPATTN_BF16;
    if (p.cache_dtype == HIPATTN_U8) {
        if (p.head_dim <= 64)
            hipLaunchKernelGGL((flash_small::paged_tiles_kernel<false, 64, true>), grid, block, 0, stream, p);
        else if (p.head_dim <= 96)
            hipLaunchKernelGGL((flash_small::paged_tiles_kernel<false, 128, true, 96>), grid, block, 0, stream, p);
        else if (p.head_dim <= 128)
            hipLaunchKernelGGL((flash_small::paged_tiles_kernel<false, 128, true>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((flash_small::paged_tiles_kernel<false, 256, true>), grid, block, 0, stream, p);
    } else if (p.head_dim <= 64) {
        if (bf16)
            hipLaunchKernelGGL((flash_small::paged_tiles_kernel<true, 64>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((flash_small::paged_tiles_kernel<false, 64>), grid, block, 0, stream, p);
    } else if (p.head_dim > 128) {
        if (bf16)
            hipLaunchKernelGGL((flash_small::paged_tiles_kernel<true, 256>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((flash_small::paged_tiles_kernel<false, 256>), grid, block, 0, stream, p);
    } else if (p.head_dim <= 96) {
        if (bf16)
            hipLaunchKernelGGL((flash_small::paged_tiles_kernel<true, 128, false, 96>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((flash_small::paged_tiles_kernel<false, 128, false, 96>), grid, block, 0, stream, p);
    } else {
        if (bf16)
            hipLaunchKernelGGL((flash_small::paged_tiles_kernel<true, 128>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((flash_small::paged_tiles_kernel<false, 128>), grid, block, 0, stream, p);
    }
}

// The multi-token sequences of a batch planned by the decode path (p.tile_prefix, p.max_q_tiles), head size 64.
hipError_t launch_paged_prefill_small(const PagedParams& p, hipStream_t stream) {
    const int64_t groups = (int64_t)p.max_q_tiles * p.num_heads_q;
    if (groups == 0) return hipSuccess;
    if (groups > 0x7fffffffLL) return hipErrorInvalidValue;
    launch_tiles(p, (unsigned)groups, stream);
    return hipGetLastError();
}

// Whole batches through the tile kernel: 16-bit queries on 16-bit or u8 caches whose shape the decode path
// does not take -- head sizes that are multiples of 8 up to 256, block sizes that are powers of
// two, up to 128 query heads per kv head.
bool paged_tiles_supported(const PagedParams& p) {
    const int G = p.num_heads_q / p.num_heads_kv;
    return p.head_dim >= 8 && p.head_dim <= 256 && p.head_dim % 8 == 0 && G <= flash_small::kTileQ &&
           p.block_size > 0 && (p.block_size & (p.block_size - 1)) == 0 &&
           (p.q_dtype == HIPATTN_F16 || p.q_dtype == HIPATTN_BF16) &&
           (p.cache_dtype == HIPATTN_F16 || p.cache_dtype == HIPATTN_BF16 || p.cache_dtype == HIPATTN_U8) && aligned16(p.q) && aligned16(p.key_cache) &&
           aligned16(p.value_cache) && ((uintptr_t)p.out % (p.out_dtype == HIPATTN_F32 ? 16 : 8)) == 0;
}

static int64_t tiles_bound(const PagedParams& p) {  // every sequence with tokens wastes at most one tile
    return (int64_t)p.num_tokens / flash_small::kTileQ + std::min(p.num_seqs, p.num_tokens);
}

size_t paged_tiles_workspace_bytes(const PagedParams& p) { return ((size_t)p.num_seqs + 1) * sizeof(int32_t); }

// (the new tokens are in the cache already)
hipError_t launch_paged_tiles(const PagedParams& p_in, void* workspace, hipStream_t stream, const KernelProbe& probe) {
    PagedParams p = p_in;
    p.tile_prefix = (int32_t*)workspace;
    p.tiles_only = 1;
    const int64_t groups = tiles_bound(p) * p.num_heads_q;
    if (groups == 0) return hipSuccess;
    if (groups > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(flash_small::paged_tiles_plan_kernel, dim3(1), dim3(256), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (probe.before) (void)hipEventRecord(probe.before, stream);
    launch_tiles(p, (unsigned)groups, stream);
    e = hipGetLastError();
    if (probe.after) (void)hipEventRecord(probe.after, stream);
    return e;
}

}  // namespace hipattn
