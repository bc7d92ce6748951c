// Flash-style attention for prefill on gfx950: dense v13::ScaledDotProductAttention and the
// multi-token (chunked prefill) sequences of PagedAttentionExtension share one kernel body.
//
// A workgroup has eight wavefronts in two groups of four.  Each group owns 128 query rows (32
// per wavefront) of one query head; the two groups work on two heads of the same K/V head (or on
// two consecutive query tiles of one head), so they share every K and V tile.  Keys are walked
// in tiles of 64.  K and V tiles go from global memory straight into LDS
// (global_load_lds_dwordx4: no staging registers, no LDS write instructions), row-major with
// the 16-byte chunks of a row XOR-swizzled so that fragment reads are free of bank conflicts;
// the V^T operand is read with the transposing LDS load ds_read_b64_tr_b16.  LDS holds a ring of
// three K and three V stages, filled two tiles ahead, and 8 KB per wavefront through which its
// query rows come in and its output rows go out as whole rows (160 KB in all: one workgroup per
// compute unit).
//
// One wavefront of each group sits on every SIMD, and the two alternate between a matrix phase
// (O += P V of one tile, then the scores of the next) and a vector phase (mask, running
// reference, exp2, conversion and row sums of the scores just computed, plus the issue of the
// global->LDS loads), separated by workgroup barriers: while one group feeds the matrix core the
// other keeps the vector ALU busy, by construction rather than by chance.  (A variant in which
// every wavefront interleaves the exponentials of one tile with its own score MFMAs of the next
// needs about 5 % fewer cycles and takes the same time: with real data the kernel runs at the
// machine's power limit, and the clock settles lower for the denser instruction stream.)
//
// Both products run on v_mfma_f32_32x32x16 (f16 or bf16) with fp32 accumulation:
//   S^T = K Q^T   (M = 32 keys, N = 32 query rows, contraction over head_dim)
//   O^T = V^T P^T (M = 32 head-dim rows, N = 32 query rows, contraction over keys)
// Computing the scores transposed leaves each lane with 8 consecutive-in-operand keys of one
// query row, i.e. the accumulator of the first product already is the B operand of the
// second; the softmax statistics of a row live in the two lanes l and l+32 and need a single
// cross-lane exchange.  Scale, causal mask, sliding window and the online softmax (exp2
// domain) are fused; fully masked key tiles are never visited.
//
// Replaces the reference's decomposed chain, which writes and re-reads the [B,H,Lq,Lk] score
// tensor four times: MatMulOp::Execute (src/ops/matmul.cpp:185-227), Multiply
// (src/ops/multiply.cpp:43), Select/Add mask (src/ops/select.cpp:50-91, src/ops/add.cpp:17-43),
// SoftmaxOp::Execute (src/ops/softmax.cpp:178-193), TransposeOp (src/ops/transpose.cpp:87-135)
// and ConvertOp (src/ops/convert.cpp:60).
#include "device_common.hpp"
#include "kernels.hpp"

namespace hipattn {

namespace flash {

constexpr int kD = 128;
constexpr int kTileQ = 128;   // query rows per group of four wavefronts
constexpr int kTileK = 64;    // keys per LDS tile
constexpr int kThreads = 512;
constexpr int kStages = 3;    // ring of K stages and ring of V stages
constexpr int kRowBytes = kD * 2;                // a K or V row in LDS: 16 chunks of 16 bytes
constexpr int kKBytes = kTileK * kRowBytes;      // one K or V stage
constexpr int kRingBytes = 2 * kStages * kKBytes;
constexpr int kWaveStageBytes = 32 * kRowBytes;  // a wavefront's 32 query rows (in) or output rows (out), 16-bit
constexpr int kLdsBytes = kRingBytes + 8 * kWaveStageBytes;

// global -> LDS load of 16 bytes per lane: lane l's data lands at LDS byte lds_base + 16 l
// (lds_base wave-uniform, carried in M0).  Issued as inline assembly on purpose: the compiler
// treats the intrinsic form as a flat access that may touch LDS and from then on waits for all
// outstanding LDS reads and loads at every use (s_waitcnt 0), which serialises the fragment
// prefetch.  The waiting these loads need is done by hand (barrier_keeping_loads).
typedef __attribute__((address_space(3))) uint8_t lds_byte;
__device__ __forceinline__ void load_to_lds_16(const uint8_t* global_base, uint32_t lane_offset, lds_byte* lds_base) {
    // global_base wave-uniform, lane_offset per lane
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(lane_offset), "s"(global_base), "s"((uint32_t)(uintptr_t)lds_base)
                 : "memory", "m0");
}
__device__ __forceinline__ void load_to_lds_16(const uint8_t* lane_address, lds_byte* lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(lane_address), "s"((uint32_t)(uintptr_t)lds_base)
                 : "memory", "m0");
}

template <bool kBf16>
struct Mfma;
template <>
struct Mfma<false> {
    using vec8 = half8_t;
    static __device__ __forceinline__ float16_t mma(vec8 a, vec8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint16_t cvt(float x) { return float_to_f16_bits(x); }
    static __device__ __forceinline__ uint32_t cvt2(float lo, float hi) {
        typedef float float2_t __attribute__((ext_vector_type(2)));
        const half2_t h = __builtin_convertvector((float2_t){lo, hi}, half2_t);
        return __builtin_bit_cast(uint32_t, h);
    }
};
template <>
struct Mfma<true> {
    using vec8 = bf16x8_t;
    static __device__ __forceinline__ float16_t mma(vec8 a, vec8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint16_t cvt(float x) {
        __bf16 b = (__bf16)x;
        return __builtin_bit_cast(uint16_t, b);
    }
    static __device__ __forceinline__ uint32_t cvt2(float lo, float hi) {
        typedef float float2_t __attribute__((ext_vector_type(2)));
        typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
        const bf16x2_t h = __builtin_convertvector((float2_t){lo, hi}, bf16x2_t);
        return __builtin_bit_cast(uint32_t, h);
    }
};

// What one group of four wavefronts works on.
struct Tile {
    const uint16_t* q;   // first query row of the tile, this head
    int64_t q_stride;    // elements between consecutive query rows
    void* out;           // output base (element (0,0) of the tile's first row, this head)
    int64_t out_stride;
    int rows;            // valid query rows (<= 128); 0: this group has nothing to do
    int pos0;            // sequence position of query row 0
    int kv_len;          // keys available
    int causal;
    int window;
    int q_dtype;         // HIPATTN_F16 / HIPATTN_BF16 (converted to the MFMA type when they differ)
    int out_dtype;
    int head_dim;        // columns of a row in memory: kD, or fewer in the kPad form of the dense kernel
    // keys / values: the same for both groups of a workgroup
    const uint8_t* k;
    const uint8_t* v;
    const int32_t* table;   // paged: this sequence's block ids; dense: nullptr
    int table_len;
    int num_blocks;
    int64_t block_stride;   // paged: bytes between physical blocks
    int block_size;
    int block_shift;        // log2(block_size)
    // dense SDPA with an attention mask (kMask variants of the kernel): the mask element of the
    // tile's query row 0 and key 0 for this batch and head; rows mask_row_bytes apart (0: one row
    // for every query), keys side by side
    const uint8_t* mask;
    int64_t mask_row_bytes;
};

// u8 caches: rows of 8 bytes (float scale, float zero-point) + 128 payload bytes.  The u8 variant
// of the kernel loads them into registers, dequantises to fp16 and writes the result into the
// same LDS stages (same layout) the 16-bit caches are loaded into directly; everything behind
// that is the fp16 kernel.
constexpr int kU8RowBytes = kD + 8;
struct U8Rows {
    uint2_t k_lo, k_hi, v_lo, v_hi;  // this lane's 16 payload bytes of a K row and of a V row
    float2 k_sz, v_sz;               // the rows' (scale, zero-point)
    int jk, jv;                      // tiles they belong to (-1: none)
};
// two bytes of a word (selected by `sel`) as fp16 numbers 1024 + byte
__device__ __forceinline__ half2_t biased_half2(uint32_t w, uint32_t sel) {
    return __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, w, sel));
}
// 8 payload bytes -> 8 dequantised fp16 values: (byte - zp) * scale, as (byte) * scale + off in
// packed fp16 (1024 + byte is exact in fp16, and so is the subtraction of 1024)
__device__ __forceinline__ uint4_t dequant8(uint2_t w, half2_t scale, half2_t off) {
    const half2_t bias = {(half_t)1024.0f, (half_t)1024.0f};
    uint4_t r;
    r[0] = __builtin_bit_cast(uint32_t, (biased_half2(w[0], 0x04010400u) - bias) * scale + off);
    r[1] = __builtin_bit_cast(uint32_t, (biased_half2(w[0], 0x04030402u) - bias) * scale + off);
    r[2] = __builtin_bit_cast(uint32_t, (biased_half2(w[1], 0x04010400u) - bias) * scale + off);
    r[3] = __builtin_bit_cast(uint32_t, (biased_half2(w[1], 0x04030402u) - bias) * scale + off);
    return r;
}

// Keys [lo, hi) a tile has to visit, lo rounded down to a tile boundary.
__device__ __forceinline__ void key_range(const Tile& t, int& lo, int& hi) {
    if (t.rows <= 0) {
        lo = hi = 0;
        return;
    }
    hi = t.kv_len;
    if (t.causal) hi = min(hi, t.pos0 + t.rows);
    lo = 0;
    if (t.window > 0) lo = max(0, t.pos0 - t.window + 1);
    lo = (lo / kTileK) * kTileK;
    if (hi < lo) hi = lo;
}

// Byte offset of a key's row from t.k / t.v.  Keys past the end are redirected to the last valid
// key and block ids outside the cache are clamped (the loads stay unconditional and inside the
// cache): such rows only ever meet a probability of zero -- the softmax masks the keys of a block
// the table does not name -- but they must be readable and finite.
__device__ __forceinline__ int64_t kv_row_offset(const Tile& t, int key, int row_bytes = kRowBytes) {
    key = min(key, t.kv_len - 1);
    if (t.table == nullptr) return (int64_t)key * row_bytes;
    const int lb = key >> t.block_shift;  // block_size is a power of two on this path
    const int pb = min(max(t.table[lb], 0), t.num_blocks - 1);
    return (int64_t)pb * t.block_stride + (int64_t)(key & (t.block_size - 1)) * row_bytes;
}

// Q fragment, multiplied by c = scale * log2(e) and rounded to the MFMA element type: the first
// product then yields the exponents of the softmax directly.
template <bool kBf16, bool kFromBf16>
__device__ __forceinline__ typename Mfma<kBf16>::vec8 convert_q_frag(uint4_t raw, float c) {
    using vec8 = typename Mfma<kBf16>::vec8;
    uint4_t cv;
#pragma unroll
    for (int w = 0; w < 4; w++) {
        float lo, hi;
        if constexpr (kFromBf16) {
            lo = __uint_as_float(raw[w] << 16);
            hi = __uint_as_float(raw[w] & 0xffff0000u);
        } else {
            lo = f16_bits_to_float((uint16_t)(raw[w] & 0xffffu));
            hi = f16_bits_to_float((uint16_t)(raw[w] >> 16));
        }
        cv[w] = Mfma<kBf16>::cvt2(lo * c, hi * c);
    }
    return __builtin_bit_cast(vec8, cv);
}

typedef short short4_t __attribute__((ext_vector_type(4)));

// Lanes l and l + 32 exchange a value in the vector ALU (v_permlane32_swap: the upper half of the
// first operand is swapped with the lower half of the second); both get (value of l, value of l + 32).
__device__ __forceinline__ void pair_values(float x, float& lo, float& hi) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    lo = __uint_as_float(r[0]);
    hi = __uint_as_float(r[1]);
}

// LDS layout of a K or V tile: row r (a key) at byte r * 256, its 16-byte chunk c stored at chunk
// position c ^ swz(r), with swz(r) = r % 16 for K and 4 * (r % 4) for V.
//
// K fragment (A operand of S^T = K Q^T, k-step i): lane (n32, hi) reads chunk 2i + hi of row
// mt*32 + n32 with one ds_read_b128; sixteen consecutive lanes hit sixteen different positions.
//
// V^T fragment (A operand of O^T = V^T P^T, k-step ks, head-dim tile dt): the lane holding
// head-dim d = dt*32 + n32 needs V[key][d] for the keys 16ks + 4hi + {0..3} and 16ks + 8 + 4hi +
// {0..3}.  ds_read_b64_tr_b16 gives lane i of a 16-lane group element j = what lane 4j + i/4 of
// the group addressed, taken at 16-bit index i % 4: so lane i addresses row key0 + i/4, head-dim
// d0 + 4 (i % 4) .. +3 (d0 = dt*32 + 16 * (group & 1), key0 = 16ks + 4 * (group >> 1)), and
// receives V[key0 + j][d0 + i].  Two such reads, eight rows apart, make one fragment.
//
// Both fragment addresses are (one per-lane base) ^ (a compile-time constant): the swizzle term
// of the lane sits in address bits that the base leaves zero.
struct FragOffsets {
    int k;  // K fragment (mt, i):  (k ^ (i << 5)) + mt * 32 rows
    int v;  // V^T fragment (ks, dt): (v ^ (dt << 6)) + ks * 16 rows (+ 8 rows for the second half)
};

__device__ __forceinline__ FragOffsets frag_offsets(int lane) {
    FragOffsets f;
    const int n32 = lane & 31, hi = lane >> 5, x = n32 & 15;
    // chunk (2i + hi) ^ x = 2 (i ^ (x >> 1)) + (hi ^ (x & 1))
    f.k = n32 * kRowBytes + ((x >> 1) << 5) + ((hi ^ (x & 1)) << 4);
    const int g = lane >> 4, i16 = lane & 15;
    const int vrow = 4 * (g >> 1) + (i16 >> 2);  // row % 4 == i16 / 4
    // chunk (4dt + 2(g&1) + (i16 % 4) / 2) ^ 4 (i16 / 4) = 4 (dt ^ (i16 / 4)) + 2 (g & 1) + (i16 % 4) / 2
    f.v = vrow * kRowBytes + ((i16 >> 2) << 6) + ((2 * (g & 1) + ((i16 & 3) >> 1)) << 4) + 8 * (i16 & 1);
    return f;
}

template <bool kBf16>
__device__ __forceinline__ typename Mfma<kBf16>::vec8 read_v_frag(const lds_byte* v_lds, int v_off, int ks, int dt) {
    typedef __attribute__((address_space(3))) short4_t lds_short4;
    const lds_byte* p = v_lds + (v_off ^ (dt << 6)) + ks * 16 * kRowBytes;
    const short4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)p);
    const short4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(p + 8 * kRowBytes));
    typedef short short8_t __attribute__((ext_vector_type(8)));
    const short8_t a = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
    return __builtin_bit_cast(typename Mfma<kBf16>::vec8, a);
}

// Online softmax with a lazily updated reference.  The scores come out of the first product as
// exponents x = s c - ref, because Q carries the factor c and the accumulator of the product is
// initialised with -ref (a 16-register tuple per lane: all sixteen belong to one query row), so
// a probability costs one v_exp_f32 and half a conversion.  p = exp2(x) is a valid numerator for
// any reference as long as it cannot overflow: ref is raised, and the accumulators rescaled,
// only when some row's largest exponent exceeds 8, which after the first few tiles is rare.
struct SoftmaxState {
    float16_t neg_ref;  // -ref in every element
    float l_run;        // this lane's half of the row sum
    bool started;       // the row has met a key it may attend to
    bool all_started;   // wave-uniform: every row of the wavefront has
};

// Mask, reference update and probabilities of the tile that starts at key ts (register r of s[mt]
// is key ts + mt*32 + 8*(r/4) + 4*hi + r%4).  `masked` is false for tiles that every query row of
// the group sees completely (the common case).
// kMask: 0 no attention mask; 2 a mask of the operands' 16-bit type, added to the scaled scores;
// 1 a boolean mask of one byte per key (zero: the key takes no part).  mask_lds: this wavefront's
// 32 rows x 64 keys of the mask in LDS (mask_tile_* below), or nullptr for a tile that reaches past
// the last key, whose mask values are fetched from global memory one by one.
// bad16 (paged caches; wave-uniform): bit b set when keys ts + 16 b .. + 15 lie in a block whose table
// entry names no block of the cache -- they take no part, like keys past the end (`masked` must be set).
template <bool kBf16, int kMask = 0>
__device__ __forceinline__ void tile_softmax(const Tile& t, float16_t (&s)[2], float16_t (&o)[4], SoftmaxState& st,
                                             typename Mfma<kBf16>::vec8 (&pf)[4], int ts, int my_pos, int hi, bool masked,
                                             const lds_byte* mask_lds = nullptr, int row = 0, uint32_t bad16 = 0) {
    using M = Mfma<kBf16>;
    using vec8 = typename M::vec8;
    if (masked) {
#pragma unroll
        for (int mt = 0; mt < 2; mt++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int key = ts + mt * 32 + 8 * (r >> 2) + 4 * hi + (r & 3);  // in sixteenth 2 mt + r / 8 of the tile
                bool ok = key < t.kv_len && ((bad16 >> (2 * mt + (r >> 3))) & 1u) == 0;
                if (t.causal) ok = ok && key <= my_pos;
                if (t.window > 0) ok = ok && key > my_pos - t.window;
                s[mt][r] = ok ? s[mt][r] : -INFINITY;
            }
    }
    if constexpr (kMask != 0) {
        const int n32 = row & 31;
        auto add16 = [&](uint32_t bits, float x) __attribute__((always_inline)) -> float {
            const float m = kBf16 ? bf16_bits_to_float((uint16_t)bits) : f16_bits_to_float((uint16_t)bits);
            return fmaf(m, kLog2e, x);  // the scores are exponents to base 2
        };
        if (mask_lds != nullptr) {
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    if constexpr (kMask == 2) {
                        typedef __attribute__((address_space(3))) uint2_t lds_uint2;
                        const int c = mt * 4 + g;
                        const uint2_t w = *(const lds_uint2*)(mask_lds + n32 * 128 + ((c ^ (n32 & 7)) << 4) + hi * 8);
                        s[mt][4 * g] = add16(w[0] & 0xffffu, s[mt][4 * g]);
                        s[mt][4 * g + 1] = add16(w[0] >> 16, s[mt][4 * g + 1]);
                        s[mt][4 * g + 2] = add16(w[1] & 0xffffu, s[mt][4 * g + 2]);
                        s[mt][4 * g + 3] = add16(w[1] >> 16, s[mt][4 * g + 3]);
                    } else {
                        typedef __attribute__((address_space(3))) uint32_t lds_uint;
                        const int c = mt * 2 + (g >> 1);
                        const uint32_t w = *(const lds_uint*)(mask_lds + n32 * 64 + ((c ^ (n32 & 3)) << 4) + 8 * (g & 1) + 4 * hi);
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (((w >> (8 * e)) & 0xffu) == 0) s[mt][4 * g + e] = -INFINITY;
                    }
                }
        } else if (row < t.rows) {
            const uint8_t* mrow = t.mask + (int64_t)row * t.mask_row_bytes;
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int key = ts + mt * 32 + 8 * (r >> 2) + 4 * hi + (r & 3);
                    if (key < t.kv_len) {
                        if constexpr (kMask == 2)
                            s[mt][r] = add16(((const uint16_t*)mrow)[key], s[mt][r]);
                        else if (mrow[key] == 0)
                            s[mt][r] = -INFINITY;
                    }
                }
        }
    }
    // probabilities of the tile against the current reference, and this lane's share of their sum
    auto probabilities = [&]() __attribute__((always_inline)) -> float {
        float sum = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            uint4_t pw;
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const float p0 = fast_exp2(s[ks >> 1][(ks & 1) * 8 + 2 * w]);
                const float p1 = fast_exp2(s[ks >> 1][(ks & 1) * 8 + 2 * w + 1]);
                pw[w] = M::cvt2(p0, p1);
                sum += p0 + p1;  // (not v_dot2: dot instructions wait for the matrix core, which the other group keeps busy)
            }
            pf[ks] = __builtin_bit_cast(vec8, pw);
        }
        return sum;
    };
    // Common case (an unmasked tile, every row already has a reference): no row maximum at all.
    // The exponentials are taken against the standing reference and the tile's row sums tell
    // whether that was safe: a sum below the bound (2^24; 2^15 where the probabilities become fp16,
    // which ends at 65504) bounds every probability, and anything else (large, infinite, NaN)
    // sends the wavefront through the careful path below, which redoes the tile from the
    // untouched scores.  Sixteen v_max3, the cross-lane exchange and the compare of the
    // maximum are then spent only on the first tile of a row, on masked tiles and on outliers.
    if (!masked && st.all_started) {
        const float sum = probabilities();
        constexpr float kSafeSum = kBf16 ? 16777216.0f : 32768.0f;
        if (!__builtin_amdgcn_ballot_w64(!(sum < kSafeSum))) {
            st.l_run += sum;
            return;
        }
    }
    float m_tile = -INFINITY;
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int r = 0; r < 16; r++) m_tile = fmaxf(m_tile, s[mt][r]);
    {  // the row lives in lanes l and l + 32
        float lo, hi2;
        pair_values(m_tile, lo, hi2);
        m_tile = fmaxf(lo, hi2);
    }
    const bool seen = m_tile != -INFINITY;
    if (__builtin_amdgcn_ballot_w64(m_tile > 8.0f || (seen && !st.started))) {
        // move the reference to this tile's maximum: up for a started row, anywhere for a new one
        // (whose accumulators are still zero)
        const float delta = st.started ? fmaxf(m_tile, 0.0f) : (seen ? m_tile : 0.0f);
        const float alpha = fast_exp2(-fmaxf(delta, 0.0f));
        st.l_run *= alpha;
#pragma unroll
        for (int dt = 0; dt < 4; dt++) o[dt] *= alpha;
#pragma unroll
        for (int mt = 0; mt < 2; mt++) s[mt] -= delta;
        st.neg_ref -= delta;
        st.started = st.started || seen;
        st.all_started = __builtin_amdgcn_ballot_w64(!st.started) == 0;
    }
    st.l_run += probabilities();
}

// The fragments of a product are read from LDS in batches of four, each batch one batch of MFMAs
// ahead of its use; sched_barrier keeps the compiler from sinking the reads back to their uses.
template <bool kBf16>
__device__ __forceinline__ void read_v_batch(const lds_byte* v_lds, const FragOffsets& f, int ks,
                                             typename Mfma<kBf16>::vec8 (&vf)[4]) {
#pragma unroll
    for (int dt = 0; dt < 4; dt++) vf[dt] = read_v_frag<kBf16>(v_lds, f.v, ks, dt);
}
template <bool kBf16>
__device__ __forceinline__ void read_k_batch(const lds_byte* k_lds, const FragOffsets& f, int b,
                                             typename Mfma<kBf16>::vec8 (&kf)[4]) {  // k-steps 2b, 2b+1 of both key halves
    typedef __attribute__((address_space(3))) typename Mfma<kBf16>::vec8 lds_vec8;
#pragma unroll
    for (int u = 0; u < 4; u++)
        kf[u] = *(const lds_vec8*)(k_lds + (f.k ^ ((2 * b + (u >> 1)) << 5)) + (u & 1) * 32 * kRowBytes);
}

// O^T += V^T P^T for one tile
template <bool kBf16>
__device__ __forceinline__ void tile_accumulate(const lds_byte* v_lds, const FragOffsets& f,
                                                const typename Mfma<kBf16>::vec8 (&pf)[4], float16_t (&o)[4]) {
    using M = Mfma<kBf16>;
    using vec8 = typename M::vec8;
    vec8 vf[2][4];
    read_v_batch<kBf16>(v_lds, f, 0, vf[0]);
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        __builtin_amdgcn_sched_barrier(0);
        if (ks < 3) read_v_batch<kBf16>(v_lds, f, ks + 1, vf[(ks + 1) & 1]);
#pragma unroll
        for (int dt = 0; dt < 4; dt++) o[dt] = M::mma(vf[ks & 1][dt], pf[ks], o[dt]);
    }
}

// S^T = K Q^T - ref for one 64-key tile
template <bool kBf16>
__device__ __forceinline__ void tile_scores(const lds_byte* k_lds, const FragOffsets& f,
                                            const typename Mfma<kBf16>::vec8 (&qf)[8], const float16_t& neg_ref,
                                            float16_t (&s)[2]) {
    using M = Mfma<kBf16>;
    using vec8 = typename M::vec8;
    vec8 kf[2][4];
    read_k_batch<kBf16>(k_lds, f, 0, kf[0]);
#pragma unroll
    for (int b = 0; b < 4; b++) {
        __builtin_amdgcn_sched_barrier(0);
        if (b < 3) read_k_batch<kBf16>(k_lds, f, b + 1, kf[(b + 1) & 1]);
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int i = 2 * b + (u >> 1), mt = u & 1;
            s[mt] = M::mma(kf[b & 1][u], qf[i], i == 0 ? neg_ref : s[mt]);
        }
    }
}

// The matrix phase of the steady state: O^T += V^T P^T for one tile, then the scores of the next;
// the first K fragments are read while the last P V MFMAs run.
template <bool kBf16>
__device__ __forceinline__ void tile_accumulate_and_scores(const lds_byte* v_lds, const lds_byte* k_lds,
                                                           const FragOffsets& f,
                                                           const typename Mfma<kBf16>::vec8 (&pf)[4], float16_t (&o)[4],
                                                           const typename Mfma<kBf16>::vec8 (&qf)[8],
                                                           const float16_t& neg_ref, float16_t (&s)[2]) {
    using M = Mfma<kBf16>;
    using vec8 = typename M::vec8;
    vec8 fr[3][4];  // batches b, b+1, b+2: reads run two batches (8 MFMAs) ahead of their use
    auto read_batch = [&](int b) {
        if (b < 4)
            read_v_batch<kBf16>(v_lds, f, b, fr[b % 3]);
        else
            read_k_batch<kBf16>(k_lds, f, b - 4, fr[b % 3]);
    };
    read_batch(0);
    read_batch(1);
#pragma unroll
    for (int b = 0; b < 8; b++) {  // batches 0..3: P V (ks = b); 4..7: scores (k-steps 2(b-4), 2(b-4)+1)
        __builtin_amdgcn_sched_barrier(0);
        if (b + 2 < 8) read_batch(b + 2);
        if (b < 4) {
#pragma unroll
            for (int dt = 0; dt < 4; dt++) o[dt] = M::mma(fr[b % 3][dt], pf[b], o[dt]);
        } else {
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int i = 2 * (b - 4) + (u >> 1), mt = u & 1;
                s[mt] = M::mma(fr[b % 3][u], qf[i], i == 0 ? neg_ref : s[mt]);
            }
        }
    }
}

template <int kOutDtype>
__device__ __forceinline__ void store_rows(const Tile& t, const float16_t (&o)[4], float inv, int row, int hi) {
    // o[dt][r] is head-dim dt*32 + 8*(r/4) + 4*hi + r%4 of `row`: four consecutive outputs per (dt, r/4)
    const int64_t obase = (int64_t)row * t.out_stride;
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int rq = 0; rq < 4; rq++) {
            const int d = dt * 32 + 8 * rq + 4 * hi;
            if (d >= t.head_dim) continue;  // (columns the rows in memory do not have)
            const float x0 = o[dt][rq * 4] * inv, x1 = o[dt][rq * 4 + 1] * inv, x2 = o[dt][rq * 4 + 2] * inv,
                        x3 = o[dt][rq * 4 + 3] * inv;
            if constexpr (kOutDtype == HIPATTN_F32) {
                *(float4*)((float*)t.out + obase + d) = make_float4(x0, x1, x2, x3);
            } else if constexpr (kOutDtype == HIPATTN_F16) {
                const uint2_t w = {Mfma<false>::cvt2(x0, x1), Mfma<false>::cvt2(x2, x3)};
                *(uint2_t*)((uint16_t*)t.out + obase + d) = w;
            } else {
                const uint2_t w = {Mfma<true>::cvt2(x0, x1), Mfma<true>::cvt2(x2, x3)};
                *(uint2_t*)((uint16_t*)t.out + obase + d) = w;
            }
        }
}

// 16-bit outputs of a wavefront's 32 rows, transposed through 8 KB of LDS (free once the key loop
// is over) so that the global stores are whole rows: the accumulator layout gives a lane 8 bytes
// in each of 16 places of one row, a wavefront-wide store of which touches 32 rows 16 bytes at a
// time.  LDS rows are 256 bytes with the 16-byte chunks XOR-swizzled by the row number; one store
// instruction then writes four complete rows (16 lanes x 16 bytes each).
template <bool kOutBf16>
__device__ __forceinline__ void store_rows_via_lds(const Tile& t, const float16_t (&o)[4], float inv, lds_byte* stage,
                                                   int row0, int lane) {
    const int n32 = lane & 31, hi = lane >> 5;
    typedef __attribute__((address_space(3))) uint2_t lds_uint2;
    typedef __attribute__((address_space(3))) uint4_t lds_uint4;
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int rq = 0; rq < 4; rq++) {
            const float x0 = o[dt][rq * 4] * inv, x1 = o[dt][rq * 4 + 1] * inv, x2 = o[dt][rq * 4 + 2] * inv,
                        x3 = o[dt][rq * 4 + 3] * inv;
            const uint2_t w = {Mfma<kOutBf16>::cvt2(x0, x1), Mfma<kOutBf16>::cvt2(x2, x3)};
            const int chunk = dt * 4 + rq;  // head-dim dt*32 + 8*rq .. +8; this lane has its half `hi`
            *(lds_uint2*)(stage + n32 * kRowBytes + ((chunk ^ (n32 & 15)) << 4) + hi * 8) = w;
        }
    const int lrow = lane >> 4, chunk = lane & 15;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const int r = 4 * k + lrow;
        const uint4_t w = *(const lds_uint4*)(stage + r * kRowBytes + ((chunk ^ (r & 15)) << 4));
        if (row0 + r < t.rows && chunk * 8 < t.head_dim) *(uint4_t*)((uint16_t*)t.out + (int64_t)(row0 + r) * t.out_stride + chunk * 8) = w;
    }
}

// Wave-uniform address of the 8 consecutive rows that start at key0 (a multiple of 8 below
// kv_len): they lie in one block of a paged cache, whose table entry is `entry`.
__device__ __forceinline__ const uint8_t* row_group_base(const Tile& t, const uint8_t* base, int key0, int entry,
                                                         int row_bytes = kRowBytes) {
    if (t.table == nullptr) return base + (int64_t)key0 * row_bytes;
    const int pb = min(max(entry, 0), t.num_blocks - 1);
    return base + (int64_t)pb * t.block_stride + (int64_t)(key0 & (t.block_size - 1)) * row_bytes;
}

// Workgroup barrier that lets the `keep` most recent global->LDS loads of this wavefront stay in
// flight (__syncthreads would wait for all of them): s_waitcnt vmcnt(keep) lgkmcnt(0), then
// s_barrier.  Loads complete in order, so everything issued earlier has landed in LDS.
template <int kKeep>
__device__ __forceinline__ void barrier_keeping() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0070 | (kKeep & 15) | ((kKeep >> 4) << 14));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}
// Waits until at most `keep` (even, <= 10, wave-uniform) of this wavefront's global->LDS loads are
// in flight, without a barrier: enough for data that only this wavefront reads.
template <int kKeep>
__device__ __forceinline__ void wait_keeping() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0f70 | (kKeep & 15) | ((kKeep >> 4) << 14));  // vmcnt only
    asm volatile("" ::: "memory");
}
__device__ __forceinline__ void wait_keeping_loads(int keep) {
    if (keep >= 10)
        wait_keeping<10>();
    else if (keep >= 8)
        wait_keeping<8>();
    else if (keep >= 6)
        wait_keeping<6>();
    else if (keep >= 4)
        wait_keeping<4>();
    else if (keep >= 2)
        wait_keeping<2>();
    else
        wait_keeping<0>();
}
__device__ __forceinline__ void barrier_keeping_loads(int keep) {  // keep is even, at most 8 (wave-uniform)
    if (keep >= 8)
        barrier_keeping<8>();
    else if (keep >= 6)
        barrier_keeping<6>();
    else if (keep >= 4)
        barrier_keeping<4>();
    else if (keep >= 2)
        barrier_keeping<2>();
    else
        barrier_keeping<0>();
}

// The loop of one wavefront.  t is the tile of this wavefront's group; [kv_lo, kv_hi) is the key
// range of the workgroup (the union of both groups' ranges, kv_lo a multiple of 64).
//
// Phases, numbered from 0: group 0 computes the scores of tile j in phase 2j, their softmax in
// phase 2j+1 and P V in phase 2j+2 (together with the scores of tile j+1); group 1 does the same
// one phase later.  K(j) is therefore read in phases 2j and 2j+1, V(j) in phases 2j+2 and 2j+3.
// Load batch B(x) = {K(x+2), V(x+1)} goes into the ring stages of K(x-1) and V(x-2); every
// wavefront issues its rows of B(x) in a vector phase (group 0 in phase 2x+1, group 1 in phase
// 2x).
//
// One workgroup barrier per tile: before every even phase, i.e. for group 0 between its vector
// and its matrix phase, for group 1 behind its matrix phase; at it a wavefront waits for all of
// its loads except the latest batch.  That is all the data needs.  What is read from phase 2j+2
// on -- K(j+1) and V(j) -- was issued by group 0 in phase 2j-1 and by group 1 in phase 2j-2, and
// at the barrier before phase 2j+2 neither batch is the issuing wavefront's latest any more.  What
// is overwritten by loads issued from phase 2j+2 on -- the stages of K(j) and V(j-1) -- was last
// read in phase 2j+1.  Between the barriers each group runs one matrix and one vector phase, in
// opposite order, so that the matrix core and the vector units are both in use; the odd phase
// boundaries are not enforced, the two groups only drift by what their phases differ in length.
// kPad (16-bit K/V): the rows of Q, K, V and the output have t.head_dim < kD columns in memory (a
// multiple of 8).  Everything in LDS and in registers keeps the layout of kD columns: a lane whose 16-byte
// chunk of a row does not exist fetches the row's first chunk instead -- valid, finite data that only
// ever meets the zeros the query fragments hold in those columns, or lands in output columns that
// are not stored.
template <bool kBf16, bool kU8 = false, bool kPaged = true, int kMask = 0, bool kPad = false>
__device__ __forceinline__ void run_pair(const Tile& t, int kv_lo, int kv_hi, uint8_t* lds_generic, float scale) {
    static_assert(kPaged || !kU8, "dense K/V are 16-bit");
    static_assert(!kPad || !kU8, "smaller head sizes: 16-bit K/V");
    const int grow = kPad ? 2 * t.head_dim : kRowBytes;  // bytes from row to row in memory
    const int head_chunks = kPad ? t.head_dim >> 3 : kD / 8;
    static_assert(kMask == 0 || !kPaged, "attention masks belong to the dense operator");
    static_assert(!(kU8 && kBf16), "u8 caches are dequantised to fp16");
    using M = Mfma<kBf16>;
    using vec8 = typename M::vec8;
    lds_byte* const lds = (lds_byte*)lds_generic;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int group = wave >> 2;
    const int n32 = lane & 31, hi = lane >> 5;
    const int row = (wave & 3) * 32 + n32;  // query row inside the group's tile
    const float c = scale * kLog2e;
    const int n = (kv_hi - kv_lo + kTileK - 1) / kTileK;  // tiles of the workgroup
    if (n <= 0) {
        // nothing to attend to: rows of zeros (the reference's softmax over an empty set is undefined)
        if (row < t.rows) {
            float16_t z[4];
#pragma unroll
            for (int dt = 0; dt < 4; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) z[dt][r] = 0.0f;
            if (t.out_dtype == HIPATTN_F32)
                store_rows<HIPATTN_F32>(t, z, 0.0f, row, hi);
            else
                store_rows<HIPATTN_F16>(t, z, 0.0f, row, hi);  // zero bits are the same in f16 and bf16
        }
        return;
    }
    auto unmasked = [&](int j) {
        if constexpr (kMask != 0) return false;
        const int ts = kv_lo + j * kTileK;
        return (ts + kTileK <= t.kv_len) && (!t.causal || ts + kTileK <= t.pos0 + 1) &&
               (t.window <= 0 || ts >= t.pos0 + t.rows - t.window);
    };
    // Paged caches: table entries that name no block of the cache ([0, num_blocks)) stand for keys that
    // take no part.  Almost no call has one, so every wavefront looks through the table in windows of 256
    // entries (four loads per lane and a ballot): the first window of the workgroup's key range is loaded
    // ahead of everything else and looked at only after the query rows have been converted, later windows
    // when the loop reaches them (one stall in 64 to 256 key tiles).  Only the tiles of a window that has
    // such an entry get their own entries checked and their keys masked (bad_sixteenths).
    constexpr int kScanWindow = 256;
    uint32_t scan_ids[4] = {0u, 0u, 0u, 0u};
    int scan_end = 0, last_entry = -1;  // entries below scan_end have been looked at; the range's last entry
    // a window looked at on the spot (the loop's later windows)
    auto scan_now = [&](int first) __attribute__((always_inline)) -> bool {
        bool bad_lane = false;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int e = first + lane + 64 * u;
            const uint32_t id = e <= last_entry ? (uint32_t)t.table[e] : 0u;
            bad_lane = bad_lane || id >= (uint32_t)t.num_blocks;
        }
        scan_end = first + kScanWindow;
        return __builtin_amdgcn_ballot_w64(bad_lane) != 0;
    };
    if constexpr (kPaged) {
        if (t.table != nullptr && t.kv_len > 0) {
            last_entry = (min(kv_hi, t.kv_len) - 1) >> t.block_shift;
            const int first = kv_lo >> t.block_shift;
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int e = first + lane + 64 * u;
                if (e <= last_entry) scan_ids[u] = (uint32_t)t.table[e];
            }
            scan_end = first + kScanWindow;
        }
    }

    // The wavefront's 32 query rows go to its own 8 KB of LDS with eight global->LDS loads of four
    // whole rows each, laid out like a K tile (chunk c of row r at position c ^ (r % 16)): the
    // fragment of k-step i, head-dim i*16 + hi*8 .. +8 of row n32, is then one conflict-free
    // ds_read_b128.  Rows past the end of the tile repeat its last row (never stored).  A lane
    // loading its fragments straight from global memory would touch 32 rows per instruction.
    lds_byte* const wave_stage = lds + kRingBytes + wave * kWaveStageBytes;
    if (t.rows > 0) {
        const int lr = lane >> 4, lp = lane & 15;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int r = 4 * k + lr;
            const int qrow = min((wave & 3) * 32 + r, t.rows - 1);
            int q_chunk = lp ^ (r & 15);
            if constexpr (kPad) q_chunk = q_chunk < head_chunks ? q_chunk : 0;
            const uint8_t* src = (const uint8_t*)(t.q + (int64_t)qrow * t.q_stride) + (q_chunk << 4);
            load_to_lds_16(src, wave_stage + 4 * k * kRowBytes);
        }
    }

    float16_t o[4];
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[dt][r] = 0.0f;
    SoftmaxState st;
#pragma unroll
    for (int r = 0; r < 16; r++) st.neg_ref[r] = 0.0f;
    st.l_run = 0.0f;
    st.started = false;
    st.all_started = false;
    const int my_pos = t.pos0 + row;  // position of this lane's query row
    const FragOffsets f = frag_offsets(lane);

    // global -> LDS: one instruction moves four rows (64 lanes x 16 bytes, LDS address = wave-uniform
    // base + lane * 16); wavefront w issues the two instructions of rows 8w .. 8w + 7 of a K or V
    // tile.  Lane l fills chunk position l % 16 of row r = 8w + 4k + l / 16, i.e. it fetches chunk
    // (l % 16) ^ swz(r): for K that is ((l%16) ^ (l/16) ^ 8(w%2)) ^ 4k, for V (l%16) ^ 4(l/16).
    const int lrow = lane >> 4, lpos = lane & 15;
    // (kPad: chunks past the end of a row in memory become chunk 0, rows are grow bytes apart)
    auto mem_chunk = [&](int chunk) __attribute__((always_inline)) { return kPad ? (chunk < head_chunks ? chunk : 0) : chunk; };
    const int k_chunk0 = lpos ^ lrow ^ (8 * (wave & 1)), v_chunk0 = lpos ^ (4 * lrow);
    const uint32_t k_lane = (uint32_t)((mem_chunk(k_chunk0) << 4) + lrow * grow);
    const uint32_t v_lane = (uint32_t)((mem_chunk(v_chunk0) << 4) + lrow * grow);
    // the second instruction of a wavefront's eight rows (four rows further on: K's chunk index has bit 2 flipped)
    const uint32_t k_lane1 = kPad ? (uint32_t)((mem_chunk(k_chunk0 ^ 4) << 4) + (lrow + 4) * grow) : (k_lane ^ 64u) + 4 * kRowBytes;
    const uint32_t v_lane1 = v_lane + 4 * grow;
    lds_byte* const k_ring = lds;
    lds_byte* const v_ring = lds + kStages * kKBytes;
    // this wavefront's rows of tile j into `stage`; returns the number of instructions issued
    // (entry: the block table entry of these rows, see table_entry below; ignored for dense K/V)
    auto load_rows = [&](bool is_k, int j, lds_byte* stage, int entry) -> int {
        if (j >= n) return 0;
        const uint8_t* base = is_k ? t.k : t.v;
        lds_byte* const dst = stage + 8 * wave * kRowBytes;
        const int key0 = kv_lo + j * kTileK + 8 * wave;
        if (key0 + 8 <= t.kv_len) {
            const uint8_t* gb = row_group_base(t, base, key0, entry, grow);
#pragma unroll
            for (int k = 0; k < 2; k++) {
                uint32_t off;
                if constexpr (kPad)
                    off = (is_k ? (k ? k_lane1 : k_lane) : (k ? v_lane1 : v_lane));
                else
                    off = (is_k ? (k_lane ^ (uint32_t)(k << 6)) : v_lane) + (uint32_t)(4 * k * kRowBytes);
                load_to_lds_16(gb, off, dst + 4 * k * kRowBytes);
            }
        } else {  // the rows at the end of the sequence: per-lane clamped
#pragma unroll
            for (int k = 0; k < 2; k++) {
                const int r = 8 * (wave & 1) + 4 * k + lrow;
                const int chunk = mem_chunk(is_k ? (lpos ^ r) : (lpos ^ (4 * lrow)));
                const int64_t off = kv_row_offset(t, key0 + 4 * k + lrow, grow) + (chunk << 4);
                load_to_lds_16(base + off, dst + 4 * k * kRowBytes);
            }
        }
        return 2;
    };
    // Block table entry of this wavefront's rows of tile j (0 when there is none), read through
    // the scalar cache at the end of a matrix phase, behind its last fragment wait: a scalar load
    // outstanding while fragments are still being waited for would turn every partial wait for LDS
    // fragments into a full one.
    // (As inline assembly, because behind the compiler fences of the barriers an ordinary load of
    // the table becomes a vector load that is waited for at once, together with every load to LDS
    // in flight.  The wait for the scalar load is part of the statement: the compiler takes the
    // output register as written when the statement ends and may reuse it at any time after.)
    auto table_entry = [&](int j) -> int {
        if constexpr (!kPaged) return 0;
        const int key0 = kv_lo + j * kTileK + 8 * wave;
        if (t.table == nullptr || j >= n || key0 + 8 > t.kv_len) return 0;
        int entry;
        asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(entry) : "s"(t.table + (key0 >> t.block_shift)));
        return entry;
    };
    auto k_stage = [&](int j) { return k_ring + (j % kStages) * kKBytes; };
    auto v_stage = [&](int j) { return v_ring + (j % kStages) * kKBytes; };
    // Attention mask: the wavefront's 32 query rows x the 64 keys of tile j go global -> LDS into one
    // half of the wavefront's own stage (which holds query rows before the loop and output rows after
    // it, and nothing in between), tile j into half j % 2, one tile ahead of its use.  16-bit masks:
    // four loads, row r at r * 128 with its 16-byte chunk c at position c ^ (r % 8); boolean masks:
    // two loads, row r at r * 64, chunk c at c ^ (r % 4).  A tile that reaches past the last key is
    // not staged (a 16-byte piece would run past the mask row): tile_softmax reads it element-wise.
    auto mask_tile_staged = [&](int j) { return kMask != 0 && j < n && kv_lo + (j + 1) * kTileK <= t.kv_len; };
    auto mask_stage = [&](int j) { return wave_stage + (j & 1) * (kWaveStageBytes / 2); };
    auto load_mask_tile = [&](int j) -> int {
        if (!mask_tile_staged(j) || t.rows <= 0) return 0;
        const int ts = kv_lo + j * kTileK;
        constexpr int kLoads = kMask == 2 ? 4 : 2, kRowsPerLoad = 32 / kLoads, kChunks = 64 / kRowsPerLoad;
#pragma unroll
        for (int k = 0; k < kLoads; k++) {
            const int r = kRowsPerLoad * k + lane / kChunks, q = lane % kChunks;
            const int c = q ^ (r & (kChunks - 1));
            const int qrow = min((wave & 3) * 32 + r, t.rows - 1);
            const uint8_t* src = t.mask + (int64_t)qrow * t.mask_row_bytes + (int64_t)(ts * (kMask == 2 ? 2 : 1)) + (c << 4);
            load_to_lds_16(src, mask_stage(j) + k * 1024);
        }
        return kLoads;
    };
    // ---- u8 caches: lane l of wavefront w handles 16 payload bytes (piece l % 8) of row 8w + l / 8
    const int u8_row = 8 * wave + (lane >> 3), u8_piece = lane & 7;
    // address of this lane's row of tile j (entry: the block table entry of the wavefront's rows)
    auto u8_row_address = [&](const uint8_t* base, int j, int entry) __attribute__((always_inline)) -> const uint8_t* {
        const int key0 = kv_lo + j * kTileK + 8 * wave;
        int key = kv_lo + j * kTileK + u8_row;
        int pb;
        if (key0 + 8 <= t.kv_len) {
            pb = entry;
        } else {  // rows at the end of the sequence repeat its last row
            key = min(key, t.kv_len - 1);
            pb = t.table[key >> t.block_shift];
        }
        pb = min(max(pb, 0), t.num_blocks - 1);
        return base + (int64_t)pb * t.block_stride + (int64_t)(key & (t.block_size - 1)) * kU8RowBytes;
    };
    auto u8_fetch = [&](int jk, int ek, int jv, int ev) __attribute__((always_inline)) -> U8Rows {
        U8Rows x;
        x.k_lo = x.k_hi = x.v_lo = x.v_hi = uint2_t{0u, 0u};
        x.k_sz = x.v_sz = make_float2(0.0f, 0.0f);
        x.jk = jk < n ? jk : -1;
        x.jv = jv < n ? jv : -1;
        if (x.jk >= 0) {
            const uint8_t* row = u8_row_address(t.k, jk, ek);
            x.k_sz = *(const float2*)row;
            x.k_lo = *(const uint2_t*)(row + 8 + 16 * u8_piece);
            x.k_hi = *(const uint2_t*)(row + 16 + 16 * u8_piece);
        }
        if (x.jv >= 0) {
            const uint8_t* row = u8_row_address(t.v, jv, ev);
            x.v_sz = *(const float2*)row;
            x.v_lo = *(const uint2_t*)(row + 8 + 16 * u8_piece);
            x.v_hi = *(const uint2_t*)(row + 16 + 16 * u8_piece);
        }
        return x;
    };
    // dequantises the rows and writes them where the 16-bit path loads them (chunk c of row r at
    // position c ^ (r % 16) for K, c ^ 4 (r % 4) for V); this lane has chunks 2 piece and 2 piece + 1
    auto u8_store = [&](const U8Rows& x) __attribute__((always_inline)) {
        typedef __attribute__((address_space(3))) uint4_t lds_uint4;
        if (x.jk >= 0) {
            const half2_t sc = {(half_t)x.k_sz.x, (half_t)x.k_sz.x};
            const float o32 = -x.k_sz.y * x.k_sz.x;
            const half2_t of = {(half_t)o32, (half_t)o32};
            lds_byte* const rowp = k_stage(x.jk) + u8_row * kRowBytes;
            *(lds_uint4*)(rowp + (((2 * u8_piece) ^ (u8_row & 15)) << 4)) = dequant8(x.k_lo, sc, of);
            *(lds_uint4*)(rowp + (((2 * u8_piece + 1) ^ (u8_row & 15)) << 4)) = dequant8(x.k_hi, sc, of);
        }
        if (x.jv >= 0) {
            const half2_t sc = {(half_t)x.v_sz.x, (half_t)x.v_sz.x};
            const float o32 = -x.v_sz.y * x.v_sz.x;
            const half2_t of = {(half_t)o32, (half_t)o32};
            lds_byte* const rowp = v_stage(x.jv) + u8_row * kRowBytes;
            *(lds_uint4*)(rowp + (((2 * u8_piece) ^ (4 * (u8_row & 3))) << 4)) = dequant8(x.v_lo, sc, of);
            *(lds_uint4*)(rowp + (((2 * u8_piece + 1) ^ (4 * (u8_row & 3))) << 4)) = dequant8(x.v_hi, sc, of);
        }
    };
    // the workgroup barrier of the u8 variant: LDS writes done, register loads may stay in flight
    auto phase_barrier = [&](int keep) __attribute__((always_inline)) {
        if constexpr (kU8)
            barrier_keeping<63>();
        else
            barrier_keeping_loads(keep);
    };

    // Dense K/V: tile j's eight rows of this wavefront are keys kv_lo + 64 j + 8 wave + [0, 8); for the
    // first fast_tiles tiles all of them exist, and their loads are two instructions on a source
    // address that advances by one tile per iteration (fill_k / fill_v: the rows of the tiles that
    // iteration j fills, K(j + group + 2) and V(j + group + 1)).
    int fast_tiles = 0;
    const uint8_t* fill_k = nullptr;
    const uint8_t* fill_v = nullptr;
    if constexpr (!kPaged) {
        const int room = t.kv_len - kv_lo - 8 * wave - 8;
        fast_tiles = room >= 0 ? min(n, room / kTileK + 1) : 0;
        fill_k = t.k + (int64_t)(kv_lo + (group + 2) * kTileK + 8 * wave) * grow;
        fill_v = t.v + (int64_t)(kv_lo + (group + 1) * kTileK + 8 * wave) * grow;
    }
    // Paged 16-bit caches: the same two instructions per tile whenever all eight rows exist; their source
    // addresses (block table entry times block stride plus the rows' place in the block) are worked out one
    // iteration ahead, at the end of a matrix phase.  fill_whole: both tiles of the coming batch are of that kind.
    bool fill_whole = false;
    auto whole_rows = [&](int j) __attribute__((always_inline)) { return j < n && kv_lo + j * kTileK + 8 * wave + 8 <= t.kv_len; };

    // ---- prologue: K(0), V(0), K(1); group 1 also issues its rows of B(0)
    const int e0 = table_entry(0), e1 = table_entry(1), e2 = table_entry(2), e3 = table_entry(3);
    int first = 0, recent = 0;
    U8Rows pending;  // u8: rows fetched in one iteration, dequantised and written in the next
    pending.jk = pending.jv = -1;
    if constexpr (kU8) {
        const U8Rows a = u8_fetch(0, e0, 0, e0), b = u8_fetch(1, e1, n, 0);
        if (group == 1) pending = u8_fetch(2, e2, 1, e1);  // its rows of B(0), written in the first iteration
        u8_store(a);
        u8_store(b);
    } else {
        first = load_rows(true, 0, k_stage(0), e0) + load_rows(false, 0, v_stage(0), e0) +
                load_rows(true, 1, k_stage(1), e1);
        if (group == 1) recent = load_rows(true, 2, k_stage(2), e2) + load_rows(false, 1, v_stage(1), e1);
    }
    // entries of the tiles the first iteration loads: K(group + 2) and V(group + 1)
    int entry_v = group ? e2 : e1, entry_k = group ? e3 : e2;
    if constexpr (kPaged && !kU8) {
        fill_whole = whole_rows(group + 2);  // (then the rows of V(group + 1) exist as well)
        fill_k = row_group_base(t, t.k, kv_lo + (group + 2) * kTileK + 8 * wave, entry_k, grow);
        fill_v = row_group_base(t, t.v, kv_lo + (group + 1) * kTileK + 8 * wave, entry_v, grow);
    }
    // The query rows were issued first and nobody else reads them: they are converted while the
    // K and V tiles are still on their way.
    if constexpr (kU8)
        wait_keeping<0>();
    else
        wait_keeping_loads(first + recent);
    // Q^T operand: k-step i covers head-dim i*16 + hi*8 .. +8
    vec8 qf[8];
    {
        typedef __attribute__((address_space(3))) uint4_t lds_uint4;
        uint4_t raw[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            raw[i] = uint4_t{0u, 0u, 0u, 0u};
            if (t.rows > 0 && (!kPad || 2 * i + hi < head_chunks)) raw[i] = *(const lds_uint4*)(wave_stage + (f.k ^ (i << 5)));
        }
        if (t.q_dtype == HIPATTN_BF16) {  // (one wave-uniform branch, not a choice per element)
#pragma unroll
            for (int i = 0; i < 8; i++) qf[i] = convert_q_frag<kBf16, true>(raw[i], c);
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) qf[i] = convert_q_frag<kBf16, false>(raw[i], c);
        }
    }
#pragma unroll
    for (int i = 0; i < 8; i++) asm volatile("" : "+v"(qf[i]));  // (converted before the wait below, not after)
    bool check_blocks = false;  // wave-uniform: the window of the table the loop is in has an entry outside the cache
    if constexpr (kPaged) {
        bool bad_lane = false;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            asm volatile("" : "+v"(scan_ids[u]));  // (looked at here, not where they were loaded)
            bad_lane = bad_lane || scan_ids[u] >= (uint32_t)t.num_blocks;
        }
        check_blocks = __builtin_amdgcn_ballot_w64(bad_lane) != 0;
    }
    // which sixteenths of tile j lie in blocks the table does not name (only ever called when check_blocks)
    auto bad_sixteenths = [&](int j) -> uint32_t {
        uint32_t bits = 0;
        if constexpr (kPaged) {
            const int key0 = kv_lo + j * kTileK;
            const int32_t* const first = t.table + (key0 >> t.block_shift);
            const auto bad = [&](int entry) { return (uint32_t)entry >= (uint32_t)t.num_blocks; };
            if (key0 + kTileK <= t.kv_len && t.block_shift >= 4) {
                // the whole tile exists: its one, two or four entries in one scalar load (waited for inside the
                // statement: no LDS read is outstanding at the head of a vector phase)
                if (t.block_shift >= 6) {
                    int e0;
                    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(e0) : "s"(first));
                    bits = bad(e0) ? 0xfu : 0u;
                } else if (t.block_shift == 5) {
                    uint2_t e;
                    asm volatile("s_load_dwordx2 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(e) : "s"(first));
                    bits = (bad((int)e[0]) ? 0x3u : 0u) | (bad((int)e[1]) ? 0xcu : 0u);
                } else {
                    uint4_t e;
                    asm volatile("s_load_dwordx4 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(e) : "s"(first));
#pragma unroll
                    for (int b = 0; b < 4; b++) bits |= bad((int)e[b]) ? 1u << b : 0u;
                }
            } else {
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    const int k = key0 + 16 * b;
                    if (k >= t.kv_len) continue;  // (keys past the end are masked as such)
                    int entry;
                    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(entry) : "s"(t.table + (k >> t.block_shift)));
                    if (bad(entry)) bits |= 1u << b;
                }
            }
        }
        return bits;
    };
    if constexpr (kMask != 0) recent += load_mask_tile(0);  // the query rows have left the stage
    phase_barrier(recent);
    if (group == 1) phase_barrier(recent);  // group 1 sits out phase 0

    float16_t s[2];
    vec8 pf[4];
    tile_scores<kBf16>(k_stage(0), f, qf, st.neg_ref, s);
    phase_barrier(recent);
    // The two phases of tile j.  Both groups run every tile of the workgroup's key range: a tile
    // outside a group's own range is fully masked and contributes probabilities of zero.  The
    // restrict qualifiers tell the compiler that the LDS writes of the asynchronous loads cannot
    // alias the fragment reads, so that it does not wait for all loads before every LDS read; the
    // barriers do the waiting that is needed.
    // The four stages an iteration touches walk round their rings in step: their indices are carried
    // (add, compare, select) instead of taking j modulo the ring length four times per iteration;
    // index * 16 KB keeps the stage addresses visibly aligned for the fragment address arithmetic.
    int i_kn = 1 % kStages, i_vc = 0, i_kf = (group + 2) % kStages, i_vf = (group + 1) % kStages;
    auto bump = [](int& i) __attribute__((always_inline)) { i = (i + 1 == kStages) ? 0 : i + 1; };
    auto two_phases = [&](int j, bool last) {
        const lds_byte* __restrict__ const k_next = k_ring + i_kn * kKBytes;
        const lds_byte* __restrict__ const v_cur = v_ring + i_vc * kKBytes;
        lds_byte* __restrict__ const k_fill = k_ring + i_kf * kKBytes;
        lds_byte* __restrict__ const v_fill = v_ring + i_vf * kKBytes;
        // ---- vector phase
        if constexpr (kU8) {
            // rows fetched one iteration ago go into their stages, two phases before their first
            // use; the rows of this iteration's batch are fetched into registers
            u8_store(pending);
            pending = u8_fetch(j + group + 2, entry_k, j + group + 1, entry_v);
        } else if constexpr (!kPaged) {
            if (j + group + 2 < fast_tiles) {  // then the rows of V(j + group + 1) exist as well
                lds_byte* const kd = k_fill + 8 * wave * kRowBytes;
                lds_byte* const vd = v_fill + 8 * wave * kRowBytes;
                load_to_lds_16(fill_k, k_lane, kd);
                load_to_lds_16(fill_k, k_lane1, kd + 4 * kRowBytes);
                load_to_lds_16(fill_v, v_lane, vd);
                load_to_lds_16(fill_v, v_lane1, vd + 4 * kRowBytes);
                recent = 4;
            } else {
                recent = load_rows(true, j + group + 2, k_fill, 0) + load_rows(false, j + group + 1, v_fill, 0);
            }
        } else {
            if (fill_whole) {
                lds_byte* const kd = k_fill + 8 * wave * kRowBytes;
                lds_byte* const vd = v_fill + 8 * wave * kRowBytes;
                load_to_lds_16(fill_k, k_lane, kd);
                load_to_lds_16(fill_k, k_lane1, kd + 4 * kRowBytes);
                load_to_lds_16(fill_v, v_lane, vd);
                load_to_lds_16(fill_v, v_lane1, vd + 4 * kRowBytes);
                recent = 4;
            } else {
                recent = load_rows(true, j + group + 2, k_fill, entry_k) + load_rows(false, j + group + 1, v_fill, entry_v);
            }
        }
        if constexpr (kMask != 0) {
            recent += load_mask_tile(j + 1);
            // tile j's mask was issued a vector phase ago, ahead of everything issued in this one
            wait_keeping_loads(recent);
            tile_softmax<kBf16, kMask>(t, s, o, st, pf, kv_lo + j * kTileK, my_pos, hi, true,
                                       mask_tile_staged(j) ? mask_stage(j) : nullptr, row);
        } else if constexpr (kPaged) {
            // the loop has reached entries nobody has looked at: the next window of the table
            const int tile_entry = (kv_lo + j * kTileK) >> t.block_shift;
            if (tile_entry + (kTileK >> t.block_shift) >= scan_end && tile_entry <= last_entry) {
                check_blocks = scan_now(tile_entry);
            }
            const uint32_t bad16 = check_blocks ? bad_sixteenths(j) : 0u;
            tile_softmax<kBf16>(t, s, o, st, pf, kv_lo + j * kTileK, my_pos, hi, !unmasked(j) || bad16 != 0, nullptr, 0, bad16);
        } else {
            tile_softmax<kBf16>(t, s, o, st, pf, kv_lo + j * kTileK, my_pos, hi, !unmasked(j));
        }
        // (the probabilities are complete before the barrier: the compiler may not move their
        // arithmetic into the matrix phase)
#pragma unroll
        for (int ks = 0; ks < 4; ks++) asm volatile("" : "+v"(pf[ks]));
        // the matrix phase runs at raised priority (set before the barrier, so that it holds from
        // the first instruction after it): otherwise the other group's instruction stream, which
        // never stalls for long, keeps this wavefront's MFMAs from issuing
        __builtin_amdgcn_s_setprio(3);
        if (group == 0) phase_barrier(recent);  // (group 1 passes from its vector phase straight into its matrix phase)
        // ---- matrix phase
        // fragment addresses of this tile: per-lane offset + stage address, so that every read is
        // one XOR with a constant plus an immediate offset (the stage addresses are multiples of
        // 16 KB and leave the XORed bits alone)
        FragOffsets fs;
        fs.k = f.k + (int)(uintptr_t)k_next;
        fs.v = f.v + (int)(uintptr_t)v_cur;
        const lds_byte* const zero = (const lds_byte*)0;
        if (!last)
            tile_accumulate_and_scores<kBf16>(zero, zero, fs, pf, o, qf, st.neg_ref, s);
        else
            tile_accumulate<kBf16>(zero, fs, pf, o);
        __builtin_amdgcn_s_setprio(0);
        // The next iteration's stages and source rows are worked out here, where the wavefront would
        // otherwise only wait at the barrier for the other group's vector phase; behind the barrier
        // this scalar arithmetic would sit at the head of its own vector phase.
        bump(i_kn);
        bump(i_vc);
        bump(i_kf);
        bump(i_vf);
        if constexpr (kPaged) {
            // (every fragment read of the matrix phase has been waited for by now, so the scalar
            // load's own wait costs the phase nothing)
            entry_v = entry_k;  // the next iteration loads V of the tile whose K was loaded now
            entry_k = table_entry(j + group + 3);
            if constexpr (!kU8) {
                fill_v = t.v + (fill_k - t.k);  // the same rows of the same block
                fill_whole = whole_rows(j + group + 3);
                fill_k = row_group_base(t, t.k, kv_lo + (j + group + 3) * kTileK + 8 * wave, entry_k, grow);
                asm volatile("" : "+s"(fill_k), "+s"(fill_v));
            }
        }
        if constexpr (!kPaged) {
            fill_k += kTileK * grow;
            fill_v += kTileK * grow;
            asm volatile("" : "+s"(fill_k), "+s"(fill_v));
        }
        asm volatile("" : "+s"(i_kn), "+s"(i_vc), "+s"(i_kf), "+s"(i_vf));
        if (group == 1) phase_barrier(recent);
    };
    for (int j = 0; j < n - 1; j++) two_phases(j, false);
    two_phases(n - 1, true);

    // ---- normalise and store
    float l_lo, l_hi;
    pair_values(st.l_run, l_lo, l_hi);
    const float l_row = l_lo + l_hi;
    const float inv = l_row > 0.0f ? 1.0f / l_row : 0.0f;
    lds_byte* const out_stage = wave_stage;
    const int row0 = (wave & 3) * 32;
    if (t.out_dtype == HIPATTN_F32) {
        if (row < t.rows) store_rows<HIPATTN_F32>(t, o, inv, row, hi);
    } else if (t.out_dtype == HIPATTN_F16) {
        store_rows_via_lds<false>(t, o, inv, out_stage, row0, lane);
    } else {
        store_rows_via_lds<true>(t, o, inv, out_stage, row0, lane);
    }
    // as many barriers as group 1, whose last phase runs while group 0 stores its rows
    if (group == 0) phase_barrier(0);
}

// Launch index -> work item: workgroups go to the eight XCDs round-robin by launch index and
// each XCD has its own L2, so index i becomes item (i % 8) * (n / 8) + i / 8.  An XCD then walks
// a contiguous range of items ordered (batch, kv head, query tile descending, pair): the
// workgroups resident on it at one time share one K/V head, which stays in that L2, and the
// heaviest (latest) causal tiles of a head come first.  With an even number of query heads per
// kv head the two groups of a workgroup take two heads at the same query tile; otherwise they
// take two consecutive query tiles of one head.
// a / b for wave-uniform 0 <= a < 2^22 and 1 <= b < 2^22: a float reciprocal and one correction
// step instead of the long 32-bit division sequence.
__device__ __forceinline__ int small_div(int a, int b) {
    int q = (int)((float)a * __builtin_amdgcn_rcpf((float)b));  // off by at most one
    const int r = a - q * b;
    q += (r >= b) ? 1 : 0;
    q -= (r < 0) ? 1 : 0;
    return q;
}
template <bool kPad = false>
__device__ __forceinline__ Tile sdpa_group_tile(const SdpaParams& p, int group) {
    const int D = kPad ? p.head_dim : kD;
    const int G = small_div(p.num_heads_q, p.num_heads_kv);
    const int n_qt = (p.len_q + kTileQ - 1) / kTileQ;
    const bool pair_heads = (G & 1) == 0;
    const int slots = pair_heads ? n_qt : (n_qt + 1) / 2;  // query positions of a head's workgroups
    const int lanes = pair_heads ? G / 2 : G;              // workgroups per query position
    const int n_items = (int)gridDim.x;
    int item = (int)blockIdx.x;
    if ((n_items & 7) == 0) item = (item & 7) * (n_items >> 3) + (item >> 3);
    const int by_lane = small_div(item, lanes), li = item - by_lane * lanes;
    const int by_slot = small_div(by_lane, slots), slot = slots - 1 - (by_lane - by_slot * slots);
    const int b = small_div(by_slot, p.num_heads_kv), hkv = by_slot - b * p.num_heads_kv;
    const int h = hkv * G + (pair_heads ? 2 * li + group : li);
    const int qt = pair_heads ? slot : 2 * slot + group;
    Tile t;
    const int64_t qoff = (((int64_t)b * p.num_heads_q + h) * p.len_q + (int64_t)min(qt, n_qt - 1) * kTileQ) * D;
    t.q = (const uint16_t*)p.q + qoff;
    t.q_stride = D;
    t.out = (uint16_t*)p.out + qoff;
    t.out_stride = D;
    t.head_dim = D;
    t.rows = qt < n_qt ? min(kTileQ, p.len_q - qt * kTileQ) : 0;
    t.pos0 = qt * kTileQ;
    t.kv_len = p.len_kv;
    t.causal = p.causal;
    t.window = 0;
    t.q_dtype = p.dtype;
    t.out_dtype = p.dtype;
    const int64_t kvoff = ((int64_t)b * p.num_heads_kv + hkv) * p.len_kv * (D * 2);
    t.k = (const uint8_t*)p.k + kvoff;
    t.v = (const uint8_t*)p.v + kvoff;
    t.table = nullptr;
    t.table_len = 0;
    t.num_blocks = 0;
    t.block_stride = 0;
    t.block_size = 1;
    t.block_shift = 0;
    t.mask = nullptr;
    t.mask_row_bytes = 0;
    if (p.mask != nullptr) {
        const int64_t esz = p.mask_dtype == HIPATTN_U8 ? 1 : 2;
        t.mask = (const uint8_t*)p.mask +
                 ((int64_t)b * p.mask_stride[0] + (int64_t)h * p.mask_stride[1] + (int64_t)t.pos0 * p.mask_stride[2]) * esz;
        t.mask_row_bytes = p.mask_stride[2] * esz;
    }
    return t;
}

template <bool kBf16, bool kU8 = false, bool kPaged = true, int kMask = 0, bool kPad = false>
__device__ __forceinline__ void run_both(const Tile& t0, const Tile& t1, uint8_t* lds, float scale) {
    int lo0, hi0, lo1, hi1;
    key_range(t0, lo0, hi0);
    key_range(t1, lo1, hi1);
    int kv_lo, kv_hi;
    if (hi0 <= lo0) {
        kv_lo = lo1;
        kv_hi = hi1;
    } else if (hi1 <= lo1) {
        kv_lo = lo0;
        kv_hi = hi0;
    } else {
        kv_lo = min(lo0, lo1);
        kv_hi = max(hi0, hi1);
    }
    const int group = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8);
    run_pair<kBf16, kU8, kPaged, kMask, kPad>(group ? t1 : t0, kv_lo, kv_hi, lds, scale);
}

template <bool kBf16>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void sdpa_flash_kernel(SdpaParams p) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[kLdsBytes];
    const Tile t0 = sdpa_group_tile(p, 0), t1 = sdpa_group_tile(p, 1);
    run_both<kBf16, false, false>(t0, t1, lds, p.scale);
}

// The same for a head size between 64 and 128 (p.head_dim, a multiple of 8): the kPad form of the loop.
template <bool kBf16>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void sdpa_flash_padded_kernel(SdpaParams p) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[kLdsBytes];
    const Tile t0 = sdpa_group_tile<true>(p, 0), t1 = sdpa_group_tile<true>(p, 1);
    run_both<kBf16, false, false, 0, true>(t0, t1, lds, p.scale);
}

// The same with an attention mask (kMask 2: of the operands' type, added; 1: boolean bytes).
template <bool kBf16, int kMask>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void sdpa_flash_masked_kernel(SdpaParams p) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[kLdsBytes];
    const Tile t0 = sdpa_group_tile(p, 0), t1 = sdpa_group_tile(p, 1);
    run_both<kBf16, false, false, kMask>(t0, t1, lds, p.scale);
}

// ... and for a head size between 64 and 128.
template <bool kBf16, int kMask>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void sdpa_flash_masked_padded_kernel(SdpaParams p) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[kLdsBytes];
    const Tile t0 = sdpa_group_tile<true>(p, 0), t1 = sdpa_group_tile<true>(p, 1);
    run_both<kBf16, false, false, kMask, true>(t0, t1, lds, p.scale);
}

// One workgroup per (128-row query tile of a multi-token sequence, pair of query heads) or, with an
// odd number of query heads per kv head, per (pair of query tiles, query head).
template <bool kPad = false>
__device__ __forceinline__ Tile paged_group_tile(const PagedParams& p, int s, int qt, int h, bool has_work) {
    const int D = kPad ? p.head_dim : kD;
    const int G = p.num_heads_q / p.num_heads_kv;
    const int t0 = p.subsequence_begins[s];
    const int qlen = p.subsequence_begins[s + 1] - t0;
    const int past = p.past_lens[s];
    const int tb0 = p.block_indices_begins[s];
    const int table_len = p.block_indices_begins[s + 1] - tb0;
    Tile t;
    const int64_t row0 = (int64_t)(t0 + qt * kTileQ) * p.num_heads_q + h;
    t.q = (const uint16_t*)p.q + row0 * D;
    t.q_stride = (int64_t)p.num_heads_q * D;
    t.out = (p.out_dtype == HIPATTN_F32) ? (void*)((float*)p.out + row0 * D) : (void*)((uint16_t*)p.out + row0 * D);
    t.out_stride = (int64_t)p.num_heads_q * D;
    t.rows = has_work ? min(kTileQ, qlen - qt * kTileQ) : 0;
    t.pos0 = past + qt * kTileQ;
    t.kv_len = min(past + qlen, table_len * p.block_size);
    t.causal = 1;
    t.window = p.sliding_window;
    t.q_dtype = p.q_dtype;
    t.out_dtype = p.out_dtype;
    t.head_dim = D;
    const int row_bytes = p.cache_dtype == HIPATTN_U8 ? kU8RowBytes : D * 2;
    const int64_t head_off = (int64_t)(h / G) * p.block_size * row_bytes;
    t.k = p.key_cache + head_off;
    t.v = p.value_cache + head_off;
    t.table = p.block_indices + tb0;
    t.table_len = table_len;
    t.num_blocks = p.num_blocks;
    t.block_stride = (int64_t)p.num_heads_kv * p.block_size * row_bytes;
    t.block_size = p.block_size;
    t.block_shift = __builtin_ctz(p.block_size);
    t.mask = nullptr;
    t.mask_row_bytes = 0;
    return t;
}

// kPad: a head size between 64 and 128 (p.head_dim, a multiple of 8; 16-bit caches).
template <bool kBf16, bool kU8, bool kPad>
__device__ __forceinline__ void paged_prefill_item(const PagedParams& p, uint8_t* lds) {
    // Launch index -> work item.  The workgroups that run on one XCD at a time should share K/V in
    // its L2, and the XCDs should get equal work although sequences differ in length.  With a
    // multiple of eight kv heads, XCD x (launch index modulo 8) takes kv heads x, x + 8, ... of
    // every sequence; its items are ordered (sequence, kv head, query tile descending, head slot),
    // so the workgroups of one (sequence, kv head), which read the same K/V, run together.  Other
    // head counts keep that order without the split.  The number of items is only known here (the
    // grid is an upper bound): indices past the end leave at once.
    const int G = p.num_heads_q / p.num_heads_kv;
    const bool pair_heads = (G & 1) == 0;
    const int slots = pair_heads ? G / 2 : G;  // workgroups per (query tile, kv head)
    const bool split = (p.num_heads_kv & 7) == 0;
    const int heads_here = split ? p.num_heads_kv >> 3 : p.num_heads_kv;  // kv heads per sequence in this list
    const int per_tile = heads_here * slots;                              // items of the list per query tile
    const int items = p.tile_prefix[p.num_seqs] * per_tile;
    const int item = split ? (int)blockIdx.x >> 3 : (int)blockIdx.x;
    if (item >= items) return;
    // sequence owning the item: largest s with tile_prefix[s] * per_tile <= item
    int lo = 0, hi_s = p.num_seqs;
    while (hi_s - lo > 1) {
        const int mid = (lo + hi_s) >> 1;
        if (p.tile_prefix[mid] * per_tile <= item)
            lo = mid;
        else
            hi_s = mid;
    }
    const int s = lo;
    const int tiles_s = p.tile_prefix[s + 1] - p.tile_prefix[s];
    int r = item - p.tile_prefix[s] * per_tile;
    const int head_here = r / (tiles_s * slots);
    r -= head_here * tiles_s * slots;
    const int qt = tiles_s - 1 - r / slots;  // the later (heavier) tiles of a sequence first
    const int li = r % slots;
    const int hkv = split ? ((int)blockIdx.x & 7) + 8 * head_here : head_here;
    const int h0 = hkv * G + (pair_heads ? 2 * li : li);
    // The two groups take two query heads of the kv head at one query tile or, with an odd number
    // of query heads per kv head, two consecutive query tiles of one head: the item of the even
    // tile does both, the item of the odd tile has nothing left to do.
    if (!pair_heads && (qt & 1)) return;
    const Tile t0 = paged_group_tile<kPad>(p, s, qt, h0, true);
    const Tile t1 = pair_heads ? paged_group_tile<kPad>(p, s, qt, h0 + 1, true) : paged_group_tile<kPad>(p, s, qt + 1, h0, qt + 1 < tiles_s);
    run_both<kBf16, kU8, true, 0, kPad>(t0, t1, lds, p.scale);
}

template <bool kBf16, bool kU8>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void paged_prefill_kernel(PagedParams p) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[kLdsBytes];
    paged_prefill_item<kBf16, kU8, false>(p, lds);
}

// The same for a head size between 64 and 128 (16-bit caches): the kPad form of the loop.
template <bool kBf16>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void paged_prefill_padded_kernel(PagedParams p) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[kLdsBytes];
    paged_prefill_item<kBf16, false, true>(p, lds);
}

}  // namespace flash

// Head size 128, and the smaller head sizes that are multiples of 8, which run the same kernel with rows of
// fewer columns in memory (16-byte aligned operands; the option sdpa_padded_rows = 0 leaves them to the
// plain kernels).  Measured on 4 x 2,048 tokens, 32 / 8 heads, causal: head size 64 0.124 ms against 0.153 ms
// in the plain head-64 kernel, head size 32 0.120 ms.
bool sdpa_flash_supported(const SdpaParams& p) {
    if (!(p.dtype == HIPATTN_F16 || p.dtype == HIPATTN_BF16)) return false;
    if (p.head_dim != flash::kD) {
        const auto aligned16 = [](const void* q) { return ((uintptr_t)q & 15) == 0; };
        if (p.head_dim < 8 || p.head_dim > flash::kD || p.head_dim % 8 != 0 || !sdpa_padded_rows_enabled()) return false;
        if (!aligned16(p.q) || !aligned16(p.k) || !aligned16(p.v) || !aligned16(p.out)) return false;
    }
    // the kernel decodes its launch index with small_div: the number of workgroups must stay below 2^22
    const int64_t q_tiles = ((int64_t)p.len_q + flash::kTileQ - 1) / flash::kTileQ;
    return (int64_t)p.batch * p.num_heads_q * q_tiles < (int64_t(1) << 22);
}

// An attention mask the flash kernel takes: of the operands' type or boolean, its keys side by
// side, and every 16-byte piece the kernel loads aligned (the mask itself, and the steps from row
// to row, head to head and batch to batch; a step of 0 broadcasts).
bool sdpa_flash_mask_supported(const SdpaParams& p) {
    if (p.mask == nullptr || p.causal) return false;
    if (p.mask_dtype != p.dtype && p.mask_dtype != HIPATTN_U8) return false;
    if (p.mask_stride[3] != 1) return false;
    const int64_t per16 = p.mask_dtype == HIPATTN_U8 ? 16 : 8;
    if (((uintptr_t)p.mask & 15) != 0) return false;
    for (int i = 0; i < 3; i++)
        if (p.mask_stride[i] % per16 != 0) return false;
    return true;
}

hipError_t launch_sdpa_flash(const SdpaParams& p, hipStream_t stream, const KernelProbe& probe) {
    if (p.batch == 0 || p.len_q == 0) return hipSuccess;
    const int G = p.num_heads_q / p.num_heads_kv;
    const int n_qt = (p.len_q + flash::kTileQ - 1) / flash::kTileQ;
    const bool pair_heads = (G & 1) == 0;
    const int per_kv_head = pair_heads ? (G / 2) * n_qt : G * ((n_qt + 1) / 2);
    dim3 grid(per_kv_head * p.num_heads_kv * p.batch);
    if (probe.before) (void)hipEventRecord(probe.before, stream);
    const int mask = p.mask == nullptr ? 0 : (p.mask_dtype == HIPATTN_U8 ? 1 : 2);
    const dim3 block(flash::kThreads);
    if (p.head_dim != flash::kD) {  // (the kPad forms)
        if (p.dtype == HIPATTN_BF16) {
            if (mask == 0)
                hipLaunchKernelGGL(flash::sdpa_flash_padded_kernel<true>, grid, block, 0, stream, p);
            else if (mask == 2)
                hipLaunchKernelGGL((flash::sdpa_flash_masked_padded_kernel<true, 2>), grid, block, 0, stream, p);
            else
                hipLaunchKernelGGL((flash::sdpa_flash_masked_padded_kernel<true, 1>), grid, block, 0, stream, p);
        } else {
            if (mask == 0)
                hipLaunchKernelGGL(flash::sdpa_flash_padded_kernel<false>, grid, block, 0, stream, p);
            else if (mask == 2)
                hipLaunchKernelGGL((flash::sdpa_flash_masked_padded_kernel<false, 2>), grid, block, 0, stream, p);
            else
                hipLaunchKernelGGL((flash::sdpa_flash_masked_padded_kernel<false, 1>), grid, block, 0, stream, p);
        }
    } else if (p.dtype == HIPATTN_BF16) {
        if (mask == 0)
            hipLaunchKernelGGL(flash::sdpa_flash_kernel<true>, grid, block, 0, stream, p);
        else if (mask == 2)
            hipLaunchKernelGGL((flash::sdpa_flash_masked_kernel<true, 2>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((flash::sdpa_flash_masked_kernel<true, 1>), grid, block, 0, stream, p);
    } else {
        if (mask == 0)
            hipLaunchKernelGGL(flash::sdpa_flash_kernel<false>, grid, block, 0, stream, p);
        else if (mask == 2)
            hipLaunchKernelGGL((flash::sdpa_flash_masked_kernel<false, 2>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((flash::sdpa_flash_masked_kernel<false, 1>), grid, block, 0, stream, p);
    }
    hipError_t e = hipGetLastError();
    if (probe.after) (void)hipEventRecord(probe.after, stream);
    return e;
}

hipError_t launch_paged_prefill(const PagedParams& p, hipStream_t stream) {
    // the head sizes between 64 and 128 of a 16-bit cache: this kernel on rows of fewer columns
    const bool padded = p.head_dim > 64 && p.head_dim < flash::kD && p.head_dim % 8 == 0 && p.cache_dtype != HIPATTN_U8 &&
                        (((uintptr_t)p.q | (uintptr_t)p.key_cache | (uintptr_t)p.value_cache | (uintptr_t)p.out) & 15) == 0;
    // (ALiBi, attention sinks: the plain kernel has the distance term and the sink in its denominator; the tuned one
    // has no vector slot to spare for the one and was not given the other)
    if ((p.head_dim != flash::kD && !padded) || p.alibi_slopes || p.sinks) return launch_paged_prefill_small(p, stream);  // the plain kernel, padded columns
    const int G = p.num_heads_q / p.num_heads_kv;
    dim3 grid((unsigned)((int64_t)p.max_q_tiles * ((G & 1) == 0 ? p.num_heads_q / 2 : p.num_heads_q)));
    if (padded) {
        if (p.cache_dtype == HIPATTN_BF16)
            hipLaunchKernelGGL(flash::paged_prefill_padded_kernel<true>, grid, dim3(flash::kThreads), 0, stream, p);
        else
            hipLaunchKernelGGL(flash::paged_prefill_padded_kernel<false>, grid, dim3(flash::kThreads), 0, stream, p);
    } else if (p.cache_dtype == HIPATTN_BF16)
        hipLaunchKernelGGL((flash::paged_prefill_kernel<true, false>), grid, dim3(flash::kThreads), 0, stream, p);
    else if (p.cache_dtype == HIPATTN_U8)
        hipLaunchKernelGGL((flash::paged_prefill_kernel<false, true>), grid, dim3(flash::kThreads), 0, stream, p);
    else
        hipLaunchKernelGGL((flash::paged_prefill_kernel<false, false>), grid, dim3(flash::kThreads), 0, stream, p);
    return hipGetLastError();
}

}  // namespace hipattn
