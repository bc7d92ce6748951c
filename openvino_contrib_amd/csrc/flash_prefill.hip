// Flash-style attention for prefill on gfx950: dense v13::ScaledDotProductAttention and the
// multi-token (chunked prefill) sequences of PagedAttentionExtension share one kernel body.
//
// A workgroup of four wavefronts owns 128 query rows of one query head (32 rows per
// wavefront) and walks the keys in tiles of 64.  K and V tiles go from global memory straight
// into LDS (global_load_lds_dwordx4: no staging registers, no LDS write instructions), both
// row-major with the 16-byte chunks of a row XOR-swizzled so that fragment reads are free of
// bank conflicts; the V^T operand is read with the transposing LDS load ds_read_b64_tr_b16.
// LDS holds two stages: the loads of tile i+1 are issued at the top of iteration i into the
// stage that tile i-1 occupied, with one workgroup barrier per tile.  The kernel is held to 256
// registers so that two workgroups share a compute unit.  Both products run on
// v_mfma_f32_32x32x16 (f16 or bf16) with fp32 accumulation:
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

// Diagnostic build only (a probe that includes this file with HIPATTN_FLASH_TRACE defined):
// lane 0 of selected wavefronts stores the shader clock at the phase boundaries of every tile.
#ifdef HIPATTN_FLASH_TRACE
__device__ long long* g_flash_trace = nullptr;
__device__ long long* g_flash_wg_trace = nullptr;  // per workgroup: wall start/end (100 MHz), cycles start/end, hw id
struct PhaseClock {
    long long acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    long long last = 0;
};
// phase k = time since the previous stamp; totals are stored once, after the last tile
#define FLASH_STAMP(t, tile, k)                                                   \
    do {                                                                          \
        __builtin_amdgcn_sched_barrier(0);                                        \
        const long long stamp_ = (long long)__builtin_readcyclecounter();         \
        __builtin_amdgcn_sched_barrier(0);                                        \
        (t).clk.acc[k] += stamp_ - (t).clk.last;                                  \
        (t).clk.last = stamp_;                                                    \
    } while (0)
#else
#define FLASH_STAMP(t, tile, k) \
    do {                        \
    } while (0)
#endif

constexpr int kD = 128;
constexpr int kTileQ = 128;   // query rows per workgroup
constexpr int kTileK = 64;    // keys per LDS tile
constexpr int kThreads = 256;
constexpr int kRowBytes = kD * 2;                // a K or V row in LDS: 16 chunks of 16 bytes
constexpr int kKBytes = kTileK * kRowBytes;      // K part of a stage
constexpr int kStageBytes = 2 * kKBytes;         // K tile + V tile

#define HIPATTN_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define HIPATTN_GLOBAL_PTR(p) ((__attribute__((address_space(1))) void*)(p))

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
    // acc + lo + hi of a packed pair (v_dot2_f32_f16 against ones)
    static __device__ __forceinline__ float add_pair(uint32_t packed, float acc) {
        const half2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, packed), ones, acc, false);
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
    // acc + lo + hi of a packed pair (v_dot2_f32_bf16 against ones)
    static __device__ __forceinline__ float add_pair(uint32_t packed, float acc) {
        typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
        const bf16x2_t ones = {(__bf16)1.0f, (__bf16)1.0f};
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, packed), ones, acc, false);
    }
};

// What one workgroup works on.
struct Tile {
    const uint16_t* q;   // first query row of the tile, this head
    int64_t q_stride;    // elements between consecutive query rows
    void* out;           // output base (element (0,0) of the tile's first row, this head)
    int64_t out_stride;
    int rows;            // valid query rows (<= 128)
    int pos0;            // sequence position of query row 0
    int kv_len;          // keys available
    int causal;
    int window;
    int q_dtype;         // HIPATTN_F16 / HIPATTN_BF16 (converted to the MFMA type when they differ)
    int out_dtype;
    // keys / values
    const uint8_t* k;
    const uint8_t* v;
    const int32_t* table;   // paged: this sequence's block ids; dense: nullptr
    int table_len;
    int num_blocks;
    int64_t block_stride;   // paged: bytes between physical blocks
    int block_size;
    int block_shift;        // log2(block_size)
#ifdef HIPATTN_FLASH_TRACE
    long long* trace;
    mutable PhaseClock clk;
#endif
};

// Byte offset of a key's row from t.k / t.v.  Keys past the end are redirected to the last valid
// key and block ids outside the cache are clamped: such rows only ever meet a probability of
// zero (or are unspecified input), but they must be readable and finite.
__device__ __forceinline__ int64_t kv_row_offset(const Tile& t, int key) {
    key = min(key, t.kv_len - 1);
    if (t.table == nullptr) return (int64_t)key * kRowBytes;
    const int lb = key >> t.block_shift;  // block_size is a power of two on this path
    const int pb = min(max(t.table[lb], 0), t.num_blocks - 1);
    return (int64_t)pb * t.block_stride + (int64_t)(key & (t.block_size - 1)) * kRowBytes;
}

// Q fragment, multiplied by c = scale * log2(e) and rounded to the MFMA element type: the first
// product then yields the exponents of the softmax directly.
template <bool kBf16>
__device__ __forceinline__ typename Mfma<kBf16>::vec8 load_q_frag(const Tile& t, int row, int d0, float c) {
    using vec8 = typename Mfma<kBf16>::vec8;
    uint4_t raw = {0u, 0u, 0u, 0u};
    if (row < t.rows) raw = *(const uint4_t*)(t.q + (int64_t)row * t.q_stride + d0);
    const bool q_is_bf16 = (t.q_dtype == HIPATTN_BF16);
    uint4_t cv;
#pragma unroll
    for (int w = 0; w < 4; w++) {
        float lo, hi;
        if (q_is_bf16) {
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

typedef __attribute__((address_space(3))) uint8_t lds_byte;
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
struct FragOffsets {
    int k[8];  // + mt * 32 rows
    int v[4];  // per dt; + ks * 16 rows (+ 8 rows for the second half)
};

__device__ __forceinline__ FragOffsets frag_offsets(int lane) {
    FragOffsets f;
    const int n32 = lane & 31, hi = lane >> 5;
#pragma unroll
    for (int i = 0; i < 8; i++) f.k[i] = n32 * kRowBytes + (((2 * i + hi) ^ (n32 & 15)) << 4);
    const int g = lane >> 4, i16 = lane & 15;
    const int vrow = 4 * (g >> 1) + (i16 >> 2);  // row % 4 == i16 / 4
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
        f.v[dt] = vrow * kRowBytes + (((4 * dt + 2 * (g & 1) + ((i16 & 3) >> 1)) ^ (4 * (i16 >> 2))) << 4) + 8 * (i16 & 1);
    return f;
}

template <bool kBf16>
__device__ __forceinline__ typename Mfma<kBf16>::vec8 read_v_frag(const lds_byte* v_lds, const FragOffsets& f, int ks,
                                                                  int dt) {
    typedef __attribute__((address_space(3))) short4_t lds_short4;
    const lds_byte* p = v_lds + f.v[dt] + ks * 16 * kRowBytes;
    const short4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)p);
    const short4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(p + 8 * kRowBytes));
    typedef short short8_t __attribute__((ext_vector_type(8)));
    const short8_t a = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
    return __builtin_bit_cast(typename Mfma<kBf16>::vec8, a);
}

// One 64-key tile against this wavefront's 32 query rows.  `masked` is false for tiles that every
// query row of the workgroup sees completely (the common case).
//
// LDS latency is taken out of the MFMA chains by issuing fragment reads in batches ahead of
// their use: all sixteen K fragments before the first score MFMA, and the first half of the V^T
// fragments right behind the score MFMAs, so that they arrive during the softmax arithmetic.
//
// Online softmax with a lazily updated reference.  The scores come out of the first product as
// exponents x = s c - ref, because Q carries the factor c and the accumulator of the product is
// initialised with -ref (a 16-register tuple per lane: all sixteen belong to one query row), so
// a probability costs one v_exp_f32 and half a conversion.  p = exp2(x) is a valid numerator for
// any reference as long as it cannot overflow: ref is raised, and the accumulators rescaled,
// only when some row's largest exponent exceeds 8, which after the first few tiles is rare.
// Row sums are taken from the rounded probabilities, two per v_dot2 instruction.
struct SoftmaxState {
    float16_t neg_ref;  // -ref in every element
    float l_run;        // this lane's half of the row sum
    bool started;       // the row has met a key it may attend to
};

template <bool kBf16, typename AfterScores>
__device__ __forceinline__ void consume_tile(const Tile& t, const lds_byte* k_lds, const lds_byte* v_lds,
                                             const FragOffsets& f, const typename Mfma<kBf16>::vec8 (&qf)[8],
                                             float16_t (&o)[4], SoftmaxState& st, int ts, int my_pos, int hi, bool masked,
                                             AfterScores&& after_scores) {
    using M = Mfma<kBf16>;
    using vec8 = typename M::vec8;
    typedef __attribute__((address_space(3))) vec8 lds_vec8;
    // ---- S^T = K Q^T
    vec8 kf[2][8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int mt = 0; mt < 2; mt++) kf[mt][i] = *(const lds_vec8*)(k_lds + f.k[i] + mt * 32 * kRowBytes);
    __builtin_amdgcn_sched_barrier(0);
    float16_t s[2];
#pragma unroll
    for (int mt = 0; mt < 2; mt++) s[mt] = M::mma(kf[mt][0], qf[0], st.neg_ref);
#pragma unroll
    for (int i = 1; i < 8; i++)
#pragma unroll
        for (int mt = 0; mt < 2; mt++) s[mt] = M::mma(kf[mt][i], qf[i], s[mt]);
    vec8 vf[2][4];
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++) vf[ks][dt] = read_v_frag<kBf16>(v_lds, f, ks, dt);
    after_scores();
    FLASH_STAMP(t, ts / kTileK, 1);
    // ---- mask (register r of tile mt is key ts + mt*32 + 8*(r/4) + 4*hi + r%4) and row maximum
    if (masked) {
#pragma unroll
        for (int mt = 0; mt < 2; mt++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int key = ts + mt * 32 + 8 * (r >> 2) + 4 * hi + (r & 3);
                bool ok = key < t.kv_len;
                if (t.causal) ok = ok && key <= my_pos;
                if (t.window > 0) ok = ok && key > my_pos - t.window;
                s[mt][r] = ok ? s[mt][r] : -INFINITY;
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
    }
    float lsum = st.l_run;
    vec8 pf[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        uint4_t pw;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float p0 = fast_exp2(s[ks >> 1][(ks & 1) * 8 + 2 * w]);
            const float p1 = fast_exp2(s[ks >> 1][(ks & 1) * 8 + 2 * w + 1]);
            pw[w] = M::cvt2(p0, p1);
            lsum = M::add_pair(pw[w], lsum);
        }
        pf[ks] = __builtin_bit_cast(vec8, pw);
    }
    st.l_run = lsum;
    FLASH_STAMP(t, ts / kTileK, 2);
    // ---- O^T += V^T P^T
    vec8 vg[2][4];
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++) vg[ks][dt] = read_v_frag<kBf16>(v_lds, f, 2 + ks, dt);
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++) o[dt] = M::mma(vf[ks][dt], pf[ks], o[dt]);
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++) o[dt] = M::mma(vg[ks][dt], pf[2 + ks], o[dt]);
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

// lds: two stages of (K tile, V tile); stage (i+1)%2 is filled while tile i is consumed, so the
// loop needs one workgroup barrier per tile.
template <bool kBf16>
__device__ __forceinline__ void run_tile(const Tile& t, uint8_t* lds_generic, float scale) {
    using M = Mfma<kBf16>;
    using vec8 = typename M::vec8;
    lds_byte* const lds = (lds_byte*)lds_generic;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int n32 = lane & 31, hi = lane >> 5;
    const int row = wave * 32 + n32;  // query row inside the tile
    const float c = scale * kLog2e;

    // Q^T operand: k-step i covers head-dim i*16 + hi*8 .. +8
    vec8 qf[8];
#pragma unroll
    for (int i = 0; i < 8; i++) qf[i] = load_q_frag<kBf16>(t, row, i * 16 + hi * 8, c);

    // key range this tile has to visit
    int kv_hi = t.kv_len;
    if (t.causal) kv_hi = min(kv_hi, t.pos0 + t.rows);
    int kv_lo = 0;
    if (t.window > 0) kv_lo = max(0, t.pos0 - t.window + 1);
    kv_lo = (kv_lo / kTileK) * kTileK;

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
    const int my_pos = t.pos0 + row;  // position of this lane's query row
    const FragOffsets f = frag_offsets(lane);

    // global -> LDS: one instruction moves four rows (64 lanes x 16 bytes, LDS address = wave-uniform
    // base + lane * 16); wavefront w issues the four instructions of rows 16w .. 16w + 15 of the K
    // tile and of the V tile.  Lane l fills chunk position l % 16 of row 16w + 4k + l / 16, i.e. it
    // fetches chunk (l % 16) ^ swz(row).
    const int lrow = lane >> 4, lpos = lane & 15;
    auto load_k_tile = [&](int tile_start, lds_byte* k_lds) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int r = 16 * wave + 4 * k + lrow;
            const int64_t off = kv_row_offset(t, tile_start + r) + ((lpos ^ (r & 15)) << 4);
            __builtin_amdgcn_global_load_lds(HIPATTN_GLOBAL_PTR(t.k + off), HIPATTN_LDS_PTR(k_lds + (16 * wave + 4 * k) * kRowBytes),
                                             16, 0, 0);
        }
    };
    auto load_v_tile = [&](int tile_start, lds_byte* v_lds) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int r = 16 * wave + 4 * k + lrow;
            const int64_t off = kv_row_offset(t, tile_start + r) + ((lpos ^ (4 * (r & 3))) << 4);
            __builtin_amdgcn_global_load_lds(HIPATTN_GLOBAL_PTR(t.v + off), HIPATTN_LDS_PTR(v_lds + (16 * wave + 4 * k) * kRowBytes),
                                             16, 0, 0);
        }
    };

    if (kv_lo < kv_hi) {
        load_k_tile(kv_lo, lds);
        load_v_tile(kv_lo, lds + kKBytes);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wavefront's rows are in LDS
    __syncthreads();
    int stage = 0;
#ifdef HIPATTN_FLASH_TRACE
    t.clk.last = (long long)__builtin_readcyclecounter();
#endif
    // `cur` and `next` are the two stages: the restrict qualifiers tell the compiler that the LDS
    // writes of the asynchronous loads cannot alias the fragment reads of the same iteration, so
    // that it does not wait for the loads before every LDS read.
    auto iteration = [&](int ts, const lds_byte* __restrict__ cur, lds_byte* __restrict__ next) {
        const bool has_next = ts + kTileK < kv_hi;
        FLASH_STAMP(t, ts / kTileK, 0);
        if (has_next) {
            load_k_tile(ts + kTileK, next);
            load_v_tile(ts + kTileK, next + kKBytes);
        }
        FLASH_STAMP(t, ts / kTileK, 5);
        const bool all_valid = (ts + kTileK <= t.kv_len) && (!t.causal || ts + kTileK <= t.pos0 + 1) &&
                               (t.window <= 0 || ts >= t.pos0 + t.rows - t.window);
        consume_tile<kBf16>(t, cur, cur + kKBytes, f, qf, o, st, ts, my_pos, hi, !all_valid, [&] {});
        FLASH_STAMP(t, ts / kTileK, 3);
    };
    for (int ts = kv_lo; ts < kv_hi; ts += kTileK) {
        // the other stage was last read one iteration ago; every wavefront has passed the barrier
        // that ended that iteration
        iteration(ts, lds + stage * kStageBytes, lds + (stage ^ 1) * kStageBytes);
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
        __syncthreads();
        FLASH_STAMP(t, ts / kTileK, 6);
        stage ^= 1;
    }

#ifdef HIPATTN_FLASH_TRACE
    if (t.trace)
        for (int k = 0; k < 8; k++) t.trace[k] = t.clk.acc[k];
#endif
    // ---- normalise and store
    float l_lo, l_hi;
    pair_values(st.l_run, l_lo, l_hi);
    const float l_row = l_lo + l_hi;
    const float inv = l_row > 0.0f ? 1.0f / l_row : 0.0f;
    if (row < t.rows) {
        if (t.out_dtype == HIPATTN_F32)
            store_rows<HIPATTN_F32>(t, o, inv, row, hi);
        else if (t.out_dtype == HIPATTN_F16)
            store_rows<HIPATTN_F16>(t, o, inv, row, hi);
        else
            store_rows<HIPATTN_BF16>(t, o, inv, row, hi);
    }
}

// Launch index -> work item: workgroups go to the eight XCDs round-robin by launch index and
// each XCD has its own L2, so index i becomes item (i % 8) * (n / 8) + i / 8.  An XCD then walks
// a contiguous range of items ordered (batch, kv head, query tile descending, query head in
// group): the workgroups resident on it at one time share one K/V head, which stays in that L2,
// and the heaviest (latest) causal tiles of a head come first.
struct SdpaItem {
    int b, h, qt;
};
__device__ __forceinline__ SdpaItem sdpa_item(const SdpaParams& p, int n_tiles) {
    const int G = p.num_heads_q / p.num_heads_kv;
    const int n_items = (int)gridDim.x;
    int item = (int)blockIdx.x;
    if ((n_items & 7) == 0) item = (item & 7) * (n_items >> 3) + (item >> 3);
    SdpaItem it;
    it.qt = n_tiles - 1 - (item / G) % n_tiles;
    it.h = ((item / (G * n_tiles)) % p.num_heads_kv) * G + item % G;
    it.b = item / (G * n_tiles * p.num_heads_kv);
    return it;
}

__device__ __forceinline__ Tile sdpa_tile(const SdpaParams& p, const SdpaItem& it, int tile_rows) {
    const int G = p.num_heads_q / p.num_heads_kv;
    Tile t;
    const int64_t qoff = (((int64_t)it.b * p.num_heads_q + it.h) * p.len_q + (int64_t)it.qt * tile_rows) * kD;
    t.q = (const uint16_t*)p.q + qoff;
    t.q_stride = kD;
    t.out = (uint16_t*)p.out + qoff;
    t.out_stride = kD;
    t.rows = min(tile_rows, p.len_q - it.qt * tile_rows);
    t.pos0 = it.qt * tile_rows;
    t.kv_len = p.len_kv;
    t.causal = p.causal;
    t.window = 0;
    t.q_dtype = p.dtype;
    t.out_dtype = p.dtype;
    const int64_t kvoff = ((int64_t)it.b * p.num_heads_kv + it.h / G) * p.len_kv * (kD * 2);
    t.k = (const uint8_t*)p.k + kvoff;
    t.v = (const uint8_t*)p.v + kvoff;
    t.table = nullptr;
    t.table_len = 0;
    t.num_blocks = 0;
    t.block_stride = 0;
    t.block_size = 1;
    t.block_shift = 0;
    return t;
}

template <bool kBf16>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void sdpa_flash_kernel(SdpaParams p) {
#ifdef HIPATTN_FLASH_LDS_PAD  // diagnostic: forces one workgroup per compute unit
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * kStageBytes + HIPATTN_FLASH_LDS_PAD];
#else
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * kStageBytes];
#endif
    const int n_tiles = (p.len_q + kTileQ - 1) / kTileQ;
    const SdpaItem it = sdpa_item(p, n_tiles);
    Tile t = sdpa_tile(p, it, kTileQ);
#ifdef HIPATTN_FLASH_TRACE
    {
        const int wg = it.h + p.num_heads_q * it.b;
        t.trace = (g_flash_trace && it.qt == n_tiles - 1 && (threadIdx.x & 63) == 0)
                      ? g_flash_trace + (int64_t)(wg * 4 + (threadIdx.x >> 6)) * 8
                      : nullptr;
    }
#endif
#ifdef HIPATTN_FLASH_TRACE
    long long w0 = 0, c0 = 0;
    if (g_flash_wg_trace) {
        w0 = wall_clock64();
        c0 = (long long)__builtin_readcyclecounter();
    }
#endif
    run_tile<kBf16>(t, lds, p.scale);
#ifdef HIPATTN_FLASH_TRACE
    if (g_flash_wg_trace && threadIdx.x == 0) {
        long long* r = g_flash_wg_trace + (int64_t)blockIdx.x * 8;
        r[0] = w0;
        r[1] = wall_clock64();
        r[2] = c0;
        r[3] = (long long)__builtin_readcyclecounter();
        r[4] = __builtin_amdgcn_s_getreg((31 << 11) | 4);   // HW_ID
        r[5] = __builtin_amdgcn_s_getreg((31 << 11) | 20);  // XCC_ID
        r[6] = it.qt;
    }
#endif
}

// (not held to 256 registers: with the block-table addressing on top that would spill)
template <bool kBf16>
__global__ __launch_bounds__(kThreads) void paged_prefill_kernel(PagedParams p) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * kStageBytes];
    const int total = p.tile_prefix[p.num_seqs];
    const int tile_id = total - 1 - (int)blockIdx.x;
    if (tile_id < 0) return;
    // sequence owning this tile: largest s with tile_prefix[s] <= tile_id
    int lo = 0, hi_s = p.num_seqs;
    while (hi_s - lo > 1) {
        const int mid = (lo + hi_s) >> 1;
        if (p.tile_prefix[mid] <= tile_id)
            lo = mid;
        else
            hi_s = mid;
    }
    const int s = lo;
    const int qt = tile_id - p.tile_prefix[s];
    const int h = blockIdx.y;
    const int G = p.num_heads_q / p.num_heads_kv;
    const int t0 = p.subsequence_begins[s];
    const int qlen = p.subsequence_begins[s + 1] - t0;
    const int past = p.past_lens[s];
    const int tb0 = p.block_indices_begins[s];
    const int table_len = p.block_indices_begins[s + 1] - tb0;
    Tile t;
    const int64_t row0 = (int64_t)(t0 + qt * kTileQ) * p.num_heads_q + h;
    t.q = (const uint16_t*)p.q + row0 * kD;
    t.q_stride = (int64_t)p.num_heads_q * kD;
    t.out = (p.out_dtype == HIPATTN_F32) ? (void*)((float*)p.out + row0 * kD) : (void*)((uint16_t*)p.out + row0 * kD);
    t.out_stride = (int64_t)p.num_heads_q * kD;
    t.rows = min(kTileQ, qlen - qt * kTileQ);
    t.pos0 = past + qt * kTileQ;
    t.kv_len = min(past + qlen, table_len * p.block_size);
    t.causal = 1;
    t.window = p.sliding_window;
    t.q_dtype = p.q_dtype;
    t.out_dtype = p.out_dtype;
    const int64_t head_off = (int64_t)(h / G) * p.block_size * (kD * 2);
    t.k = p.key_cache + head_off;
    t.v = p.value_cache + head_off;
    t.table = p.block_indices + tb0;
    t.table_len = table_len;
    t.num_blocks = p.num_blocks;
    t.block_stride = (int64_t)p.num_heads_kv * p.block_size * (kD * 2);
    t.block_size = p.block_size;
    t.block_shift = __builtin_ctz(p.block_size);
#ifdef HIPATTN_FLASH_TRACE
    t.trace = nullptr;
#endif
    run_tile<kBf16>(t, lds, p.scale);
}

}  // namespace flash

bool sdpa_flash_supported(const SdpaParams& p) {
    return p.head_dim == flash::kD && (p.dtype == HIPATTN_F16 || p.dtype == HIPATTN_BF16);
}

hipError_t launch_sdpa_flash(const SdpaParams& p, hipStream_t stream, const KernelProbe& probe) {
    if (p.batch == 0 || p.len_q == 0) return hipSuccess;
    const int n_tiles = (p.len_q + flash::kTileQ - 1) / flash::kTileQ;
    dim3 grid(n_tiles * p.num_heads_q * p.batch);
    if (probe.before) (void)hipEventRecord(probe.before, stream);
    if (p.dtype == HIPATTN_BF16)
        hipLaunchKernelGGL(flash::sdpa_flash_kernel<true>, grid, dim3(flash::kThreads), 0, stream, p);
    else
        hipLaunchKernelGGL(flash::sdpa_flash_kernel<false>, grid, dim3(flash::kThreads), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (probe.after) (void)hipEventRecord(probe.after, stream);
    return e;
}

hipError_t launch_paged_prefill(const PagedParams& p, hipStream_t stream) {
    dim3 grid(p.max_q_tiles, p.num_heads_q);
    if (p.cache_dtype == HIPATTN_BF16)
        hipLaunchKernelGGL(flash::paged_prefill_kernel<true>, grid, dim3(flash::kThreads), 0, stream, p);
    else
        hipLaunchKernelGGL(flash::paged_prefill_kernel<false>, grid, dim3(flash::kThreads), 0, stream, p);
    return hipGetLastError();
}

}  // namespace hipattn
