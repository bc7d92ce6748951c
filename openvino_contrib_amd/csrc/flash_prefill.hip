// Flash-style attention for prefill on gfx950: dense v13::ScaledDotProductAttention and the
// multi-token (chunked prefill) sequences of PagedAttentionExtension share one kernel body.
//
// A workgroup of four wavefronts owns 128 query rows of one query head (32 rows per
// wavefront) and walks the keys in tiles of 64.  K tiles are staged in LDS row-major, V tiles
// transposed (the 4x8 patch each thread loads is transposed in registers on the way in).  LDS
// holds two stages: while tile i is consumed, tile i+1 is written to the other stage and the
// global loads of tile i+2 are in flight, with one workgroup barrier per tile.  The kernel is
// held to 256 registers so that two workgroups share a compute unit and one workgroup's MFMA
// phase overlaps the other's softmax arithmetic.  Both products
// run on v_mfma_f32_32x32x16 (f16 or bf16) with fp32 accumulation:
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
constexpr int kKRow = 272;    // bytes per K row in LDS (256 + 16 pad)
constexpr int kVRow = 136;    // bytes per V^T row in LDS (64 keys * 2 + 8 pad)
constexpr int kKBytes = kTileK * kKRow;          // K part of a stage
constexpr int kStageBytes = kKBytes + kD * kVRow;  // K tile + V^T tile

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

__device__ __forceinline__ int64_t kv_row_offset(const Tile& t, int key, bool& ok) {
    ok = key < t.kv_len;
    if (!ok) return 0;
    if (t.table == nullptr) return (int64_t)key * (kD * 2);
    const int lb = key >> t.block_shift;  // block_size is a power of two on this path
    const int pb = t.table[lb];
    if (pb < 0 || pb >= t.num_blocks) {
        ok = false;
        return 0;
    }
    return (int64_t)pb * t.block_stride + (int64_t)(key & (t.block_size - 1)) * (kD * 2);
}

template <bool kBf16>
__device__ __forceinline__ typename Mfma<kBf16>::vec8 load_q_frag(const Tile& t, int row, int d0) {
    using vec8 = typename Mfma<kBf16>::vec8;
    uint4_t raw = {0u, 0u, 0u, 0u};
    if (row < t.rows) raw = *(const uint4_t*)(t.q + (int64_t)row * t.q_stride + d0);
    const bool q_is_bf16 = (t.q_dtype == HIPATTN_BF16);
    if (q_is_bf16 == kBf16) return __builtin_bit_cast(vec8, raw);
    // widen through fp32 and round to the MFMA element type
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
        cv[w] = (uint32_t)Mfma<kBf16>::cvt(lo) | ((uint32_t)Mfma<kBf16>::cvt(hi) << 16);
    }
    return __builtin_bit_cast(vec8, cv);
}

// One 64-key tile against this wavefront's 32 query rows.  kMasked is false for tiles that every
// query row of the workgroup sees completely (the common case), so that the inner loops carry no
// per-element predicate at all.
//
// Online softmax with a lazily updated reference: p = exp2((s - m_ref) c) is a valid numerator
// for any reference m_ref as long as it cannot overflow, so the accumulators are rescaled only
// when some row's maximum has grown by more than 2^8 (exp2 domain) over its reference, which
// after the first few tiles is rare.
template <bool kBf16, bool kMasked>
__device__ __forceinline__ void consume_tile(const Tile& t, const uint8_t* k_lds, const uint8_t* v_lds,
                                             const typename Mfma<kBf16>::vec8 (&qf)[8], float16_t (&o)[4],
                                             float& m_ref, float& l_run, float c, int ts, int my_pos, int n32,
                                             int hi) {
    using M = Mfma<kBf16>;
    using vec8 = typename M::vec8;
    // ---- S^T = K Q^T
    float16_t s[2];
#pragma unroll
    for (int mt = 0; mt < 2; mt++) {
#pragma unroll
        for (int r = 0; r < 16; r++) s[mt][r] = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const vec8 a = *(const vec8*)(k_lds + (mt * 32 + n32) * kKRow + (i * 16 + hi * 8) * 2);
            s[mt] = M::mma(a, qf[i], s[mt]);
        }
    }
    FLASH_STAMP(t, ts / kTileK, 1);
    // ---- mask (register r of tile mt is key ts + mt*32 + 8*(r/4) + 4*hi + r%4) and row maximum
    float m_tile = -INFINITY;
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            if constexpr (kMasked) {
                const int key = ts + mt * 32 + 8 * (r >> 2) + 4 * hi + (r & 3);
                bool ok = key < t.kv_len;
                if (t.causal) ok = ok && key <= my_pos;
                if (t.window > 0) ok = ok && key > my_pos - t.window;
                s[mt][r] = ok ? s[mt][r] : -INFINITY;
            }
            m_tile = fmaxf(m_tile, s[mt][r]);
        }
    m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, 64));  // the row lives in lanes l and l + 32
    const bool grow = m_tile * c > m_ref * c + 8.0f || (m_ref == -INFINITY && m_tile != -INFINITY);
    if (__builtin_amdgcn_ballot_w64(grow)) {
        const float m_new = fmaxf(m_ref, m_tile);
        const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;  // row with nothing to attend yet
        const float alpha = fast_exp2((m_ref - m_safe) * c);        // exp2(-inf) = 0 the first time
        l_run *= alpha;
#pragma unroll
        for (int dt = 0; dt < 4; dt++) o[dt] *= alpha;
        m_ref = m_new;
    }
    const float neg_mc = (m_ref == -INFINITY) ? 0.0f : -m_ref * c;
    float lsum = 0.0f;
    vec8 pf[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        uint4_t pw;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float p0 = fast_exp2(fmaf(s[ks >> 1][(ks & 1) * 8 + 2 * w], c, neg_mc));
            const float p1 = fast_exp2(fmaf(s[ks >> 1][(ks & 1) * 8 + 2 * w + 1], c, neg_mc));
            lsum += p0 + p1;
            pw[w] = M::cvt2(p0, p1);
        }
        pf[ks] = __builtin_bit_cast(vec8, pw);
    }
    l_run += lsum;
    FLASH_STAMP(t, ts / kTileK, 2);
    // ---- O^T += V^T P^T
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
            const uint8_t* vrow = v_lds + (dt * 32 + n32) * kVRow + (ks * 16 + 4 * hi) * 2;
            const uint2_t a0 = *(const uint2_t*)(vrow);
            const uint2_t a1 = *(const uint2_t*)(vrow + 16);
            const uint4_t aw = {a0[0], a0[1], a1[0], a1[1]};
            o[dt] = M::mma(__builtin_bit_cast(vec8, aw), pf[ks], o[dt]);
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

// lds: two stages of (K tile, V^T tile); the stage for tile i+1 is filled while tile i is consumed,
// so the loop needs one workgroup barrier per tile.
template <bool kBf16>
__device__ __forceinline__ void run_tile(const Tile& t, uint8_t* lds, float scale) {
    using M = Mfma<kBf16>;
    using vec8 = typename M::vec8;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int n32 = lane & 31, hi = lane >> 5;
    const int row = wave * 32 + n32;  // query row inside the tile
    const float c = scale * kLog2e;

    // Q^T operand: k-step i covers head-dim i*16 + hi*8 .. +8
    vec8 qf[8];
#pragma unroll
    for (int i = 0; i < 8; i++) qf[i] = load_q_frag<kBf16>(t, row, i * 16 + hi * 8);

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
    float m_ref = -INFINITY, l_run = 0.0f;
    const int my_pos = t.pos0 + row;  // position of this lane's query row

    // global -> register staging: thread (c16, r16) loads 16-byte chunk c16 of K rows r16 + 16k
    // and chunk r16 of V rows c16*4 + j: the 16 lanes that share an LDS write instruction then
    // hold 16 consecutive key quads of one V^T row (a contiguous 128-byte write, no bank conflicts)
    const int c16 = tid & 15, r16 = tid >> 4;
    uint4_t kreg[4], vreg[4];
    auto load_regs = [&](int tile_start) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            bool ok;
            int64_t off = kv_row_offset(t, tile_start + r16 + 16 * k, ok);
            kreg[k] = ok ? *(const uint4_t*)(t.k + off + c16 * 16) : (uint4_t){0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            bool ok;
            int64_t off = kv_row_offset(t, tile_start + c16 * 4 + j, ok);
            vreg[j] = ok ? *(const uint4_t*)(t.v + off + r16 * 16) : (uint4_t){0u, 0u, 0u, 0u};
        }
    };
    auto store_lds = [&](uint8_t* k_lds, uint8_t* v_lds) {
#pragma unroll
        for (int k = 0; k < 4; k++) *(uint4_t*)(k_lds + (r16 + 16 * k) * kKRow + c16 * 16) = kreg[k];
#pragma unroll
        for (int e = 0; e < 8; e++) {
            uint2_t w;
            if (e & 1) {
                w[0] = (vreg[0][e >> 1] >> 16) | (vreg[1][e >> 1] & 0xffff0000u);
                w[1] = (vreg[2][e >> 1] >> 16) | (vreg[3][e >> 1] & 0xffff0000u);
            } else {
                w[0] = (vreg[0][e >> 1] & 0xffffu) | (vreg[1][e >> 1] << 16);
                w[1] = (vreg[2][e >> 1] & 0xffffu) | (vreg[3][e >> 1] << 16);
            }
            *(uint2_t*)(v_lds + (r16 * 8 + e) * kVRow + c16 * 8) = w;
        }
    };

    if (kv_lo < kv_hi) {
        load_regs(kv_lo);
        store_lds(lds, lds + kKBytes);
        if (kv_lo + kTileK < kv_hi) load_regs(kv_lo + kTileK);
    }
    __syncthreads();
    int stage = 0;
#ifdef HIPATTN_FLASH_TRACE
    t.clk.last = (long long)__builtin_readcyclecounter();
#endif
    for (int ts = kv_lo; ts < kv_hi; ts += kTileK) {
        const uint8_t* k_lds = lds + stage * kStageBytes;
        const uint8_t* v_lds = k_lds + kKBytes;
        FLASH_STAMP(t, ts / kTileK, 0);
        const bool all_valid = (ts + kTileK <= t.kv_len) && (!t.causal || ts + kTileK <= t.pos0 + 1) &&
                               (t.window <= 0 || ts >= t.pos0 + t.rows - t.window);
        if (all_valid)
            consume_tile<kBf16, false>(t, k_lds, v_lds, qf, o, m_ref, l_run, c, ts, my_pos, n32, hi);
        else
            consume_tile<kBf16, true>(t, k_lds, v_lds, qf, o, m_ref, l_run, c, ts, my_pos, n32, hi);
        FLASH_STAMP(t, ts / kTileK, 3);
        if (ts + kTileK < kv_hi) {
            // the other stage was last read one iteration ago; every wavefront has passed the
            // barrier that ended that iteration
            uint8_t* nk = lds + (stage ^ 1) * kStageBytes;
            store_lds(nk, nk + kKBytes);
            FLASH_STAMP(t, ts / kTileK, 4);
            if (ts + 2 * kTileK < kv_hi) load_regs(ts + 2 * kTileK);
        }
        FLASH_STAMP(t, ts / kTileK, 5);
        __syncthreads();
        FLASH_STAMP(t, ts / kTileK, 6);
        stage ^= 1;
    }

#ifdef HIPATTN_FLASH_TRACE
    if (t.trace)
        for (int k = 0; k < 8; k++) t.trace[k] = t.clk.acc[k];
#endif
    // ---- normalise and store
    l_run += __shfl_xor(l_run, 32, 64);
    const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
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
    run_tile<kBf16>(t, lds, p.scale);
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
