/*
 * CPU oracle for the attention hot path.  TEST INFRASTRUCTURE ONLY: this file is the
 * checker that tests, the smoke check and the benchmark's cpu_baseline leg compare the
 * HIP kernels against.  Nothing in the shipped library links or calls it.
 *
 * The reference plugin holds no attention kernel of its own: it rewrites
 * v13::ScaledDotProductAttention into Multiply / MatMul / Select / Add / Softmax / MatMul
 * (modules/nvidia_plugin/src/transformer/cuda_graph_transformer.cpp:151-156) and runs
 * those on cuBLAS and cuDNN (src/ops/matmul.cpp:204-226, src/ops/softmax.cpp:184-192).
 * The arithmetic itself lives in OpenVINO 2025.3.0 (wheel/requirements.txt:4), which is
 * not part of the reference tree, so this file restates the published operator
 * definitions:
 *
 *   oracle_sdpa_f32            softmax(scale * Q K^T + causal mask) V, fp32, GQA by head
 *                              group, top-left aligned lower-triangular mask
 *                              (model built as in tests/functional/shared_tests_instances/
 *                              single_layer_tests/scaled_dot_product_attention.cpp:48-69;
 *                              batch broadcast rules as src/ops/matmul.cpp:128-175;
 *                              max-subtracted softmax as src/ops/softmax.cpp:75-147).
 *                              Pinned by: fp64 brute force, torch's CPU
 *                              scaled_dot_product_attention fixtures, invariants.
 *   oracle_sdpa_mask_f32       the same with the operator's attention_mask input (additive;
 *                              boolean masks converted to 0 / -inf), the Add node of the
 *                              decomposed graph (src/ops/add.cpp:17-43).  Pinned by torch's
 *                              CPU routine with attn_mask (float, boolean, broadcast) and by
 *                              explicit causal mask == causal flag.
 *   oracle_kv_cache_write      slot(s, p) = block_indices[begins[s] + p / bs] * bs + p % bs,
 *                              row scatter in the spirit of
 *                              src/kernels/scatter_nd_update.cu:19-34; out-of-range block
 *                              ids are skipped, never written
 *                              (tests/unit/kernels/scatter_update.cpp:59-86).
 *                              Pinned by: brute force in numpy, write-then-gather identity,
 *                              canary fill.
 *   oracle_paged_attention     PagedAttentionExtension: cache write, then every query token
 *                              attends cache positions (p - W, p] of its own sequence.
 *                              PARITY UNPINNED against OpenVINO: the op does not occur in
 *                              the reference tree and OpenVINO is not installed.  Pinned
 *                              by reduction to oracle_sdpa_f32 after a gather through the
 *                              block table, and by block-permutation invariance.
 *   oracle_paged_attention_scores   the operator's second output: attention probability per
 *                              cache position, summed over heads and the aggregated query
 *                              tokens.  PARITY UNPINNED against OpenVINO.  Pinned by a numpy
 *                              restatement over a dense gather, by sum = heads x aggregated
 *                              tokens, and by scores-weighted values = attention output for a
 *                              one-head, one-token sequence.
 *   oracle_quant_u8_row /      asymmetric per-token, per-head u8 rows
 *   oracle_dequant_u8_row      [scale f32][zero-point f32][D bytes].  PARITY UNPINNED
 *                              against OpenVINO (rounding mode and row layout are restated
 *                              from the published CPU plugin behaviour, not checked).
 *                              Pinned by |x - x^| <= scale/2 and min/max round trip.
 *
 * All arithmetic is fp32 with fp64 softmax sums.  Compiled with OpenMP; the number of
 * threads is whatever omp_get_max_threads() says (reported by oracle_num_threads()).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <float.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

enum { ORACLE_F32 = 0, ORACLE_F16 = 1, ORACLE_BF16 = 2, ORACLE_U8 = 3 };

ORACLE_API int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

ORACLE_API void oracle_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* ---------------------------------------------------------------- scalar conversions */

static inline uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float bits_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* IEEE binary16 -> binary32, exact. */
ORACLE_API float oracle_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-8f;
        return sign ? -v : v;
    }
    if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* binary32 -> binary16, round to nearest even, subnormals kept, overflow to inf. */
ORACLE_API uint16_t oracle_f32_to_f16(float f) {
    uint32_t x = f32_bits(f);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) { /* inf / nan */
        if (ax > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((ax >> 13) & 0x3ffu));
        return (uint16_t)(sign | 0x7c00u);
    }
    if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to inf */
    if (ax < 0x33000001u) return sign;                        /* <= 2^-25 rounds to zero */
    int32_t e = (int32_t)(ax >> 23) - 127;
    uint32_t m = (ax & 0x7fffffu) | 0x800000u;
    if (e < -14) {
        /* subnormal half: shift so that the unit is 2^-24 */
        int shift = -14 - e + 13; /* 14..24 */
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t q = ((uint32_t)(e + 15) << 10) | ((m >> 13) & 0x3ffu);
    uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;
    return (uint16_t)(sign | q);
}

ORACLE_API float oracle_bf16_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

/* binary32 -> bfloat16, round to nearest even. */
ORACLE_API uint16_t oracle_f32_to_bf16(float f) {
    uint32_t x = f32_bits(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7fffu + lsb;
    return (uint16_t)(x >> 16);
}

ORACLE_API void oracle_f32_to_f16_array(const float* src, uint16_t* dst, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) dst[i] = oracle_f32_to_f16(src[i]);
}
ORACLE_API void oracle_f16_to_f32_array(const uint16_t* src, float* dst, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) dst[i] = oracle_f16_to_f32(src[i]);
}
ORACLE_API void oracle_f32_to_bf16_array(const float* src, uint16_t* dst, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) dst[i] = oracle_f32_to_bf16(src[i]);
}
ORACLE_API void oracle_bf16_to_f32_array(const uint16_t* src, float* dst, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) dst[i] = oracle_bf16_to_f32(src[i]);
}

/* ------------------------------------------------------------------- u8 quantisation */

/*
 * One cache row of a u8 cache: [scale f32][zp f32][D x u8].
 *   scale = (max - min) / 255   (0 -> 1e-4 so that a constant row survives)
 *   zp    = -min / scale + 0   (the sum turns -0 into +0)
 *   q     = clamp(rint(fma(x, 1/scale, zp)), 0, 255)     (round half to even)
 *   x^    = (q - zp) * scale
 */
ORACLE_API void oracle_quant_u8_row(const float* x, int D, uint8_t* row) {
    float mn = FLT_MAX, mx = -FLT_MAX;
    for (int d = 0; d < D; d++) {
        mn = x[d] < mn ? x[d] : mn;
        mx = x[d] > mx ? x[d] : mx;
    }
    float scale = (mx - mn) / 255.0f;
    if (scale == 0.0f) scale = 0.0001f;
    float zp = -mn / scale + 0.0f;
    float inv = 1.0f / scale;
    memcpy(row, &scale, 4);
    memcpy(row + 4, &zp, 4);
    for (int d = 0; d < D; d++) {
        float t = rintf(fmaf(x[d], inv, zp));
        t = t < 0.0f ? 0.0f : (t > 255.0f ? 255.0f : t);
        row[8 + d] = (uint8_t)t;
    }
}

ORACLE_API void oracle_dequant_u8_row(const uint8_t* row, int D, float* x) {
    float scale, zp;
    memcpy(&scale, row, 4);
    memcpy(&zp, row + 4, 4);
    for (int d = 0; d < D; d++) x[d] = ((float)row[8 + d] - zp) * scale;
}

ORACLE_API void oracle_quant_u8_rows(const float* x, int64_t n, int D, uint8_t* rows) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) oracle_quant_u8_row(x + i * D, D, rows + i * (D + 8));
}

ORACLE_API void oracle_dequant_u8_rows(const uint8_t* rows, int64_t n, int D, float* x) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) oracle_dequant_u8_row(rows + i * (D + 8), D, x + i * D);
}

static inline int64_t cache_row_bytes(int dtype, int D) {
    switch (dtype) {
        case ORACLE_F32: return 4 * (int64_t)D;
        case ORACLE_F16:
        case ORACLE_BF16: return 2 * (int64_t)D;
        default: return (int64_t)D + 8;
    }
}

static void cache_row_store(int dtype, const float* x, int D, uint8_t* row) {
    switch (dtype) {
        case ORACLE_F32: memcpy(row, x, 4 * (size_t)D); break;
        case ORACLE_F16:
            for (int d = 0; d < D; d++) ((uint16_t*)row)[d] = oracle_f32_to_f16(x[d]);
            break;
        case ORACLE_BF16:
            for (int d = 0; d < D; d++) ((uint16_t*)row)[d] = oracle_f32_to_bf16(x[d]);
            break;
        default: oracle_quant_u8_row(x, D, row);
    }
}

static void cache_row_load(int dtype, const uint8_t* row, int D, float* x) {
    switch (dtype) {
        case ORACLE_F32: memcpy(x, row, 4 * (size_t)D); break;
        case ORACLE_F16:
            for (int d = 0; d < D; d++) x[d] = oracle_f16_to_f32(((const uint16_t*)row)[d]);
            break;
        case ORACLE_BF16:
            for (int d = 0; d < D; d++) x[d] = oracle_bf16_to_f32(((const uint16_t*)row)[d]);
            break;
        default: oracle_dequant_u8_row(row, D, x);
    }
}

/* ------------------------------------------------------------------------ dense SDPA */

static inline float dotf(const float* a, const float* b, int n) {
    float s = 0.0f;
#pragma omp simd reduction(+ : s)
    for (int i = 0; i < n; i++) s += a[i] * b[i];
    return s;
}

/*
 * One query row against keys [j0, j1) given as row pointers computed by the caller's
 * stride; scores buffer must hold j1 - j0 floats.
 */
/* sink: -INFINITY, or a logit that takes part in the row's softmax without a value row of its own (an
 * "attention sink": the row's probabilities then sum to less than one). */
static void attend_row_sink(const float* q, const float* kbase, const float* vbase, int64_t kv_stride, int j0,
                            int j1, int D, float scale, const float* bias, int64_t bias_stride, float sink, float* scores,
                            float* out) {
    int n = j1 - j0;
    if (n <= 0) {
        for (int d = 0; d < D; d++) out[d] = 0.0f;
        return;
    }
    float m = -INFINITY;
    for (int j = 0; j < n; j++) {
        float s = scale * dotf(q, kbase + (int64_t)(j0 + j) * kv_stride, D);
        if (bias) s += bias[(int64_t)(j0 + j) * bias_stride];
        scores[j] = s;
        m = s > m ? s : m;
    }
    if (sink > m) m = sink;
    double l = sink > -INFINITY ? exp((double)sink - (double)m) : 0.0;
    for (int j = 0; j < n; j++) {
        float p = expf(scores[j] - m);
        scores[j] = p;
        l += (double)p;
    }
    for (int d = 0; d < D; d++) out[d] = 0.0f;
    for (int j = 0; j < n; j++) {
        const float* v = vbase + (int64_t)(j0 + j) * kv_stride;
        float p = scores[j];
        for (int d = 0; d < D; d++) out[d] += p * v[d];
    }
    float inv = (float)(1.0 / l);
    for (int d = 0; d < D; d++) out[d] *= inv;
}

static void attend_row_biased(const float* q, const float* kbase, const float* vbase, int64_t kv_stride, int j0,
                              int j1, int D, float scale, const float* bias, int64_t bias_stride, float* scores,
                              float* out) {
    attend_row_sink(q, kbase, vbase, kv_stride, j0, j1, D, scale, bias, bias_stride, -INFINITY, scores, out);
}

static void attend_row(const float* q, const float* kbase, const float* vbase, int64_t kv_stride, int j0, int j1,
                       int D, float scale, float* scores, float* out) {
    attend_row_biased(q, kbase, vbase, kv_stride, j0, j1, D, scale, NULL, 0, scores, out);
}

/*
 * q [B,Hq,Lq,D], k,v [B,Hkv,Lk,D], out [B,Hq,Lq,D]; query head h reads kv head
 * h / (Hq/Hkv).  causal: row i sees keys j <= i (top-left aligned, as the operator
 * specification's tril(ones(Lq,Lk))).  scale <= 0 selects 1/sqrt(D).
 */
ORACLE_API int oracle_sdpa_f32(const float* q, const float* k, const float* v, float* out, int B, int Hq, int Hkv,
                               int Lq, int Lk, int D, int causal, float scale) {
    if (B < 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || Lq < 0 || Lk < 0 || D <= 0) return 1;
    if (scale <= 0.0f) scale = 1.0f / sqrtf((float)D);
    int G = Hq / Hkv;
    int64_t rows = (int64_t)B * Hq * Lq;
#pragma omp parallel
    {
        float* scores = (float*)malloc(sizeof(float) * (size_t)(Lk > 0 ? Lk : 1));
#pragma omp for schedule(dynamic, 16)
        for (int64_t r = 0; r < rows; r++) {
            int i = (int)(r % Lq);
            int h = (int)((r / Lq) % Hq);
            int b = (int)(r / ((int64_t)Lq * Hq));
            const float* kb = k + ((int64_t)b * Hkv + h / G) * Lk * D;
            const float* vb = v + ((int64_t)b * Hkv + h / G) * Lk * D;
            int j1 = causal ? (i + 1 < Lk ? i + 1 : Lk) : Lk;
            attend_row(q + r * D, kb, vb, D, 0, j1, D, scale, scores, out + r * D);
        }
        free(scores);
    }
    return 0;
}

/*
 * The same operator with its attention_mask input: softmax(scale * Q K^T + mask) V.  mask is the
 * additive form (a boolean mask is 0 where true and -inf where false, as the operator
 * specification converts it), addressed as [B,Hq,Lq,Lk] through element strides, 0 = broadcast;
 * it replaces the Add node of the decomposed graph (src/ops/add.cpp:17-43, numpy broadcast as
 * src/ops/elementwise_binary.hpp:15-77).  With causal set the mask is ignored, as the operator
 * specifies.  A row whose keys are all masked with -inf comes out as NaN (exp(-inf - -inf)),
 * like the library routine that pins this function.
 * Pinned by torch's CPU scaled_dot_product_attention(attn_mask=...) fixtures (float and boolean,
 * broadcast and full) and by reduction: a causal mask passed explicitly equals causal = 1.
 */
ORACLE_API int oracle_sdpa_mask_f32(const float* q, const float* k, const float* v, float* out, int B, int Hq,
                                    int Hkv, int Lq, int Lk, int D, int causal, float scale, const float* mask,
                                    const int64_t* mask_stride) {
    if (!mask || causal) return oracle_sdpa_f32(q, k, v, out, B, Hq, Hkv, Lq, Lk, D, causal, scale);
    if (B < 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || Lq < 0 || Lk < 0 || D <= 0) return 1;
    if (scale <= 0.0f) scale = 1.0f / sqrtf((float)D);
    int G = Hq / Hkv;
    int64_t rows = (int64_t)B * Hq * Lq;
#pragma omp parallel
    {
        float* scores = (float*)malloc(sizeof(float) * (size_t)(Lk > 0 ? Lk : 1));
#pragma omp for schedule(dynamic, 16)
        for (int64_t r = 0; r < rows; r++) {
            int i = (int)(r % Lq);
            int h = (int)((r / Lq) % Hq);
            int b = (int)(r / ((int64_t)Lq * Hq));
            const float* kb = k + ((int64_t)b * Hkv + h / G) * Lk * D;
            const float* vb = v + ((int64_t)b * Hkv + h / G) * Lk * D;
            const float* mrow = mask + b * mask_stride[0] + h * mask_stride[1] + i * mask_stride[2];
            attend_row_biased(q + r * D, kb, vb, D, 0, Lk, D, scale, mrow, mask_stride[3], scores, out + r * D);
        }
        free(scores);
    }
    return 0;
}

/* ------------------------------------------------------------------ paged KV cache */

/*
 * Scatter the new key/value rows of a batch into the paged caches.
 *   k_new, v_new        [T, Hkv*D] fp32 (already rounded to the activation type by the caller)
 *   key_cache/value_cache  [num_blocks, Hkv, block_size, row_bytes(dtype, D)]
 *   past_lens [S], subsequence_begins [S+1], block_indices [..], block_indices_begins [S+1]
 * Token i of sequence s goes to logical position p = past_lens[s] + i, i.e. physical
 * block block_indices[block_indices_begins[s] + p / block_size], row p % block_size.
 * A logical block beyond the sequence's table, or a physical id outside [0, num_blocks),
 * is skipped.  Returns the number of skipped token rows.
 */
ORACLE_API int64_t oracle_kv_cache_write(const float* k_new, const float* v_new, uint8_t* key_cache,
                                         uint8_t* value_cache, int cache_dtype, const int32_t* past_lens,
                                         const int32_t* subsequence_begins, const int32_t* block_indices,
                                         const int32_t* block_indices_begins, int S, int Hkv, int D, int block_size,
                                         int num_blocks) {
    int64_t rb = cache_row_bytes(cache_dtype, D);
    int64_t skipped = 0;
    for (int s = 0; s < S; s++) {
        int t0 = subsequence_begins[s], t1 = subsequence_begins[s + 1];
        int nb = block_indices_begins[s + 1] - block_indices_begins[s];
        for (int t = t0; t < t1; t++) {
            int p = past_lens[s] + (t - t0);
            int lb = p / block_size;
            if (p < 0 || lb >= nb) {
                skipped++;
                continue;
            }
            int pb = block_indices[block_indices_begins[s] + lb];
            if (pb < 0 || pb >= num_blocks) {
                skipped++;
                continue;
            }
            for (int h = 0; h < Hkv; h++) {
                int64_t off = (((int64_t)pb * Hkv + h) * block_size + p % block_size) * rb;
                cache_row_store(cache_dtype, k_new + ((int64_t)t * Hkv + h) * D, D, key_cache + off);
                cache_row_store(cache_dtype, v_new + ((int64_t)t * Hkv + h) * D, D, value_cache + off);
            }
        }
    }
    return skipped;
}

/*
 * Gather one sequence's first n cache rows of kv head h through its block table into a
 * contiguous fp32 [n, D] array (used by the oracle itself and by tests that reduce the
 * paged case to the dense one).  A table entry outside [0, num_blocks) names no block: its rows
 * come out as zeros and, when valid is not NULL, valid[p] is 0 for them (1 for every other row).
 * num_blocks <= 0: every entry is taken as it is.
 */
ORACLE_API void oracle_gather_cache_rows_checked(const uint8_t* cache, int cache_dtype, const int32_t* seq_blocks, int n,
                                                 int h, int Hkv, int D, int block_size, int num_blocks, float* dst,
                                                 uint8_t* valid) {
    int64_t rb = cache_row_bytes(cache_dtype, D);
    for (int p = 0; p < n; p++) {
        int pb = seq_blocks[p / block_size];
        int ok = num_blocks <= 0 || (pb >= 0 && pb < num_blocks);
        if (valid) valid[p] = (uint8_t)ok;
        if (!ok) {
            memset(dst + (int64_t)p * D, 0, sizeof(float) * (size_t)D);
            continue;
        }
        int64_t off = (((int64_t)pb * Hkv + h) * block_size + p % block_size) * rb;
        cache_row_load(cache_dtype, cache + off, D, dst + (int64_t)p * D);
    }
}

ORACLE_API void oracle_gather_cache_rows(const uint8_t* cache, int cache_dtype, const int32_t* seq_blocks, int n,
                                         int h, int Hkv, int D, int block_size, float* dst) {
    oracle_gather_cache_rows_checked(cache, cache_dtype, seq_blocks, n, h, Hkv, D, block_size, 0, dst, NULL);
}

/*
 * PagedAttentionExtension, restated.
 *   q [T, Hq*D] fp32, out [T, Hq*D] fp32.
 *   do_write != 0: first scatter k_new / v_new (oracle_kv_cache_write).
 * Query token i of sequence s sits at position p = past_lens[s] + i and attends cache
 * positions j with max(0, p - W + 1) <= j <= p when W = sliding_window > 0, else 0..p.
 * A table entry outside [0, num_blocks) names no block: the positions it stands for take no part
 * (probability zero, like the new tokens that oracle_kv_cache_write could not store there), and a
 * row left with nothing to attend is zeros.
 * alibi_slopes (NULL, or one float per query head): slope[h] * (j - p) is added to the scaled score
 * of position j, the linear distance bias of ALiBi (0 at the token itself, more negative with
 * distance for a positive slope).  A constant added to a whole row does not change its softmax,
 * so a kernel may measure the distance from any fixed position of the row.
 * PARITY UNPINNED against OpenVINO for this input (sign and origin restated from the operator's
 * documentation); pinned against an explicit additive mask through torch's fp64
 * scaled_dot_product_attention (tests/golden/make_alibi_golden.py) and against the fp64 closed form.
 * sinks (NULL, or one float per query head): a logit that joins every row's softmax of that head without a
 * value row ("attention sink"): out = sum_j exp(s_j) v_j / (sum_j exp(s_j) + exp(sink)); a row left with
 * nothing to attend is zeros all the same.  PARITY UNPINNED against OpenVINO (restated from the operator's
 * documentation and the models that carry the input); pinned by the fp64 closed form, by "a sink of -inf
 * changes nothing" and by the equivalent extra key with a value row of zeros (tests/test_oracle_cpu.py).
 * scale <= 0 selects 1/sqrt(D).
 */
ORACLE_API int oracle_paged_attention(const float* q, const float* k_new, const float* v_new, uint8_t* key_cache,
                                      uint8_t* value_cache, int cache_dtype, const int32_t* past_lens,
                                      const int32_t* subsequence_begins, const int32_t* block_indices,
                                      const int32_t* block_indices_begins, int S, int Hq, int Hkv, int D,
                                      int block_size, int num_blocks, float scale, int sliding_window, int do_write,
                                      const float* alibi_slopes, const float* sinks, float* out) {
    if (S < 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || D <= 0 || block_size <= 0) return 1;
    if (scale <= 0.0f) scale = 1.0f / sqrtf((float)D);
    if (do_write)
        oracle_kv_cache_write(k_new, v_new, key_cache, value_cache, cache_dtype, past_lens, subsequence_begins,
                              block_indices, block_indices_begins, S, Hkv, D, block_size, num_blocks);
    int G = Hq / Hkv;
    /* work items: (sequence, kv head); gathered K/V are shared by the G query heads */
    int64_t items = (int64_t)S * Hkv;
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t it = 0; it < items; it++) {
        int s = (int)(it / Hkv), h = (int)(it % Hkv);
        int t0 = subsequence_begins[s], qlen = subsequence_begins[s + 1] - t0;
        if (qlen <= 0) continue;
        int ctx = past_lens[s] + qlen;
        /* positions beyond the sequence's block table do not exist (their writes were skipped) */
        int table_tokens = (block_indices_begins[s + 1] - block_indices_begins[s]) * block_size;
        if (ctx > table_tokens) ctx = table_tokens;
        if (ctx <= 0) {
            for (int i = 0; i < qlen; i++)
                for (int g = 0; g < G; g++)
                    memset(out + ((int64_t)(t0 + i) * Hq + (h * G + g)) * D, 0, sizeof(float) * (size_t)D);
            continue;
        }
        float* kbuf = (float*)malloc(sizeof(float) * (size_t)ctx * D);
        float* vbuf = (float*)malloc(sizeof(float) * (size_t)ctx * D);
        float* scores = (float*)malloc(sizeof(float) * (size_t)ctx);
        uint8_t* valid = (uint8_t*)malloc((size_t)ctx);
        float* bias = (float*)malloc(sizeof(float) * (size_t)ctx); /* 0, or -inf where the table names no block */
        float* rowbias = (float*)malloc(sizeof(float) * (size_t)ctx); /* bias plus a row's distance term */
        const int32_t* blocks = block_indices + block_indices_begins[s];
        oracle_gather_cache_rows_checked(key_cache, cache_dtype, blocks, ctx, h, Hkv, D, block_size, num_blocks, kbuf, valid);
        oracle_gather_cache_rows_checked(value_cache, cache_dtype, blocks, ctx, h, Hkv, D, block_size, num_blocks, vbuf, NULL);
        int holes = 0;
        for (int j = 0; j < ctx; j++) {
            bias[j] = valid[j] ? 0.0f : -INFINITY;
            holes += !valid[j];
        }
        for (int i = 0; i < qlen; i++) {
            int p = past_lens[s] + i;
            int j0 = 0;
            if (sliding_window > 0 && p - sliding_window + 1 > 0) j0 = p - sliding_window + 1;
            int j1 = p + 1 < ctx ? p + 1 : ctx;
            if (j0 > ctx) j0 = ctx;
            int any = 0;
            for (int j = j0; j < j1 && !any; j++) any = valid[j];
            for (int g = 0; g < G; g++) {
                int64_t row = ((int64_t)(t0 + i) * Hq + (h * G + g)) * D;
                if (!any) {
                    memset(out + row, 0, sizeof(float) * (size_t)D);
                } else if (alibi_slopes) {
                    float slope = alibi_slopes[h * G + g];
                    for (int j = j0; j < j1; j++) rowbias[j] = bias[j] + slope * (float)(j - p);
                    attend_row_sink(q + row, kbuf, vbuf, D, j0, j1, D, scale, rowbias, 1, sinks ? sinks[h * G + g] : -INFINITY, scores,
                                    out + row);
                } else {
                    attend_row_sink(q + row, kbuf, vbuf, D, j0, j1, D, scale, holes ? bias : NULL, 1, sinks ? sinks[h * G + g] : -INFINITY,
                                    scores, out + row);
                }
            }
        }
        free(kbuf);
        free(vbuf);
        free(scores);
        free(valid);
        free(bias);
        free(rowbias);
    }
    return 0;
}

/*
 * Cache rotation of PagedAttentionExtension (inputs rotated_block_indices, rotation_deltas,
 * rotation_trig_lut): the keys of the listed cache blocks are turned by a rotary-embedding angle, which is
 * what moving a token to another position does to a key that was stored with its rotary embedding applied
 * (a cache-eviction policy closes the gaps it leaves and re-rotates the blocks behind them).
 *   rotated_block_indices [n]        blocks of the cache (ids outside [0, num_blocks) are skipped)
 *   rotation_deltas [n, per_block]   per_block = 1: one row of the table for the whole block;
 *                                    per_block = block_size: one per token of the block
 *   rotation_trig_lut [lut_rows, D]  row r: D/2 cosines, then D/2 sines (a delta outside [0, lut_rows)
 *                                    leaves its token as it is)
 * Every key row x of a listed block (all kv heads) becomes, for i < D/2,
 *   x'[i] = x[i] cos[i] - x[i + D/2] sin[i],   x'[i + D/2] = x[i] sin[i] + x[i + D/2] cos[i]
 * (the "rotate-half" pairing), computed in fp32 and stored in the cache's type (u8 rows are dequantised,
 * turned and quantised again).  The value cache is not touched.  In the operator this happens before the
 * step's new keys are stored.
 * PARITY UNPINNED against OpenVINO (the operator is not in the reference tree, OpenVINO is not installed):
 * table layout, pairing and order restated from the operator's documentation.  Pinned by: two rotations
 * compose to the rotation by the summed angle, a rotation and its inverse restore the rows, norms are kept,
 * and a key stored with the rotary embedding of position p (oracle_rope_f32, itself pinned by transformers'
 * apply_rotary_pos_emb) and turned by delta equals the key embedded at position p + delta
 * (tests/test_oracle_cpu.py).
 */
ORACLE_API int oracle_rotate_key_cache(uint8_t* key_cache, int cache_dtype, const int32_t* rotated_block_indices, int n,
                                       const int32_t* rotation_deltas, int per_block, const float* rotation_trig_lut,
                                       int lut_rows, int Hkv, int D, int block_size, int num_blocks) {
    if (n < 0 || Hkv <= 0 || D <= 0 || (D & 1) || block_size <= 0 || (per_block != 1 && per_block != block_size)) return 1;
    const int64_t rb = cache_row_bytes(cache_dtype, D);
    const int half = D / 2;
    float* x = (float*)malloc(sizeof(float) * (size_t)D);
    float* y = (float*)malloc(sizeof(float) * (size_t)D);
    for (int b = 0; b < n; b++) {
        const int pb = rotated_block_indices[b];
        if (pb < 0 || pb >= num_blocks) continue;
        for (int t = 0; t < block_size; t++) {
            const int delta = rotation_deltas[(int64_t)b * per_block + (per_block == 1 ? 0 : t)];
            if (delta < 0 || delta >= lut_rows) continue;
            const float* cs = rotation_trig_lut + (int64_t)delta * D;
            for (int h = 0; h < Hkv; h++) {
                uint8_t* row = key_cache + (((int64_t)pb * Hkv + h) * block_size + t) * rb;
                cache_row_load(cache_dtype, row, D, x);
                for (int i = 0; i < half; i++) { /* (one product rounded, the other fused: spelled out so that a kernel can match to the bit) */
                    const float t0 = x[i + half] * cs[half + i], t1 = x[i + half] * cs[i];
                    y[i] = fmaf(x[i], cs[i], -t0);
                    y[i + half] = fmaf(x[i], cs[half + i], t1);
                }
                cache_row_store(cache_dtype, y, D, row);
            }
        }
    }
    free(x);
    free(y);
    return 0;
}

/* Second output of PagedAttentionExtension ("scores"): for every cache position of every
 * sequence, the probability it received, summed over the query heads and over the last
 * score_window[s] query tokens of the sequence (all of them when score_window is NULL).
 * Reads the cache as it stands (call after the write).  scores must hold
 * sum(past_lens[s] + new_tokens(s)) floats; sequence s starts where s-1 ends.  fp64 throughout.
 * A table entry outside [0, num_blocks) names no block, as in oracle_paged_attention: its positions
 * get probability zero and take no part in a row's softmax; a row with nothing left adds nothing
 * (num_blocks <= 0: every entry is taken as it is).
 * PARITY UNPINNED against OpenVINO (which tokens and heads are aggregated is restated from its
 * operator documentation).  Pinned by: a numpy restatement over a dense gather of the keys, the sum
 * of a sequence's scores (= heads x aggregated tokens), and agreement of the probabilities with
 * the attention output (scores-weighted values of one head, one token). */
ORACLE_API int oracle_paged_attention_scores(const float* q, const uint8_t* key_cache, int cache_dtype,
                                             const int32_t* past_lens, const int32_t* subsequence_begins,
                                             const int32_t* block_indices, const int32_t* block_indices_begins,
                                             const int32_t* score_window, int S, int Hq, int Hkv, int D, int block_size,
                                             int num_blocks, float scale, int sliding_window, float* scores) {
    if (S < 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || D <= 0 || block_size <= 0) return 1;
    if (scale <= 0.0f) scale = 1.0f / sqrtf((float)D);
    const int G = Hq / Hkv;
    int64_t* starts = (int64_t*)malloc(sizeof(int64_t) * (size_t)(S + 1));
    starts[0] = 0;
    for (int s = 0; s < S; s++) starts[s + 1] = starts[s] + past_lens[s] + (subsequence_begins[s + 1] - subsequence_begins[s]);
#pragma omp parallel for schedule(dynamic, 1)
    for (int s = 0; s < S; s++) {
        const int t0 = subsequence_begins[s], qlen = subsequence_begins[s + 1] - t0;
        const int ctx_full = past_lens[s] + qlen;
        float* out = scores + starts[s];
        for (int j = 0; j < ctx_full; j++) out[j] = 0.0f;
        int ctx = ctx_full;
        const int table_tokens = (block_indices_begins[s + 1] - block_indices_begins[s]) * block_size;
        if (ctx > table_tokens) ctx = table_tokens;
        int w = qlen;
        if (score_window) w = score_window[s] < 0 ? 0 : (score_window[s] < qlen ? score_window[s] : qlen);
        if (ctx <= 0 || w <= 0) continue;
        double* acc = (double*)calloc((size_t)ctx, sizeof(double));
        double* sc = (double*)malloc(sizeof(double) * (size_t)ctx);
        float* kbuf = (float*)malloc(sizeof(float) * (size_t)ctx * D);
        uint8_t* valid = (uint8_t*)malloc((size_t)ctx);
        const int32_t* blocks = block_indices + block_indices_begins[s];
        for (int h = 0; h < Hkv; h++) {
            oracle_gather_cache_rows_checked(key_cache, cache_dtype, blocks, ctx, h, Hkv, D, block_size, num_blocks, kbuf, valid);
            for (int i = qlen - w; i < qlen; i++) {
                const int p = past_lens[s] + i;
                int j0 = 0, j1 = p + 1 < ctx ? p + 1 : ctx;
                if (sliding_window > 0 && p - sliding_window + 1 > 0) j0 = p - sliding_window + 1;
                if (j0 >= j1) continue;
                for (int g = 0; g < G; g++) {
                    const float* qr = q + ((int64_t)(t0 + i) * Hq + (h * G + g)) * D;
                    double m = -INFINITY, l = 0.0;
                    for (int j = j0; j < j1; j++) {
                        if (!valid[j]) continue;
                        double d = 0.0;
                        for (int e = 0; e < D; e++) d += (double)qr[e] * (double)kbuf[(int64_t)j * D + e];
                        sc[j] = d * (double)scale;
                        if (sc[j] > m) m = sc[j];
                    }
                    if (m == -INFINITY) continue; /* every attended position lies in a block the table does not name */
                    for (int j = j0; j < j1; j++)
                        if (valid[j]) l += exp(sc[j] - m);
                    for (int j = j0; j < j1; j++)
                        if (valid[j]) acc[j] += exp(sc[j] - m) / l;
                }
            }
        }
        for (int j = 0; j < ctx; j++) out[j] = (float)acc[j];
        free(acc);
        free(sc);
        free(kbuf);
        free(valid);
    }
    free(starts);
    return 0;
}
