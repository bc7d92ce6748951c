/*
 * CPU oracle for the operators either side of attention in a decoder layer.  TEST INFRASTRUCTURE
 * ONLY: the checker that tests and the benchmark's cpu_baseline leg compare libhipops.so against.
 * Nothing in the shipped libraries links or calls it.
 *
 *   oracle_rms_norm_f32   out = x / sqrt(mean(x^2) + eps) * gamma over the last axis: OpenVINO's
 *                         internal RMS operator, which the reference would execute as the unfused
 *                         Power / ReduceMean / Add / Sqrt / Divide / Multiply chain
 *                         (modules/nvidia_plugin/src/ops/reduce.cpp, elementwise_binary.hpp).
 *                         Pinned by torch.nn.functional.rms_norm in fp64 (fixtures), unit mean
 *                         square of the output, and scale invariance at eps = 0.
 *   oracle_rope_f32       rotary position embedding, rotate-half (LLaMA) and adjacent-pair (GPT-J)
 *                         layouts of OpenVINO's internal RoPE operator; the reference runs the
 *                         unfused Slice / Multiply / Concat / Add chain (src/ops/concat.cpp:20-102,
 *                         src/ops/multiply.cpp:43, src/ops/add.cpp:17-43).  Pinned by the
 *                         transformers library's apply_rotary_pos_emb for both layouts
 *                         (fixtures), by complex multiplication in numpy, norm preservation and
 *                         the identity at angle 0.  Which tensor layouts OpenVINO's fused operator
 *                         accepts (its slice / transpose attributes) is PARITY UNPINNED: OpenVINO
 *                         is not installed; the entry point takes strides instead.
 *   oracle_matmul_f32     C[b] = op(A[b]) op(B[b]) with fp64 accumulation; shape and broadcast
 *                         rules of MatMulOp (src/ops/matmul.cpp:22-76, 128-175).  Pinned by
 *                         numpy.matmul in fp64.
 *   oracle_gather_bytes   Gather with batch_dims as src/ops/gather.cpp:60-127 sets it up and
 *                         src/kernels/gather.cu:19-47 executes it (negative indices wrap once,
 *                         out-of-range rows are zero).  Pinned by numpy.take and the zero rule on
 *                         hand-written cases.
 *   oracle_concat_bytes   Concat along an axis (src/ops/concat.cpp:31-56).  Pinned by
 *                         numpy.concatenate.
 *   oracle_transpose_bytes  Transpose, output axis k = input axis order[k] (src/ops/transpose.cpp:54-135), elements
 *                         of any size moved as bytes.  Pinned by numpy.transpose.
 *   oracle_convert        Convert as a C cast, through float where a 16-bit floating type is involved
 *                         (src/kernels/convert.cuh:24-49), with the two cases C leaves undefined fixed:
 *                         floating values beyond an integer target's range saturate, NaN gives 0.
 *                         Pinned by numpy.astype for every pair of types on values inside the range,
 *                         by torch for the roundings to f16 / bf16, and by hand-written cases for the
 *                         saturation, NaN and boolean rules.
 *   oracle_binary_f32     Add / Subtract / Multiply / Divide with numpy broadcasting (src/ops/elementwise_binary.hpp:16-76,
 *                         src/kernels/details/elementwise_binary.cuh:24-46), one fp32 operation per element.
 *                         Pinned by numpy's own broadcasting arithmetic in float32, bit for bit.
 *   oracle_softmax_f32    Softmax over the middle axis of [outer, length, inner] (src/ops/softmax.cpp:73-196)
 *                         in fp64.  Pinned by scipy.special.softmax and torch.softmax in fp64, rows that sum
 *                         to 1, shift invariance, and the uniform row.
 *   oracle_swish_f32 /    Swish (src/ops/swish.cpp:41-59) and OpenVINO's fused gated linear unit
 *   oracle_glu_f32        act(gate) * up with Swish, Gelu (erf) or Gelu (tanh).  Pinned by
 *                         torch.nn.functional.silu / gelu in fp64 (fixtures) and the explicit product.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

ORACLE_API void oracle_rms_norm_f32(const float* x, const float* gamma, float* out, int64_t rows, int64_t hidden,
                                    float eps) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        const float* xr = x + r * hidden;
        double sq = 0.0;
        for (int64_t i = 0; i < hidden; i++) sq += (double)xr[i] * (double)xr[i];
        const double inv = 1.0 / sqrt(sq / (double)hidden + (double)eps);
        for (int64_t i = 0; i < hidden; i++) {
            const double v = (double)xr[i] * inv;
            out[r * hidden + i] = (float)(gamma ? v * (double)gamma[i] : v);
        }
    }
}

/* x, out: [tokens, heads, head_size] contiguous; cos, sin: rows of `table_stride` floats */
ORACLE_API void oracle_rope_f32(const float* x, const float* cos_t, const float* sin_t, const int32_t* positions,
                                float* out, int64_t tokens, int heads, int head_size, int rotary, int interleaved,
                                int64_t table_stride) {
    const int half = rotary / 2;
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < tokens; t++) {
        const int64_t pos = positions ? positions[t] : t;
        const float* c = cos_t + pos * table_stride;
        const float* s = sin_t + pos * table_stride;
        for (int h = 0; h < heads; h++) {
            const float* xr = x + (t * heads + h) * (int64_t)head_size;
            float* o = out + (t * heads + h) * (int64_t)head_size;
            for (int i = 0; i < half; i++) {
                if (interleaved) {
                    const double a = xr[2 * i], b = xr[2 * i + 1];
                    o[2 * i] = (float)(a * c[i] - b * s[i]);
                    o[2 * i + 1] = (float)(b * c[i] + a * s[i]);
                } else {
                    const double a = xr[i], b = xr[i + half];
                    o[i] = (float)(a * c[i] - b * s[i]);
                    o[i + half] = (float)(b * c[i + half] + a * s[i + half]);
                }
            }
            for (int i = rotary; i < head_size; i++) o[i] = xr[i];
        }
    }
}

/* stride_a / stride_b == 0 broadcasts the operand over the batch */
ORACLE_API void oracle_matmul_f32(const float* a, const float* b, float* c, int64_t m, int64_t n, int64_t k, int64_t batch,
                                  int transpose_a, int transpose_b, int64_t stride_a, int64_t stride_b) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t bi = 0; bi < batch; bi++) {
        for (int64_t i = 0; i < m; i++) {
            const float* ab = a + bi * stride_a;
            const float* bb = b + bi * stride_b;
            for (int64_t j = 0; j < n; j++) {
                double acc = 0.0;
                for (int64_t l = 0; l < k; l++) {
                    const double av = transpose_a ? ab[l * m + i] : ab[i * k + l];
                    const double bv = transpose_b ? bb[j * k + l] : bb[l * n + j];
                    acc += av * bv;
                }
                c[(bi * m + i) * n + j] = (float)acc;
            }
        }
    }
}

ORACLE_API void oracle_gather_bytes(const uint8_t* data, const int64_t* indices, uint8_t* out, int64_t batch, int64_t outer,
                                    int64_t axis_dim, int64_t inner_bytes, int64_t num_indices) {
    for (int64_t b = 0; b < batch; b++)
        for (int64_t o = 0; o < outer; o++)
            for (int64_t k = 0; k < num_indices; k++) {
                int64_t idx = indices[b * num_indices + k];
                if (idx < 0) idx += axis_dim;
                uint8_t* dst = out + (((b * outer + o) * num_indices) + k) * inner_bytes;
                if (idx >= 0 && idx < axis_dim)
                    memcpy(dst, data + (((b * outer + o) * axis_dim) + idx) * inner_bytes, (size_t)inner_bytes);
                else
                    memset(dst, 0, (size_t)inner_bytes);
            }
}

ORACLE_API void oracle_concat_bytes(const uint8_t* const* inputs, const int64_t* axis_bytes, int num_inputs, int64_t outer,
                                    uint8_t* out) {
    int64_t total = 0;
    for (int i = 0; i < num_inputs; i++) total += axis_bytes[i];
    for (int64_t o = 0; o < outer; o++) {
        int64_t offset = 0;
        for (int i = 0; i < num_inputs; i++) {
            if (axis_bytes[i] > 0) memcpy(out + o * total + offset, inputs[i] + o * axis_bytes[i], (size_t)axis_bytes[i]);
            offset += axis_bytes[i];
        }
    }
}

/* Swish x / (1 + exp(-beta x)) (src/ops/swish.cpp:41-59, src/kernels/swish.cu:17-19 of the reference);
 * activation 1: Gelu with erf, 2: Gelu with the tanh approximation (OpenVINO's Gelu modes ERF and
 * TANH).  Pinned by torch.nn.functional.silu / gelu fixtures in fp64. */
static double oracle_activate(double x, int activation, double beta) {
    switch (activation) {
        case 1: return 0.5 * x * (1.0 + erf(x * 0.70710678118654752440));
        case 2: return 0.5 * x * (1.0 + tanh(0.79788456080286535588 * (x + 0.044715 * x * x * x)));
        default: return x / (1.0 + exp(-beta * x));
    }
}

ORACLE_API void oracle_swish_f32(const float* x, float* out, int64_t count, float beta) {
    for (int64_t i = 0; i < count; i++) out[i] = (float)oracle_activate(x[i], 0, beta);
}

/* out[r, i] = act(x[r, g + i]) * x[r, u + i], x of 2 * width columns: OpenVINO's fused gated linear
 * unit.  Pinned by act(gate) * up from the torch fixtures and by the plain product for multiply. */
ORACLE_API void oracle_glu_f32(const float* x, float* out, int64_t rows, int64_t width, int activation, int gate_first) {
    const int64_t g = gate_first ? 0 : width, u = width - g;
    for (int64_t r = 0; r < rows; r++)
        for (int64_t i = 0; i < width; i++)
            out[r * width + i] = (float)(oracle_activate(x[r * 2 * width + g + i], activation, 1.0) * (double)x[r * 2 * width + u + i]);
}

/* out = in with output axis k taken from input axis order[k]; dims are the input's extents */
ORACLE_API int oracle_transpose_bytes(const uint8_t* in, uint8_t* out, int rank, const int64_t* dims, const int32_t* order,
                                      int64_t element_bytes) {
    if (rank < 0 || rank > 16) return 1;
    int64_t in_stride[16], out_dims[16], step[16], coord[16], total = 1;
    for (int k = rank - 1; k >= 0; k--) in_stride[k] = k == rank - 1 ? 1 : in_stride[k + 1] * dims[k + 1];
    for (int k = 0; k < rank; k++) {
        if (order[k] < 0 || order[k] >= rank) return 1;
        out_dims[k] = dims[order[k]];
        step[k] = in_stride[order[k]];
        coord[k] = 0;
        total *= out_dims[k];
    }
    int64_t src = 0;
    for (int64_t i = 0; i < total; i++) {
        memcpy(out + i * element_bytes, in + src * element_bytes, (size_t)element_bytes);
        for (int k = rank - 1; k >= 0; k--) {  /* odometer over the output's coordinates */
            src += step[k];
            if (++coord[k] < out_dims[k]) break;
            src -= step[k] * out_dims[k];
            coord[k] = 0;
        }
    }
    return 0;
}

/* element types as in hipops.h: 0 f32, 1 f16, 2 bf16, 100 i32, 101 i64, 102 u8, 103 i8, 104 boolean */
float oracle_f16_to_f32(uint16_t h);
uint16_t oracle_f32_to_f16(float f);
float oracle_bf16_to_f32(uint16_t b);
uint16_t oracle_f32_to_bf16(float f);

static int64_t oracle_saturate(float f, float lowest, float beyond, int64_t min_value, int64_t max_value) {
    if (f != f) return 0;
    if (f <= lowest) return min_value;
    if (f >= beyond) return max_value;
    return (int64_t)f;
}

ORACLE_API int oracle_convert(const void* in, void* out, int64_t count, int from, int to) {
    for (int64_t i = 0; i < count; i++) {
        int is_float = 1;
        float f = 0.f;
        int64_t v = 0;
        switch (from) {
            case 0: f = ((const float*)in)[i]; break;
            case 1: f = oracle_f16_to_f32(((const uint16_t*)in)[i]); break;
            case 2: f = oracle_bf16_to_f32(((const uint16_t*)in)[i]); break;
            case 100: is_float = 0, v = ((const int32_t*)in)[i]; break;
            case 101: is_float = 0, v = ((const int64_t*)in)[i]; break;
            case 102: is_float = 0, v = ((const uint8_t*)in)[i]; break;
            case 103: is_float = 0, v = ((const int8_t*)in)[i]; break;
            case 104: is_float = 0, v = ((const uint8_t*)in)[i] != 0; break;
            default: return 1;
        }
        switch (to) {
            case 0: ((float*)out)[i] = is_float ? f : (float)v; break;
            case 1: ((uint16_t*)out)[i] = oracle_f32_to_f16(is_float ? f : (float)v); break;
            case 2: ((uint16_t*)out)[i] = oracle_f32_to_bf16(is_float ? f : (float)v); break;
            case 100: ((int32_t*)out)[i] = is_float ? (int32_t)oracle_saturate(f, -2147483648.f, 2147483648.f, INT32_MIN, INT32_MAX) : (int32_t)(uint32_t)(uint64_t)v; break;
            case 101: ((int64_t*)out)[i] = is_float ? oracle_saturate(f, -9223372036854775808.f, 9223372036854775808.f, INT64_MIN, INT64_MAX) : v; break;
            case 102: ((uint8_t*)out)[i] = is_float ? (uint8_t)oracle_saturate(f, 0.f, 255.f, 0, 255) : (uint8_t)(uint64_t)v; break;
            case 103: ((int8_t*)out)[i] = is_float ? (int8_t)oracle_saturate(f, -128.f, 127.f, -128, 127) : (int8_t)(uint8_t)(uint64_t)v; break;
            case 104: ((uint8_t*)out)[i] = is_float ? (f != 0.f) : (v != 0); break;
            default: return 1;
        }
    }
    return 0;
}

/* out = a (op) b, the three shapes given at one rank; op: 0 add, 1 subtract, 2 multiply, 3 divide */
ORACLE_API int oracle_binary_f32(int op, const float* a, const float* b, float* out, int rank, const int64_t* out_dims,
                                 const int64_t* a_dims, const int64_t* b_dims) {
    if (rank < 0 || rank > 16) return 1;
    int64_t sa[16], sb[16], coord[16], total = 1, ra = 1, rb = 1;
    for (int k = rank - 1; k >= 0; k--) {
        if ((a_dims[k] != out_dims[k] && a_dims[k] != 1) || (b_dims[k] != out_dims[k] && b_dims[k] != 1)) return 1;
        sa[k] = a_dims[k] == 1 ? 0 : ra;
        sb[k] = b_dims[k] == 1 ? 0 : rb;
        ra *= a_dims[k];
        rb *= b_dims[k];
        total *= out_dims[k];
        coord[k] = 0;
    }
    int64_t ia = 0, ib = 0;
    for (int64_t i = 0; i < total; i++) {
        const float x = a[ia], y = b[ib];
        out[i] = op == 1 ? x - y : op == 2 ? x * y : op == 3 ? x / y : x + y;
        for (int k = rank - 1; k >= 0; k--) {
            ia += sa[k];
            ib += sb[k];
            if (++coord[k] < out_dims[k]) break;
            ia -= sa[k] * out_dims[k];
            ib -= sb[k] * out_dims[k];
            coord[k] = 0;
        }
    }
    return 0;
}

ORACLE_API void oracle_softmax_f32(const float* x, float* out, int64_t outer, int64_t length, int64_t inner) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t o = 0; o < outer; o++)
        for (int64_t n = 0; n < inner; n++) {
            const float* xr = x + o * length * inner + n;
            float* yr = out + o * length * inner + n;
            double m = -INFINITY, sum = 0.0;
            for (int64_t i = 0; i < length; i++)
                if ((double)xr[i * inner] > m) m = xr[i * inner];
            for (int64_t i = 0; i < length; i++) sum += exp((double)xr[i * inner] - m);
            for (int64_t i = 0; i < length; i++) yr[i * inner] = (float)(exp((double)xr[i * inner] - m) / sum);
        }
}
