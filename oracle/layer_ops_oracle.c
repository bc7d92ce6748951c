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
