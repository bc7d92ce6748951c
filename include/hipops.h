/*
 * hipops - thin C ABI over the operators that stand either side of attention in a decoder layer
 * on MI355X (gfx950): RMS normalisation, rotary position embedding, MatMul, Gather, Concat, the gated
 * MLP's Swish, Multiply and GLU, Transpose and Convert between them, and the broadcasting
 * arithmetic and Softmax of attention in its decomposed form.
 *
 * Same conventions as hipattn.h, whose status codes, dtype codes and stream type it uses: plain C,
 * device pointers of the current HIP device, asynchronous on the given stream, nothing allocated
 * behind the caller's back (MatMul scratch comes in through a workspace argument), no exceptions;
 * hipops_last_error_string() describes the last failure on the calling thread.  The library
 * (libhipops.so) is separate from libhipattn.so because it links hipBLASLt.
 *
 * Reference citations are relative to modules/nvidia_plugin/ of openvino_contrib.
 */
#ifndef HIPOPS_H_
#define HIPOPS_H_

#include "hipattn.h"

#ifdef __cplusplus
extern "C" {
#endif

#define HIPOPS_VERSION_MAJOR 0
#define HIPOPS_VERSION_MINOR 4

#define HIPOPS_I64 101 /* element types beyond hipattn.h's: 64-bit integers (indices, shapes) */

const char* hipops_last_error_string(void);
int hipops_version(void); /* major * 1000 + minor */

/* ---- RMS normalisation ----------------------------------------------------------------
 * out[r, i] = x[r, i] * 1/sqrt(mean_i(x[r, i]^2) + eps) * gamma[i]  over the last axis.
 * The reference has no fused form: a model carrying this pattern reaches it as Power/ReduceMean/
 * Add/Sqrt/Divide/Multiply nodes (src/ops/elementwise_binary.hpp, src/ops/reduce.cpp); OpenVINO
 * fuses the pattern into its internal RMS operator, which is what this entry point serves.
 * x, out: [rows, hidden] contiguous; gamma: [hidden] or NULL (all ones).  Sums and products are
 * fp32, the result is rounded once to out_dtype.  dtypes: HIPATTN_F32 / F16 / BF16. */
hipattn_status hipops_rms_norm(const void* device_x, const void* device_gamma, void* device_out, int64_t rows,
                               int64_t hidden, float eps, int x_dtype, int gamma_dtype, int out_dtype,
                               hipattn_stream stream);

/* ---- rotary position embedding ----------------------------------------------------------
 * OpenVINO's internal RoPE operator for the two layouts of the LLaMA and GPT-J families; the
 * reference runs the unfused Slice/Multiply/Concat/Add chain (src/ops/strided_slice.cpp,
 * src/ops/concat.cpp:20-102, src/ops/multiply.cpp:43, src/ops/add.cpp:17-43).
 *
 * x: num_tokens x num_heads rows of head_size elements; element (t, h, i) lies at
 *    x + t * x_token_stride + h * x_head_stride + i (strides in elements), so a slice of a packed
 *    q/k/v projection is addressed in place.  out likewise with its own strides.
 * The first rotary_ndims elements of a head are rotated, the rest copied.
 * cos, sin: tables of table_dtype, row p at cos + p * table_row_stride.
 *   interleaved == 0 (rotate-half):  rows of rotary_ndims values, half = rotary_ndims / 2,
 *       out[i]        = x[i] * cos[i]               - x[i + half] * sin[i]
 *       out[i + half] = x[i + half] * cos[i + half] + x[i]        * sin[i + half]      for i < half
 *   interleaved != 0 (adjacent pairs): rows of rotary_ndims / 2 values,
 *       out[2i]     = x[2i] * cos[i]     - x[2i + 1] * sin[i]
 *       out[2i + 1] = x[2i + 1] * cos[i] + x[2i]     * sin[i]                          for i < half
 * The table row of token t is positions[t] when positions is not NULL (the operator's gather
 * input), otherwise t.  Products and sums are fp32, rounded once to `dtype`.
 * A row index outside [0, table_rows) is an error the kernel cannot report: the caller
 * guarantees the range. */
typedef struct hipops_rope_desc {
    int dtype;        /* x and out: HIPATTN_F32 / F16 / BF16 */
    int table_dtype;  /* cos and sin: HIPATTN_F32 / F16 / BF16 */
    int64_t num_tokens;
    int num_heads;
    int head_size;
    int rotary_ndims; /* even, <= head_size; 0 selects head_size */
    int interleaved;
    int64_t x_token_stride, x_head_stride;
    int64_t out_token_stride, out_head_stride;
    int64_t table_rows;
    int64_t table_row_stride;
} hipops_rope_desc;
hipattn_status hipops_rope(const hipops_rope_desc* desc, const void* device_x, const void* device_cos,
                           const void* device_sin, const int32_t* device_positions, void* device_out,
                           hipattn_stream stream);

/* ---- MatMul -----------------------------------------------------------------------------
 * C[b] = op(A[b]) * op(B[b]), row-major, through hipBLASLt.  Replaces MatMulOp
 * (src/ops/matmul.cpp:22-76 for the shape rules, :185-227 for cublasGemmStridedBatchedEx).
 * op(A) is m x k (A stored k x m when transpose_a), op(B) is k x n (B stored n x k when
 * transpose_b - the weight layout of a projection).  batch_stride_a / _b == 0 broadcasts that
 * operand over the batch, as the reference does for an operand without batch dimensions.
 * Leading dimensions are the row lengths of the stored matrices (no padding): that is what the
 * operator's contiguous tensors have.  A and B share ab_dtype (F32 / F16 / BF16); C is c_dtype
 * (same, or F32); accumulation is always fp32 (the reference lets cuBLAS accumulate f16 x f16 ->
 * f16 in half precision, matmul.cpp:84-87; fp32 is the tighter of the two).
 * The workspace may be NULL / 0; hipops_matmul_workspace_size gives the size that lets the
 * library choose among all of its algorithms.  The first call with a new shape on a device times
 * the library's candidate algorithms on the given operands (a few extra launches that write the
 * same C, and one event synchronisation) and keeps the fastest; under stream capture it takes the
 * library's first choice instead. */
typedef struct hipops_matmul_desc {
    int ab_dtype;
    int c_dtype;
    int64_t m, n, k;
    int64_t batch;
    int transpose_a, transpose_b;
    int64_t batch_stride_a, batch_stride_b; /* in elements; 0 = broadcast */
} hipops_matmul_desc;
hipattn_status hipops_matmul_workspace_size(const hipops_matmul_desc* desc, size_t* bytes);
hipattn_status hipops_matmul(const hipops_matmul_desc* desc, const void* device_a, const void* device_b,
                             void* device_c, void* device_workspace, size_t workspace_bytes, hipattn_stream stream);

/* ---- gated MLP pieces: Swish, Multiply, GLU --------------------------------------------------
 * hipops_swish:    out = x / (1 + exp(-beta x))   SwishOp (src/ops/swish.cpp:41-59,
 *                  src/kernels/swish.cu:17-19), beta from the operator's second input (default 1).
 * hipops_multiply: out = a * b, equal shapes       MultiplyOp (src/ops/multiply.cpp:43 over
 *                  src/kernels/details/elementwise_binary.cuh:24-46, without broadcasting).
 * hipops_glu:      OpenVINO's fused gated linear unit (internal operator GLU, the fusion of
 *                  VariadicSplit + Swish/Gelu + Multiply; the reference would run the three):
 *                  x is [rows, 2 * width]; out[r, i] = act(x[r, g + i]) * x[r, u + i] with
 *                  g = gate_first ? 0 : width and u = width - g, act one of HIPOPS_GLU_*.
 * All three: fp32 arithmetic, one rounding to `dtype` (HIPATTN_F32 / F16 / BF16). */
#define HIPOPS_GLU_SWISH 0
#define HIPOPS_GLU_GELU 1      /* x * 0.5 (1 + erf(x / sqrt 2)) */
#define HIPOPS_GLU_GELU_TANH 2 /* x * 0.5 (1 + tanh(sqrt(2 / pi) (x + 0.044715 x^3))) */
hipattn_status hipops_swish(const void* device_x, void* device_out, int64_t count, float beta, int dtype,
                            hipattn_stream stream);
hipattn_status hipops_multiply(const void* device_a, const void* device_b, void* device_out, int64_t count, int dtype,
                               hipattn_stream stream);
hipattn_status hipops_glu(const void* device_x, void* device_out, int64_t rows, int64_t width, int activation,
                          int gate_first, int dtype, hipattn_stream stream);

/* ---- Add / Subtract / Multiply / Divide with broadcasting ---------------------------------------
 * out = a (op) b under numpy's broadcasting rule, as the reference's ElementwiseBinaryOp
 * (src/ops/elementwise_binary.hpp:16-76 over src/kernels/details/elementwise_binary.cuh:24-46 and
 * numpy_broadcast_mapper.cuh; AddOp src/ops/add.cpp:17-43, MultiplyOp src/ops/multiply.cpp:43,
 * SubtractOp, DivideOp).  The three shapes have one rank (<= HIPOPS_BINARY_MAX_RANK; the caller
 * pads the shorter ones with leading 1s); an operand's extent is the output's or 1.  fp32
 * arithmetic, one rounding to `dtype` (HIPATTN_F32 / F16 / BF16); division is correctly rounded.
 * out may be a or b when that operand has the output's shape. */
#define HIPOPS_BINARY_MAX_RANK 8
#define HIPOPS_ADD 0
#define HIPOPS_SUBTRACT 1
#define HIPOPS_MULTIPLY 2
#define HIPOPS_DIVIDE 3
hipattn_status hipops_binary(int operation, const void* device_a, const void* device_b, void* device_out, int rank,
                             const int64_t* out_dims, const int64_t* a_dims, const int64_t* b_dims, int dtype,
                             hipattn_stream stream);

/* ---- Softmax --------------------------------------------------------------------------------
 * x seen as [outer, length, inner]: out[o, i, n] = exp(x[o, i, n] - max_i) / sum_i exp(x[o, i, n] - max_i),
 * SoftmaxOp (src/ops/softmax.cpp:73-196: cudnnSoftmaxForward, accurate algorithm, channel mode, after
 * folding the axes around `axis` the same way).  fp32 arithmetic, one rounding to `dtype`
 * (HIPATTN_F32 / F16 / BF16).  A slice that is -inf throughout gives NaN.  In place is allowed. */
hipattn_status hipops_softmax(const void* device_x, void* device_out, int64_t outer, int64_t length, int64_t inner,
                              int dtype, hipattn_stream stream);

/* ---- Transpose -----------------------------------------------------------------------------
 * out = in with its axes permuted: output axis k is input axis order[k], as TransposeOp
 * (src/ops/transpose.cpp:54-135; the reference calls cuTENSOR, or its own gather kernel where
 * cuTENSOR has no code for the GPU, :215-270).  dims: the input's extents, rank <=
 * HIPOPS_TRANSPOSE_MAX_RANK; both tensors contiguous; the operator moves elements of
 * element_bytes (1, 2, 4 or 8) whatever their type.  dims and order are host arrays.  Not in place.
 * A permutation that keeps the innermost axis moves contiguous runs in pieces of up to 16 bytes;
 * one that changes it goes through 64 x 64 tiles in LDS. */
#define HIPOPS_TRANSPOSE_MAX_RANK 8
hipattn_status hipops_transpose(const void* device_in, void* device_out, int rank, const int64_t* dims,
                                const int32_t* order, int element_bytes, hipattn_stream stream);

/* ---- Convert -------------------------------------------------------------------------------
 * out[i] = (to_dtype) in[i], ConvertOp (src/ops/convert.cpp:19-58, src/kernels/convert.cuh:24-49:
 * static_cast, through float where a 16-bit floating type is involved).  Types: HIPATTN_F32 / F16 /
 * BF16 / I32, HIPOPS_I64 / U8 / I8 / BOOL (one byte, 0 or 1).
 *   floating -> floating   one rounding to nearest even
 *   integer  -> floating   through float, to nearest even
 *   floating -> integer    towards zero; values beyond the target's range saturate and NaN gives 0
 *                          (C leaves both undefined)
 *   integer  -> integer    modulo 2^bits, as a C cast
 *   any      -> boolean    1 where the value is not zero (NaN included)
 * Equal types copy (nothing at all when in == out). */
#define HIPOPS_U8 102 /* plain bytes; HIPATTN_U8 names the quantised KV-cache rows */
#define HIPOPS_I8 103
#define HIPOPS_BOOL 104
hipattn_status hipops_convert(const void* device_in, void* device_out, int64_t count, int from_dtype, int to_dtype,
                              hipattn_stream stream);

/* ---- Gather -----------------------------------------------------------------------------
 * Gather (opset 1/7/8) with batch_dims, as GatherOp sets it up (src/ops/gather.cpp:60-127) and
 * the kernel executes it (src/kernels/gather.cu:19-47): data seen as
 * [batch, outer, axis_dim, inner], indices as [batch, num_indices], out as
 * [batch, outer, num_indices, inner].  A negative index counts from the end; an index outside
 * the axis after that yields zeros.  inner_bytes = elements after the axis x element size: the
 * operator moves bytes, whatever the element type.  index_dtype: HIPATTN_I32 or HIPOPS_I64. */
hipattn_status hipops_gather(const void* device_data, const void* device_indices, void* device_out, int64_t batch,
                             int64_t outer, int64_t axis_dim, int64_t inner_bytes, int64_t num_indices,
                             int index_dtype, hipattn_stream stream);

/* ---- Concat -----------------------------------------------------------------------------
 * Concat along one axis, ConcatOp (src/ops/concat.cpp:31-56, src/kernels/concat.cu): input i seen
 * as [outer, axis_bytes[i]] (axis_bytes = its extent along the axis x elements after the axis x
 * element size), out as [outer, sum of axis_bytes].  device_inputs is a HOST array of
 * num_inputs device pointers, axis_bytes a host array; inputs with axis_bytes 0 are skipped. */
hipattn_status hipops_concat(const void* const* device_inputs, const int64_t* axis_bytes, int num_inputs,
                             int64_t outer, void* device_out, hipattn_stream stream);

#ifdef __cplusplus
}
#endif
#endif /* HIPOPS_H_ */
