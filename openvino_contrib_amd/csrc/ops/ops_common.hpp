// Internal declarations shared by the sources of libhipops.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hipops.h"

namespace hipops {

// records the message for hipops_last_error_string() on this thread and returns `status`
hipattn_status fail(hipattn_status status, const char* format, ...) __attribute__((format(printf, 2, 3)));

hipattn_status rms_norm(const void* x, const void* gamma, void* out, int64_t rows, int64_t hidden, float eps, int x_dtype,
                        int gamma_dtype, int out_dtype, hipStream_t stream);
hipattn_status rope(const hipops_rope_desc* desc, const void* x, const void* cos, const void* sin, const int32_t* positions,
                    void* out, hipStream_t stream);
hipattn_status gather(const void* data, const void* indices, void* out, int64_t batch, int64_t outer, int64_t axis_dim,
                      int64_t inner_bytes, int64_t num_indices, int index_dtype, hipStream_t stream);
hipattn_status concat(const void* const* inputs, const int64_t* axis_bytes, int num_inputs, int64_t outer, void* out,
                      hipStream_t stream);
hipattn_status swish(const void* x, void* out, int64_t count, float beta, int dtype, hipStream_t stream);
hipattn_status multiply(const void* a, const void* b, void* out, int64_t count, int dtype, hipStream_t stream);
hipattn_status glu(const void* x, void* out, int64_t rows, int64_t width, int activation, int gate_first, int dtype,
                   hipStream_t stream);
hipattn_status transpose(const void* in, void* out, int rank, const int64_t* dims, const int32_t* order, int element_bytes,
                         hipStream_t stream);
hipattn_status convert(const void* in, void* out, int64_t count, int from_dtype, int to_dtype, hipStream_t stream);
hipattn_status binary(int op, const void* a, const void* b, void* out, int rank, const int64_t* out_dims, const int64_t* a_dims,
                      const int64_t* b_dims, int dtype, hipStream_t stream);
hipattn_status softmax(const void* x, void* out, int64_t outer, int64_t length, int64_t inner, int dtype, hipStream_t stream);
hipattn_status matmul_workspace_size(const hipops_matmul_desc* desc, size_t* bytes);
hipattn_status matmul(const hipops_matmul_desc* desc, const void* a, const void* b, void* c, void* workspace,
                      size_t workspace_bytes, hipStream_t stream);

}  // namespace hipops
