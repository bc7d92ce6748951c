// The extern "C" surface of libhipops.so: argument checks that need no kernel knowledge, the
// thread-local error string, and the hand-over to the launchers.  Nothing is thrown across it.
#include <cstdarg>
#include <cstdio>
#include <exception>

#include "ops/ops_common.hpp"

#define HIPOPS_API extern "C" __attribute__((visibility("default")))

namespace hipops {

static thread_local char g_error[512] = "";

hipattn_status fail(hipattn_status status, const char* format, ...) {
    va_list args;
    va_start(args, format);
    vsnprintf(g_error, sizeof(g_error), format, args);
    va_end(args);
    return status;
}

template <typename F>
static hipattn_status guarded(const char* what, F&& body) {
    try {
        return body();
    } catch (const std::exception& e) {
        return fail(HIPATTN_HIP_ERROR, "%s: %s", what, e.what());
    } catch (...) {
        return fail(HIPATTN_HIP_ERROR, "%s: unknown exception", what);
    }
}

}  // namespace hipops

using namespace hipops;

HIPOPS_API const char* hipops_last_error_string(void) { return g_error; }
HIPOPS_API int hipops_version(void) { return HIPOPS_VERSION_MAJOR * 1000 + HIPOPS_VERSION_MINOR; }

HIPOPS_API hipattn_status hipops_rms_norm(const void* x, const void* gamma, void* out, int64_t rows, int64_t hidden, float eps,
                                          int x_dtype, int gamma_dtype, int out_dtype, hipattn_stream stream) {
    return guarded("hipops_rms_norm", [&] {
        return rms_norm(x, gamma, out, rows, hidden, eps, x_dtype, gamma_dtype, out_dtype, (hipStream_t)stream);
    });
}

HIPOPS_API hipattn_status hipops_rope(const hipops_rope_desc* desc, const void* x, const void* cos, const void* sin,
                                      const int32_t* positions, void* out, hipattn_stream stream) {
    return guarded("hipops_rope", [&] { return rope(desc, x, cos, sin, positions, out, (hipStream_t)stream); });
}

HIPOPS_API hipattn_status hipops_matmul_workspace_size(const hipops_matmul_desc* desc, size_t* bytes) {
    return guarded("hipops_matmul_workspace_size", [&] { return matmul_workspace_size(desc, bytes); });
}

HIPOPS_API hipattn_status hipops_matmul(const hipops_matmul_desc* desc, const void* a, const void* b, void* c, void* workspace,
                                        size_t workspace_bytes, hipattn_stream stream) {
    return guarded("hipops_matmul", [&] { return matmul(desc, a, b, c, workspace, workspace_bytes, (hipStream_t)stream); });
}

HIPOPS_API hipattn_status hipops_gather(const void* data, const void* indices, void* out, int64_t batch, int64_t outer,
                                        int64_t axis_dim, int64_t inner_bytes, int64_t num_indices, int index_dtype,
                                        hipattn_stream stream) {
    return guarded("hipops_gather", [&] {
        return gather(data, indices, out, batch, outer, axis_dim, inner_bytes, num_indices, index_dtype, (hipStream_t)stream);
    });
}

HIPOPS_API hipattn_status hipops_concat(const void* const* inputs, const int64_t* axis_bytes, int num_inputs, int64_t outer,
                                        void* out, hipattn_stream stream) {
    return guarded("hipops_concat", [&] { return concat(inputs, axis_bytes, num_inputs, outer, out, (hipStream_t)stream); });
}

HIPOPS_API hipattn_status hipops_swish(const void* x, void* out, int64_t count, float beta, int dtype, hipattn_stream stream) {
    return guarded("hipops_swish", [&] { return swish(x, out, count, beta, dtype, (hipStream_t)stream); });
}

HIPOPS_API hipattn_status hipops_multiply(const void* a, const void* b, void* out, int64_t count, int dtype,
                                          hipattn_stream stream) {
    return guarded("hipops_multiply", [&] { return multiply(a, b, out, count, dtype, (hipStream_t)stream); });
}

HIPOPS_API hipattn_status hipops_transpose(const void* in, void* out, int rank, const int64_t* dims, const int32_t* order,
                                           int element_bytes, hipattn_stream stream) {
    return guarded("hipops_transpose", [&] { return transpose(in, out, rank, dims, order, element_bytes, (hipStream_t)stream); });
}

HIPOPS_API hipattn_status hipops_convert(const void* in, void* out, int64_t count, int from_dtype, int to_dtype,
                                         hipattn_stream stream) {
    return guarded("hipops_convert", [&] { return convert(in, out, count, from_dtype, to_dtype, (hipStream_t)stream); });
}

HIPOPS_API hipattn_status hipops_binary(int operation, const void* a, const void* b, void* out, int rank, const int64_t* out_dims,
                                        const int64_t* a_dims, const int64_t* b_dims, int dtype, hipattn_stream stream) {
    return guarded("hipops_binary", [&] { return binary(operation, a, b, out, rank, out_dims, a_dims, b_dims, dtype, (hipStream_t)stream); });
}

HIPOPS_API hipattn_status hipops_softmax(const void* x, void* out, int64_t outer, int64_t length, int64_t inner, int dtype,
                                         hipattn_stream stream) {
    return guarded("hipops_softmax", [&] { return softmax(x, out, outer, length, inner, dtype, (hipStream_t)stream); });
}

HIPOPS_API hipattn_status hipops_glu(const void* x, void* out, int64_t rows, int64_t width, int activation, int gate_first,
                                     int dtype, hipattn_stream stream) {
    return guarded("hipops_glu", [&] { return glu(x, out, rows, width, activation, gate_first, dtype, (hipStream_t)stream); });
}
