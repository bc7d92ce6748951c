// MatMul through hipBLASLt: a plain library GEMM with fp32 accumulation.  The operator's tensors
// are row-major; hipBLASLt is column-major, so the product is taken transposed
// (C^T = op(B)^T * op(A)^T) with the operands swapped and no data movement.  Descriptors and the
// algorithm are kept per (device, shape), so a repeated shape costs one hipblasLtMatmul call; the
// algorithm is the fastest of the heuristic's candidates, timed once when the shape is first seen
// outside a stream capture (that call synchronises with its stream; calls on other devices are not
// held up by it: every device has a lock of its own).
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

#include "ops/ops_common.hpp"

namespace hipops {

namespace {

constexpr size_t kRecommendedWorkspace = 32u << 20;

struct Plan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t first = nullptr, second = nullptr, result = nullptr;
    hipblasLtMatmulAlgo_t algo{};
    size_t workspace = 0;
    bool tuned = false;  // false: the heuristic's first candidate (picked under a stream capture); timed by the next call outside one
    void destroy() {
        if (desc) hipblasLtMatmulDescDestroy(desc);
        if (first) hipblasLtMatrixLayoutDestroy(first);
        if (second) hipblasLtMatrixLayoutDestroy(second);
        if (result) hipblasLtMatrixLayoutDestroy(result);
        desc = nullptr;
        first = second = result = nullptr;
    }
};
// destroys what a plan under construction holds unless it reaches the cache
struct PlanGuard {
    Plan& plan;
    bool keep = false;
    ~PlanGuard() {
        if (!keep) plan.destroy();
    }
};

using Key = std::tuple<int, int, int, int64_t, int64_t, int64_t, int64_t, int, int, int64_t, int64_t, size_t>;

struct DeviceState {
    std::mutex mutex;  // the handle and the plans of this device
    hipblasLtHandle_t handle = nullptr;
    std::map<Key, Plan> plans;
};

std::mutex g_mutex;  // the map of devices only
std::map<int, DeviceState> g_devices;  // never destroyed: the library may outlive static teardown order

bool blas_type(int dtype, hipDataType* t) {
    switch (dtype) {
        case HIPATTN_F32: *t = HIP_R_32F; return true;
        case HIPATTN_F16: *t = HIP_R_16F; return true;
        case HIPATTN_BF16: *t = HIP_R_16BF; return true;
        default: return false;
    }
}

#define BLAS_CHECK(call)                                                                                          \
    do {                                                                                                          \
        const hipblasStatus_t st_ = (call);                                                                       \
        if (st_ != HIPBLAS_STATUS_SUCCESS) return fail(HIPATTN_HIP_ERROR, "matmul: %s failed with status %d", #call, (int)st_); \
    } while (0)

hipattn_status make_layout(hipblasLtMatrixLayout_t* layout, hipDataType type, int64_t rows, int64_t cols, int64_t ld,
                           int64_t batch, int64_t stride) {
    BLAS_CHECK(hipblasLtMatrixLayoutCreate(layout, type, (uint64_t)rows, (uint64_t)cols, ld));
    const int32_t count = (int32_t)batch;
    BLAS_CHECK(hipblasLtMatrixLayoutSetAttribute(*layout, HIPBLASLT_MATRIX_LAYOUT_BATCH_COUNT, &count, sizeof(count)));
    BLAS_CHECK(hipblasLtMatrixLayoutSetAttribute(*layout, HIPBLASLT_MATRIX_LAYOUT_STRIDED_BATCH_OFFSET, &stride, sizeof(stride)));
    return HIPATTN_OK;
}

hipattn_status validate(const hipops_matmul_desc* d) {
    if (!d) return fail(HIPATTN_INVALID_ARGUMENT, "matmul: null descriptor");
    hipDataType t;
    if (!blas_type(d->ab_dtype, &t) || !blas_type(d->c_dtype, &t)) return fail(HIPATTN_UNSUPPORTED, "matmul: dtypes must be f32, f16 or bf16");
    if (d->c_dtype != d->ab_dtype && d->c_dtype != HIPATTN_F32)
        return fail(HIPATTN_UNSUPPORTED, "matmul: the result is of the operands' type or f32");
    // zero extents are refused as the reference refuses them (matmul.cpp:66-72)
    if (d->m <= 0 || d->n <= 0 || d->k <= 0 || d->batch <= 0)
        return fail(HIPATTN_INVALID_ARGUMENT, "matmul: m %lld n %lld k %lld batch %lld must be positive", (long long)d->m, (long long)d->n,
                    (long long)d->k, (long long)d->batch);
    if (d->m > 0x7fffffffLL || d->n > 0x7fffffffLL || d->k > 0x7fffffffLL || d->batch > 0x7fffffffLL)
        return fail(HIPATTN_UNSUPPORTED, "matmul: extent beyond 2^31");
    if (d->batch_stride_a < 0 || d->batch_stride_b < 0 || (d->batch_stride_a != 0 && d->batch_stride_a < d->m * d->k) ||
        (d->batch_stride_b != 0 && d->batch_stride_b < d->k * d->n))
        return fail(HIPATTN_INVALID_ARGUMENT, "matmul: batch strides must be 0 or at least one matrix");
    return HIPATTN_OK;
}

}  // namespace

hipattn_status matmul_workspace_size(const hipops_matmul_desc* d, size_t* bytes) {
    if (!bytes) return fail(HIPATTN_INVALID_ARGUMENT, "matmul: null size pointer");
    const hipattn_status st = validate(d);
    if (st != HIPATTN_OK) return st;
    *bytes = kRecommendedWorkspace;
    return HIPATTN_OK;
}

hipattn_status matmul(const hipops_matmul_desc* d, const void* a, const void* b, void* c, void* workspace, size_t workspace_bytes,
                      hipStream_t stream) {
    hipattn_status st = validate(d);
    if (st != HIPATTN_OK) return st;
    if (!a || !b || !c) return fail(HIPATTN_INVALID_ARGUMENT, "matmul: null pointer");
    if (!workspace) workspace_bytes = 0;
    if (workspace && ((uintptr_t)workspace % 256) != 0) return fail(HIPATTN_INVALID_ARGUMENT, "matmul: workspace must be 256-byte aligned");
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return fail(HIPATTN_NO_DEVICE, "matmul: no current device");

    DeviceState* dev_ptr = nullptr;
    {
        std::lock_guard<std::mutex> devices_lock(g_mutex);
        dev_ptr = &g_devices[device];  // (map nodes do not move)
    }
    DeviceState& dev = *dev_ptr;
    std::lock_guard<std::mutex> lock(dev.mutex);
    if (!dev.handle) BLAS_CHECK(hipblasLtCreate(&dev.handle));
    const Key key{device, d->ab_dtype, d->c_dtype, d->m, d->n, d->k, d->batch, d->transpose_a != 0, d->transpose_b != 0,
                  d->batch_stride_a, d->batch_stride_b, workspace_bytes};
    auto it = dev.plans.find(key);
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    const bool can_time = hipStreamIsCapturing(stream, &capturing) == hipSuccess && capturing == hipStreamCaptureStatusNone;
    if (it != dev.plans.end() && !it->second.tuned && can_time) {  // picked under a capture: time the candidates now
        it->second.destroy();
        dev.plans.erase(it);
        it = dev.plans.end();
    }
    if (it == dev.plans.end()) {
        Plan plan;
        PlanGuard guard{plan};
        hipDataType ab, ct;
        blas_type(d->ab_dtype, &ab);
        blas_type(d->c_dtype, &ct);
        BLAS_CHECK(hipblasLtMatmulDescCreate(&plan.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
        // first operand of the library call = this operator's B, second = its A
        const hipblasOperation_t op_first = d->transpose_b ? HIPBLAS_OP_T : HIPBLAS_OP_N;
        const hipblasOperation_t op_second = d->transpose_a ? HIPBLAS_OP_T : HIPBLAS_OP_N;
        BLAS_CHECK(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_first, sizeof(op_first)));
        BLAS_CHECK(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_second, sizeof(op_second)));
        // B stored [k, n] row-major is the column-major n x k matrix with ld n; stored [n, k] it is k x n with ld k
        st = d->transpose_b ? make_layout(&plan.first, ab, d->k, d->n, d->k, d->batch, d->batch_stride_b)
                            : make_layout(&plan.first, ab, d->n, d->k, d->n, d->batch, d->batch_stride_b);
        if (st != HIPATTN_OK) return st;
        // A stored [m, k] row-major is the column-major k x m matrix with ld k; stored [k, m] it is m x k with ld m
        st = d->transpose_a ? make_layout(&plan.second, ab, d->m, d->k, d->m, d->batch, d->batch_stride_a)
                            : make_layout(&plan.second, ab, d->k, d->m, d->k, d->batch, d->batch_stride_a);
        if (st != HIPATTN_OK) return st;
        st = make_layout(&plan.result, ct, d->n, d->m, d->n, d->batch, d->m * d->n);
        if (st != HIPATTN_OK) return st;
        hipblasLtMatmulPreference_t pref = nullptr;
        BLAS_CHECK(hipblasLtMatmulPreferenceCreate(&pref));
        const uint64_t max_ws = workspace_bytes;
        BLAS_CHECK(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws, sizeof(max_ws)));
        constexpr int kAsk = 16;
        hipblasLtMatmulHeuristicResult_t found[kAsk];
        int n_found = 0;
        const hipblasStatus_t hs = hipblasLtMatmulAlgoGetHeuristic(dev.handle, plan.desc, plan.first, plan.second, plan.result,
                                                                   plan.result, pref, kAsk, found, &n_found);
        hipblasLtMatmulPreferenceDestroy(pref);
        if (hs != HIPBLAS_STATUS_SUCCESS) return fail(HIPATTN_HIP_ERROR, "matmul: heuristic query failed with status %d", (int)hs);
        int pick = -1, usable = 0;
        for (int i = 0; i < n_found; i++)
            if (found[i].state == HIPBLAS_STATUS_SUCCESS && found[i].workspaceSize <= workspace_bytes) {
                if (pick < 0) pick = i;
                usable++;
            }
        if (pick < 0)
            return fail(HIPATTN_UNSUPPORTED, "matmul: hipBLASLt has no algorithm for m %lld n %lld k %lld batch %lld with %zu bytes of workspace",
                        (long long)d->m, (long long)d->n, (long long)d->k, (long long)d->batch, workspace_bytes);
        // The heuristic's order is a guess: the first time a shape is seen, and unless the stream is
        // being captured, every candidate runs a few times on the caller's own operands (each writes the
        // same C) and the fastest is kept.  A candidate that fails to run is skipped.
        if (usable > 1 && can_time) {
            hipEvent_t e0 = nullptr, e1 = nullptr;
            if (hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess) {
                const float one = 1.0f, zero = 0.0f;
                float best = 0.f;
                for (int i = 0; i < n_found; i++) {
                    if (found[i].state != HIPBLAS_STATUS_SUCCESS || found[i].workspaceSize > workspace_bytes) continue;
                    constexpr int kRuns = 4;
                    bool ok = true;
                    for (int r = 0; r < kRuns + 1 && ok; r++) {  // the first run is not timed
                        if (r == 1) ok = hipEventRecord(e0, stream) == hipSuccess;
                        ok = ok && hipblasLtMatmul(dev.handle, plan.desc, &one, b, plan.first, a, plan.second, &zero, c, plan.result, c,
                                                   plan.result, &found[i].algo, workspace, workspace_bytes, stream) == HIPBLAS_STATUS_SUCCESS;
                    }
                    float ms = 0.f;
                    ok = ok && hipEventRecord(e1, stream) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
                         hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
                    if (ok && (best == 0.f || ms < best)) best = ms, pick = i;
                }
            }
            if (e0) (void)hipEventDestroy(e0);
            if (e1) (void)hipEventDestroy(e1);
            (void)hipGetLastError();  // a candidate that could not launch must not poison the caller's next check
        }
        plan.algo = found[pick].algo;
        plan.workspace = found[pick].workspaceSize;
        plan.tuned = can_time || usable <= 1;
        it = dev.plans.emplace(key, plan).first;
        guard.keep = true;
    }
    const Plan& plan = it->second;
    const float alpha = 1.0f, beta = 0.0f;
    BLAS_CHECK(hipblasLtMatmul(dev.handle, plan.desc, &alpha, b, plan.first, a, plan.second, &beta, c, plan.result, c, plan.result,
                               &plan.algo, workspace, workspace_bytes, stream));
    return HIPATTN_OK;
}

}  // namespace hipops
