// Element-wise Add / Subtract / Multiply / Divide with numpy broadcasting, and Softmax along an
// axis: the operators the decomposed form of attention is made of (scores scaled, a mask added,
// softmax taken).  HBM-bound; fp32 arithmetic, one rounding to the tensor's type.
#include <algorithm>

#include "ops/ops_common.hpp"
#include "ops/vec8.hpp"

namespace hipops {

namespace {

constexpr int kAxes = HIPOPS_BINARY_MAX_RANK;

bool aligned(const void* ptr, size_t a) { return ((uintptr_t)ptr % a) == 0; }
bool float_dtype(int d) { return d == HIPATTN_F32 || d == HIPATTN_F16 || d == HIPATTN_BF16; }

hipattn_status launched(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HIPATTN_HIP_ERROR, "%s: %s", what, hipGetErrorString(e));
    return HIPATTN_OK;
}

// ------------------------------------------------------------------------------ binary, broadcasting
struct BinaryParams {
    const void* a;
    const void* b;
    void* out;
    int axes;                                     // of the output after merging, outermost first
    uint32_t extent[kAxes];
    int64_t stride_a[kAxes], stride_b[kAxes];     // in elements; 0 where the operand is broadcast
    int64_t count;                                // elements of the output
    int op;
    int dtype;
};

__device__ __forceinline__ float apply(int op, float x, float y) {
    switch (op) {
        case HIPOPS_SUBTRACT: return x - y;
        case HIPOPS_MULTIPLY: return x * y;
        case HIPOPS_DIVIDE: return x / y;
        default: return x + y;
    }
}

// kWide: eight output elements a lane along the innermost axis (whose extent is then a multiple of
// 8, and an operand's innermost stride is 1 -- read as eight -- or 0 -- one value for all eight)
// Index: uint32_t when the output has fewer than 2^32 elements (its divisions are a fraction of the 64-bit ones)
template <bool kWide, typename Index>
__global__ __launch_bounds__(256) void binary_kernel(BinaryParams p) {
    constexpr int kPer = kWide ? 8 : 1;
    const int64_t first = ((int64_t)blockIdx.x * 256 + threadIdx.x) * kPer;
    if (first >= p.count) return;
    Index rest = (Index)first;
    int64_t oa = 0, ob = 0;
#pragma unroll 1
    for (int k = p.axes - 1; k > 0; k--) {
        const Index next = rest / p.extent[k], c = rest - next * p.extent[k];
        oa += (int64_t)c * p.stride_a[k];
        ob += (int64_t)c * p.stride_b[k];
        rest = next;
    }
    oa += (int64_t)rest * p.stride_a[0];
    ob += (int64_t)rest * p.stride_b[0];
    if constexpr (kWide) {
        const int last = p.axes - 1;
        Float8 x, y, o;
        if (p.stride_a[last] != 0) {
            x = load8(p.a, oa, p.dtype);
        } else {
            const float v = load_scalar(p.a, oa, p.dtype);
#pragma unroll
            for (int i = 0; i < 8; i++) x.v[i] = v;
        }
        if (p.stride_b[last] != 0) {
            y = load8(p.b, ob, p.dtype);
        } else {
            const float v = load_scalar(p.b, ob, p.dtype);
#pragma unroll
            for (int i = 0; i < 8; i++) y.v[i] = v;
        }
#pragma unroll
        for (int i = 0; i < 8; i++) o.v[i] = apply(p.op, x.v[i], y.v[i]);
        store8(p.out, first, p.dtype, o);
    } else {
        store_scalar(p.out, first, p.dtype, apply(p.op, load_scalar(p.a, oa, p.dtype), load_scalar(p.b, ob, p.dtype)));
    }
}

// ------------------------------------------------------------------------------ softmax
// f32 tensors get the accurate exponential (the fast one's error grows with the argument, to a few
// 1e-6 of the result at |x| = 30, which an f32 result shows and a 16-bit one does not)
__device__ __forceinline__ float exp_of(int dtype, float x) { return dtype == HIPATTN_F32 ? expf(x) : __expf(x); }

struct SoftmaxParams {
    const void* x;
    void* out;
    int64_t outer, length, inner;  // x seen as [outer, length, inner]; softmax over `length`
    int dtype;
};

// inner == 1: a wavefront per row, eight elements a lane per step; the row is read twice (running
// maximum and sum first, then the quotients), the second time from cache
template <bool kWide>
__global__ __launch_bounds__(256) void softmax_rows_kernel(SoftmaxParams p) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= p.outer) return;
    const int lane = threadIdx.x & 63;
    const int64_t base = row * p.length;
    constexpr int kPer = kWide ? 8 : 1;
    float m = -INFINITY, l = 0.f;
    for (int64_t i = (int64_t)lane * kPer; i < p.length; i += 64 * kPer) {
        float v[kPer];
        if constexpr (kWide) {
            const Float8 r = load8(p.x, base + i, p.dtype);
#pragma unroll
            for (int k = 0; k < 8; k++) v[k] = r.v[k];
        } else {
            v[0] = load_scalar(p.x, base + i, p.dtype);
        }
        float chunk = v[0];
#pragma unroll
        for (int k = 1; k < kPer; k++) chunk = fmaxf(chunk, v[k]);
        const float m_new = fmaxf(m, chunk);
        if (m_new > -INFINITY) {  // a row of -inf so far keeps l = 0
            float add = 0.f;
#pragma unroll
            for (int k = 0; k < kPer; k++) add += exp_of(p.dtype, v[k] - m_new);
            l = l * exp_of(p.dtype, m - m_new) + add;
            m = m_new;
        }
    }
    const float row_max = wave_max(m);
    l = row_max > -INFINITY ? l * exp_of(p.dtype, m - row_max) : 0.f;
    const float inv = 1.0f / wave_sum(l);  // a row that is -inf throughout divides 0 by 0: NaN, as exp(-inf + inf) gives
    for (int64_t i = (int64_t)lane * kPer; i < p.length; i += 64 * kPer) {
        if constexpr (kWide) {
            Float8 r = load8(p.x, base + i, p.dtype);
#pragma unroll
            for (int k = 0; k < 8; k++) r.v[k] = exp_of(p.dtype, r.v[k] - row_max) * inv;
            store8(p.out, base + i, p.dtype, r);
        } else {
            store_scalar(p.out, base + i, p.dtype, exp_of(p.dtype, load_scalar(p.x, base + i, p.dtype) - row_max) * inv);
        }
    }
}

// inner == 1 and rows of at most 64 * 8 * kKeep elements: the row stays in registers between the
// maximum, the sum and the quotients, so it is read once
template <int kKeep>
__global__ __launch_bounds__(256) void softmax_kept_rows_kernel(SoftmaxParams p) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= p.outer) return;
    const int lane = threadIdx.x & 63;
    const int64_t base = row * p.length;
    Float8 keep[kKeep];
    float m = -INFINITY;
#pragma unroll
    for (int c = 0; c < kKeep; c++) {
        const int64_t i = ((int64_t)c * 64 + lane) * 8;
        if (i < p.length) {
            keep[c] = load8(p.x, base + i, p.dtype);
#pragma unroll
            for (int k = 0; k < 8; k++) m = fmaxf(m, keep[c].v[k]);
        }
    }
    m = wave_max(m);
    float l = 0.f;
#pragma unroll
    for (int c = 0; c < kKeep; c++) {
        const int64_t i = ((int64_t)c * 64 + lane) * 8;
        if (i < p.length) {
#pragma unroll
            for (int k = 0; k < 8; k++) {
                keep[c].v[k] = exp_of(p.dtype, keep[c].v[k] - m);  // a row of -inf throughout: exp(nan), as the other kernels give
                l += keep[c].v[k];
            }
        }
    }
    const float inv = 1.0f / wave_sum(l);
#pragma unroll
    for (int c = 0; c < kKeep; c++) {
        const int64_t i = ((int64_t)c * 64 + lane) * 8;
        if (i < p.length) {
#pragma unroll
            for (int k = 0; k < 8; k++) keep[c].v[k] *= inv;
            store8(p.out, base + i, p.dtype, keep[c]);
        }
    }
}

// inner > 1: a lane per (outer, inner) position walks the axis; neighbouring lanes are neighbours in memory
__global__ __launch_bounds__(256) void softmax_strided_kernel(SoftmaxParams p) {
    const int64_t pos = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (pos >= p.outer * p.inner) return;
    const int64_t o = pos / p.inner, in = pos - o * p.inner;
    const int64_t base = o * p.length * p.inner + in;
    float m = -INFINITY, l = 0.f;
    for (int64_t i = 0; i < p.length; i++) {
        const float v = load_scalar(p.x, base + i * p.inner, p.dtype);
        const float m_new = fmaxf(m, v);
        if (m_new > -INFINITY) {
            l = l * exp_of(p.dtype, m - m_new) + exp_of(p.dtype, v - m_new);
            m = m_new;
        }
    }
    const float inv = 1.0f / l;
    for (int64_t i = 0; i < p.length; i++)
        store_scalar(p.out, base + i * p.inner, p.dtype, exp_of(p.dtype, load_scalar(p.x, base + i * p.inner, p.dtype) - m) * inv);
}

}  // namespace

hipattn_status binary(int op, const void* a, const void* b, void* out, int rank, const int64_t* out_dims, const int64_t* a_dims,
                      const int64_t* b_dims, int dtype, hipStream_t stream) {
    if (op < HIPOPS_ADD || op > HIPOPS_DIVIDE) return fail(HIPATTN_INVALID_ARGUMENT, "binary: operation %d", op);
    if (!float_dtype(dtype)) return fail(HIPATTN_UNSUPPORTED, "binary: dtype must be f32, f16 or bf16");
    if (rank < 0 || rank > kAxes || (rank > 0 && (!out_dims || !a_dims || !b_dims)))
        return fail(HIPATTN_INVALID_ARGUMENT, "binary: rank %d (0 to %d expected, with the three shapes)", rank, kAxes);
    int64_t count = 1;
    for (int k = 0; k < rank; k++) {
        if (out_dims[k] < 0) return fail(HIPATTN_INVALID_ARGUMENT, "binary: negative extent");
        for (const int64_t* dims : {a_dims, b_dims})
            if (dims[k] != out_dims[k] && dims[k] != 1)
                return fail(HIPATTN_INVALID_ARGUMENT, "binary: extent %lld of an operand does not broadcast to %lld (axis %d)",
                            (long long)dims[k], (long long)out_dims[k], k);
        if (out_dims[k] > 0xffffffffLL) return fail(HIPATTN_UNSUPPORTED, "binary: extent beyond 2^32");
        count *= out_dims[k];
    }
    if (count == 0) return HIPATTN_OK;
    if (!a || !b || !out) return fail(HIPATTN_INVALID_ARGUMENT, "binary: null pointer");

    // strides of the operands along the output's axes (0 where broadcast); axes of extent 1 go, and
    // neighbours merge when both operands step over them like over one axis
    int64_t sa[kAxes], sb[kAxes];
    {
        int64_t ra = 1, rb = 1;
        for (int k = rank - 1; k >= 0; k--) {
            sa[k] = a_dims[k] == 1 ? 0 : ra;
            sb[k] = b_dims[k] == 1 ? 0 : rb;
            ra *= a_dims[k];
            rb *= b_dims[k];
        }
    }
    BinaryParams p{};
    p.a = a, p.b = b, p.out = out, p.count = count, p.op = op, p.dtype = dtype;
    int n = 0;
    int64_t extent[kAxes];
    for (int k = 0; k < rank; k++) {
        if (out_dims[k] == 1) continue;
        const bool merges = n > 0 && p.stride_a[n - 1] == sa[k] * out_dims[k] && p.stride_b[n - 1] == sb[k] * out_dims[k];
        if (merges) {
            extent[n - 1] *= out_dims[k];
            p.stride_a[n - 1] = sa[k];
            p.stride_b[n - 1] = sb[k];
        } else {
            extent[n] = out_dims[k];
            p.stride_a[n] = sa[k];
            p.stride_b[n] = sb[k];
            n++;
        }
    }
    if (n == 0) {  // one element
        extent[0] = 1, p.stride_a[0] = p.stride_b[0] = 0, n = 1;
    }
    for (int k = 0; k < n; k++) {
        if (extent[k] > 0xffffffffLL) return fail(HIPATTN_UNSUPPORTED, "binary: merged extent beyond 2^32");
        p.extent[k] = (uint32_t)extent[k];
    }
    p.axes = n;
    // eight elements a lane: the innermost extent a multiple of 8, and every operand either read as
    // eight consecutive elements from 16-byte aligned addresses or broadcast along that axis
    bool wide = extent[n - 1] % 8 == 0 && aligned(out, 16);
    const size_t esz = dtype == HIPATTN_F32 ? 4 : 2;
    auto operand_ok = [&](const void* ptr, const int64_t* stride) {
        if (stride[n - 1] == 0) return true;
        if (!aligned(ptr, 8 * esz > 16 ? 16 : 8 * esz)) return false;
        for (int k = 0; k < n - 1; k++)
            if (stride[k] % 8) return false;
        return true;
    };
    wide = wide && operand_ok(a, p.stride_a) && operand_ok(b, p.stride_b);
    const int64_t items = wide ? count / 8 : count;
    if ((items + 255) / 256 > 0x7fffffffLL) return fail(HIPATTN_UNSUPPORTED, "binary: too many elements for one launch");
    const dim3 grid((unsigned)((items + 255) / 256));
    const bool small = count < 0xffffffffLL;
    if (wide && small)
        hipLaunchKernelGGL((binary_kernel<true, uint32_t>), grid, dim3(256), 0, stream, p);
    else if (wide)
        hipLaunchKernelGGL((binary_kernel<true, int64_t>), grid, dim3(256), 0, stream, p);
    else if (small)
        hipLaunchKernelGGL((binary_kernel<false, uint32_t>), grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL((binary_kernel<false, int64_t>), grid, dim3(256), 0, stream, p);
    return launched("binary");
}

hipattn_status softmax(const void* x, void* out, int64_t outer, int64_t length, int64_t inner, int dtype, hipStream_t stream) {
    if (outer < 0 || length < 0 || inner < 0) return fail(HIPATTN_INVALID_ARGUMENT, "softmax: negative extent");
    if (!float_dtype(dtype)) return fail(HIPATTN_UNSUPPORTED, "softmax: dtype must be f32, f16 or bf16");
    if (outer * length * inner == 0) return HIPATTN_OK;
    if (!x || !out) return fail(HIPATTN_INVALID_ARGUMENT, "softmax: null pointer");
    SoftmaxParams p{x, out, outer, length, inner, dtype};
    if (inner == 1) {
        const int64_t blocks = (outer + 3) / 4;
        if (blocks > 0x7fffffffLL) return fail(HIPATTN_UNSUPPORTED, "softmax: too many rows for one launch");
        const bool wide = length % 8 == 0 && aligned(x, 16) && aligned(out, 16);
        if (wide && length <= 64 * 8)
            hipLaunchKernelGGL(softmax_kept_rows_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, stream, p);
        else if (wide && length <= 64 * 8 * 4)
            hipLaunchKernelGGL(softmax_kept_rows_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, stream, p);
        else if (wide)
            hipLaunchKernelGGL(softmax_rows_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, stream, p);
        else
            hipLaunchKernelGGL(softmax_rows_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, stream, p);
    } else {
        const int64_t blocks = (outer * inner + 255) / 256;
        if (blocks > 0x7fffffffLL) return fail(HIPATTN_UNSUPPORTED, "softmax: too many positions for one launch");
        hipLaunchKernelGGL(softmax_strided_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p);
    }
    return launched("softmax");
}

}  // namespace hipops
