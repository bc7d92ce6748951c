// The operators either side of attention in a decoder layer that move bytes or do a few flops per
// byte: RMS normalisation, rotary position embedding, Gather, Concat.  All are HBM-bound on
// MI355X: the kernels read every input byte once with 16-byte accesses where the layout allows,
// keep a row in registers between the two passes of a normalisation, and write every output byte
// once.  A scalar path covers shapes and alignments the vector path does not.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <string>

#include "device_common.hpp"
#include "hipops.h"
#include "ops/ops_common.hpp"
#include "ops/vec8.hpp"

namespace hipops {

using namespace hipattn;

// ------------------------------------------------------------------------------ RMS norm
struct RmsParams {
    const void* x;
    const void* gamma;
    void* out;
    int64_t rows, hidden;
    float eps;
    int x_dtype, gamma_dtype, out_dtype;
};

constexpr int kRmsKeep = 8;  // chunks of eight elements a lane keeps between the two passes

// kWavesPerRow wavefronts share a row; a workgroup of four wavefronts holds 4 / kWavesPerRow rows.
// Pass 1 sums the squares (the first kRmsKeep chunks of a lane stay in registers), pass 2 scales;
// a row of up to kWavesPerRow * 4096 elements is read from memory once.
template <int kWavesPerRow>
__global__ __launch_bounds__(256) void rms_norm_vec_kernel(RmsParams p) {
    constexpr int kLanes = kWavesPerRow * kWave;
    constexpr int kRowsPerGroup = 4 / kWavesPerRow;
    __shared__ float partial[4];
    const int slot = threadIdx.x / kLanes, t = threadIdx.x % kLanes;
    const int64_t row = (int64_t)blockIdx.x * kRowsPerGroup + slot;
    const bool live = row < p.rows;
    const int64_t chunks = p.hidden / 8;
    const int64_t base = row * p.hidden;
    Float8 keep[kRmsKeep];
    float sq = 0.f;
    if (live) {
#pragma unroll
        for (int c = 0; c < kRmsKeep; c++) {
            const int64_t ch = t + (int64_t)c * kLanes;
            if (ch < chunks) {
                keep[c] = load8(p.x, base + ch * 8, p.x_dtype);
#pragma unroll
                for (int i = 0; i < 8; i++) sq = fmaf(keep[c].v[i], keep[c].v[i], sq);
            }
        }
        for (int64_t ch = t + (int64_t)kRmsKeep * kLanes; ch < chunks; ch += kLanes) {
            const Float8 r = load8(p.x, base + ch * 8, p.x_dtype);
#pragma unroll
            for (int i = 0; i < 8; i++) sq = fmaf(r.v[i], r.v[i], sq);
        }
    }
    sq = wave_sum(sq);
    if constexpr (kWavesPerRow > 1) {
        if ((threadIdx.x & (kWave - 1)) == 0) partial[threadIdx.x / kWave] = sq;
        __syncthreads();
        sq = (partial[0] + partial[1]) + (partial[2] + partial[3]);
    }
    if (!live) return;
    const float inv = 1.0f / sqrtf(sq / (float)p.hidden + p.eps);
    auto finish = [&](const Float8& r, int64_t ch) {
        Float8 o;
        if (p.gamma != nullptr) {
            const Float8 g = load8(p.gamma, ch * 8, p.gamma_dtype);
#pragma unroll
            for (int i = 0; i < 8; i++) o.v[i] = (r.v[i] * inv) * g.v[i];
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) o.v[i] = r.v[i] * inv;
        }
        store8(p.out, base + ch * 8, p.out_dtype, o);
    };
#pragma unroll
    for (int c = 0; c < kRmsKeep; c++) {
        const int64_t ch = t + (int64_t)c * kLanes;
        if (ch < chunks) finish(keep[c], ch);
    }
    for (int64_t ch = t + (int64_t)kRmsKeep * kLanes; ch < chunks; ch += kLanes)
        finish(load8(p.x, base + ch * 8, p.x_dtype), ch);
}

// any hidden size and alignment: one wavefront per row, element by element
__global__ __launch_bounds__(256) void rms_norm_scalar_kernel(RmsParams p) {
    const int64_t row = (int64_t)blockIdx.x * 4 + threadIdx.x / kWave;
    const int lane = threadIdx.x % kWave;
    if (row >= p.rows) return;
    const int64_t base = row * p.hidden;
    float sq = 0.f;
    for (int64_t i = lane; i < p.hidden; i += kWave) {
        const float v = load_scalar(p.x, base + i, p.x_dtype);
        sq = fmaf(v, v, sq);
    }
    sq = wave_sum(sq);
    const float inv = 1.0f / sqrtf(sq / (float)p.hidden + p.eps);
    for (int64_t i = lane; i < p.hidden; i += kWave) {
        float v = load_scalar(p.x, base + i, p.x_dtype) * inv;
        if (p.gamma != nullptr) v *= load_scalar(p.gamma, i, p.gamma_dtype);
        store_scalar(p.out, base + i, p.out_dtype, v);
    }
}

// ------------------------------------------------------------------------------ RoPE
struct RopeParams {
    hipops_rope_desc d;
    const void* x;
    const void* cos;
    const void* sin;
    const int32_t* positions;
    void* out;
    int rotary, half;
    int items_per_head;  // vector kernel: work items of a head
    int rot_items;       // of which rotate (the rest copy)
};

constexpr int kRopeMaxTable = 512;  // floats per table row the vector kernel stages (rotary_ndims up to 512)

// One workgroup per token: its cos / sin rows go to LDS once, as floats, and every (head, piece)
// of the token reads them from there.  One lane takes both halves of a rotation (eight elements
// i.. and eight elements i + half.., or eight adjacent elements = four pairs), so out may alias x.
__global__ __launch_bounds__(256) void rope_vec_kernel(RopeParams p) {
    __shared__ float cs[2][kRopeMaxTable];
    const int64_t t = blockIdx.x;
    const int64_t pos = p.positions ? (int64_t)p.positions[t] : t;
    const int64_t tb = pos * p.d.table_row_stride;
    const int width = p.d.interleaved ? p.half : p.rotary;
    for (int i = threadIdx.x; i < 2 * width; i += blockDim.x) {
        const int which = i >= width, k = i - which * width;
        cs[which][k] = load_scalar(which ? p.sin : p.cos, tb + k, p.d.table_dtype);
    }
    __syncthreads();
    const int per_token = p.d.num_heads * p.items_per_head;
    for (int item = threadIdx.x; item < per_token; item += blockDim.x) {
        const int h = item / p.items_per_head;
        const int it = item - h * p.items_per_head;
        const int64_t xb = t * p.d.x_token_stride + (int64_t)h * p.d.x_head_stride;
        const int64_t ob = t * p.d.out_token_stride + (int64_t)h * p.d.out_head_stride;
        if (it >= p.rot_items) {  // pass-through tail of the head
            const int i = p.rotary + (it - p.rot_items) * 8;
            store8(p.out, ob + i, p.d.dtype, load8(p.x, xb + i, p.d.dtype));
            continue;
        }
        const int i = it * 8;
        if (p.d.interleaved) {  // elements i..i+7 = pairs i/2..i/2+3
            const Float8 v = load8(p.x, xb + i, p.d.dtype);
            Float8 o;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const float c = cs[0][i / 2 + k], s = cs[1][i / 2 + k];
                o.v[2 * k] = v.v[2 * k] * c - v.v[2 * k + 1] * s;
                o.v[2 * k + 1] = v.v[2 * k + 1] * c + v.v[2 * k] * s;
            }
            store8(p.out, ob + i, p.d.dtype, o);
        } else {
            const Float8 lo = load8(p.x, xb + i, p.d.dtype), hi = load8(p.x, xb + i + p.half, p.d.dtype);
            Float8 ol, oh;
#pragma unroll
            for (int k = 0; k < 8; k++) {
                ol.v[k] = lo.v[k] * cs[0][i + k] - hi.v[k] * cs[1][i + k];
                oh.v[k] = hi.v[k] * cs[0][i + p.half + k] + lo.v[k] * cs[1][i + p.half + k];
            }
            store8(p.out, ob + i, p.d.dtype, ol);
            store8(p.out, ob + i + p.half, p.d.dtype, oh);
        }
    }
}

// one lane per rotation pair (or pass-through element); any size and alignment
__global__ __launch_bounds__(256) void rope_scalar_kernel(RopeParams p) {
    const int per_head = p.half + (p.d.head_size - p.rotary);
    const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t th = item / per_head;
    const int it = (int)(item - th * per_head);
    if (th >= p.d.num_tokens * p.d.num_heads) return;
    const int64_t t = th / p.d.num_heads;
    const int h = (int)(th - t * p.d.num_heads);
    const int64_t xb = t * p.d.x_token_stride + (int64_t)h * p.d.x_head_stride;
    const int64_t ob = t * p.d.out_token_stride + (int64_t)h * p.d.out_head_stride;
    if (it >= p.half) {
        const int i = p.rotary + (it - p.half);
        store_scalar(p.out, ob + i, p.d.dtype, load_scalar(p.x, xb + i, p.d.dtype));
        return;
    }
    const int64_t pos = p.positions ? (int64_t)p.positions[t] : t;
    const int64_t tb = pos * p.d.table_row_stride;
    if (p.d.interleaved) {
        const float a = load_scalar(p.x, xb + 2 * it, p.d.dtype), b = load_scalar(p.x, xb + 2 * it + 1, p.d.dtype);
        const float c = load_scalar(p.cos, tb + it, p.d.table_dtype), s = load_scalar(p.sin, tb + it, p.d.table_dtype);
        store_scalar(p.out, ob + 2 * it, p.d.dtype, a * c - b * s);
        store_scalar(p.out, ob + 2 * it + 1, p.d.dtype, b * c + a * s);
    } else {
        const float a = load_scalar(p.x, xb + it, p.d.dtype), b = load_scalar(p.x, xb + it + p.half, p.d.dtype);
        const float cl = load_scalar(p.cos, tb + it, p.d.table_dtype), sl = load_scalar(p.sin, tb + it, p.d.table_dtype);
        const float ch = load_scalar(p.cos, tb + it + p.half, p.d.table_dtype);
        const float sh = load_scalar(p.sin, tb + it + p.half, p.d.table_dtype);
        store_scalar(p.out, ob + it, p.d.dtype, a * cl - b * sl);
        store_scalar(p.out, ob + it + p.half, p.d.dtype, b * ch + a * sh);
    }
}

// ------------------------------------------------------------------------------ Swish, Multiply, GLU
__device__ __forceinline__ float activate(float x, int activation, float beta) {
    switch (activation) {
        case HIPOPS_GLU_GELU: return 0.5f * x * (1.0f + erff(x * 0.70710678118654752f));
        case HIPOPS_GLU_GELU_TANH: return 0.5f * x * (1.0f + tanhf(0.79788456080286536f * (x + 0.044715f * x * x * x)));
        default: return x / (1.0f + __expf(-beta * x));
    }
}

struct EltwiseParams {
    const void* a;  // x (swish), a (multiply), the gate half's row 0 (glu)
    const void* b;  // multiply: b; glu: the other half's row 0
    void* out;
    int64_t count;      // elements of out
    int64_t width;      // glu: elements per output row (input rows are twice as long)
    int op;             // 0 swish, 1 multiply, 2 glu
    int activation;
    float beta;
    int dtype;
};

// eight output elements per lane
__global__ __launch_bounds__(256) void eltwise_vec_kernel(EltwiseParams p) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (i >= p.count) return;
    int64_t ia = i;
    if (p.op == 2) {  // row r of the output lies in row r of a 2 * width wide input
        const int64_t r = i / p.width;
        ia = r * 2 * p.width + (i - r * p.width);
    }
    const Float8 x = load8(p.a, ia, p.dtype);
    Float8 o;
    if (p.op == 0) {
#pragma unroll
        for (int k = 0; k < 8; k++) o.v[k] = activate(x.v[k], HIPOPS_GLU_SWISH, p.beta);
    } else {
        const Float8 y = load8(p.b, ia, p.dtype);
#pragma unroll
        for (int k = 0; k < 8; k++) o.v[k] = (p.op == 1 ? x.v[k] : activate(x.v[k], p.activation, 1.0f)) * y.v[k];
    }
    store8(p.out, i, p.dtype, o);
}

__global__ __launch_bounds__(256) void eltwise_scalar_kernel(EltwiseParams p) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= p.count) return;
    int64_t ia = i;
    if (p.op == 2) {
        const int64_t r = i / p.width;
        ia = r * 2 * p.width + (i - r * p.width);
    }
    const float x = load_scalar(p.a, ia, p.dtype);
    float o;
    if (p.op == 0)
        o = activate(x, HIPOPS_GLU_SWISH, p.beta);
    else
        o = (p.op == 1 ? x : activate(x, p.activation, 1.0f)) * load_scalar(p.b, ia, p.dtype);
    store_scalar(p.out, i, p.dtype, o);
}

// ------------------------------------------------------------------------------ Gather / Concat
template <typename V>
__device__ __forceinline__ V zero_of() {
    V z;
    __builtin_memset(&z, 0, sizeof(V));
    return z;
}

struct GatherParams {
    const uint8_t* data;
    const void* indices;
    uint8_t* out;
    int64_t batch, outer, axis_dim, inner_chunks, num_indices;  // inner in units of sizeof(V)
    int index_i64;
};

// one lane per sizeof(V)-byte piece of the output
template <typename V>
__global__ __launch_bounds__(256) void gather_kernel(GatherParams p) {
    const int64_t piece = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t out_row = piece / p.inner_chunks;  // (batch, outer, index)
    const int64_t c = piece - out_row * p.inner_chunks;
    if (out_row >= p.batch * p.outer * p.num_indices) return;
    const int64_t bo = out_row / p.num_indices;      // (batch, outer)
    const int64_t k = out_row - bo * p.num_indices;
    const int64_t b = bo / p.outer;
    int64_t idx = p.index_i64 ? ((const int64_t*)p.indices)[b * p.num_indices + k]
                              : (int64_t)((const int32_t*)p.indices)[b * p.num_indices + k];
    if (idx < 0) idx += p.axis_dim;
    V v = zero_of<V>();
    if (idx >= 0 && idx < p.axis_dim) v = ((const V*)p.data)[(bo * p.axis_dim + idx) * p.inner_chunks + c];
    ((V*)p.out)[piece] = v;
}

constexpr int kConcatInputsPerLaunch = 8;
struct ConcatParams {
    const uint8_t* src[kConcatInputsPerLaunch];
    int64_t width[kConcatInputsPerLaunch];   // pieces of sizeof(V) per row of this input
    int64_t offset[kConcatInputsPerLaunch];  // pieces from the start of an output row
    int64_t outer, out_width;
    uint8_t* out;
};

// blockIdx.y picks the input, one lane per sizeof(V)-byte piece of it
template <typename V>
__global__ __launch_bounds__(256) void concat_kernel(ConcatParams p) {
    const int in = blockIdx.y;
    const int64_t w = p.width[in];
    const int64_t piece = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (w == 0 || piece >= p.outer * w) return;
    const int64_t row = piece / w, c = piece - row * w;
    ((V*)p.out)[row * p.out_width + p.offset[in] + c] = ((const V*)p.src[in])[piece];
}

// ------------------------------------------------------------------------------ host side
static bool aligned(const void* ptr, size_t a) { return ((uintptr_t)ptr % a) == 0; }
static bool float_dtype(int d) { return d == HIPATTN_F32 || d == HIPATTN_F16 || d == HIPATTN_BF16; }

static hipattn_status launched(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HIPATTN_HIP_ERROR, "%s: %s", what, hipGetErrorString(e));
    return HIPATTN_OK;
}

static int64_t blocks_for(int64_t items) { return (items + 255) / 256; }

hipattn_status rms_norm(const void* x, const void* gamma, void* out, int64_t rows, int64_t hidden, float eps, int x_dtype,
                        int gamma_dtype, int out_dtype, hipStream_t stream) {
    if (rows < 0 || hidden <= 0) return fail(HIPATTN_INVALID_ARGUMENT, "rms_norm: rows %lld hidden %lld", (long long)rows, (long long)hidden);
    if (!float_dtype(x_dtype) || !float_dtype(out_dtype) || (gamma && !float_dtype(gamma_dtype)))
        return fail(HIPATTN_UNSUPPORTED, "rms_norm: dtypes must be f32, f16 or bf16");
    if (!(eps >= 0.f)) return fail(HIPATTN_INVALID_ARGUMENT, "rms_norm: eps must be >= 0");
    if (rows == 0) return HIPATTN_OK;
    if (!x || !out) return fail(HIPATTN_INVALID_ARGUMENT, "rms_norm: null pointer");
    if (rows > 0x7fffffffLL) return fail(HIPATTN_UNSUPPORTED, "rms_norm: too many rows");
    RmsParams p{x, gamma, out, rows, hidden, eps, x_dtype, gamma_dtype, out_dtype};
    const bool vec = hidden % 8 == 0 && aligned(x, 16) && aligned(out, 16) && (!gamma || aligned(gamma, 16));
    if (!vec) {
        hipLaunchKernelGGL(rms_norm_scalar_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, p);
    } else if (rows >= 2048 && hidden <= 1024) {
        // enough rows to fill the device with one wavefront each
        hipLaunchKernelGGL(rms_norm_vec_kernel<1>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, p);
    } else {
        hipLaunchKernelGGL(rms_norm_vec_kernel<4>, dim3((unsigned)rows), dim3(256), 0, stream, p);
    }
    return launched("rms_norm");
}

hipattn_status rope(const hipops_rope_desc* d, const void* x, const void* cos, const void* sin, const int32_t* positions,
                    void* out, hipStream_t stream) {
    if (!d) return fail(HIPATTN_INVALID_ARGUMENT, "rope: null descriptor");
    if (d->num_tokens < 0 || d->num_heads <= 0 || d->head_size <= 0)
        return fail(HIPATTN_INVALID_ARGUMENT, "rope: tokens %lld heads %d head_size %d", (long long)d->num_tokens, d->num_heads, d->head_size);
    const int rotary = d->rotary_ndims == 0 ? d->head_size : d->rotary_ndims;
    if (rotary < 0 || rotary > d->head_size || rotary % 2)
        return fail(HIPATTN_INVALID_ARGUMENT, "rope: rotary_ndims %d must be even and at most head_size %d", rotary, d->head_size);
    if (!float_dtype(d->dtype) || !float_dtype(d->table_dtype)) return fail(HIPATTN_UNSUPPORTED, "rope: dtypes must be f32, f16 or bf16");
    const int table_width = d->interleaved ? rotary / 2 : rotary;
    if (d->table_rows <= 0 || d->table_row_stride < table_width)
        return fail(HIPATTN_INVALID_ARGUMENT, "rope: table of %lld rows, row stride %lld, needs rows of %d", (long long)d->table_rows,
                    (long long)d->table_row_stride, table_width);
    if (!positions && d->num_tokens > d->table_rows)
        return fail(HIPATTN_INVALID_ARGUMENT, "rope: %lld tokens but %lld table rows and no positions", (long long)d->num_tokens,
                    (long long)d->table_rows);
    if (d->x_head_stride < d->head_size || d->out_head_stride < d->head_size || d->x_token_stride < 0 || d->out_token_stride < 0)
        return fail(HIPATTN_INVALID_ARGUMENT, "rope: strides smaller than a head");
    if (d->num_tokens == 0) return HIPATTN_OK;
    if (!x || !cos || !sin || !out) return fail(HIPATTN_INVALID_ARGUMENT, "rope: null pointer");
    RopeParams p{};
    p.d = *d;
    p.x = x, p.cos = cos, p.sin = sin, p.positions = positions, p.out = out;
    p.rotary = rotary, p.half = rotary / 2;
    const bool vec = d->head_size % 8 == 0 && rotary % 8 == 0 && (d->interleaved || p.half % 8 == 0) && rotary <= kRopeMaxTable &&
                     d->x_token_stride % 8 == 0 && d->x_head_stride % 8 == 0 && d->out_token_stride % 8 == 0 &&
                     d->out_head_stride % 8 == 0 && aligned(x, 16) && aligned(out, 16);
    if (vec) {
        if (d->num_tokens > 0x7fffffffLL) return fail(HIPATTN_UNSUPPORTED, "rope: too many tokens for one launch");
        p.rot_items = d->interleaved ? rotary / 8 : p.half / 8;
        p.items_per_head = p.rot_items + (d->head_size - rotary) / 8;
        const int per_token = d->num_heads * p.items_per_head;
        const int threads = std::min(256, (per_token + kWave - 1) / kWave * kWave);
        hipLaunchKernelGGL(rope_vec_kernel, dim3((unsigned)d->num_tokens), dim3(threads), 0, stream, p);
    } else {
        const int64_t items = d->num_tokens * d->num_heads * (int64_t)(p.half + (d->head_size - rotary));
        if (blocks_for(items) > 0x7fffffffLL) return fail(HIPATTN_UNSUPPORTED, "rope: too many elements for one launch");
        hipLaunchKernelGGL(rope_scalar_kernel, dim3((unsigned)blocks_for(items)), dim3(256), 0, stream, p);
    }
    return launched("rope");
}

hipattn_status swish(const void* x, void* out, int64_t count, float beta, int dtype, hipStream_t stream) {
    if (count < 0) return fail(HIPATTN_INVALID_ARGUMENT, "swish: negative count");
    if (!float_dtype(dtype)) return fail(HIPATTN_UNSUPPORTED, "swish: dtype must be f32, f16 or bf16");
    if (count == 0) return HIPATTN_OK;
    if (!x || !out) return fail(HIPATTN_INVALID_ARGUMENT, "swish: null pointer");
    EltwiseParams p{x, nullptr, out, count, 0, 0, HIPOPS_GLU_SWISH, beta, dtype};
    const bool vec = count % 8 == 0 && aligned(x, 16) && aligned(out, 16);
    const int64_t items = vec ? count / 8 : count;
    if (blocks_for(items) > 0x7fffffffLL) return fail(HIPATTN_UNSUPPORTED, "swish: too many elements for one launch");
    if (vec)
        hipLaunchKernelGGL(eltwise_vec_kernel, dim3((unsigned)blocks_for(items)), dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(eltwise_scalar_kernel, dim3((unsigned)blocks_for(items)), dim3(256), 0, stream, p);
    return launched("swish");
}

hipattn_status multiply(const void* a, const void* b, void* out, int64_t count, int dtype, hipStream_t stream) {
    if (count < 0) return fail(HIPATTN_INVALID_ARGUMENT, "multiply: negative count");
    if (!float_dtype(dtype)) return fail(HIPATTN_UNSUPPORTED, "multiply: dtype must be f32, f16 or bf16");
    if (count == 0) return HIPATTN_OK;
    if (!a || !b || !out) return fail(HIPATTN_INVALID_ARGUMENT, "multiply: null pointer");
    EltwiseParams p{a, b, out, count, 0, 1, 0, 1.0f, dtype};
    const bool vec = count % 8 == 0 && aligned(a, 16) && aligned(b, 16) && aligned(out, 16);
    const int64_t items = vec ? count / 8 : count;
    if (blocks_for(items) > 0x7fffffffLL) return fail(HIPATTN_UNSUPPORTED, "multiply: too many elements for one launch");
    if (vec)
        hipLaunchKernelGGL(eltwise_vec_kernel, dim3((unsigned)blocks_for(items)), dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(eltwise_scalar_kernel, dim3((unsigned)blocks_for(items)), dim3(256), 0, stream, p);
    return launched("multiply");
}

hipattn_status glu(const void* x, void* out, int64_t rows, int64_t width, int activation, int gate_first, int dtype,
                   hipStream_t stream) {
    if (rows < 0 || width <= 0) return fail(HIPATTN_INVALID_ARGUMENT, "glu: rows %lld width %lld", (long long)rows, (long long)width);
    if (!float_dtype(dtype)) return fail(HIPATTN_UNSUPPORTED, "glu: dtype must be f32, f16 or bf16");
    if (activation < HIPOPS_GLU_SWISH || activation > HIPOPS_GLU_GELU_TANH) return fail(HIPATTN_INVALID_ARGUMENT, "glu: activation %d", activation);
    if (rows == 0) return HIPATTN_OK;
    if (!x || !out) return fail(HIPATTN_INVALID_ARGUMENT, "glu: null pointer");
    const int esz = dtype == HIPATTN_F32 ? 4 : 2;
    const char* gate = (const char*)x + (gate_first ? 0 : width * esz);
    const char* up = (const char*)x + (gate_first ? width * esz : 0);
    EltwiseParams p{gate, up, out, rows * width, width, 2, activation, 1.0f, dtype};
    const bool vec = width % 8 == 0 && aligned(x, 16) && aligned(out, 16);
    const int64_t items = vec ? p.count / 8 : p.count;
    if (blocks_for(items) > 0x7fffffffLL) return fail(HIPATTN_UNSUPPORTED, "glu: too many elements for one launch");
    if (vec)
        hipLaunchKernelGGL(eltwise_vec_kernel, dim3((unsigned)blocks_for(items)), dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(eltwise_scalar_kernel, dim3((unsigned)blocks_for(items)), dim3(256), 0, stream, p);
    return launched("glu");
}

// widest power-of-two piece (<= 16 bytes) that divides every size and address given
static int common_piece(std::initializer_list<int64_t> sizes, std::initializer_list<const void*> ptrs) {
    int piece = 16;
    for (int64_t s : sizes)
        while (piece > 1 && s % piece) piece >>= 1;
    for (const void* q : ptrs)
        while (piece > 1 && !aligned(q, piece)) piece >>= 1;
    return piece;
}

template <template <typename> class Launch, typename... Args>
static void by_piece(int piece, Args&&... args) {
    switch (piece) {
        case 16: Launch<uint4_t>::run(args...); break;
        case 8: Launch<uint2_t>::run(args...); break;
        case 4: Launch<uint32_t>::run(args...); break;
        case 2: Launch<uint16_t>::run(args...); break;
        default: Launch<uint8_t>::run(args...); break;
    }
}

template <typename V>
struct LaunchGather {
    static void run(const GatherParams& p, int64_t pieces, hipStream_t stream) {
        hipLaunchKernelGGL(gather_kernel<V>, dim3((unsigned)blocks_for(pieces)), dim3(256), 0, stream, p);
    }
};
template <typename V>
struct LaunchConcat {
    static void run(const ConcatParams& p, int64_t pieces, int inputs, hipStream_t stream) {
        hipLaunchKernelGGL(concat_kernel<V>, dim3((unsigned)blocks_for(pieces), (unsigned)inputs), dim3(256), 0, stream, p);
    }
};

hipattn_status gather(const void* data, const void* indices, void* out, int64_t batch, int64_t outer, int64_t axis_dim,
                      int64_t inner_bytes, int64_t num_indices, int index_dtype, hipStream_t stream) {
    if (batch < 0 || outer < 0 || axis_dim < 0 || inner_bytes < 0 || num_indices < 0)
        return fail(HIPATTN_INVALID_ARGUMENT, "gather: negative extent");
    if (index_dtype != HIPATTN_I32 && index_dtype != HIPOPS_I64) return fail(HIPATTN_UNSUPPORTED, "gather: indices must be i32 or i64");
    // the reference returns without a launch for an empty output (gather.cpp:96-101)
    if (batch * outer * num_indices * inner_bytes == 0) return HIPATTN_OK;
    if (!indices || !out || (!data && axis_dim > 0)) return fail(HIPATTN_INVALID_ARGUMENT, "gather: null pointer");
    const int piece = common_piece({inner_bytes}, {data, out});
    GatherParams p{(const uint8_t*)data, indices, (uint8_t*)out, batch, outer, axis_dim, inner_bytes / piece, num_indices,
                   index_dtype == HIPOPS_I64};
    const int64_t pieces = batch * outer * num_indices * p.inner_chunks;
    if (blocks_for(pieces) > 0x7fffffffLL) return fail(HIPATTN_UNSUPPORTED, "gather: output too large for one launch");
    by_piece<LaunchGather>(piece, p, pieces, stream);
    return launched("gather");
}

hipattn_status concat(const void* const* inputs, const int64_t* axis_bytes, int num_inputs, int64_t outer, void* out,
                      hipStream_t stream) {
    if (num_inputs <= 0 || !inputs || !axis_bytes || outer < 0) return fail(HIPATTN_INVALID_ARGUMENT, "concat: bad argument");
    int64_t total = 0;
    for (int i = 0; i < num_inputs; i++) {
        if (axis_bytes[i] < 0) return fail(HIPATTN_INVALID_ARGUMENT, "concat: negative extent of input %d", i);
        if (axis_bytes[i] > 0 && outer > 0 && !inputs[i]) return fail(HIPATTN_INVALID_ARGUMENT, "concat: input %d is null", i);
        total += axis_bytes[i];
    }
    if (total == 0 || outer == 0) return HIPATTN_OK;
    if (!out) return fail(HIPATTN_INVALID_ARGUMENT, "concat: null output");
    int piece = common_piece({total}, {out});
    for (int i = 0; i < num_inputs; i++)
        if (axis_bytes[i] > 0) piece = std::min(piece, common_piece({axis_bytes[i]}, {inputs[i]}));
    int64_t offset = 0;
    for (int first = 0; first < num_inputs; first += kConcatInputsPerLaunch) {
        const int n = std::min(kConcatInputsPerLaunch, num_inputs - first);
        ConcatParams p{};
        int64_t widest = 0;
        for (int i = 0; i < n; i++) {
            p.src[i] = (const uint8_t*)inputs[first + i];
            p.width[i] = axis_bytes[first + i] / piece;
            p.offset[i] = offset / piece;
            offset += axis_bytes[first + i];
            widest = std::max(widest, p.width[i]);
        }
        if (widest == 0) continue;
        p.outer = outer, p.out_width = total / piece, p.out = (uint8_t*)out;
        if (blocks_for(outer * widest) > 0x7fffffffLL) return fail(HIPATTN_UNSUPPORTED, "concat: input too large for one launch");
        by_piece<LaunchConcat>(piece, p, outer * widest, n, stream);
        const hipattn_status st = launched("concat");
        if (st != HIPATTN_OK) return st;
    }
    return HIPATTN_OK;
}

}  // namespace hipops
