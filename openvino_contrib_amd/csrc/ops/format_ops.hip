// Transpose and Convert: the operators that change a tensor's layout or element type between the
// others of a decoder layer.  Both are HBM-bound byte movers.
//
// Transpose.  The host reduces the permutation first: axes of extent 1 go, output axes that are
// neighbours in the input in the same order become one.  What is left falls into one of two forms:
//   rows   the innermost axis stays innermost ([b, l, h, d] <-> [b, h, l, d]): contiguous runs move
//          whole, a lane per piece of up to 16 bytes, the source address built from the coordinates
//          of the piece's row;
//   tiles  the innermost axis changes: 64 x 64 elements go through LDS, read along the input's
//          innermost axis and written along the output's, 16 bytes a lane on both sides where the
//          strides allow; the other axes are spread over blockIdx.z.
//
// Convert.  Eight elements per lane through 16-byte loads and stores where the addresses allow.
#include <algorithm>

#include "ops/ops_common.hpp"

namespace hipops {

namespace {

typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

constexpr int kMaxAxes = HIPOPS_TRANSPOSE_MAX_RANK;

bool aligned(const void* ptr, size_t a) { return ((uintptr_t)ptr % a) == 0; }

hipattn_status launched(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HIPATTN_HIP_ERROR, "%s: %s", what, hipGetErrorString(e));
    return HIPATTN_OK;
}

// ------------------------------------------------------------------------------ Transpose
struct RowsParams {
    const uint8_t* in;
    uint8_t* out;
    int axes;                     // output axes outside the run, outermost first
    uint32_t extent[kMaxAxes];    // their extents
    int64_t in_stride[kMaxAxes];  // and what a step along each is worth in the input, in pieces
    uint32_t run;                 // pieces per contiguous run
    int64_t pieces;               // in all
};

// one lane per piece of the output
template <typename V, typename Index>
__global__ __launch_bounds__(256) void transpose_rows_kernel(RowsParams p) {
    const Index piece = (Index)blockIdx.x * 256 + threadIdx.x;
    if (piece >= (Index)p.pieces) return;
    Index row = piece / p.run;
    int64_t src = (int64_t)(piece - row * p.run);
#pragma unroll 1
    for (int a = p.axes - 1; a > 0; a--) {
        const Index next = row / p.extent[a];
        src += (int64_t)(row - next * p.extent[a]) * p.in_stride[a];
        row = next;
    }
    if (p.axes > 0) src += (int64_t)row * p.in_stride[0];
    ((V*)p.out)[piece] = ((const V*)p.in)[src];
}

struct TilesParams {
    const uint8_t* in;
    uint8_t* out;
    uint32_t extent_a, extent_b;  // a: innermost in the input, b: innermost in the output
    int64_t in_stride_b;          // a step along b in the input, in elements (a's is 1)
    int64_t out_stride_a;         // a step along a in the output, in elements (b's is 1)
    int axes;                     // the other axes, outermost first
    uint32_t extent[kMaxAxes];
    int64_t in_stride[kMaxAxes], out_stride[kMaxAxes];
    uint32_t batches;             // product of their extents
    int wide_in, wide_out;        // every row start on that side is aligned for the kernel's widest access
};

// A lane moves kWide elements at a time on either side (16 bytes; 8 bytes of single-byte elements)
// where the addresses allow it: p.wide_in / p.wide_out say so for the whole launch.
template <typename E>
__global__ __launch_bounds__(256) void transpose_tiles_kernel(TilesParams p) {
    constexpr int kWide = sizeof(E) >= 2 ? 16 / sizeof(E) : 8;
    constexpr int kLanesPerRow = 64 / kWide, kRowsPerPass = 256 / kLanesPerRow;
    struct alignas(sizeof(E) * kWide) Wide {
        E v[kWide];
    };
    __shared__ alignas(16) E tile[64][64 + kWide];  // rows: b, columns: a
    const uint32_t a0 = blockIdx.x * 64, b0 = blockIdx.y * 64;
    const uint32_t column = (threadIdx.x % kLanesPerRow) * kWide, first_row = threadIdx.x / kLanesPerRow;
    for (uint32_t batch = blockIdx.z; batch < p.batches; batch += gridDim.z) {
        int64_t src = 0, dst = 0;
        uint32_t rest = batch;
#pragma unroll 1
        for (int k = p.axes - 1; k >= 0; k--) {
            const uint32_t next = rest / p.extent[k], c = rest - next * p.extent[k];
            src += (int64_t)c * p.in_stride[k];
            dst += (int64_t)c * p.out_stride[k];
            rest = next;
        }
        const E* in = (const E*)p.in + src;
        E* out = (E*)p.out + dst;
#pragma unroll
        for (uint32_t row = first_row; row < 64; row += kRowsPerPass) {
            const uint32_t a = a0 + column, b = b0 + row;
            if (b >= p.extent_b || a >= p.extent_a) continue;
            const E* from = in + (int64_t)b * p.in_stride_b + a;
            if (p.wide_in && a + kWide <= p.extent_a) {
                *(Wide*)&tile[row][column] = *(const Wide*)from;
            } else {
                for (uint32_t i = 0; i < kWide && a + i < p.extent_a; i++) tile[row][column + i] = from[i];
            }
        }
        __syncthreads();
#pragma unroll
        for (uint32_t row = first_row; row < 64; row += kRowsPerPass) {
            const uint32_t a = a0 + row, b = b0 + column;
            if (a >= p.extent_a || b >= p.extent_b) continue;
            E* to = out + (int64_t)a * p.out_stride_a + b;
            if (p.wide_out && b + kWide <= p.extent_b) {
                Wide w;
#pragma unroll
                for (int i = 0; i < kWide; i++) w.v[i] = tile[column + i][row];
                *(Wide*)to = w;
            } else {
                for (uint32_t i = 0; i < kWide && b + i < p.extent_b; i++) to[i] = tile[column + i][row];
            }
        }
        __syncthreads();
    }
}

template <typename V>
void launch_rows(const RowsParams& p, hipStream_t stream) {
    const unsigned blocks = (unsigned)((p.pieces + 255) / 256);
    if (p.pieces < 0x7fffffffLL)
        hipLaunchKernelGGL((transpose_rows_kernel<V, uint32_t>), dim3(blocks), dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL((transpose_rows_kernel<V, int64_t>), dim3(blocks), dim3(256), 0, stream, p);
}

// ------------------------------------------------------------------------------ Convert
// Values travel as float (floating types) or int64_t (integer types and boolean).
template <int kType>
struct Element;
template <>
struct Element<HIPATTN_F32> {
    using Storage = float;
    using Value = float;
    static __device__ __forceinline__ Value load(Storage s) { return s; }
};
template <>
struct Element<HIPATTN_F16> {
    using Storage = _Float16;
    using Value = float;
    static __device__ __forceinline__ Value load(Storage s) { return (float)s; }
};
template <>
struct Element<HIPATTN_BF16> {
    using Storage = uint16_t;
    using Value = float;
    static __device__ __forceinline__ Value load(Storage s) { return __uint_as_float((uint32_t)s << 16); }
};
template <>
struct Element<HIPATTN_I32> {
    using Storage = int32_t;
    using Value = int64_t;
    static __device__ __forceinline__ Value load(Storage s) { return s; }
};
template <>
struct Element<HIPOPS_I64> {
    using Storage = int64_t;
    using Value = int64_t;
    static __device__ __forceinline__ Value load(Storage s) { return s; }
};
template <>
struct Element<HIPOPS_U8> {
    using Storage = uint8_t;
    using Value = int64_t;
    static __device__ __forceinline__ Value load(Storage s) { return s; }
};
template <>
struct Element<HIPOPS_I8> {
    using Storage = int8_t;
    using Value = int64_t;
    static __device__ __forceinline__ Value load(Storage s) { return s; }
};
template <>
struct Element<HIPOPS_BOOL> {
    using Storage = uint8_t;
    using Value = int64_t;
    static __device__ __forceinline__ Value load(Storage s) { return s != 0; }
};

__device__ __forceinline__ uint16_t bf16_bits(float f) {  // round to nearest even, NaN stays NaN
    const uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

// float to integer: towards zero, saturating at the target's range, NaN gives 0
template <typename I>
__device__ __forceinline__ I float_to_int(float f, float lowest, float beyond, I min_value, I max_value) {
    if (f != f) return 0;
    if (f <= lowest) return min_value;
    if (f >= beyond) return max_value;
    return (I)f;
}

template <int kType>
struct Store;
template <>
struct Store<HIPATTN_F32> {
    static __device__ __forceinline__ float from(float v) { return v; }
    static __device__ __forceinline__ float from(int64_t v) { return (float)v; }
};
template <>
struct Store<HIPATTN_F16> {
    static __device__ __forceinline__ _Float16 from(float v) { return (_Float16)v; }
    static __device__ __forceinline__ _Float16 from(int64_t v) { return (_Float16)(float)v; }
};
template <>
struct Store<HIPATTN_BF16> {
    static __device__ __forceinline__ uint16_t from(float v) { return bf16_bits(v); }
    static __device__ __forceinline__ uint16_t from(int64_t v) { return bf16_bits((float)v); }
};
template <>
struct Store<HIPATTN_I32> {
    static __device__ __forceinline__ int32_t from(float v) { return float_to_int<int32_t>(v, -2147483648.f, 2147483648.f, INT32_MIN, INT32_MAX); }
    static __device__ __forceinline__ int32_t from(int64_t v) { return (int32_t)v; }
};
template <>
struct Store<HIPOPS_I64> {
    static __device__ __forceinline__ int64_t from(float v) {
        return float_to_int<int64_t>(v, -9223372036854775808.f, 9223372036854775808.f, INT64_MIN, INT64_MAX);
    }
    static __device__ __forceinline__ int64_t from(int64_t v) { return v; }
};
template <>
struct Store<HIPOPS_U8> {
    static __device__ __forceinline__ uint8_t from(float v) { return float_to_int<uint8_t>(v, 0.f, 255.f, 0, 255); }
    static __device__ __forceinline__ uint8_t from(int64_t v) { return (uint8_t)v; }
};
template <>
struct Store<HIPOPS_I8> {
    static __device__ __forceinline__ int8_t from(float v) { return float_to_int<int8_t>(v, -128.f, 127.f, -128, 127); }
    static __device__ __forceinline__ int8_t from(int64_t v) { return (int8_t)v; }
};
template <>
struct Store<HIPOPS_BOOL> {
    static __device__ __forceinline__ uint8_t from(float v) { return v != 0.f; }  // NaN is true, as in C
    static __device__ __forceinline__ uint8_t from(int64_t v) { return v != 0; }
};

template <typename T>
struct alignas(sizeof(T) * 8 > 16 ? 16 : sizeof(T) * 8) Pack8 {
    T v[8];
};

// `first` .. `first + count`; kPacked: eight elements a lane, count a multiple of 8
template <int kFrom, int kTo, bool kPacked>
__global__ __launch_bounds__(256) void convert_kernel(const void* in, void* out, int64_t first, int64_t count) {
    using From = typename Element<kFrom>::Storage;
    using To = decltype(Store<kTo>::from(typename Element<kFrom>::Value{}));
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if constexpr (kPacked) {
        if (i * 8 >= count) return;
        const Pack8<From> src = ((const Pack8<From>*)((const From*)in + first))[i];
        Pack8<To> dst;
#pragma unroll
        for (int k = 0; k < 8; k++) dst.v[k] = Store<kTo>::from(Element<kFrom>::load(src.v[k]));
        ((Pack8<To>*)((To*)out + first))[i] = dst;
    } else {
        if (i >= count) return;
        ((To*)out)[first + i] = Store<kTo>::from(Element<kFrom>::load(((const From*)in)[first + i]));
    }
}

size_t type_size(int dtype) {
    switch (dtype) {
        case HIPATTN_F32:
        case HIPATTN_I32: return 4;
        case HIPATTN_F16:
        case HIPATTN_BF16: return 2;
        case HIPOPS_I64: return 8;
        case HIPOPS_U8:
        case HIPOPS_I8:
        case HIPOPS_BOOL: return 1;
        default: return 0;
    }
}

template <int kFrom, int kTo>
void launch_convert(const void* in, void* out, int64_t count, hipStream_t stream) {
    const size_t a_in = std::min<size_t>(16, type_size(kFrom) * 8), a_out = std::min<size_t>(16, type_size(kTo) * 8);
    const int64_t packed = aligned(in, a_in) && aligned(out, a_out) ? count / 8 * 8 : 0;
    if (packed) hipLaunchKernelGGL((convert_kernel<kFrom, kTo, true>), dim3((unsigned)((packed / 8 + 255) / 256)), dim3(256), 0, stream, in, out, (int64_t)0, packed);
    if (count > packed)
        hipLaunchKernelGGL((convert_kernel<kFrom, kTo, false>), dim3((unsigned)((count - packed + 255) / 256)), dim3(256), 0, stream, in, out, packed, count - packed);
}

template <int kFrom>
bool convert_from(int to, const void* in, void* out, int64_t count, hipStream_t stream) {
    switch (to) {
        case HIPATTN_F32: launch_convert<kFrom, HIPATTN_F32>(in, out, count, stream); return true;
        case HIPATTN_F16: launch_convert<kFrom, HIPATTN_F16>(in, out, count, stream); return true;
        case HIPATTN_BF16: launch_convert<kFrom, HIPATTN_BF16>(in, out, count, stream); return true;
        case HIPATTN_I32: launch_convert<kFrom, HIPATTN_I32>(in, out, count, stream); return true;
        case HIPOPS_I64: launch_convert<kFrom, HIPOPS_I64>(in, out, count, stream); return true;
        case HIPOPS_U8: launch_convert<kFrom, HIPOPS_U8>(in, out, count, stream); return true;
        case HIPOPS_I8: launch_convert<kFrom, HIPOPS_I8>(in, out, count, stream); return true;
        case HIPOPS_BOOL: launch_convert<kFrom, HIPOPS_BOOL>(in, out, count, stream); return true;
        default: return false;
    }
}

}  // namespace

hipattn_status transpose(const void* in, void* out, int rank, const int64_t* dims, const int32_t* order, int element_bytes,
                         hipStream_t stream) {
    if (rank < 0 || rank > kMaxAxes || (rank > 0 && (!dims || !order)))
        return fail(HIPATTN_INVALID_ARGUMENT, "transpose: rank %d (0 to %d expected, with extents and order)", rank, kMaxAxes);
    if (element_bytes != 1 && element_bytes != 2 && element_bytes != 4 && element_bytes != 8)
        return fail(HIPATTN_UNSUPPORTED, "transpose: elements of %d bytes", element_bytes);
    bool seen[kMaxAxes] = {};
    int64_t count = 1;
    for (int k = 0; k < rank; k++) {
        if (order[k] < 0 || order[k] >= rank || seen[order[k]]) return fail(HIPATTN_INVALID_ARGUMENT, "transpose: order is not a permutation of the axes");
        seen[order[k]] = true;
        if (dims[k] < 0) return fail(HIPATTN_INVALID_ARGUMENT, "transpose: negative extent");
        if (dims[k] > 0xffffffffLL) return fail(HIPATTN_UNSUPPORTED, "transpose: extent beyond 2^32");
        count *= dims[k];
    }
    if (count == 0) return HIPATTN_OK;
    if (!in || !out) return fail(HIPATTN_INVALID_ARGUMENT, "transpose: null pointer");
    if (in == out) return fail(HIPATTN_INVALID_ARGUMENT, "transpose: in place is not supported");

    // input strides in elements, then the output's axes without those of extent 1, merged where two
    // neighbours are neighbours in the input too
    int64_t stride[kMaxAxes];
    for (int k = rank - 1; k >= 0; k--) stride[k] = k == rank - 1 ? 1 : stride[k + 1] * dims[k + 1];
    int n = 0;
    int64_t extent[kMaxAxes], in_stride[kMaxAxes];
    for (int k = 0; k < rank; k++) {
        const int src = order[k];
        if (dims[src] == 1) continue;
        if (n > 0 && in_stride[n - 1] == stride[src] * dims[src]) {  // the previous output axis steps over exactly this one
            extent[n - 1] *= dims[src];
            in_stride[n - 1] = stride[src];
        } else {
            extent[n] = dims[src];
            in_stride[n] = stride[src];
            n++;
        }
    }
    if (n <= 1) {  // nothing moves
        const hipError_t e = hipMemcpyAsync(out, in, (size_t)count * element_bytes, hipMemcpyDeviceToDevice, stream);
        if (e != hipSuccess) return fail(HIPATTN_HIP_ERROR, "transpose: copy: %s", hipGetErrorString(e));
        return HIPATTN_OK;
    }
    for (int k = 0; k < n; k++)
        if (extent[k] > 0xffffffffLL) return fail(HIPATTN_UNSUPPORTED, "transpose: merged extent beyond 2^32");

    if (in_stride[n - 1] == 1) {
        const int64_t run_bytes = extent[n - 1] * element_bytes;
        int piece = 16;
        while (piece > 1 && (run_bytes % piece || !aligned(in, piece) || !aligned(out, piece))) piece >>= 1;
        RowsParams p{};
        p.in = (const uint8_t*)in, p.out = (uint8_t*)out;
        p.axes = n - 1;
        for (int k = 0; k < n - 1; k++) {
            p.extent[k] = (uint32_t)extent[k];
            p.in_stride[k] = in_stride[k] * element_bytes / piece;  // every other input stride is a multiple of the run
        }
        p.run = (uint32_t)(run_bytes / piece);
        p.pieces = count * element_bytes / piece;
        if ((p.pieces + 255) / 256 > 0x7fffffffLL) return fail(HIPATTN_UNSUPPORTED, "transpose: tensor too large for one launch");
        switch (piece) {
            case 16: launch_rows<uint4_t>(p, stream); break;
            case 8: launch_rows<uint2_t>(p, stream); break;
            case 4: launch_rows<uint32_t>(p, stream); break;
            case 2: launch_rows<uint16_t>(p, stream); break;
            default: launch_rows<uint8_t>(p, stream); break;
        }
        return launched("transpose");
    }

    // the input's innermost axis sits somewhere else in the output
    int64_t out_stride[kMaxAxes];
    for (int k = n - 1; k >= 0; k--) out_stride[k] = k == n - 1 ? 1 : out_stride[k + 1] * extent[k + 1];
    int pos_a = -1;
    for (int k = 0; k < n; k++)
        if (in_stride[k] == 1) pos_a = k;
    if (pos_a < 0) return fail(HIPATTN_INVALID_ARGUMENT, "transpose: no axis of stride 1 left (internal)");
    TilesParams p{};
    p.in = (const uint8_t*)in, p.out = (uint8_t*)out;
    p.extent_a = (uint32_t)extent[pos_a], p.extent_b = (uint32_t)extent[n - 1];
    p.in_stride_b = in_stride[n - 1], p.out_stride_a = out_stride[pos_a];
    int64_t batches = 1;
    for (int k = 0; k < n - 1; k++) {
        if (k == pos_a) continue;
        p.extent[p.axes] = (uint32_t)extent[k];
        p.in_stride[p.axes] = in_stride[k];
        p.out_stride[p.axes] = out_stride[k];
        p.axes++;
        batches *= extent[k];
    }
    if (batches > 0xffffffffLL) return fail(HIPATTN_UNSUPPORTED, "transpose: too many tiles' batches for one launch");
    p.batches = (uint32_t)batches;
    const int64_t wide = element_bytes >= 2 ? 16 / element_bytes : 8;  // elements per access, as in the kernel
    p.wide_in = aligned(in, wide * element_bytes) && p.in_stride_b % wide == 0;
    p.wide_out = aligned(out, wide * element_bytes) && p.out_stride_a % wide == 0;
    for (int k = 0; k < p.axes; k++) {
        p.wide_in = p.wide_in && p.in_stride[k] % wide == 0;
        p.wide_out = p.wide_out && p.out_stride[k] % wide == 0;
    }
    const dim3 grid((p.extent_a + 63) / 64, (p.extent_b + 63) / 64, (unsigned)std::min<int64_t>(batches, 65535));
    if (grid.y > 65535) return fail(HIPATTN_UNSUPPORTED, "transpose: innermost output axis too long for one launch");
    switch (element_bytes) {
        case 8: hipLaunchKernelGGL(transpose_tiles_kernel<uint64_t>, grid, dim3(256), 0, stream, p); break;
        case 4: hipLaunchKernelGGL(transpose_tiles_kernel<uint32_t>, grid, dim3(256), 0, stream, p); break;
        case 2: hipLaunchKernelGGL(transpose_tiles_kernel<uint16_t>, grid, dim3(256), 0, stream, p); break;
        default: hipLaunchKernelGGL(transpose_tiles_kernel<uint8_t>, grid, dim3(256), 0, stream, p); break;
    }
    return launched("transpose");
}

hipattn_status convert(const void* in, void* out, int64_t count, int from_dtype, int to_dtype, hipStream_t stream) {
    if (count < 0) return fail(HIPATTN_INVALID_ARGUMENT, "convert: negative count");
    if (!type_size(from_dtype) || !type_size(to_dtype))
        return fail(HIPATTN_UNSUPPORTED, "convert: element types %d -> %d (f32, f16, bf16, i32, i64, u8, i8 or boolean expected)", from_dtype, to_dtype);
    if (count == 0) return HIPATTN_OK;
    if (!in || !out) return fail(HIPATTN_INVALID_ARGUMENT, "convert: null pointer");
    if ((count + 255) / 256 > 0x7fffffffLL) return fail(HIPATTN_UNSUPPORTED, "convert: too many elements for one launch");
    if (from_dtype == to_dtype && from_dtype != HIPOPS_BOOL) {  // as the reference: a copy, or nothing in place (kernels/convert.cu:30-41)
        if (in == out) return HIPATTN_OK;
        const hipError_t e = hipMemcpyAsync(out, in, (size_t)count * type_size(from_dtype), hipMemcpyDeviceToDevice, stream);
        if (e != hipSuccess) return fail(HIPATTN_HIP_ERROR, "convert: copy: %s", hipGetErrorString(e));
        return HIPATTN_OK;
    }
    bool ok = false;
    switch (from_dtype) {
        case HIPATTN_F32: ok = convert_from<HIPATTN_F32>(to_dtype, in, out, count, stream); break;
        case HIPATTN_F16: ok = convert_from<HIPATTN_F16>(to_dtype, in, out, count, stream); break;
        case HIPATTN_BF16: ok = convert_from<HIPATTN_BF16>(to_dtype, in, out, count, stream); break;
        case HIPATTN_I32: ok = convert_from<HIPATTN_I32>(to_dtype, in, out, count, stream); break;
        case HIPOPS_I64: ok = convert_from<HIPOPS_I64>(to_dtype, in, out, count, stream); break;
        case HIPOPS_U8: ok = convert_from<HIPOPS_U8>(to_dtype, in, out, count, stream); break;
        case HIPOPS_I8: ok = convert_from<HIPOPS_I8>(to_dtype, in, out, count, stream); break;
        case HIPOPS_BOOL: ok = convert_from<HIPOPS_BOOL>(to_dtype, in, out, count, stream); break;
    }
    if (!ok) return fail(HIPATTN_UNSUPPORTED, "convert: element types %d -> %d", from_dtype, to_dtype);
    return launched("convert");
}

}  // namespace hipops
