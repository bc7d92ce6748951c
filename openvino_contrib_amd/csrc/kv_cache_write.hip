// Device-side KV-cache block writer: scatters the new key/value rows of a batch into the
// paged caches, converting or quantising on the way.  HBM-bound byte moving: one wavefront
// per (token, kv head) -- per token for large batches --, contiguous rows, no staging.
//
// Nearest reference analogue: the row scatter of src/kernels/scatter_nd_update.cu:19-34,
// 36-79 (which first copies the whole input, scatter_nd_update.cu:170-171; this writer
// touches only the new rows) and the whole-state copies of
// src/cuda_variable_state.hpp:135-160.  Out-of-range targets are skipped as in
// tests/unit/kernels/scatter_update.cpp:59-86.
#include "kv_cache_write.hpp"

namespace hipattn {

template <int kMaxPerLane>
__global__ __launch_bounds__(256) void kv_cache_write_kernel(KvWriteParams p) {
    kv_cache_write_wave<kMaxPerLane>(p, (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6), threadIdx.x & 63);
}

hipError_t launch_kv_cache_write(const KvWriteParams& params, hipStream_t stream) {
    if (params.num_tokens == 0 || params.num_seqs == 0) return hipSuccess;
    KvWriteParams p = params;
    dim3 grid((unsigned)((kv_write_wavefronts(p) + 3) / 4));
    if (p.head_dim <= 128)
        hipLaunchKernelGGL(kv_cache_write_kernel<2>, grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(kv_cache_write_kernel<8>, grid, dim3(256), 0, stream, p);
    return hipGetLastError();
}

}  // namespace hipattn
