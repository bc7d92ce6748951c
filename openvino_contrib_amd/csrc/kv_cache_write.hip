// Device-side KV-cache block writer: scatters the new key/value rows of a batch into the
// paged caches, converting or quantising on the way.  HBM-bound byte moving: one wavefront
// per (token, kv head), contiguous rows, no staging.
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
    const int pair = blockIdx.x * 4 + (threadIdx.x >> 6);  // (token, kv head) pair of this wavefront
    if (pair >= p.num_tokens * p.num_heads_kv) return;
    kv_cache_write_pair<kMaxPerLane>(p, pair / p.num_heads_kv, pair % p.num_heads_kv, threadIdx.x & 63);
}

hipError_t launch_kv_cache_write(const KvWriteParams& p, hipStream_t stream) {
    if (p.num_tokens == 0 || p.num_seqs == 0) return hipSuccess;
    const int64_t pairs = (int64_t)p.num_tokens * p.num_heads_kv;
    dim3 grid((unsigned)((pairs + 3) / 4));
    if (p.head_dim <= 128)
        hipLaunchKernelGGL(kv_cache_write_kernel<2>, grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(kv_cache_write_kernel<8>, grid, dim3(256), 0, stream, p);
    return hipGetLastError();
}

}  // namespace hipattn
