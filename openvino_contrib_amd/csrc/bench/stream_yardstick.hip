// A yardstick for the HBM-bound kernels on PART of the device: what do N compute units sustain when each
// runs one workgroup that does nothing but read, sixteen-byte loads with eight of them in flight per lane
// (64 KB per compute unit; four and thirty-two per lane measure the same)?  The paged decode kernel of a
// mixed batch runs on a share of the compute units beside the chunks' flash kernel; this reader, launched
// on a stream of its own ahead of that kernel, shows what the share could stream at best.  Not part of the
// attention path: it lives in the yardstick library that only bench.py loads (--workload stream).
#include <stdint.h>

#include <hip/hip_runtime.h>

namespace hipattn {

namespace {

constexpr int kReaderThreads = 512;
constexpr int kReaderDepth = 8;

// One workgroup to a compute unit: the LDS array is all of a compute unit's LDS, so no second workgroup fits.
__global__ __launch_bounds__(kReaderThreads) void stream_reader_kernel(const uint4* src, long long vecs_per_workgroup, uint32_t* sink) {
    __shared__ uint8_t whole_lds[160 * 1024 - 64];
    whole_lds[threadIdx.x] = 0;
    const uint4* p = src + (long long)blockIdx.x * vecs_per_workgroup + threadIdx.x;
    uint4 acc = make_uint4(0u, 0u, 0u, 0u);
    const long long rounds = vecs_per_workgroup / (kReaderThreads * kReaderDepth);
    for (long long r = 0; r < rounds; r++) {
        uint4 x[kReaderDepth];
#pragma unroll
        for (int u = 0; u < kReaderDepth; u++) x[u] = p[u * kReaderThreads];
#pragma unroll
        for (int u = 0; u < kReaderDepth; u++) {
            acc.x ^= x[u].x;
            acc.y += x[u].y;
            acc.z ^= x[u].z;
            acc.w += x[u].w;
        }
        p += kReaderThreads * kReaderDepth;
    }
    // (keeps the loads alive; the buffer bench.py fills never produces this value)
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = whole_lds[(threadIdx.x * 13) & 1023];
}

}  // namespace

}  // namespace hipattn

// Enqueues the reader on `stream`: `workgroups` workgroups share the first `bytes` bytes of `src` equally (each
// share rounded down to whole rounds of 64 KB) and read them once.  *bytes_read: what the launch reads.
// Returns 0 on success, a hipError_t value otherwise.
extern "C" __attribute__((visibility("default"))) int stream_yardstick_launch(const void* src, long long bytes, int workgroups,
                                                                              void* sink, void* stream, long long* bytes_read) {
    using namespace hipattn;
    if (!src || !sink || !bytes_read || workgroups < 1 || workgroups > 4096 || bytes < 0) return (int)hipErrorInvalidValue;
    const long long round_vecs = (long long)kReaderThreads * kReaderDepth;
    const long long vecs = bytes / 16 / workgroups / round_vecs * round_vecs;
    *bytes_read = vecs * 16 * workgroups;
    if (vecs == 0) return 0;
    hipLaunchKernelGGL(stream_reader_kernel, dim3(workgroups), dim3(kReaderThreads), 0, (hipStream_t)stream, (const uint4*)src, vecs,
                       (uint32_t*)sink);
    return (int)hipGetLastError();
}
