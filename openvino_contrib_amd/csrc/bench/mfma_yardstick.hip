// A yardstick for the MFMA-bound kernels, as a plain copy is one for the HBM-bound ones: what does
// this device sustain when every wavefront issues nothing but register-fed
// v_mfma_f32_32x32x16_bf16, and at which shader clock?  The published peak (2.5 PFLOP/s dense
// bf16) assumes 2.4 GHz; under load the clock is set by the power management, and the power an
// MFMA draws depends on how many operand bits toggle, so the answer differs between all-zero
// operands and random ones.  Not part of the attention path and not part of libhipattn: built into a
// library of its own (libmfma_yardstick.so) that only bench.py --workload mfma loads.
#include <vector>

#include <hip/hip_runtime.h>

#include "device_common.hpp"

namespace hipattn {

namespace {

constexpr int kYardstickIters = 4000;  // rounds of 4 MFMAs per wavefront and launch

// One workgroup of eight wavefronts per compute unit (two per SIMD), four accumulators each.
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void mfma_yardstick_kernel(int zero_data,
                                                                                                       long long* clocks,
                                                                                                       float* sink) {
    const long long w0 = wall_clock64();
    const long long c0 = (long long)__builtin_readcyclecounter();
    float16_t acc[4];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[a][r] = 0.0f;
    bf16x8_t x[4], y[4];
    uint32_t s = 12345u + 7919u * (blockIdx.x * 512u + threadIdx.x);
#pragma unroll
    for (int k = 0; k < 4; k++)
#pragma unroll
        for (int i = 0; i < 8; i++) {
            s = s * 1664525u + 1013904223u;
            const float fx = zero_data ? 0.0f : (float)((int)(s >> 8) % 2001 - 1000) * 0.001f;
            s = s * 1664525u + 1013904223u;
            const float fy = zero_data ? 0.0f : (float)((int)(s >> 8) % 2001 - 1000) * 0.001f;
            x[k][i] = (__bf16)fx;
            y[k][i] = (__bf16)fy;
        }
    for (int it = 0; it < kYardstickIters; it += 4) {
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int a = 0; a < 4; a++)
                acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x[a], y[(a + u) & 3], acc[a], 0, 0, 0);
    }
    float t = 0.0f;
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int r = 0; r < 16; r++) t += acc[a][r];
    if (t == 12345.678f) *sink = t;  // keeps the products alive
    if (threadIdx.x == 0) {
        clocks[blockIdx.x * 2] = wall_clock64() - w0;  // 100 MHz
        clocks[blockIdx.x * 2 + 1] = (long long)__builtin_readcyclecounter() - c0;
    }
}

}  // namespace

// Runs the kernel `launches` times after as many untimed ones (clock ramp) on the default stream and
// synchronises it.
static hipError_t run_mfma_yardstick(int zero_data, int launches, double* tflops, double* shader_ghz) {
    hipStream_t stream = nullptr;
    int dev = 0, cus = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return e;
    long long* clocks = nullptr;
    float* sink = nullptr;
    e = hipMalloc(&clocks, (size_t)cus * 2 * sizeof(long long));
    if (e != hipSuccess) return e;
    e = hipMalloc(&sink, sizeof(float));
    if (e != hipSuccess) {
        (void)hipFree(clocks);
        return e;
    }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    for (int i = 0; i < launches; i++)
        hipLaunchKernelGGL(mfma_yardstick_kernel, dim3(cus), dim3(512), 0, stream, zero_data, clocks, sink);
    (void)hipEventRecord(e0, stream);
    for (int i = 0; i < launches; i++)
        hipLaunchKernelGGL(mfma_yardstick_kernel, dim3(cus), dim3(512), 0, stream, zero_data, clocks, sink);
    (void)hipEventRecord(e1, stream);
    e = hipStreamSynchronize(stream);
    float ms = 0.0f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    std::vector<long long> h((size_t)cus * 2);
    if (e == hipSuccess) e = hipMemcpy(h.data(), clocks, h.size() * sizeof(long long), hipMemcpyDeviceToHost);
    if (e == hipSuccess) {
        double wall = 0.0, clk = 0.0;
        for (int i = 0; i < cus; i++) {
            wall += (double)h[2 * i];
            clk += (double)h[2 * i + 1];
        }
        const double flops = (double)cus * 8.0 * kYardstickIters * 4.0 * 2.0 * 32.0 * 32.0 * 16.0;
        *tflops = flops / ((double)ms / launches * 1e-3) / 1e12;
        *shader_ghz = wall > 0.0 ? clk / wall * 0.1 : 0.0;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(clocks);
    (void)hipFree(sink);
    return e;
}

}  // namespace hipattn

// Returns 0 on success, a hipError_t value otherwise.
extern "C" __attribute__((visibility("default"))) int mfma_yardstick(int zero_data, int launches, double* tflops,
                                                                     double* shader_ghz) {
    if (!tflops || !shader_ghz || launches < 1 || launches > 100000) return (int)hipErrorInvalidValue;
    return (int)hipattn::run_mfma_yardstick(zero_data, launches, tflops, shader_ghz);
}
