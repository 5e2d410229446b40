// Benchmark-only object (libmhffn_probe.so), not part of the product library or its header.
// Diagnostic: what the matrix cores of this device sustain on a register-resident loop of the instruction the kernels
// use (v_mfma_f32_32x32x16_bf16), one wave per SIMD with four independent accumulator chains, no memory traffic.  The
// benchmark prints its rate next to the kernels' so that a figure can be read against the clock the chip actually holds
// under matrix load as well as against the nominal peak.
#include "mhffn_common.hpp"

namespace mhffn {

__global__ __launch_bounds__(256) void mfma_peak_probe_kernel(float* sink, int iters)
{
    const int lane = threadIdx.x & 63;
    bf16x8 a, b;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        a[j] = (bf16_t)(0.001f * (float)(lane + j));
        b[j] = (bf16_t)(0.002f * (float)(lane - j));
    }
    f32x16 c0, c1, c2, c3;
#pragma unroll
    for (int i = 0; i < 16; ++i) c0[i] = c1[i] = c2[i] = c3[i] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            c0 = mfma32(a, b, c0);
            c1 = mfma32(a, b, c1);
            c2 = mfma32(a, b, c2);
            c3 = mfma32(a, b, c3);
        }
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
    if (s == 12345.678f) sink[0] = s;   // keeps the loop alive; practically never true
}

}  // namespace mhffn

// Enqueues `blocks` workgroups of four waves, `iters` x 32 matrix instructions of 2*32*32*16 flops per wave, no memory
// traffic, and writes the number of floating-point operations executed to *flops (host memory).  `sink` is one device
// float.  Returns 0, or -1 on bad arguments or a failed launch.
extern "C" int mhffn_probe_mfma_peak(float* sink, int blocks, int iters, void* stream, double* flops)
{
    if (!sink || !flops || blocks <= 0 || iters <= 0 || blocks > (1 << 20)) return -1;
    *flops = 2.0 * 32 * 32 * 16 * 32.0 * (double)iters * 4.0 * (double)blocks;
    hipLaunchKernelGGL(mhffn::mfma_peak_probe_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, sink, iters);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}
