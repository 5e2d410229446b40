// Benchmark-only object (libmhffn_probe.so), not part of the product library or its header.
// Diagnostic: what the matrix cores of this device sustain on a register-resident loop of the instruction the kernels
// use (v_mfma_f32_32x32x16_bf16), one wave per SIMD with four independent accumulator chains, no memory traffic.  The
// benchmark prints its rate next to the kernels' so that a figure can be read against the clock the chip actually holds
// under matrix load as well as against the nominal peak -- once on smooth operand values and once on values in which
// every bit varies, which is what the kernels multiply.
#include "mhffn_common.hpp"

namespace mhffn {

// Operand values: `random_data` = 0 gives small, smoothly varying numbers (few mantissa and exponent bits differ between
// lanes and elements), 1 gives hashed values spread over (-2, 2) in which every bit varies, as in real activations and
// weights.  The matrix cores' power draw, and with it the clock the package grants, depends on how many bits toggle.
__global__ __launch_bounds__(256) void mfma_peak_probe_kernel(float* sink, int iters, int random_data)
{
    const int lane = threadIdx.x & 63;
    bf16x8 a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (random_data) {
                unsigned h = (unsigned)lane * 2654435761u ^ (unsigned)(j + 1) * 40503u ^ (unsigned)(i + 1) * 97u;
                h ^= h >> 13;
                h *= 0x5bd1e995u;
                h ^= h >> 15;
                a[i][j] = (bf16_t)((float)((int)(h & 0xffffu) - 32768) * (1.0f / 16384.0f));
                b[i][j] = (bf16_t)((float)((int)(h >> 16) - 32768) * (1.0f / 16384.0f));
            } else {
                a[i][j] = (bf16_t)(0.001f * (float)(lane + j));
                b[i][j] = (bf16_t)(0.002f * (float)(lane - j));
            }
        }
    f32x16 c0, c1, c2, c3;
#pragma unroll
    for (int i = 0; i < 16; ++i) c0[i] = c1[i] = c2[i] = c3[i] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            c0 = mfma32(a[r & 3], b[0], c0);
            c1 = mfma32(a[r & 3], b[1], c1);
            c2 = mfma32(a[r & 3], b[2], c2);
            c3 = mfma32(a[r & 3], b[3], c3);
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
// float; `random_data` selects the operand values (see the kernel).  Returns 0, or -1 on bad arguments or a failed launch.
extern "C" int mhffn_probe_mfma_loop(float* sink, int blocks, int iters, int random_data, void* stream, double* flops)
{
    if (!sink || !flops || blocks <= 0 || iters <= 0 || blocks > (1 << 20)) return -1;
    *flops = 2.0 * 32 * 32 * 16 * 32.0 * (double)iters * 4.0 * (double)blocks;
    hipLaunchKernelGGL(mhffn::mfma_peak_probe_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, sink, iters,
                       random_data);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

// The loop on smooth operand values (the form this entry point has always had).
extern "C" int mhffn_probe_mfma_peak(float* sink, int blocks, int iters, void* stream, double* flops)
{
    return mhffn_probe_mfma_loop(sink, blocks, iters, 0, stream, flops);
}
