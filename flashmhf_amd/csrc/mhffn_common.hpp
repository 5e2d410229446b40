// Shared device/host definitions for the gfx950 fused multi-head FFN kernels.
//
// Tile vocabulary used by every kernel in this directory
// -------------------------------------------------------
// * "j" indexes rows of K/U/V inside one expert (the d_e axis), "c" indexes the head dim (d_h), "t" a token.
// * The d_e axis is processed in blocks of JB = 32 rows; blocks never straddle experts (d_e % 32 == 0).
// * All matrix products use v_mfma_f32_32x32x16_bf16.  For one instruction D = A(32x16) * B(16x32) + C:
//       A: lane l holds row (l % 32), k = 8*(l / 32) .. +7        (8 bf16 = 4 VGPRs)
//       B: lane l holds col (l % 32), k = 8*(l / 32) .. +7
//       C/D: lane l holds col (l % 32), register i (0..15) holds row 8*(i/4) + 4*(l/32) + (i%4)
// * Chained products keep the first product's C registers as the second product's B operand without a trip
//   through LDS: with the first product written "transposed" (rows = j, cols = t) registers 8s..8s+7 of lane
//   (t, g = l/32) are exactly the 8 k-slots the second product's B operand wants, provided slot (s, g, kk)
//   means j = 16s + 8g + kk.  That holds when output row rho of the first product was fed K row
//   PI(rho) (see row_perm32): the permutation is applied once, when the weight tiles are packed.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

namespace mhffn {

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));   // 16-byte copy unit (native vector: stays in registers)

constexpr int JB = 32;          // rows of K/U/V per block
constexpr int PADE = 8;         // bf16 elements of padding per LDS row (16 bytes: rotates rows across banks)
constexpr float LOG2E = 1.4426950408889634f;

// MFMA output row rho (0..31) -> which row of the 32-row weight block must be fed as A-row rho so that
// C registers 8s..8s+7 of lane group g hold j = 16s + 8g + kk.  rho = 8a + 4g + b  ->  16(a/2) + 8g + 4(a%2) + b.
__host__ __device__ constexpr int row_perm32(int rho)
{
    return 16 * ((rho >> 3) >> 1) + 8 * ((rho >> 2) & 1) + 4 * ((rho >> 3) & 1) + (rho & 3);
}

// Position p (0..31) inside a transposed token tile -> token it holds, so that B-operand k-slot (s, g, kk) of a
// [t, j] product's C registers (token 16s + 8(kk/4) + 4g + kk%4) lines up with 8 contiguous positions 16s + 8g + kk.
__host__ __device__ constexpr int tok_perm32(int p)
{
    return (p & 16) + 8 * ((p >> 2) & 1) + 4 * ((p >> 3) & 1) + (p & 3);
}

// Geometry of the packed tiles, all in bf16 elements.
//   natural tile   [32 rows][DH + 8]   row rho = weight row row_perm32(rho) (or token row for Q/dO tiles)
//   transposed tile [DH rows][32 + 8]  row c, position = j (weights) or tok_perm32 position (tokens)
template <int DH>
struct Geo {
    static constexpr int NAT_LD = DH + PADE;
    static constexpr int NAT_ELEMS = JB * NAT_LD;
    static constexpr int TR_LD = JB + PADE;
    static constexpr int TR_ELEMS = DH * TR_LD;
    static constexpr int FWD_STAGE = 2 * NAT_ELEMS + TR_ELEMS;       // Kn | Un | Vt
    static constexpr int DQ_STAGE = 3 * NAT_ELEMS + 2 * TR_ELEMS;    // Kn | Un | Vn | Kt | Ut
};

// Compile-time loop: f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>).  Arrays indexed through it are
// indexed by constants from the first optimisation pass on, so they are promoted to registers (never scratch).
template <int I, int N>
struct StaticFor {
    template <class F>
    __device__ __forceinline__ static void run(F&& f)
    {
        f(std::integral_constant<int, I>{});
        StaticFor<I + 1, N>::run(f);
    }
};
template <int N>
struct StaticFor<N, N> {
    template <class F>
    __device__ __forceinline__ static void run(F&&) {}
};
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f)
{
    StaticFor<0, N>::run(f);
}

__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ float fast_sigmoid(float x)
{
    // 1 / (1 + 2^(-x log2 e)): v_mul, v_exp_f32, v_add, v_rcp_f32.  x -> -inf gives rcp(inf) = 0, x -> +inf gives 1.
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-LOG2E * x));
}

// Host-side launch entry points (defined in the per-kernel .hip files).
struct Dims {
    int B, H, Hkuv, S, d_h, E, d_e;
};

// Re-lays the K/U/V blocks of every (kuv-head, 32-row block) as one contiguous "stage image" that the main kernels
// copy verbatim into LDS.  bundle 0: forward (Kn|Un|Vt); bundle 1: dQ/dR kernel (Kn|Un|Vn|Kt|Ut).
hipError_t launch_pack_weights(const void* K, const void* U, const void* V, void* dst, int bundle, const Dims& d,
                               hipStream_t st);
size_t packed_weights_bytes(const Dims& d, int bundle);

size_t fwd_workspace_bytes_bf16(const Dims& d);
size_t bwd_workspace_bytes_bf16(const Dims& d);
hipError_t launch_fwd_bf16(const void* Q, const void* K, const void* U, const void* V, const float* R, void* O,
                           void* ws, const Dims& d, hipStream_t st, int phases);
hipError_t launch_bwd_bf16(const void* Q, const void* K, const void* U, const void* V, const float* R, const void* dO,
                           void* dQ, void* dK, void* dU, void* dV, float* dR, int grad_w_f32,
                           void* ws, const Dims& d, hipStream_t st, int phases);

}  // namespace mhffn
