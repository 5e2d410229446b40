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
//   PI(rho) (see row_perm32): the permutation is applied in the LDS read address of the K/U/V tiles.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <atomic>
#include <type_traits>

namespace mhffn {

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));   // 16-byte copy unit (native vector: stays in registers)

constexpr int JB = 32;          // rows of K/U/V per block
// Experts whose gate values the forward and the dQ/dR kernel keep in LDS at a time ([GATE_WIN][256 tokens] fp32 = 64 KB,
// next to the 96 KB weight ring); a power of two.  With more experts the forward restages the tile every GATE_WIN experts
// (a multiple of four blocks whatever d_e is, so every window starts on its LDS stage 0) and the dQ/dR kernel refills it
// as a ring, expert e in slot e % GATE_WIN.
constexpr int GATE_WIN = 64;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float FLT_MAX_F = 3.402823466e+38f;

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

// The same instruction with its accumulator forced into architectural VGPRs (the compiler picks one register file for
// the accumulators of all builtin MFMAs of a kernel; a one-wave-per-SIMD kernel gets AGPRs, from which every value the
// VALU needs costs a v_accvgpr_read).  Used for products whose result feeds element-wise VALU work directly.
// The compiler cannot see that this is an MFMA, so the caller must leave the required wait states between the last of
// these and the first VALU read of the result (mfma_result_fence).  A/B operand waits (LDS loads) are still inserted
// by the compiler, back-to-back accumulation into the same registers is interlocked by hardware.
__device__ __forceinline__ void mfma32_vgpr_first(f32x16& d, bf16x8 a, bf16x8 b)
{
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma32_vgpr_acc(f32x16& d, bf16x8 a, bf16x8 b)
{
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "v"(b));
}
// Same, with the B operand held in an accumulation register (AGPRs are legal MFMA A/B sources): used for operands that
// stay resident for a whole kernel, so they do not compete with the VALU's working set for architectural VGPRs.
__device__ __forceinline__ void mfma32_vgpr_first_bacc(f32x16& d, bf16x8 a, bf16x8 b)
{
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b));
}
__device__ __forceinline__ void mfma32_vgpr_acc_bacc(f32x16& d, bf16x8 a, bf16x8 b)
{
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "a"(b));
}
__device__ __forceinline__ void mfma_result_fence(f32x16& a, f32x16& b, f32x16& c)
{
    // 8-pass MFMA result -> VALU read needs at most 18 wait states on gfx940-class hardware; leave 32.  The results
    // are operands of the statement, so no read of them can be scheduled above it.
    asm volatile("s_nop 15\n\ts_nop 15" : "+v"(a), "+v"(b), "+v"(c));
}
// Never pass the same object twice to one fence: the compiler would materialise the extra operands as register copies
// of the result, and those copies are VALU reads issued before the wait states have passed.
__device__ __forceinline__ void mfma_result_fence(f32x16& a)
{
    asm volatile("s_nop 15\n\ts_nop 15" : "+v"(a));
}

__device__ __forceinline__ float fast_sigmoid(float x)
{
    // 1 / (1 + 2^(-x log2 e)): v_mul, v_exp_f32, v_add, v_rcp_f32.  x -> -inf gives rcp(inf) = 0, x -> +inf gives 1.
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-LOG2E * x));
}

// ---- LDS tile layout shared by the main kernels -------------------------------------------------------------------
// A staged tile is 32 rows (weight rows j, or tokens) of 256 bytes: 16 chunks of 8 bf16, d_h/8 of them used.  The chunk
// holding columns [8c, 8c+8) of row r sits at chunk position c ^ swz16(r).  With this XOR swizzle both access patterns
// -- 16-byte row reads (16 lanes = 16 different rows, same column chunk) and transposing 8-byte reads (a 16-lane group
// reads 4 consecutive rows x 32 contiguous bytes) -- are bank-conflict free without padding, so tiles can be filled
// by global_load_lds_dwordx4, whose LDS destination is (wave-uniform base) + lane * 16.
constexpr int TILE_ROW_B = 256;
constexpr int TILE_B = JB * TILE_ROW_B;   // 8 KB

__device__ __forceinline__ int swz16(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 v4bf16_t;

// One wave-instruction of an asynchronous tile fill: 4 rows (ins*4 .. ins*4+3) of a row-major [32][DH] bf16 source
// tile whose row `r` starts at src_row0 + r * row_stride (elements).  Counts as one vmcnt event.
template <int DH>
__device__ __forceinline__ void tile_fill_ins(const bf16_t* src_row0, long row_stride, unsigned char* lds_tile, int ins,
                                              int lane)
{
    const int r = 4 * ins + (lane >> 4);
    int c = (lane & 15) ^ swz16(r);
    c = c < DH / 8 ? c : 0;   // chunk positions a narrow row does not use receive a dummy chunk
    __builtin_amdgcn_global_load_lds((gptr_t)(src_row0 + r * row_stride + c * 8), (lptr_t)(lds_tile + ins * 1024), 16, 0,
                                     0);
}

// A operand (32 rows x 16 k) for k-step ks from a swizzled tile, row-major use: lane holds row `row`, columns
// 16ks + 8g .. +7.
__device__ __forceinline__ bf16x8 tile_read_rows(const unsigned char* tile, int row, int ks, int g)
{
    return *reinterpret_cast<const bf16x8*>(tile + row * TILE_ROW_B + (((2 * ks + g) ^ swz16(row)) << 4));
}

// A operand (32 rows = tile columns 32ct + l32, 16 k = tile rows) from a swizzled tile, transposed use:
// lane holds column 32ct + l32; its 8 k values are tile rows rlo + {0..3} then rhi + {0..3}.  rlo/rhi must be uniform
// within each 16-lane group (they may depend on lane / 32).
//
// The two ds_read_b64_tr_b16 are issued from inline assembly, not through the compiler builtin: behind the builtin the
// compiler cannot tell that the read does not touch the LDS stage an asynchronous LDS-direct load is filling, and puts
// a full s_waitcnt vmcnt(0) in front of it, which stalls every loop iteration for the whole global-memory latency.
// The price is that the compiler does not know these reads are in flight either: the consumer must call
// lds_tr_wait() on the operands before their first use.
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
struct TrOperand {
    u32x2 lo, hi;
};
__device__ __forceinline__ unsigned lds_addr(const void* p)
{
    return (unsigned)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}
// Per-lane byte offsets (inside a tile, for s = 0) of the two reads of a transposed operand, for every column tile ct.
// The tile rows a lane group reads are  16 s + RG * (lane / 32) + RH * hi + (lane % 16) / 4,  hi = 0, 1
//   (RG, RH) = (8, 4): k-slot (s, g, kk) is row 16 s + 8 g + kk            (weights: second products of fwd, dQ)
//   (RG, RH) = (4, 8): k-slot (s, g, kk) is row 16 s + 8 (kk / 4) + 4 g + kk % 4   (tokens: dK/dU/dV contraction)
// s only adds 16 rows = 4096 bytes (the swizzle has period 16 rows), which goes into the instruction's immediate offset.
template <int CT>
struct TrLane {
    unsigned off[CT][2];
};
template <int CT, int RG, int RH>
__device__ __forceinline__ TrLane<CT> make_tr_lane(int lane)
{
    TrLane<CT> t;
    const int lam = lane & 15, l32 = lane & 31, g = lane >> 5;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int hi = 0; hi < 2; ++hi) {
            const int r = RG * g + RH * hi + (lam >> 2);
            const int chunk = 4 * ct + 2 * (l32 >> 4) + ((lam & 3) >> 1);
            t.off[ct][hi] = r * TILE_ROW_B + ((chunk ^ swz16(r)) << 4) + (lam & 1) * 8;
        }
    return t;
}
// Requests operand (ct, s) of the tile at LDS byte address `tile_addr` (wave-uniform); IMM = 4096 * s + any
// compile-time displacement (must stay below 65536 together).
template <int IMM, int CT>
__device__ __forceinline__ TrOperand tile_read_cols_async(unsigned tile_addr, const TrLane<CT>& tl, int ct)
{
    const unsigned a0 = tile_addr + tl.off[ct][0], a1 = tile_addr + tl.off[ct][1];
    TrOperand t;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(t.lo) : "v"(a0), "n"(IMM));
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(t.hi) : "v"(a1), "n"(IMM));
    return t;
}
// Waits for every LDS operation of this wave (lgkmcnt(0)); the operands are inputs and outputs of the statement, so no
// use of them can be scheduled above it.
__device__ __forceinline__ void lds_tr_wait(TrOperand& a)
{
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a.lo), "+v"(a.hi));
}
__device__ __forceinline__ void lds_tr_wait(TrOperand& a, TrOperand& b)
{
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a.lo), "+v"(a.hi), "+v"(b.lo), "+v"(b.hi));
}
__device__ __forceinline__ void lds_tr_wait(TrOperand& a, TrOperand& b, TrOperand& c, TrOperand& d)
{
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(a.lo), "+v"(a.hi), "+v"(b.lo), "+v"(b.hi), "+v"(c.lo), "+v"(c.hi), "+v"(d.lo), "+v"(d.hi));
}
// Partial wait: at most N LDS operations of this wave still outstanding.  Only exact inside a region that the caller
// has fenced with sched_barrier(0) and that contains no other LDS instruction than the asynchronous reads above
// (LDS operations complete in order; each TrOperand is two of them).
template <int N>
__device__ __forceinline__ void lds_tr_wait_n(TrOperand& a, TrOperand& b)
{
    asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(a.lo), "+v"(a.hi), "+v"(b.lo), "+v"(b.hi) : "n"(N));
}
// The same for 16 contiguous bytes per lane (a row-major A operand as in tile_read_rows, four gate values): issued from
// inline assembly so that the waits in front of the uses can be partial -- the compiler's own bookkeeping puts a full
// lgkmcnt(0) in front of the first use of any read of a group in flight.  IMM: compile-time displacement.
template <int IMM>
__device__ __forceinline__ u32x4 lds_read16_async(unsigned addr)
{
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(IMM));
    return v;
}
// Two 4-byte values per lane, 128 bytes apart (one instruction, one LDS operation).
__device__ __forceinline__ u32x2 lds_read2x4_async(unsigned addr)
{
    u32x2 v;
    asm volatile("ds_read2_b32 %0, %1 offset1:32" : "=v"(v) : "v"(addr));
    return v;
}
// At most N LDS operations of this wave still outstanding; the operands cannot be used above it.  Same conditions as
// lds_tr_wait_n.
template <int N>
__device__ __forceinline__ void lds_wait_n(u32x4& a, u32x4& b, u32x2& c)
{
    asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(a), "+v"(b), "+v"(c) : "n"(N));
}
// The same without operands, for reads whose only consumers are matrix instructions issued from inline assembly (volatile
// statements keep their order): with the operands tied to the wait the compiler assumes the statement wrote them and puts
// a hazard s_nop in front of the matrix instruction.
template <int N>
__device__ __forceinline__ void lds_wait_n()
{
    asm volatile("s_waitcnt lgkmcnt(%0)" :: "n"(N));
}
template <int N>
__device__ __forceinline__ void lds_wait_n(u32x4& a, u32x4& b, u32x4& c, u32x4& d, u32x4& e, u32x4& f)
{
    asm volatile("s_waitcnt lgkmcnt(%6)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e), "+v"(f) : "n"(N));
}
__device__ __forceinline__ bf16x8 tr_value(const TrOperand& t)
{
    u32x4 v = {t.lo[0], t.lo[1], t.hi[0], t.hi[1]};
    return __builtin_bit_cast(bf16x8, v);
}

// s_waitcnt vmcnt(N) only (gfx9 encoding: vmcnt[3:0] at bits 3:0, vmcnt[5:4] at bits 15:14; other counters unconstrained).
template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// Dynamic LDS above 64 KB must be opted into per kernel function and per device.  One LdsOptIn per kernel function (static
// storage, zero-initialised) remembers the largest size already granted on each device, so the attribute call is made
// once per (kernel, device) whichever host thread launches first; a repeated call is harmless.
constexpr int LDS_OPTIN_MAX_DEVICES = 64;
struct LdsOptIn {
    std::atomic<int> granted[LDS_OPTIN_MAX_DEVICES];
};
inline hipError_t ensure_dynamic_lds(LdsOptIn& c, const void* fn, int bytes)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const bool tracked = dev >= 0 && dev < LDS_OPTIN_MAX_DEVICES;
    if (tracked && bytes <= c.granted[dev].load(std::memory_order_acquire)) return hipSuccess;
    e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess && tracked) c.granted[dev].store(bytes, std::memory_order_release);
    return e;
}

// Host-side launch entry points (defined in the per-kernel .hip files).
struct Dims {
    int B, H, Hkuv, S, d_h, E, d_e;
    int tokmaj;   // layout of Q, O, dO, dQ: 0 = [B, H, S, d_h], 1 = [B, S, H, d_h] (token-major, heads interleaved)
};

// Rows (units of d_h elements) of Q/O/dO/dQ: token t of (batch b, q-head h) is row base + t * stride.
struct TokRows {
    long base;
    int stride;
};
__host__ __device__ inline TokRows tok_rows(int tokmaj, int b, int h, int H, int S)
{
    return tokmaj ? TokRows{(long)b * S * H + h, H} : TokRows{((long)b * H + h) * S, 1};
}

size_t fwd_workspace_bytes_bf16(const Dims& d);
size_t bwd_workspace_bytes_bf16(const Dims& d);       // what the launch uses when it may choose freely (0: one token
                                                      // slice, no partial sums); with less it runs fewer slices
hipError_t launch_fwd_bf16(const void* Q, const void* K, const void* U, const void* V, const float* R, void* O,
                           void* ws, const Dims& d, hipStream_t st, int phases);
hipError_t launch_bwd_bf16(const void* Q, const void* K, const void* U, const void* V, const float* R, const void* dO,
                           void* dQ, void* dK, void* dU, void* dV, float* dR, int grad_w_f32,
                           void* ws, size_t ws_bytes, const Dims& d, hipStream_t st, int phases);

// fp32 instantiation (mhffn_f32.hip): d_h a multiple of 8 up to 128, any d_e, any E.
size_t bwd_workspace_bytes_f32(const Dims& d);
hipError_t launch_fwd_f32(const void* Q, const void* K, const void* U, const void* V, const float* R, void* O,
                          const Dims& d, hipStream_t st);
hipError_t launch_bwd_f32(const void* Q, const void* K, const void* U, const void* V, const float* R, const void* dO,
                          void* dQ, void* dK, void* dU, void* dV, float* dR, int grad_w_f32, void* ws, const Dims& d,
                          hipStream_t st, int phases);

// Head prologue (mhffn_gate.hip): per-head RMSNorm + expert gate over [B, S, H, d_h] bf16 rows; d_h 64/96/128, E <= 64.
hipError_t launch_gate_fwd(const void* X, const float* Wn, float eps, const float* Wr, void* Qn, float* R, const Dims& d,
                           hipStream_t st);
hipError_t launch_gate_bwd(const void* X, const float* Wn, float eps, const float* Wr, const void* dQ, int dq_tokmaj,
                           const float* dR, void* dX, float* dWn, float* dWr, const Dims& d, hipStream_t st);

// Bits of the `phases` argument of the launch functions (the values of MHFFN_FWD_* / MHFFN_BWD_* in include/mhffn.h).
constexpr int PH_FWD_MAIN = 1, PH_BWD_DQDR = 1, PH_BWD_DKDUDV = 2, PH_BWD_REDUCE = 4;

}  // namespace mhffn
