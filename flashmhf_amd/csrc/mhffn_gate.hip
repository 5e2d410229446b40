// Head prologue of the multi-head FFN block for gfx950: per-head RMSNorm of the projected heads and the expert gate, in
// one pass over the [B, S, H, d_h] activations, forward and backward.
//
//   u = x * rsqrt(mean(x^2) + eps)            fp32, per (token, head) row          (modeling_mhffnmoe.py:124-129)
//   y = bf16(u * w[h])                        the Q the fused operator reads       (:130-133)
//   z = y . router[h]      (fp32, d_h x E)    s = sigmoid(z)    R = s / max(sum_e s, 1e-20)   (:384-386)
//
// Both kernels are bound by HBM traffic, not by arithmetic: a wave owns tiles of 32 tokens of one head, loads each row
// once with 16-byte accesses (a lane holds half a row: the 8-element chunks 2ks + g), keeps everything between the load
// and the stores in registers, and takes the router products on the matrix cores:
//   * logits^T [E x 32 tokens] = router^T (A, staged once per workgroup in LDS as bf16 hi + lo parts of the fp32
//     values, so a float32 router is honoured to 2^-17) x y^T (B = the lane's own packed row chunks);
//     the sum over experts is then a sum over a lane's registers plus one exchange between the two lane halves;
//   * backward: dy += dz router^T (B = dz straight from the logits' registers: the router rows are fed in row_perm32
//     order, exactly as the main kernels chain their products) and d_router += y^T dz (contraction over tokens = lanes:
//     y and dz go through a wave-private LDS tile and come back with transposing reads).
// d_router and d_norm_weight are summed over all tokens: per-wave partial sums in registers, one atomic add per wave
// and element at the end (the caller passes zero-filled or to-be-accumulated buffers).
#include "mhffn_common.hpp"

namespace mhffn {

struct GateArgs {
    const bf16_t* X;     // [B, S, H, DH]
    const float* Wn;     // [H, DH] (NORM only)
    const float* Wr;     // [H, DH, E]
    bf16_t* Qn;          // [B, S, H, DH] (NORM only)
    float* R;            // [B, H, S, E]
    const bf16_t* dQ;    // gradient of y, rows addressed through dq_tokmaj
    const float* dR;     // [B, H, S, E]
    bf16_t* dX;          // [B, S, H, DH]
    float* dWn;          // [H, DH], accumulated
    float* dWr;          // [H, DH, E], accumulated
    int B, H, S, E, tpw, dq_tokmaj;
    float eps;
};

__device__ __forceinline__ float bf_even(unsigned w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf_odd(unsigned w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
__device__ __forceinline__ float bf_at(const u32x4& v, int j) { return (j & 1) ? bf_odd(v[j >> 1]) : bf_even(v[j >> 1]); }

// Router slice of head h as MFMA A operands in LDS.
//   part 0/1 (hi/lo), expert tile nt, k-step ks, lane (rho, g): router[(2ks+g)*8 + j][nt*32 + row_perm32(rho)], j = 0..7
// so that register 8s + kk of lane half g of the product holds expert nt*32 + 16s + 8g + kk.
template <int DH, int NT>
__device__ __forceinline__ void stage_router_rows(const float* Wr, int E, unsigned char* dst)
{
    constexpr int KS = DH / 16;
    for (int idx = threadIdx.x; idx < NT * KS * 64; idx += blockDim.x) {
        const int ln = idx & 63, ks = (idx >> 6) % KS, nt = idx / (KS * 64);
        const int e = nt * 32 + row_perm32(ln & 31), k0 = (2 * ks + (ln >> 5)) * 8;
        bf16x8 hi, lo;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float v = e < E ? Wr[(long)(k0 + j) * E + e] : 0.0f;
            hi[j] = (bf16_t)v;
            lo[j] = (bf16_t)(v - (float)hi[j]);
        }
        *reinterpret_cast<bf16x8*>(dst + idx * 16) = hi;
        *reinterpret_cast<bf16x8*>(dst + (NT * KS * 64 + idx) * 16) = lo;
    }
}

// Router slice as A operands of dy^T [d_h x tokens] = router [d_h x E] dz^T: column tile ct, k-step q = 2nt + s,
// lane (rho, g): router[ct*32 + row_perm32(rho)][nt*32 + 16s + 8g + j]  (bf16, high part only: dy is rounded to bf16).
template <int DH, int NT>
__device__ __forceinline__ void stage_router_cols(const float* Wr, int E, unsigned char* dst)
{
    constexpr int CT = DH / 32;
    for (int idx = threadIdx.x; idx < CT * 2 * NT * 64; idx += blockDim.x) {
        const int ln = idx & 63, q = (idx >> 6) % (2 * NT), ct = idx / (2 * NT * 64);
        const int col = ct * 32 + row_perm32(ln & 31), e0 = q * 16 + 8 * (ln >> 5);
        bf16x8 v;
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = (bf16_t)(e0 + j < E ? Wr[(long)col * E + e0 + j] : 0.0f);
        *reinterpret_cast<bf16x8*>(dst + idx * 16) = v;
    }
}

// Everything the forward computes for one tile, shared by both kernels.
template <int DH, int NT, bool NORM>
struct GateTile {
    static constexpr int KS = DH / 16;
    u32x4 xr[KS];       // the lane's half row of x
    bf16x8 y[KS];       // normalised, rounded
    float rstd;
    float s[NT][16];    // sigmoid(z), 0 for experts >= E
    float inv;          // 1 / max(sum s, 1e-20)
    float sum;

    __device__ __forceinline__ void load(const bf16_t* xrow, int g)
    {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) xr[ks] = *reinterpret_cast<const u32x4*>(xrow + (2 * ks + g) * 8);
    }
    __device__ __forceinline__ void normalise(const float* sW, int g)
    {
        if constexpr (NORM) {
            float ss = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float v = bf_at(xr[ks], j);
                    ss = fmaf(v, v, ss);
                }
            ss += __shfl_xor(ss, 32);
            rstd = 1.0f / sqrtf(ss / (float)DH + eps_);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const f32x4 w0 = *reinterpret_cast<const f32x4*>(sW + (2 * ks + g) * 8);
                const f32x4 w1 = *reinterpret_cast<const f32x4*>(sW + (2 * ks + g) * 8 + 4);
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    y[ks][j] = (bf16_t)((bf_at(xr[ks], j) * rstd) * (j < 4 ? w0[j & 3] : w1[j & 3]));
            }
        } else {
            rstd = 1.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) y[ks] = __builtin_bit_cast(bf16x8, xr[ks]);
        }
    }
    __device__ __forceinline__ void gate(const unsigned char* sA, int lane, int g, int E)
    {
        f32x16 acc[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[nt][i] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const unsigned char* a = sA + ((nt * KS + ks) * 64 + lane) * 16;
                acc[nt] = mfma32(*reinterpret_cast<const bf16x8*>(a), y[ks], acc[nt]);
                acc[nt] = mfma32(*reinterpret_cast<const bf16x8*>(a + NT * KS * 1024), y[ks], acc[nt]);
            }
        sum = 0.0f;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int e = nt * 32 + 16 * (i >> 3) + 8 * g + (i & 7);
                s[nt][i] = e < E ? fast_sigmoid(acc[nt][i]) : 0.0f;
                sum += s[nt][i];
            }
        sum += __shfl_xor(sum, 32);
        inv = 1.0f / fmaxf(sum, 1e-20f);
    }
    float eps_;
};

// router operands | norm weight | per wave: a [32 tokens][E] float tile of R, so that the 32 x E block (contiguous in
// memory) leaves the wave as whole cache lines instead of one scattered dword per lane and expert
constexpr size_t gate_fwd_smem(int DH, int NT) { return (size_t)2 * NT * (DH / 16) * 1024 + DH * 4 + 4 * TILE_B; }

template <int DH, int NT, bool NORM>
__global__ __launch_bounds__(256) void mhffn_gate_fwd_kernel(GateArgs p)
{
    constexpr int KS = DH / 16;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    float* sW = reinterpret_cast<float*>(smem + 2 * NT * KS * 1024);
    const int lane = threadIdx.x & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    float* rtile = sW + DH + wave * (TILE_B / 4);
    const int h = blockIdx.y, b = blockIdx.z;

    stage_router_rows<DH, NT>(p.Wr + (long)h * DH * p.E, p.E, smem);
    if constexpr (NORM)
        for (int i = threadIdx.x; i < DH; i += blockDim.x) sW[i] = p.Wn[h * DH + i];
    __syncthreads();

    const int ntiles = (p.S + 31) / 32;
    const int tile0 = (blockIdx.x * 4 + wave) * p.tpw;
    const int tile1 = min(tile0 + p.tpw, ntiles);
    for (int tile = tile0; tile < tile1; ++tile) {
        const int t = tile * 32 + l32;
        const bool valid = t < p.S;
        const long row = (((long)b * p.S + (valid ? t : p.S - 1)) * p.H + h) * DH;
        GateTile<DH, NT, NORM> T;
        T.eps_ = p.eps;
        T.load(p.X + row, g);
        T.normalise(sW, g);
        if constexpr (NORM) {
            if (valid) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    *reinterpret_cast<bf16x8*>(p.Qn + row + (2 * ks + g) * 8) = T.y[ks];
            }
        }
        T.gate(smem, lane, g, p.E);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int e = nt * 32 + 16 * (i >> 3) + 8 * g + (i & 7);
                if (e < p.E) rtile[l32 * p.E + e] = T.s[nt][i] * T.inv;
            }
        float* rblock = p.R + (((long)b * p.H + h) * p.S + tile * 32) * p.E;
        const int lim = min(32, p.S - tile * 32) * p.E;
        for (int idx = lane; idx < lim; idx += 64) rblock[idx] = rtile[idx];
    }
}

// ---- backward -------------------------------------------------------------------------------------------------------
// LDS: router rows (hi, lo) | router columns | norm weight | per wave: y tile (8 KB) + dz tile (8 KB), both in the
// swizzled 32 x 256-byte tile layout of the main kernels so the transposing reads can be shared.
// One wave per SIMD (the register partial sums leave no room for a second), so the next tile's rows are requested
// before the current tile's arithmetic starts; a wave takes enough consecutive tiles that the launch is one wave per
// SIMD of the chip where the problem allows, which also bounds the number of atomic adds per element.
// The per-wave region doubles as the staging area of the end-of-kernel reductions over the four waves: one expert
// tile of d_router partials ((d_h/32) x 16 x 64 floats <= 16 KB) or a 64 x 65 float transpose of the d_norm_weight
// partials; a [4][128] float array for the latter's cross-wave sums follows the regions.
constexpr int GATE_WAVE_REGION_B = 2 * TILE_B + 1024;
constexpr size_t gate_bwd_smem(int DH, int NT)
{
    return (size_t)2 * NT * (DH / 16) * 1024 + (size_t)(DH / 32) * 2 * NT * 1024 + DH * 4 + 4 * GATE_WAVE_REGION_B +
           4 * 128 * 4;
}

// Transposed operand (column tile ct, k-half s) of a swizzled tile.  Only column tile 0's two lane offsets are kept in
// registers: the swizzle XORs the chunk index, and a column tile is 4 chunks = 64 bytes, so tile ct's offset is tile
// 0's with bits 6..7 XORed by ct (one VALU instruction per read instead of two more registers per column tile).
__device__ __forceinline__ bf16x8 tile_cols(const unsigned char* tile, const TrLane<1>& tl, int ct, int s)
{
    typedef __attribute__((address_space(3))) v4bf16_t* lds_v4;
    const v4bf16_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_v4)(tile + (tl.off[0][0] ^ (ct << 6)) + 4096 * s));
    const v4bf16_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_v4)(tile + (tl.off[0][1] ^ (ct << 6)) + 4096 * s));
    bf16x8 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        r[j] = lo[j];
        r[4 + j] = hi[j];
    }
    return r;
}

template <int DH, int NT, bool NORM>
__global__ __launch_bounds__(256) void mhffn_gate_bwd_kernel(GateArgs p)
{
    constexpr int KS = DH / 16, CT = DH / 32;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char* sA = smem;                                   // logits operands
    unsigned char* sC = sA + 2 * NT * KS * 1024;                // dy operands
    float* sW = reinterpret_cast<float*>(sC + CT * 2 * NT * 1024);
    const int lane = threadIdx.x & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform: tile counters and tile bases stay scalar
    unsigned char* regions = reinterpret_cast<unsigned char*>(sW + DH);
    unsigned char* ytile = regions + wave * GATE_WAVE_REGION_B;
    unsigned char* ztile = ytile + TILE_B;
    const int h = blockIdx.y, b = blockIdx.z;

    stage_router_rows<DH, NT>(p.Wr + (long)h * DH * p.E, p.E, sA);
    stage_router_cols<DH, NT>(p.Wr + (long)h * DH * p.E, p.E, sC);
    if constexpr (NORM)
        for (int i = threadIdx.x; i < DH; i += blockDim.x) sW[i] = p.Wn[h * DH + i];
    // the dz tile's chunks beyond the experts in use are read by nobody, but columns e >= E inside a used chunk are:
    // they are written as zeros every tile, so nothing needs clearing here
    __syncthreads();

    const TrLane<1> trl = make_tr_lane<1, 8, 4>(lane);
    const TokRows dqrows = tok_rows(p.dq_tokmaj, b, h, p.H, p.S);
    f32x16 wacc[CT][NT];            // d_router partial: rows = columns of y, cols = experts
    float dwacc[KS][8];             // d_norm_weight partial for the lane's own columns
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 16; ++i) wacc[ct][nt][i] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int j = 0; j < 8; ++j) dwacc[ks][j] = 0.0f;

    const int ntiles = (p.S + 31) / 32;
    const int tile0 = (blockIdx.x * 4 + wave) * p.tpw;
    const int tile1 = min(tile0 + p.tpw, ntiles);
    // rows of the tile after the current one, requested one iteration ahead
    u32x4 nx[KS], ndq[KS];
    float ngr[NT * 16];
    auto request = [&](int tile) {
        const int t = tile * 32 + l32;
        const bool valid = t < p.S;
        const int tc = valid ? t : p.S - 1;
        const bf16_t* xrow = p.X + (((long)b * p.S + tc) * p.H + h) * DH;
        const bf16_t* dqrow = p.dQ + (dqrows.base + (long)tc * dqrows.stride) * DH;
        const float* dblock = p.dR + (((long)b * p.H + h) * p.S + tile * 32) * p.E;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            nx[ks] = *reinterpret_cast<const u32x4*>(xrow + (2 * ks + g) * 8);
            ndq[ks] = *reinterpret_cast<const u32x4*>(dqrow + (2 * ks + g) * 8);
        }
        // the tile's [32][E] block of dR is contiguous: dword k*64 + lane of it, zero past the last token
        const int lim = min(32, p.S - tile * 32) * p.E;
#pragma unroll
        for (int k = 0; k < NT * 16; ++k) ngr[k] = k * 64 + lane < lim ? dblock[k * 64 + lane] : 0.0f;
    };
    if (tile0 < tile1) request(tile0);
    for (int tile = tile0; tile < tile1; ++tile) {
        const int t = tile * 32 + l32;
        const bool valid = t < p.S;
        const long row = (((long)b * p.S + (valid ? t : p.S - 1)) * p.H + h) * DH;
        GateTile<DH, NT, NORM> T;
        T.eps_ = p.eps;
        u32x4 dqr[KS];
        float gr[NT][16];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            T.xr[ks] = nx[ks];
            dqr[ks] = ndq[ks];
        }
        // dR goes lane-major -> token-major through the (currently idle) dz tile
        {
            float* rt = reinterpret_cast<float*>(ztile);
#pragma unroll
            for (int k = 0; k < NT * 16; ++k) rt[k * 64 + lane] = ngr[k];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int e = nt * 32 + 16 * (i >> 3) + 8 * g + (i & 7);
                    gr[nt][i] = e < p.E ? rt[l32 * p.E + e] : 0.0f;
                }
        }
        if (tile + 1 < tile1) request(tile + 1);
        T.normalise(sW, g);
        if (!valid) {   // rows past the end contribute nothing to the sums over tokens
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) T.y[ks] = __builtin_bit_cast(bf16x8, u32x4{0u, 0u, 0u, 0u});
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            *reinterpret_cast<bf16x8*>(ytile + l32 * TILE_ROW_B + (((2 * ks + g) ^ swz16(l32)) << 4)) = T.y[ks];
        T.gate(sA, lane, g, p.E);

        // R = s * inv; d s = (dR - [sum >= 1e-20] sum_e dR R) * inv; d z = d s * s (1 - s)
        float dot = 0.0f;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 16; ++i) dot = fmaf(gr[nt][i], T.s[nt][i] * T.inv, dot);
        dot += __shfl_xor(dot, 32);
        if (T.sum < 1e-20f) dot = 0.0f;
        bf16x8 dzb[NT][2];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float sv = T.s[nt][i];
                dzb[nt][i >> 3][i & 7] = (bf16_t)((gr[nt][i] - dot) * T.inv * (sv * (1.0f - sv)));
            }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int s = 0; s < 2; ++s)
                *reinterpret_cast<bf16x8*>(ztile + l32 * TILE_ROW_B + (((4 * nt + 2 * s + g) ^ swz16(l32)) << 4)) =
                    dzb[nt][s];

        // dy^T = router dz^T, then the RMSNorm backward on the lane's own half row
        f32x16 dy[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
#pragma unroll
            for (int i = 0; i < 16; ++i) dy[ct][i] = 0.0f;
#pragma unroll
            for (int q = 0; q < 2 * NT; ++q)
                dy[ct] = mfma32(*reinterpret_cast<const bf16x8*>(sC + ((ct * 2 * NT + q) * 64 + lane) * 16),
                                dzb[q >> 1][q & 1], dy[ct]);
        }
        float du[KS][8];
        float cpart = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            [[maybe_unused]] f32x4 w0, w1;
            if constexpr (NORM) {
                w0 = *reinterpret_cast<const f32x4*>(sW + (2 * ks + g) * 8);
                w1 = *reinterpret_cast<const f32x4*>(sW + (2 * ks + g) * 8 + 4);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float d = dy[ks >> 1][8 * (ks & 1) + j] + bf_at(dqr[ks], j);
                if constexpr (NORM) {
                    const float u = bf_at(T.xr[ks], j) * T.rstd;
                    if (valid) dwacc[ks][j] = fmaf(d, u, dwacc[ks][j]);
                    d *= (j < 4 ? w0[j & 3] : w1[j & 3]);
                    cpart = fmaf(d, u, cpart);
                }
                du[ks][j] = d;
            }
        }
        if constexpr (NORM) {
            cpart += __shfl_xor(cpart, 32);
            const float c = cpart / (float)DH;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    du[ks][j] = T.rstd * (du[ks][j] - bf_at(T.xr[ks], j) * T.rstd * c);
        }
        if (valid) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                bf16x8 o;
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = (bf16_t)du[ks][j];
                *reinterpret_cast<bf16x8*>(p.dX + row + (2 * ks + g) * 8) = o;
            }
        }

        // d_router += y^T dz over this tile's tokens
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            bf16x8 bz[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) bz[nt] = tile_cols(ztile, trl, nt, s);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const bf16x8 ay = tile_cols(ytile, trl, ct, s);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) wacc[ct][nt] = mfma32(ay, bz[nt], wacc[ct][nt]);
            }
        }
    }

    // ---- sums over tokens: the four waves' partials meet in LDS, then one atomic add per workgroup and element ------
    __syncthreads();   // every wave is past its last tile: the per-wave regions are free
    float* mine = reinterpret_cast<float*>(regions + wave * GATE_WAVE_REGION_B);
    float* dWr = p.dWr + (long)h * DH * p.E;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int i = 0; i < 16; ++i) mine[(ct * 16 + i) * 64 + lane] = wacc[ct][nt][i];
        __syncthreads();
        for (int idx = threadIdx.x; idx < CT * 16 * 64; idx += 256) {
            float v = 0.0f;
#pragma unroll
            for (int w = 0; w < 4; ++w) v += reinterpret_cast<const float*>(regions + w * GATE_WAVE_REGION_B)[idx];
            const int ln = idx & 63, i = (idx >> 6) & 15, ct = idx >> 10;
            const int e = nt * 32 + (ln & 31), col = ct * 32 + 8 * (i >> 2) + 4 * (ln >> 5) + (i & 3);
            if (e < p.E) unsafeAtomicAdd(dWr + (long)col * p.E + e, v);
        }
        __syncthreads();
    }
    if constexpr (NORM) {
        // transpose inside the wave: value v = 8 ks + j of every lane goes to row v (row stride 65 floats keeps both the
        // writes and the row-wise reads conflict-free), then lane v adds up each lane half of its row
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int j = 0; j < 8; ++j) mine[(ks * 8 + j) * 65 + lane] = dwacc[ks][j];
        float* cross = reinterpret_cast<float*>(regions + 4 * GATE_WAVE_REGION_B);   // [4 waves][128 columns]
        if (lane < KS * 8) {
            float s0 = 0.0f, s1 = 0.0f;
            for (int i = 0; i < 32; ++i) {
                s0 += mine[lane * 65 + i];
                s1 += mine[lane * 65 + 32 + i];
            }
            const int ks = lane >> 3, j = lane & 7;
            cross[wave * 128 + (2 * ks) * 8 + j] = s0;
            cross[wave * 128 + (2 * ks + 1) * 8 + j] = s1;
        }
        __syncthreads();
        if (threadIdx.x < DH)
            unsafeAtomicAdd(p.dWn + h * DH + threadIdx.x, cross[threadIdx.x] + cross[128 + threadIdx.x] +
                                                              cross[256 + threadIdx.x] + cross[384 + threadIdx.x]);
    }
}

// ---- launch ---------------------------------------------------------------------------------------------------------
namespace {

int tiles_per_wave(const GateArgs& a, bool backward)
{
    const long total = (long)a.B * a.H * ((a.S + 31) / 32);
    // forward: several waves per SIMD hide the latency, so a wave only takes several tiles once there are at least 8 waves
    // per SIMD; backward: one wave per SIMD with its own prefetch, as few waves (= atomic adds) as fill the chip once
    const long tpw = backward ? total / 1024 : total / 8192;
    const long cap = backward ? 64 : 16;
    return (int)(tpw < 1 ? 1 : tpw > cap ? cap : tpw);
}

template <int DH, int NT, bool NORM>
hipError_t launch_gate(GateArgs a, bool backward, hipStream_t st)
{
    static LdsOptIn optin_fwd, optin_bwd;
    a.tpw = tiles_per_wave(a, backward);
    const int ntiles = (a.S + 31) / 32;
    const dim3 grid((ntiles + 4 * a.tpw - 1) / (4 * a.tpw), a.H, a.B);
    if (backward) {
        const size_t smem = gate_bwd_smem(DH, NT);
        const hipError_t e = ensure_dynamic_lds(optin_bwd, (const void*)mhffn_gate_bwd_kernel<DH, NT, NORM>, (int)smem);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL((mhffn_gate_bwd_kernel<DH, NT, NORM>), grid, dim3(256), smem, st, a);
    } else {
        const size_t smem = gate_fwd_smem(DH, NT);
        const hipError_t e = ensure_dynamic_lds(optin_fwd, (const void*)mhffn_gate_fwd_kernel<DH, NT, NORM>, (int)smem);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL((mhffn_gate_fwd_kernel<DH, NT, NORM>), grid, dim3(256), smem, st, a);
    }
    return hipGetLastError();
}

template <int DH>
hipError_t launch_gate_dh(const GateArgs& a, bool backward, hipStream_t st)
{
    const bool norm = a.Wn != nullptr;
    if (a.E <= 32) return norm ? launch_gate<DH, 1, true>(a, backward, st) : launch_gate<DH, 1, false>(a, backward, st);
    return norm ? launch_gate<DH, 2, true>(a, backward, st) : launch_gate<DH, 2, false>(a, backward, st);
}

hipError_t launch_gate_any(const GateArgs& a, int d_h, bool backward, hipStream_t st)
{
    switch (d_h) {
        case 64: return launch_gate_dh<64>(a, backward, st);
        case 96: return launch_gate_dh<96>(a, backward, st);
        case 128: return launch_gate_dh<128>(a, backward, st);
    }
    return hipErrorInvalidValue;
}

}  // namespace

hipError_t launch_gate_fwd(const void* X, const float* Wn, float eps, const float* Wr, void* Qn, float* R, const Dims& d,
                           hipStream_t st)
{
    GateArgs a{};
    a.X = (const bf16_t*)X;
    a.Wn = Wn;
    a.Wr = Wr;
    a.Qn = (bf16_t*)Qn;
    a.R = R;
    a.B = d.B, a.H = d.H, a.S = d.S, a.E = d.E, a.eps = eps;
    return launch_gate_any(a, d.d_h, false, st);
}

hipError_t launch_gate_bwd(const void* X, const float* Wn, float eps, const float* Wr, const void* dQ, int dq_tokmaj,
                           const float* dR, void* dX, float* dWn, float* dWr, const Dims& d, hipStream_t st)
{
    GateArgs a{};
    a.X = (const bf16_t*)X;
    a.Wn = Wn;
    a.Wr = Wr;
    a.dQ = (const bf16_t*)dQ;
    a.dR = dR;
    a.dX = (bf16_t*)dX;
    a.dWn = dWn;
    a.dWr = dWr;
    a.dq_tokmaj = dq_tokmaj;
    a.B = d.B, a.H = d.H, a.S = d.S, a.E = d.E, a.eps = eps;
    return launch_gate_any(a, d.d_h, true, st);
}

}  // namespace mhffn
