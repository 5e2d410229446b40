// fp32 instantiation of the fused multi-head FFN (forward, dQ/dR, dK/dU/dV): the correctness path for float32
// tensors.  Same fusion as the bf16 kernels -- the [tokens, E*d_e] intermediate only ever exists as a 32x32 tile in
// LDS -- but plain fp32 FMAs instead of MFMA and an exact sigmoid, so results track an fp32 eager evaluation to ~1e-6.
// Generic in d_h (multiple of 8, at most 128) and d_e (any); tiles are 32 tokens x 32 rows of K/U/V.
//
// Thread roles inside a 256-thread workgroup, per (32-token tile, 32-row chunk):
//   phase A  thread (t = tid / 8, jl = tid % 8) computes the products for rows j = jl + 8 i, i < 4
//   phase B  thread (row = tid / 8, cg = tid % 8) accumulates output columns c = cg + 8 i, i < d_h / 8
// Formulas: models/flashmhf/modeling_mhffnmoe.py:418-427 (forward), kernels/triton/flash_mlp_moe.py:401-414, 527-542,
// 720-729 (backward).
#include "mhffn_common.hpp"

namespace mhffn {

namespace {

constexpr int TT = 32;   // tokens per tile
constexpr int JC = 32;   // K/U/V rows per chunk
constexpr int MAXC = 16; // d_h / 8 at most

struct F32Args {
    const float *Q, *K, *U, *V, *R, *dO;
    float *O, *dQ, *dR, *part;
    int B, H, G, S, DH, E, DE, nslice;
    int tokmaj;   // Q, O, dO, dQ token-major ([B, S, H, d_h]) instead of [B, H, S, d_h]
};

__device__ __forceinline__ float sigmoid_exact(float x) { return 1.0f / (1.0f + __expf(-x)); }

// Loads a [rows x DH] fp32 tile (row stride `rs` rows of DH elements in global) into LDS with row stride DH + 1; rows >=
// valid are zeroed.
__device__ __forceinline__ void load_tile(float* dst, const float* src, int valid, int DH, int tid, int rs = 1)
{
    const int LD = DH + 1;
    for (int i = tid; i < 32 * DH; i += 256) {
        const int r = i / DH, c = i % DH;
        dst[r * LD + c] = r < valid ? src[(long)r * rs * DH + c] : 0.0f;
    }
}

__global__ __launch_bounds__(256) void fwd_f32_kernel(F32Args p)
{
    extern __shared__ float lds[];
    const int DH = p.DH, LD = DH + 1, NC = DH / 8;
    float* sQ = lds;
    float* sK = sQ + 32 * LD;
    float* sU = sK + 32 * LD;
    float* sV = sU + 32 * LD;
    float* sA = sV + 32 * LD;          // [TT][JC + 1]
    const int tid = threadIdx.x, t = tid >> 3, jl = tid & 7, cg = tid & 7;
    const int h = blockIdx.x, tb = blockIdx.y, b = blockIdx.z, hk = h / p.G;
    const long rowbase = ((long)b * p.H + h) * p.S + (long)tb * TT;   // rows of R
    const TokRows qr = tok_rows(p.tokmaj, b, h, p.H, p.S);
    const long qrow0 = qr.base + (long)tb * TT * qr.stride;           // rows of Q, O
    const int tvalid = min(TT, p.S - tb * TT);
    load_tile(sQ, p.Q + qrow0 * DH, tvalid, DH, tid, qr.stride);

    float acc[MAXC];
#pragma unroll
    for (int i = 0; i < MAXC; ++i) acc[i] = 0.0f;
    for (int e = 0; e < p.E; ++e) {
        const float r = t < tvalid ? p.R[(rowbase + t) * p.E + e] : 0.0f;
        for (int j0 = 0; j0 < p.DE; j0 += JC) {
            const long wrow = ((long)hk * p.E + e) * p.DE + j0;
            const int jvalid = min(JC, p.DE - j0);
            __syncthreads();
            load_tile(sK, p.K + wrow * DH, jvalid, DH, tid);
            load_tile(sU, p.U + wrow * DH, jvalid, DH, tid);
            load_tile(sV, p.V + wrow * DH, jvalid, DH, tid);
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = jl + 8 * i;
                float m = 0.0f, n = 0.0f;
                for (int c = 0; c < DH; ++c) {
                    const float q = sQ[t * LD + c];
                    m = fmaf(q, sK[j * LD + c], m);
                    n = fmaf(q, sU[j * LD + c], n);
                }
                sA[t * (JC + 1) + j] = m * sigmoid_exact(m) * n * r;
            }
            __syncthreads();
            for (int j = 0; j < JC; ++j) {
                const float a = sA[t * (JC + 1) + j];
#pragma unroll
                for (int i = 0; i < MAXC; ++i)
                    if (i < NC) acc[i] = fmaf(a, sV[j * LD + cg + 8 * i], acc[i]);
            }
        }
    }
    if (t < tvalid)
#pragma unroll
        for (int i = 0; i < MAXC; ++i)
            if (i < NC) p.O[(qrow0 + (long)t * qr.stride) * DH + cg + 8 * i] = acc[i];
}

__global__ __launch_bounds__(256) void dqdr_f32_kernel(F32Args p)
{
    extern __shared__ float lds[];
    const int DH = p.DH, LD = DH + 1, NC = DH / 8;
    float* sQ = lds;
    float* sG = sQ + 32 * LD;
    float* sK = sG + 32 * LD;
    float* sU = sK + 32 * LD;
    float* sV = sU + 32 * LD;
    float* sDM = sV + 32 * LD;          // [TT][JC + 1]
    float* sDN = sDM + TT * (JC + 1);
    float* sDR = sDN + TT * (JC + 1);   // [TT][8] per-thread partials of dR
    const int tid = threadIdx.x, t = tid >> 3, jl = tid & 7, cg = tid & 7;
    const int h = blockIdx.x, tb = blockIdx.y, b = blockIdx.z, hk = h / p.G;
    const long rowbase = ((long)b * p.H + h) * p.S + (long)tb * TT;   // rows of R, dR
    const TokRows qr = tok_rows(p.tokmaj, b, h, p.H, p.S);
    const long qrow0 = qr.base + (long)tb * TT * qr.stride;           // rows of Q, dO, dQ
    const int tvalid = min(TT, p.S - tb * TT);
    load_tile(sQ, p.Q + qrow0 * DH, tvalid, DH, tid, qr.stride);
    load_tile(sG, p.dO + qrow0 * DH, tvalid, DH, tid, qr.stride);

    float acc[MAXC];
#pragma unroll
    for (int i = 0; i < MAXC; ++i) acc[i] = 0.0f;
    for (int e = 0; e < p.E; ++e) {
        const float r = t < tvalid ? p.R[(rowbase + t) * p.E + e] : 0.0f;
        float dr = 0.0f;
        for (int j0 = 0; j0 < p.DE; j0 += JC) {
            const long wrow = ((long)hk * p.E + e) * p.DE + j0;
            const int jvalid = min(JC, p.DE - j0);
            __syncthreads();
            load_tile(sK, p.K + wrow * DH, jvalid, DH, tid);
            load_tile(sU, p.U + wrow * DH, jvalid, DH, tid);
            load_tile(sV, p.V + wrow * DH, jvalid, DH, tid);
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = jl + 8 * i;
                float m = 0.0f, n = 0.0f, da = 0.0f;
                for (int c = 0; c < DH; ++c) {
                    const float q = sQ[t * LD + c];
                    m = fmaf(q, sK[j * LD + c], m);
                    n = fmaf(q, sU[j * LD + c], n);
                    da = fmaf(sG[t * LD + c], sV[j * LD + c], da);
                }
                const float sg = sigmoid_exact(m), sl = m * sg;
                dr = fmaf(da * sl, n, dr);
                sDN[t * (JC + 1) + j] = r * da * sl;
                sDM[t * (JC + 1) + j] = r * da * n * (sg + sl * (1.0f - sg));
            }
            __syncthreads();
            for (int j = 0; j < JC; ++j) {
                const float dm = sDM[t * (JC + 1) + j], dn = sDN[t * (JC + 1) + j];
#pragma unroll
                for (int i = 0; i < MAXC; ++i)
                    if (i < NC) acc[i] = fmaf(dm, sK[j * LD + cg + 8 * i], fmaf(dn, sU[j * LD + cg + 8 * i], acc[i]));
            }
        }
        __syncthreads();
        sDR[t * 8 + jl] = dr;
        __syncthreads();
        if (jl == 0 && t < tvalid) {
            float s = 0.0f;
            for (int x = 0; x < 8; ++x) s += sDR[t * 8 + x];
            p.dR[(rowbase + t) * p.E + e] = s;
        }
    }
    if (t < tvalid)
#pragma unroll
        for (int i = 0; i < MAXC; ++i)
            if (i < NC) p.dQ[(qrow0 + (long)t * qr.stride) * DH + cg + 8 * i] = acc[i];
}

// One workgroup owns a 32-row chunk of K/U/V of one kuv-head and a slice of the token tiles; partial sums go to
// part[slice][3][Hkuv][E*d_e][d_h] (rows of a chunk beyond d_e are never written: chunks do not straddle experts).
__global__ __launch_bounds__(256) void dkdudv_f32_kernel(F32Args p)
{
    extern __shared__ float lds[];
    const int DH = p.DH, LD = DH + 1, NC = DH / 8;
    float* sQ = lds;
    float* sG = sQ + 32 * LD;
    float* sK = sG + 32 * LD;
    float* sU = sK + 32 * LD;
    float* sV = sU + 32 * LD;
    float* sDM = sV + 32 * LD;          // [TT][JC + 1]
    float* sDN = sDM + TT * (JC + 1);
    float* sP = sDN + TT * (JC + 1);
    const int tid = threadIdx.x, t = tid >> 3, jl = tid & 7, jr = tid >> 3, cg = tid & 7;
    const int nch = (p.DE + JC - 1) / JC;                 // chunks per expert
    const int e = blockIdx.x / nch, j0 = (blockIdx.x % nch) * JC;
    const int hk = blockIdx.y, z = blockIdx.z;
    const int jvalid = min(JC, p.DE - j0);
    const long wrow = ((long)hk * p.E + e) * p.DE + j0;
    load_tile(sK, p.K + wrow * DH, jvalid, DH, tid);
    load_tile(sU, p.U + wrow * DH, jvalid, DH, tid);
    load_tile(sV, p.V + wrow * DH, jvalid, DH, tid);

    float dk[MAXC], du[MAXC], dv[MAXC];
#pragma unroll
    for (int i = 0; i < MAXC; ++i) { dk[i] = 0.0f; du[i] = 0.0f; dv[i] = 0.0f; }
    const int nS = (p.S + TT - 1) / TT, ntile = p.G * p.B * nS;
    const int t_begin = (int)((long)ntile * z / p.nslice), t_end = (int)((long)ntile * (z + 1) / p.nslice);
    for (int tau = t_begin; tau < t_end; ++tau) {
        const int st = tau % nS, bb = (tau / nS) % p.B, gi = tau / (nS * p.B);
        const long rowbase = ((long)bb * p.H + hk * p.G + gi) * p.S + (long)st * TT;
        const int tvalid = min(TT, p.S - st * TT);
        __syncthreads();
        const TokRows qr = tok_rows(p.tokmaj, bb, hk * p.G + gi, p.H, p.S);
        const long qrow0 = qr.base + (long)st * TT * qr.stride;
        load_tile(sQ, p.Q + qrow0 * DH, tvalid, DH, tid, qr.stride);
        load_tile(sG, p.dO + qrow0 * DH, tvalid, DH, tid, qr.stride);
        __syncthreads();
        const float r = t < tvalid ? p.R[(rowbase + t) * p.E + e] : 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int j = jl + 8 * i;
            float m = 0.0f, n = 0.0f, da = 0.0f;
            for (int c = 0; c < DH; ++c) {
                const float q = sQ[t * LD + c];
                m = fmaf(q, sK[j * LD + c], m);
                n = fmaf(q, sU[j * LD + c], n);
                da = fmaf(sG[t * LD + c], sV[j * LD + c], da);
            }
            const float sg = sigmoid_exact(m), sl = m * sg;
            sP[t * (JC + 1) + j] = r * sl * n;
            sDN[t * (JC + 1) + j] = r * da * sl;
            sDM[t * (JC + 1) + j] = r * da * n * (sg + sl * (1.0f - sg));
        }
        __syncthreads();
        for (int tt = 0; tt < TT; ++tt) {
            const float dm = sDM[tt * (JC + 1) + jr], dn = sDN[tt * (JC + 1) + jr], pp = sP[tt * (JC + 1) + jr];
#pragma unroll
            for (int i = 0; i < MAXC; ++i)
                if (i < NC) {
                    const float q = sQ[tt * LD + cg + 8 * i], g = sG[tt * LD + cg + 8 * i];
                    dk[i] = fmaf(dm, q, dk[i]);
                    du[i] = fmaf(dn, q, du[i]);
                    dv[i] = fmaf(pp, g, dv[i]);
                }
        }
    }
    if (jr < jvalid) {
        const long wsz = (long)gridDim.y * p.E * p.DE * DH;
        float* base = p.part + (long)z * 3 * wsz + (wrow + jr) * DH;
#pragma unroll
        for (int i = 0; i < MAXC; ++i)
            if (i < NC) {
                base[cg + 8 * i] = dk[i];
                base[wsz + cg + 8 * i] = du[i];
                base[2 * wsz + cg + 8 * i] = dv[i];
            }
    }
}

template <typename OutT>
__global__ __launch_bounds__(256) void reduce_f32_kernel(const float* __restrict__ part, OutT* dK, OutT* dU, OutT* dV,
                                                         long wsz, int nslice)
{
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= wsz) return;
    OutT* outs[3] = {dK, dU, dV};
    for (int w = 0; w < 3; ++w) {
        float acc = 0.0f;
        for (int z = 0; z < nslice; ++z) acc += part[((long)z * 3 + w) * wsz + i];
        outs[w][i] = (OutT)acc;
    }
}

int f32_nslice(const Dims& d)
{
    const long cols = (long)d.E * ((d.d_e + JC - 1) / JC) * d.Hkuv;
    const long ntile = (long)(d.H / d.Hkuv) * d.B * ((d.S + TT - 1) / TT);
    long ns = (1024 + cols - 1) / cols;
    if (ns > ntile) ns = ntile;
    if (ns < 1) ns = 1;
    if (ns > 64) ns = 64;
    return (int)ns;
}

}  // namespace

size_t bwd_workspace_bytes_f32(const Dims& d)
{
    return (size_t)f32_nslice(d) * 3 * d.Hkuv * d.E * d.d_e * d.d_h * sizeof(float);
}

hipError_t launch_fwd_f32(const void* Q, const void* K, const void* U, const void* V, const float* R, void* O,
                          const Dims& d, hipStream_t st)
{
    F32Args a{};
    a.Q = (const float*)Q; a.K = (const float*)K; a.U = (const float*)U; a.V = (const float*)V; a.R = R;
    a.O = (float*)O;
    a.B = d.B; a.H = d.H; a.G = d.H / d.Hkuv; a.S = d.S; a.DH = d.d_h; a.E = d.E; a.DE = d.d_e; a.tokmaj = d.tokmaj;
    const int smem = (4 * 32 * (d.d_h + 1) + TT * (JC + 1)) * (int)sizeof(float);
    static LdsOptIn optin;
    const hipError_t e = ensure_dynamic_lds(optin, (const void*)fwd_f32_kernel, 128 * 1024);
    if (e != hipSuccess) return e;
    dim3 grid((unsigned)d.H, (unsigned)((d.S + TT - 1) / TT), (unsigned)d.B);
    hipLaunchKernelGGL(fwd_f32_kernel, grid, dim3(256), smem, st, a);
    return hipGetLastError();
}

hipError_t launch_bwd_f32(const void* Q, const void* K, const void* U, const void* V, const float* R, const void* dO,
                          void* dQ, void* dK, void* dU, void* dV, float* dR, int grad_w_f32, void* ws, const Dims& d,
                          hipStream_t st, int phases)
{
    F32Args a{};
    a.Q = (const float*)Q; a.K = (const float*)K; a.U = (const float*)U; a.V = (const float*)V; a.R = R;
    a.dO = (const float*)dO; a.dQ = (float*)dQ; a.dR = dR; a.part = (float*)ws;
    a.B = d.B; a.H = d.H; a.G = d.H / d.Hkuv; a.S = d.S; a.DH = d.d_h; a.E = d.E; a.DE = d.d_e; a.tokmaj = d.tokmaj;
    a.nslice = f32_nslice(d);
    static LdsOptIn optin_dq, optin_dw;
    hipError_t e = ensure_dynamic_lds(optin_dq, (const void*)dqdr_f32_kernel, 128 * 1024);
    if (e == hipSuccess) e = ensure_dynamic_lds(optin_dw, (const void*)dkdudv_f32_kernel, 128 * 1024);
    if (e != hipSuccess) return e;
    hipError_t err = hipSuccess;
    if (phases & PH_BWD_DQDR) {
        const int smem = (5 * 32 * (d.d_h + 1) + 2 * TT * (JC + 1) + TT * 8) * (int)sizeof(float);
        dim3 grid((unsigned)d.H, (unsigned)((d.S + TT - 1) / TT), (unsigned)d.B);
        hipLaunchKernelGGL(dqdr_f32_kernel, grid, dim3(256), smem, st, a);
        err = hipGetLastError();
        if (err != hipSuccess) return err;
    }
    if (phases & PH_BWD_DKDUDV) {
        const int smem = (5 * 32 * (d.d_h + 1) + 3 * TT * (JC + 1)) * (int)sizeof(float);
        dim3 grid((unsigned)(d.E * ((d.d_e + JC - 1) / JC)), (unsigned)d.Hkuv, (unsigned)a.nslice);
        hipLaunchKernelGGL(dkdudv_f32_kernel, grid, dim3(256), smem, st, a);
        err = hipGetLastError();
        if (err != hipSuccess) return err;
    }
    if (phases & PH_BWD_REDUCE) {
        const long wsz = (long)d.Hkuv * d.E * d.d_e * d.d_h;
        const unsigned rblocks = (unsigned)((wsz + 255) / 256);
        if (grad_w_f32)
            hipLaunchKernelGGL((reduce_f32_kernel<float>), dim3(rblocks), dim3(256), 0, st, a.part, (float*)dK, (float*)dU,
                               (float*)dV, wsz, a.nslice);
        else
            hipLaunchKernelGGL((reduce_f32_kernel<bf16_t>), dim3(rblocks), dim3(256), 0, st, a.part, (bf16_t*)dK,
                               (bf16_t*)dU, (bf16_t*)dV, wsz, a.nslice);
        err = hipGetLastError();
    }
    return err;
}

}  // namespace mhffn
