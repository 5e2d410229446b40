// Fused multi-head FFN backward for gfx950 (bf16 MFMA, fp32 accumulation), two kernels:
//
//  (1) dQ/dR kernel -- same tiling as the forward: a workgroup owns 4 * 32*NCT tokens of one (batch, q-head) and
//      streams the packed stage images (Kn | Un | Vn | Kt | Ut) through LDS.  Per 32-row block and wave:
//          M^T = Kn Q^T, N^T = Un Q^T, dA^T = Vn dO^T         (recomputed, registers only)
//          dR_e += sum_j dA * silu(M) * N                      (fp32, before any rounding)
//          dN^T = r_e dA^T silu(M^T),  dM^T = r_e dA^T N^T silu'(M^T)      (rounded once to bf16)
//          dQ^T += Kt dM^T + Ut dN^T
//      Formulas: kernels/triton/flash_mlp_moe.py:401-414, :527-542.
//
//  (2) dK/dU/dV kernel -- a wave owns one 32-row block of K/U/V (held in registers as MFMA B operands) and loops
//      over token tiles of 32 staged in LDS by its workgroup; dK^T, dU^T, dV^T (d_h x 32, fp32) stay in registers
//      for the whole token loop.  Products are written [t, j] here (M = Q K^T) so that the recomputed tile is the
//      B operand of the token contraction; the A operands Q^T / dO^T come from the natural LDS tiles through
//      ds_read_b64_tr_b16.  Token slices (grid.z) write fp32 partials that a small epilogue sums and converts.
//      Formulas: kernels/triton/flash_mlp_moe.py:683-729.
#include "mhffn_common.hpp"

namespace mhffn {

// ------------------------------------------------------------------------------------------------ dQ / dR
struct DqArgs {
    const bf16_t* Q;
    const bf16_t* dO;
    const bf16_t* W;   // packed stage images [Hkuv][E * d_e/32][DQ_STAGE]
    const float* R;
    bf16_t* dQ;
    float* dR;
    int H, G, S, E, nbe;
};

template <int DH, int NCT>
__global__ __launch_bounds__(256) void mhffn_bwd_dqdr_kernel(DqArgs p)
{
    using Ge = Geo<DH>;
    constexpr int KS = DH / 16, CT = DH / 32;
    constexpr int STAGE = Ge::DQ_STAGE;
    constexpr int CHUNKS = STAGE / 8;
    constexpr int NCH = (CHUNKS + 255) / 256;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    bf16_t* lds = reinterpret_cast<bf16_t*>(smem_raw);

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int h = blockIdx.x, tb = blockIdx.y, b = blockIdx.z;
    const int hk = h / p.G;
    const long rowbase = ((long)b * p.H + h) * p.S;
    const int tok0 = tb * (128 * NCT) + wave * (32 * NCT);
    const int nblk = p.E * p.nbe;
    const bf16_t* img = p.W + (long)hk * nblk * STAGE;

    bf16x8 q[NCT][KS], go[NCT][KS];
    long trow[NCT];
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) {
        int t = tok0 + ct * 32 + l32;
        t = t < p.S ? t : p.S - 1;
        trow[ct] = rowbase + t;
        const bf16_t* qr = p.Q + trow[ct] * DH + 8 * g;
        const bf16_t* gr = p.dO + trow[ct] * DH + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            q[ct][ks] = *reinterpret_cast<const bf16x8*>(qr + ks * 16);
            go[ct][ks] = *reinterpret_cast<const bf16x8*>(gr + ks * 16);
        }
    }

    f32x16 dq[CT][NCT];
#pragma unroll
    for (int i = 0; i < CT; ++i)
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
            for (int x = 0; x < 16; ++x) dq[i][ct][x] = 0.0f;

    u32x4 stg[NCH];
    auto gload = [&](int blk) {
        const u32x4* src = reinterpret_cast<const u32x4*>(img + (long)blk * STAGE);
        static_for<NCH>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            const int idx = tid + i * 256;
            if (i * 256 + 255 < CHUNKS || idx < CHUNKS) stg[i] = src[idx];
        });
    };
    auto lstore = [&](int st) {
        u32x4* dst = reinterpret_cast<u32x4*>(lds + st * STAGE);
        static_for<NCH>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            const int idx = tid + i * 256;
            if (i * 256 + 255 < CHUNKS || idx < CHUNKS) dst[idx] = stg[i];
        });
    };

    gload(0);
    lstore(0);
    if (nblk > 1) gload(1);

    int blk = 0;
    for (int e = 0; e < p.E; ++e) {
        float r[NCT], dr[NCT];
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) {
            r[ct] = p.R[trow[ct] * p.E + e];
            dr[ct] = 0.0f;
        }
        for (int jb = 0; jb < p.nbe; ++jb, ++blk) {
            __syncthreads();
            if (blk + 1 < nblk) lstore((blk + 1) & 1);
            if (blk + 2 < nblk) gload(blk + 2);

            const bf16_t* sK = lds + (blk & 1) * STAGE;
            const bf16_t* sU = sK + Ge::NAT_ELEMS;
            const bf16_t* sV = sU + Ge::NAT_ELEMS;
            const bf16_t* sKt = sV + Ge::NAT_ELEMS;
            const bf16_t* sUt = sKt + Ge::TR_ELEMS;

            f32x16 m[NCT], n[NCT], da[NCT];
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                for (int x = 0; x < 16; ++x) { m[ct][x] = 0.0f; n[ct][x] = 0.0f; da[ct][x] = 0.0f; }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int off = l32 * Ge::NAT_LD + ks * 16 + 8 * g;
                const bf16x8 ak = *reinterpret_cast<const bf16x8*>(sK + off);
                const bf16x8 au = *reinterpret_cast<const bf16x8*>(sU + off);
                const bf16x8 av = *reinterpret_cast<const bf16x8*>(sV + off);
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct) {
                    m[ct] = mfma32(ak, q[ct][ks], m[ct]);
                    n[ct] = mfma32(au, q[ct][ks], n[ct]);
                    da[ct] = mfma32(av, go[ct][ks], da[ct]);
                }
            }

            bf16x8 dmt[NCT][2], dnt[NCT][2];
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                for (int s = 0; s < 2; ++s)
#pragma unroll
                    for (int kk = 0; kk < 8; ++kk) {
                        const int i = 8 * s + kk;
                        const float x = m[ct][i], nn = n[ct][i], a = da[ct][i];
                        const float sg = fast_sigmoid(x);
                        const float sl = x * sg;                 // silu(m)
                        const float as = a * sl;
                        dr[ct] = __builtin_fmaf(as, nn, dr[ct]);
                        const float w = sg + sl * (1.0f - sg);    // silu'(m)
                        dnt[ct][s][kk] = (bf16_t)(r[ct] * as);
                        dmt[ct][s][kk] = (bf16_t)((r[ct] * a) * (nn * w));
                    }

#pragma unroll
            for (int i = 0; i < CT; ++i)
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const int off = (i * 32 + l32) * Ge::TR_LD + 16 * s + 8 * g;
                    const bf16x8 akt = *reinterpret_cast<const bf16x8*>(sKt + off);
                    const bf16x8 aut = *reinterpret_cast<const bf16x8*>(sUt + off);
#pragma unroll
                    for (int ct = 0; ct < NCT; ++ct) {
                        dq[i][ct] = mfma32(akt, dmt[ct][s], dq[i][ct]);
                        dq[i][ct] = mfma32(aut, dnt[ct][s], dq[i][ct]);
                    }
                }
        }
        // dR[t, e]: the two lane halves hold disjoint j rows of the same token column.
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) {
            const float tot = dr[ct] + __shfl_xor(dr[ct], 32);
            const int t = tok0 + ct * 32 + l32;
            if (g == 0 && t < p.S) p.dR[(rowbase + t) * p.E + e] = tot;
        }
    }

#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) {
        const int t = tok0 + ct * 32 + l32;
        if (t < p.S) {
            bf16_t* orow = p.dQ + (rowbase + t) * DH;
#pragma unroll
            for (int i = 0; i < CT; ++i)
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    bf16x4 v;
#pragma unroll
                    for (int x = 0; x < 4; ++x) v[x] = (bf16_t)dq[i][ct][4 * a + x];
                    *reinterpret_cast<bf16x4*>(orow + 32 * i + 8 * a + 4 * g) = v;
                }
        }
    }
}

// ------------------------------------------------------------------------------------------------ dK / dU / dV
struct DwArgs {
    const bf16_t* Q;
    const bf16_t* dO;
    const bf16_t* K;
    const bf16_t* U;
    const bf16_t* V;
    const float* R;
    float* part;        // [nslice][3][Hkuv][E*d_e][DH] fp32 partial sums
    int B, H, G, S, E, nbe, nslice;
};

__device__ __forceinline__ bf16x8 lds_read_tr8(const bf16_t* p0, const bf16_t* p1)
{
    // Each call returns, for this lane's column, 4 + 4 consecutive rows of a row-major LDS tile (see the kernel).
    typedef __attribute__((address_space(3))) v4bf16_t* lds_v4_ptr;
    v4bf16_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_v4_ptr)(p0));
    v4bf16_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_v4_ptr)(p1));
    bf16x8 r;
    r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
    r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
    return r;
}

template <int DH>
__global__ __launch_bounds__(256) void mhffn_bwd_dkdudv_kernel(DwArgs p)
{
    constexpr int KS = DH / 16, CT = DH / 32;
    constexpr int NCHUNK = DH / 8;                    // 16-byte chunks per token row
        extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
    const int e_pad = (p.E + 1) & ~1;
    const int stage_bytes = 2 * TILE_B + e_pad * 128;  // Q tile | dO tile | R tile [E][32] fp32

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int hk = blockIdx.y, z = blockIdx.z;
    const int nblk = p.E * p.nbe;
    const int jblk = blockIdx.x * 4 + wave;
    const bool active = jblk < nblk;
    const int jb_c = active ? jblk : nblk - 1;
    const int e_w = jb_c / p.nbe;
    const long wrow = ((long)hk * nblk + jb_c) * JB + l32;      // this lane's row of K/U/V (column j of the products)

    bf16x8 kB[KS], uB[KS], vB[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        kB[ks] = *reinterpret_cast<const bf16x8*>(p.K + wrow * DH + ks * 16 + 8 * g);
        uB[ks] = *reinterpret_cast<const bf16x8*>(p.U + wrow * DH + ks * 16 + 8 * g);
        vB[ks] = *reinterpret_cast<const bf16x8*>(p.V + wrow * DH + ks * 16 + 8 * g);
    }

    f32x16 dk[CT], du[CT], dv[CT];
#pragma unroll
    for (int i = 0; i < CT; ++i)
#pragma unroll
        for (int x = 0; x < 16; ++x) { dk[i][x] = 0.0f; du[i][x] = 0.0f; dv[i][x] = 0.0f; }

    const int nS = (p.S + 31) / 32;
    const int ntile = p.G * p.B * nS;
    const int t_begin = (int)((long)ntile * z / p.nslice), t_end = (int)((long)ntile * (z + 1) / p.nslice);

    // Asynchronous fill of one stage: every wave issues its share of LDS-direct loads (no staging registers).
    auto issue_tile = [&](int tau, int sidx) {
        const int st = tau % nS;
        const int bb = (tau / nS) % p.B;
        const int gi = tau / (nS * p.B);
        const long rb = ((long)bb * p.H + hk * p.G + gi) * p.S;
        unsigned char* sbase = smem_raw + sidx * stage_bytes;
        // Q and dO: 8 wave-instructions each (4 rows of 256 B per instruction); wave w takes instructions w and w+4.
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const int ins = wave + 4 * k;
            const int r = 4 * ins + (lane >> 4);
            int c = (lane & 15) ^ swz16(r);
            c = c < NCHUNK ? c : 0;                   // unused chunk positions of narrow rows load a dummy chunk
            int t = st * 32 + r;
            t = t < p.S ? t : p.S - 1;                // tail rows are neutralised by r = 0 below
            const long off = (rb + t) * DH + c * 8;
            __builtin_amdgcn_global_load_lds((gptr_t)(p.Q + off), (lptr_t)(sbase + ins * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((gptr_t)(p.dO + off), (lptr_t)(sbase + TILE_B + ins * 1024), 16, 0, 0);
        }
        // R tile: [E][32] fp32, one 4-byte element per lane, two experts per instruction.
        for (int ins = wave; 2 * ins < p.E; ins += 4) {
            int e = 2 * ins + (lane >> 5);
            e = e < p.E ? e : p.E - 1;
            int t = st * 32 + l32;
            t = t < p.S ? t : p.S - 1;
            __builtin_amdgcn_global_load_lds((gptr_t)(p.R + (rb + t) * p.E + e),
                                             (lptr_t)(sbase + 2 * TILE_B + ins * 256), 4, 0, 0);
        }
    };

    if (t_begin < t_end) issue_tile(t_begin, 0);

    const int lam = lane & 15;
    for (int tau = t_begin; tau < t_end; ++tau) {
        const int cur = (tau - t_begin) & 1;
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wave's share of stage `cur` has landed
        __syncthreads();                      // ... and everybody's; all waves are done reading the other stage
        if (tau + 1 < t_end) issue_tile(tau + 1, cur ^ 1);
        // waves beyond the last block recompute block nblk-1 (straight-line code) and drop their result at the end

        const unsigned char* sQ = smem_raw + cur * stage_bytes;
        const unsigned char* sG = sQ + TILE_B;
        const float* sR = reinterpret_cast<const float*>(sG + TILE_B) + e_w * 32;

        f32x16 m, n, da;
#pragma unroll
        for (int x = 0; x < 16; ++x) { m[x] = 0.0f; n[x] = 0.0f; da[x] = 0.0f; }
        const int fr = swz16(l32);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int off = l32 * 256 + (((2 * ks + g) ^ fr) << 4);
            const bf16x8 aq = *reinterpret_cast<const bf16x8*>(sQ + off);
            const bf16x8 ag = *reinterpret_cast<const bf16x8*>(sG + off);
            m = mfma32(aq, kB[ks], m);
            n = mfma32(aq, uB[ks], n);
            da = mfma32(ag, vB[ks], da);
        }

        // registers 4a+b of m/n/da are token 8a + 4g + b (rows), column j = l32.
        const int nvalid = p.S - (tau % nS) * 32;     // tokens of this tile that exist (>= 32 except in a tail tile)
        bf16x8 pB[2], dmB[2], dnB[2];
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            f32x4 rv = *reinterpret_cast<const f32x4*>(sR + 8 * a + 4 * g);
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) rv[bb] = (8 * a + 4 * g + bb < nvalid) ? rv[bb] : 0.0f;
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) {
                const int i = 4 * a + bb;
                const float x = m[i], nn = n[i], dA = da[i], rr = rv[bb];
                const float sg = fast_sigmoid(x);
                const float sl = x * sg;
                const float w = sg + sl * (1.0f - sg);
                const float ra = rr * dA;
                pB[i >> 3][i & 7] = (bf16_t)(rr * (sl * nn));
                dnB[i >> 3][i & 7] = (bf16_t)(ra * sl);
                dmB[i >> 3][i & 7] = (bf16_t)(ra * (nn * w));
            }
            __builtin_amdgcn_sched_barrier(0);   // bound the number of element chains in flight (register pressure)
        }

        // token contraction: A = Q^T / dO^T gathered from the row-major tiles with transposing LDS reads.
        // k-slot (s, g, kk) of the B operands is token 16s + 8(kk/4) + 4g + kk%4; a 16-lane group covers 16 columns c.
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const int row0 = 16 * s + 4 * g + (lam >> 2);
                const int chunk = 4 * ct + 2 * (l32 >> 4) + ((lam & 3) >> 1);
                const int o0 = row0 * 256 + ((chunk ^ swz16(row0)) << 4) + (lam & 1) * 8;
                const int o1 = (row0 + 8) * 256 + ((chunk ^ swz16(row0 + 8)) << 4) + (lam & 1) * 8;
                const bf16x8 aqt = lds_read_tr8(reinterpret_cast<const bf16_t*>(sQ + o0),
                                                reinterpret_cast<const bf16_t*>(sQ + o1));
                const bf16x8 agt = lds_read_tr8(reinterpret_cast<const bf16_t*>(sG + o0),
                                                reinterpret_cast<const bf16_t*>(sG + o1));
                dk[ct] = mfma32(aqt, dmB[s], dk[ct]);
                du[ct] = mfma32(aqt, dnB[s], du[ct]);
                dv[ct] = mfma32(agt, pB[s], dv[ct]);
            }
    }

    if (active) {
        // dK^T registers 4a+b of row tile ct: c = 32ct + 8a + 4g + b, column j = l32 -> 16-byte runs along c.
        const long wsz = (long)gridDim.y * nblk * JB * DH;   // elements of one weight tensor
        float* base = p.part + (long)z * 3 * wsz + wrow * DH;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const int c = 32 * ct + 8 * a + 4 * g;
                f32x4 v0, v1, v2;
#pragma unroll
                for (int x = 0; x < 4; ++x) { v0[x] = dk[ct][4 * a + x]; v1[x] = du[ct][4 * a + x]; v2[x] = dv[ct][4 * a + x]; }
                *reinterpret_cast<f32x4*>(base + c) = v0;
                *reinterpret_cast<f32x4*>(base + wsz + c) = v1;
                *reinterpret_cast<f32x4*>(base + 2 * wsz + c) = v2;
            }
    }
}

// Sums the token-slice partials and converts to the output dtype.  HBM-bound: reads nslice*3*|W| fp32 once.
template <typename OutT>
__global__ __launch_bounds__(256) void reduce_partials_kernel(const float* __restrict__ part, OutT* dK, OutT* dU, OutT* dV,
                                                              long wsz, int nslice)
{
    const long i4 = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i4 >= wsz) return;
    OutT* outs[3] = {dK, dU, dV};
#pragma unroll
    for (int w = 0; w < 3; ++w) {
        f32x4 acc = *reinterpret_cast<const f32x4*>(part + w * wsz + i4);
        for (int z = 1; z < nslice; ++z) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(part + ((long)z * 3 + w) * wsz + i4);
            acc += v;
        }
#pragma unroll
        for (int x = 0; x < 4; ++x) outs[w][i4 + x] = (OutT)acc[x];
    }
}

// ------------------------------------------------------------------------------------------------ host side
static int pick_nslice(const Dims& d)
{
    // Enough workgroups for ~2 per CU (256 CUs), but at least 8 token tiles per slice.
    const int nblk = d.E * (d.d_e / JB);
    const long cols = (long)((nblk + 3) / 4) * d.Hkuv;
    const long ntile = (long)(d.H / d.Hkuv) * d.B * ((d.S + 31) / 32);
    long ns = (512 + cols - 1) / cols;
    if (ns > ntile / 8) ns = ntile / 8;
    if (ns < 1) ns = 1;
    if (ns > 64) ns = 64;
    return (int)ns;
}

static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

size_t bwd_workspace_bytes_bf16(const Dims& d)
{
    const size_t wsz = (size_t)d.Hkuv * d.E * d.d_e * d.d_h;
    return align256(packed_weights_bytes(d, 1)) + align256((size_t)pick_nslice(d) * 3 * wsz * sizeof(float));
}

template <int DH>
static hipError_t launch_bwd_t(const void* Q, const void* K, const void* U, const void* V, const float* R,
                               const void* dO, void* dQ, void* dK, void* dU, void* dV, float* dR, int grad_w_f32,
                               void* ws, const Dims& d, hipStream_t st, int phases)
{
    constexpr int NCT = 2;
    hipError_t err = hipSuccess;
    if (phases & 1) {
        err = launch_pack_weights(K, U, V, ws, 1, d, st);
        if (err != hipSuccess) return err;
    }
    float* part = reinterpret_cast<float*>((char*)ws + align256(packed_weights_bytes(d, 1)));
    const int nbe = d.d_e / JB, G = d.H / d.Hkuv;

    if (phases & 2) {
        DqArgs a{(const bf16_t*)Q, (const bf16_t*)dO, (const bf16_t*)ws, R, (bf16_t*)dQ, dR, d.H, G, d.S, d.E, nbe};
        constexpr int smem = 2 * Geo<DH>::DQ_STAGE * (int)sizeof(bf16_t);
        static bool attr_done = false;   // raising the dynamic LDS limit is a per-process, per-kernel property
        if (!attr_done) {
            err = hipFuncSetAttribute((const void*)mhffn_bwd_dqdr_kernel<DH, NCT>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, smem);
            if (err != hipSuccess) return err;
            attr_done = true;
        }
        const int tokw = 128 * NCT;
        dim3 grid((unsigned)d.H, (unsigned)((d.S + tokw - 1) / tokw), (unsigned)d.B);
        hipLaunchKernelGGL((mhffn_bwd_dqdr_kernel<DH, NCT>), grid, dim3(256), smem, st, a);
        err = hipGetLastError();
        if (err != hipSuccess) return err;
    }
    const int nslice = pick_nslice(d);
    if (phases & 4) {
        DwArgs a{(const bf16_t*)Q, (const bf16_t*)dO, (const bf16_t*)K, (const bf16_t*)U, (const bf16_t*)V, R, part,
                 d.B, d.H, G, d.S, d.E, nbe, nslice};
        const int smem = 2 * (2 * JB * 256 + ((d.E + 1) & ~1) * 128);
        if (smem > 64 * 1024) return hipErrorInvalidValue;
        const int nblk = d.E * nbe;
        dim3 grid((unsigned)((nblk + 3) / 4), (unsigned)d.Hkuv, (unsigned)nslice);
        hipLaunchKernelGGL((mhffn_bwd_dkdudv_kernel<DH>), grid, dim3(256), smem, st, a);
        err = hipGetLastError();
        if (err != hipSuccess) return err;
    }
    if (phases & 8) {
        const long wsz = (long)d.Hkuv * d.E * d.d_e * d.d_h;
        const unsigned rblocks = (unsigned)((wsz / 4 + 255) / 256);
        if (grad_w_f32)
            hipLaunchKernelGGL((reduce_partials_kernel<float>), dim3(rblocks), dim3(256), 0, st, part, (float*)dK,
                               (float*)dU, (float*)dV, wsz, nslice);
        else
            hipLaunchKernelGGL((reduce_partials_kernel<bf16_t>), dim3(rblocks), dim3(256), 0, st, part, (bf16_t*)dK,
                               (bf16_t*)dU, (bf16_t*)dV, wsz, nslice);
        err = hipGetLastError();
    }
    return err;
}

hipError_t launch_bwd_bf16(const void* Q, const void* K, const void* U, const void* V, const float* R, const void* dO,
                           void* dQ, void* dK, void* dU, void* dV, float* dR, int grad_w_f32, void* ws, const Dims& d,
                           hipStream_t st, int phases)
{
    switch (d.d_h) {
        case 64: return launch_bwd_t<64>(Q, K, U, V, R, dO, dQ, dK, dU, dV, dR, grad_w_f32, ws, d, st, phases);
        case 96: return launch_bwd_t<96>(Q, K, U, V, R, dO, dQ, dK, dU, dV, dR, grad_w_f32, ws, d, st, phases);
        case 128: return launch_bwd_t<128>(Q, K, U, V, R, dO, dQ, dK, dU, dV, dR, grad_w_f32, ws, d, st, phases);
    }
    return hipErrorInvalidValue;
}

}  // namespace mhffn
