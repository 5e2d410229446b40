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
    const bf16_t* K;
    const bf16_t* U;
    const bf16_t* V;
    const float* R;
    bf16_t* dQ;
    float* dR;
    int H, G, S, E, nbe;
};

constexpr int DQ_NST = 4;                  // LDS stages (K | U | V tiles each)
constexpr int DQ_STAGE_B = 3 * TILE_B;

template <int DH, int NCT>
__global__ __launch_bounds__(256) void mhffn_bwd_dqdr_kernel(DqArgs p)
{
    constexpr int KS = DH / 16, CT = DH / 32;
    constexpr int BT = 128 * NCT;
    constexpr int FILL = 6;                // tile-fill wave-instructions per wave and block (3 tiles x 8 / 4 waves)
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    float* sR = reinterpret_cast<float*>(smem + DQ_NST * DQ_STAGE_B);   // [E][BT]

    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = blockIdx.x, tb = blockIdx.y, b = blockIdx.z;
    const int hk = h / p.G;
    const long rowbase = ((long)b * p.H + h) * p.S;
    const int tok0 = tb * BT + wave * (32 * NCT);
    const int nblk = p.E * p.nbe;
    const bf16_t* Kh = p.K + (long)hk * nblk * JB * DH;
    const long offU = p.U - p.K, offV = p.V - p.K;

    auto issue_block = [&](int blk) {
        const int bc = blk < nblk ? blk : nblk - 1;
        unsigned char* st = smem + (blk % DQ_NST) * DQ_STAGE_B;
        const long roff = (long)bc * JB * DH;
#pragma unroll
        for (int k = 0; k < FILL; ++k) {
            const int id = wave + 4 * k;             // 0..23: tile id/8 (K, U, V), 4-row group id%8
            const int which = id >> 3;
            const long toff = which == 0 ? 0 : (which == 1 ? offU : offV);
            tile_fill_ins<DH>(Kh + toff + roff, DH, st + which * TILE_B, id & 7, lane);
        }
    };
    issue_block(0);
    issue_block(1);

    bf16x8 q[NCT][KS], go[NCT][KS];
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) {
        int t = tok0 + ct * 32 + l32;
        t = t < p.S ? t : p.S - 1;
        const bf16_t* qr = p.Q + (rowbase + t) * DH + 8 * g;
        const bf16_t* gr = p.dO + (rowbase + t) * DH + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            q[ct][ks] = *reinterpret_cast<const bf16x8*>(qr + ks * 16);
            go[ct][ks] = *reinterpret_cast<const bf16x8*>(gr + ks * 16);
        }
    }
    for (int idx = tid; idx < BT * p.E; idx += 256) {
        int t = tb * BT + idx / p.E;
        t = t < p.S ? t : p.S - 1;
        sR[(idx % p.E) * BT + idx / p.E] = p.R[(rowbase + t) * p.E + idx % p.E];
    }

    f32x16 dq[CT][NCT];
#pragma unroll
    for (int i = 0; i < CT; ++i)
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
            for (int x = 0; x < 16; ++x) dq[i][ct][x] = 0.0f;

    const int krow = row_perm32(l32);
    int blk = 0;
    for (int e = 0; e < p.E; ++e) {
        float dr[NCT];
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) dr[ct] = 0.0f;
        for (int jb = 0; jb < p.nbe; ++jb, ++blk) {
            wait_vmcnt<FILL>();       // block blk has landed (block blk+1 may be in flight)
            __syncthreads();
            issue_block(blk + 2);

            const unsigned char* sK = smem + (blk % DQ_NST) * DQ_STAGE_B;
            const unsigned char* sU = sK + TILE_B;
            const unsigned char* sV = sU + TILE_B;
            float r[NCT];
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) r[ct] = sR[e * BT + wave * (32 * NCT) + ct * 32 + l32];

            f32x16 m[NCT], n[NCT], da[NCT];
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                for (int x = 0; x < 16; ++x) { m[ct][x] = 0.0f; n[ct][x] = 0.0f; da[ct][x] = 0.0f; }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const bf16x8 ak = tile_read_rows(sK, krow, ks, g);
                const bf16x8 au = tile_read_rows(sU, krow, ks, g);
                const bf16x8 av = tile_read_rows(sV, krow, ks, g);
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
                        const float w = __builtin_fmaf(sl, 1.0f - sg, sg);    // silu'(m)
                        dnt[ct][s][kk] = (bf16_t)(r[ct] * as);
                        dmt[ct][s][kk] = (bf16_t)((r[ct] * a) * (nn * w));
                    }

#pragma unroll
            for (int i = 0; i < CT; ++i)
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const bf16x8 akt = tile_read_cols(sK, i, 16 * s + 8 * g, 16 * s + 8 * g + 4, lane);
                    const bf16x8 aut = tile_read_cols(sU, i, 16 * s + 8 * g, 16 * s + 8 * g + 4, lane);
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
    wait_vmcnt<0>();   // drain the phantom prefetches before the workgroup's LDS is released

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

constexpr int DW_RTILE_B = 16 * 1024;                 // staged R tile: [E][32] fp32, E <= 128
constexpr int DW_STAGE_B = 2 * TILE_B + DW_RTILE_B;    // Q tile | dO tile | R tile

template <int DH>
__global__ __launch_bounds__(256) void mhffn_bwd_dkdudv_kernel(DwArgs p)
{
    constexpr int KS = DH / 16, CT = DH / 32;
    constexpr int NCHUNK = DH / 8;                    // 16-byte chunks per token row
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];

    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hk = blockIdx.y, z = blockIdx.z;
    const int nblk = p.E * p.nbe;
    const int jblk = blockIdx.x * 4 + wave;
    const bool active = jblk < nblk;
    const int jb_c = active ? jblk : nblk - 1;        // idle waves of the last column recompute the last block
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

    // Tile cursor of the prefetcher: tile index -> (q-head of the group, batch, 32-token tile), advanced incrementally.
    int pf_st = t_begin % nS, pf_bb = (t_begin / nS) % p.B, pf_gi = t_begin / (nS * p.B);

    // per-lane constants of the tile fill: this wave's two 4-row groups, swizzled source chunk
    int fill_row[2], fill_coff[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int ins = wave + 4 * k;
        const int r = 4 * ins + (lane >> 4);
        int c = (lane & 15) ^ swz16(r);
        c = c < NCHUNK ? c : 0;                       // unused chunk positions of narrow rows load a dummy chunk
        fill_row[k] = r;
        fill_coff[k] = c * 8;
    }

    // Asynchronous fill of stage `sidx` with the tile under the cursor; every wave issues its share of LDS-direct
    // loads (no staging registers), then the cursor advances.  Rows past the end of a sequence are clamped to its last
    // row and their gate value is zeroed afterwards (zero_tail), which removes them from all three products.
    auto issue_tile = [&](int sidx) {
        const long rb = ((long)pf_bb * p.H + hk * p.G + pf_gi) * p.S;
        const int t0 = pf_st * 32;
        unsigned char* sbase = smem_raw + sidx * DW_STAGE_B;
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            int t = t0 + fill_row[k];
            t = t < p.S ? t : p.S - 1;
            const long off = (rb + t) * DH + fill_coff[k];
            const int ins = wave + 4 * k;
            __builtin_amdgcn_global_load_lds((gptr_t)(p.Q + off), (lptr_t)(sbase + ins * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((gptr_t)(p.dO + off), (lptr_t)(sbase + TILE_B + ins * 1024), 16, 0, 0);
        }
        // R tile: [E][32] fp32, one 4-byte element per lane, two experts per instruction.
        for (int ins = wave; 2 * ins < p.E; ins += 4) {
            int e = 2 * ins + (lane >> 5);
            e = e < p.E ? e : p.E - 1;
            int t = t0 + l32;
            t = t < p.S ? t : p.S - 1;
            __builtin_amdgcn_global_load_lds((gptr_t)(p.R + (rb + t) * p.E + e),
                                             (lptr_t)(sbase + 2 * TILE_B + ins * 256), 4, 0, 0);
        }
        if (++pf_st == nS) {
            pf_st = 0;
            if (++pf_bb == p.B) { pf_bb = 0; ++pf_gi; }
        }
    };
    // Called by every wave after its own loads of stage `sidx` have landed and before the barrier that publishes
    // the stage: zeroes the gate values of the rows a tail tile does not have.
    auto zero_tail = [&](int sidx, int nvalid) {
        float* sR = reinterpret_cast<float*>(smem_raw + sidx * DW_STAGE_B + 2 * TILE_B);
        for (int ins = wave; 2 * ins < p.E; ins += 4)
            if (l32 >= nvalid) sR[ins * 64 + lane] = 0.0f;
    };

    int cur_st = pf_st;                                // 32-token tile index (within its sequence) of tile `tau`
    if (t_begin < t_end) issue_tile(0);

    const int fr = swz16(l32);
    f32x16 zero16;
#pragma unroll
    for (int x = 0; x < 16; ++x) zero16[x] = 0.0f;

    auto process = [&](auto stage_c, int tau) {
        constexpr int cur = decltype(stage_c)::value;
        wait_vmcnt<0>();                      // this wave's share of stage `cur` has landed
        const int nvalid = p.S - cur_st * 32;
        if (nvalid < 32) zero_tail(cur, nvalid);
        if (++cur_st == nS) cur_st = 0;
        __syncthreads();                      // ... and everybody's; all waves are done reading the other stage
        if (tau + 1 < t_end) issue_tile(cur ^ 1);

        const unsigned char* sQ = smem_raw + cur * DW_STAGE_B;
        const unsigned char* sG = sQ + TILE_B;
        const float* sR = reinterpret_cast<const float*>(sG + TILE_B) + e_w * 32;

        f32x16 m, n, da;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int off = l32 * 256 + (((2 * ks + g) ^ fr) << 4);
            const bf16x8 aq = *reinterpret_cast<const bf16x8*>(sQ + off);
            const bf16x8 ag = *reinterpret_cast<const bf16x8*>(sG + off);
            m = mfma32(aq, kB[ks], ks == 0 ? zero16 : m);
            n = mfma32(aq, uB[ks], ks == 0 ? zero16 : n);
            da = mfma32(ag, vB[ks], ks == 0 ? zero16 : da);
        }

        // registers 4a+b of m/n/da are token 8a + 4g + b (rows), column j = l32.
        bf16x8 pB[2], dmB[2], dnB[2];
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const f32x4 rv = *reinterpret_cast<const f32x4*>(sR + 8 * a + 4 * g);
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) {
                const int i = 4 * a + bb;
                const float x = m[i], nn = n[i], dA = da[i], rr = rv[bb];
                const float sg = fast_sigmoid(x);
                const float sl = x * sg;                               // silu(m)
                const float w = __builtin_fmaf(sl, 1.0f - sg, sg);     // silu'(m)
                const float rs = rr * sl;
                pB[i >> 3][i & 7] = (bf16_t)(rs * nn);
                dnB[i >> 3][i & 7] = (bf16_t)(rs * dA);
                dmB[i >> 3][i & 7] = (bf16_t)((rr * w) * (nn * dA));
            }
        }

        // token contraction: A = Q^T / dO^T gathered from the row-major tiles with transposing LDS reads.
        // k-slot (s, g, kk) of the B operands is token 16s + 8(kk/4) + 4g + kk%4; a 16-lane group covers 16 columns c.
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const bf16x8 aqt = tile_read_cols(sQ, ct, 16 * s + 4 * g, 16 * s + 4 * g + 8, lane);
                const bf16x8 agt = tile_read_cols(sG, ct, 16 * s + 4 * g, 16 * s + 4 * g + 8, lane);
                dk[ct] = mfma32(aqt, dmB[s], dk[ct]);
                du[ct] = mfma32(aqt, dnB[s], du[ct]);
                dv[ct] = mfma32(agt, pB[s], dv[ct]);
            }
    };

    // two tiles per trip so that the LDS stage (and every LDS address) is a compile-time constant
    int tau = t_begin;
    for (; tau + 1 < t_end; tau += 2) {
        process(std::integral_constant<int, 0>{}, tau);
        process(std::integral_constant<int, 1>{}, tau + 1);
    }
    if (tau < t_end) process(std::integral_constant<int, 0>{}, tau);

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
    return align256((size_t)pick_nslice(d) * 3 * wsz * sizeof(float));
}

template <int DH>
static hipError_t launch_bwd_t(const void* Q, const void* K, const void* U, const void* V, const float* R,
                               const void* dO, void* dQ, void* dK, void* dU, void* dV, float* dR, int grad_w_f32,
                               void* ws, const Dims& d, hipStream_t st, int phases)
{
    constexpr int NCT = 2;
    hipError_t err = hipSuccess;
    float* part = reinterpret_cast<float*>(ws);
    const int nbe = d.d_e / JB, G = d.H / d.Hkuv;

    if (phases & 2) {
        DqArgs a{(const bf16_t*)Q, (const bf16_t*)dO, (const bf16_t*)K, (const bf16_t*)U, (const bf16_t*)V, R,
                 (bf16_t*)dQ, dR, d.H, G, d.S, d.E, nbe};
        const int tokw = 128 * NCT;
        const int smem = DQ_NST * DQ_STAGE_B + d.E * tokw * (int)sizeof(float);
        if (smem > 160 * 1024) return hipErrorInvalidValue;
        static int attr_smem = 0;   // dynamic LDS above 64 KB must be opted into, per kernel
        if (smem > attr_smem) {
            err = hipFuncSetAttribute((const void*)mhffn_bwd_dqdr_kernel<DH, NCT>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, smem);
            if (err != hipSuccess) return err;
            attr_smem = smem;
        }
        dim3 grid((unsigned)d.H, (unsigned)((d.S + tokw - 1) / tokw), (unsigned)d.B);
        hipLaunchKernelGGL((mhffn_bwd_dqdr_kernel<DH, NCT>), grid, dim3(256), smem, st, a);
        err = hipGetLastError();
        if (err != hipSuccess) return err;
    }
    const int nslice = pick_nslice(d);
    if (phases & 4) {
        DwArgs a{(const bf16_t*)Q, (const bf16_t*)dO, (const bf16_t*)K, (const bf16_t*)U, (const bf16_t*)V, R, part,
                 d.B, d.H, G, d.S, d.E, nbe, nslice};
        const int smem = 2 * DW_STAGE_B;
        if (d.E > 128) return hipErrorInvalidValue;   // staged R tile holds at most 128 experts
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
