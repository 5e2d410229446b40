// Fused multi-head FFN forward for gfx950 (bf16 MFMA, fp32 accumulation).
//
// One workgroup (4 waves, one per SIMD) owns 128*NCT tokens of one (batch, q-head); wave w owns NCT column tiles of 32
// tokens.  The workgroup streams the K, U, V blocks (32 rows of the E*d_e axis at a time) straight from the weight
// tensors into a ring of LDS stages with asynchronous LDS-direct loads.  Per block and wave:
//     M^T = K Q^T, N^T = U Q^T               (A = rows of the K/U tiles, B = Q^T held in registers for the whole kernel)
//     P^T = silu(M^T) * N^T * r_e             (fp32 in the accumulator registers, rounded once to bf16)
//     O^T += V^T P^T                          (A = columns of the V tile via transposing LDS reads, B = P^T registers)
// so the [tokens, E*d_e] intermediate lives only in registers.  The loop is software-pipelined: the first products of
// block i+1 are issued together with the element-wise work of block i, so the MFMA pipe and the VALU overlap inside
// the single wave each SIMD runs.  Reference semantics: kernels/triton/flash_mlp_moe.py:243-266.
#include "mhffn_common.hpp"

namespace mhffn {

struct FwdArgs {
    const bf16_t* Q;
    const bf16_t* K;
    const bf16_t* U;
    const bf16_t* V;
    const float* R;
    bf16_t* O;
    int H, G, S, E, nbe;  // G = H / Hkuv, nbe = d_e / 32 blocks per expert
};

constexpr int FWD_NST = 4;                 // LDS stages (K | U | V tiles each)
constexpr int FWD_STAGE_B = 3 * TILE_B;    // 24 KB
#ifndef FWD_SKEW
#define FWD_SKEW 0   // 1: the upper half of the workgroup runs half a block behind the lower half
#endif

template <int DH, int NCT, int NW, bool PIPE>
__global__ __launch_bounds__(NW * 64) void mhffn_fwd_kernel(FwdArgs p)
{
    constexpr int KS = DH / 16;   // k-steps of the first products
    constexpr int CT = DH / 32;   // row tiles of O^T
    constexpr int BT = NW * 32 * NCT; // tokens per workgroup
    constexpr int NTHR = NW * 64;
    constexpr int FILL = 24 / NW;    // tile-fill wave-instructions per wave and block (3 tiles x 8 / NW)
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    float* sR = reinterpret_cast<float*>(smem + FWD_NST * FWD_STAGE_B);   // [E][BT]

    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: keeps tile bookkeeping on the scalar unit
    const int h = blockIdx.x, tb = blockIdx.y, b = blockIdx.z;
    const int hk = h / p.G;
    const long rowbase = ((long)b * p.H + h) * p.S;
    const int tok0 = tb * BT + wave * (32 * NCT);
    const int nblk = p.E * p.nbe;
    const long wbase = (long)hk * nblk * JB * DH;   // first element of this kuv-head's rows
    const bf16_t* Kh = p.K + wbase;
    const long offU = p.U - p.K, offV = p.V - p.K;   // U and V addressed relative to K (flat address space)

    // Asynchronous fill of one stage with block `blk` (clamped: phantom blocks past the end reload the last one).
    // 24 wave-instructions (3 tiles x 8), 6 per wave: the vmcnt bookkeeping below relies on that constant.
    auto issue_block = [&](int blk) {
        const int bc = blk < nblk ? blk : nblk - 1;
        unsigned char* st = smem + (blk % FWD_NST) * FWD_STAGE_B;
        const long roff = (long)bc * JB * DH;
#pragma unroll
        for (int k = 0; k < FILL; ++k) {
            const int id = wave + NW * k;            // 0..23: tile id/8 (K, U, V), 4-row group id%8
            const int which = id >> 3;
            const long toff = which == 0 ? 0 : (which == 1 ? offU : offV);   // integer select: no pointer table
            tile_fill_ins<DH>(Kh + toff + roff, DH, st + which * TILE_B, id & 7, lane);
        }
    };

    issue_block(0);
    issue_block(1);
    if constexpr (PIPE) issue_block(2);

    // Q^T B operands: lane holds token column l32 of each column tile, 8 consecutive c per k-step.
    bf16x8 q[NCT][KS];
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) {
        int t = tok0 + ct * 32 + l32;
        t = t < p.S ? t : p.S - 1;   // tail tokens read the last valid row; their stores are masked
        const bf16_t* qr = p.Q + (rowbase + t) * DH + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) q[ct][ks] = *reinterpret_cast<const bf16x8*>(qr + ks * 16);
    }
    // gate values of this workgroup's tokens, [E][BT] in LDS: the main loop then has no global loads of its own
    for (int idx = tid; idx < BT * p.E; idx += NTHR) {
        int t = tb * BT + idx / p.E;
        t = t < p.S ? t : p.S - 1;
        sR[(idx % p.E) * BT + idx / p.E] = p.R[(rowbase + t) * p.E + idx % p.E];
    }

    f32x16 oacc[CT][NCT];
#pragma unroll
    for (int i = 0; i < CT; ++i)
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
            for (int x = 0; x < 16; ++x) oacc[i][ct][x] = 0.0f;

    const int krow = row_perm32(l32);   // K/U row fed as MFMA A-row l32 (see mhffn_common.hpp)
    const TrLane<CT> trl = make_tr_lane<CT, 8, 4>(lane);

    auto gemm1 = [&](const unsigned char* st, f32x16 (&m)[NCT], f32x16 (&n)[NCT]) {
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
            for (int x = 0; x < 16; ++x) { m[ct][x] = 0.0f; n[ct][x] = 0.0f; }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const bf16x8 ak = tile_read_rows(st, krow, ks, g);
            const bf16x8 au = tile_read_rows(st + TILE_B, krow, ks, g);
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) {
                m[ct] = mfma32(ak, q[ct][ks], m[ct]);
                n[ct] = mfma32(au, q[ct][ks], n[ct]);
            }
        }
    };

    // One pipeline step: consumes M/N of block `blk` (mc, nc), produces M/N of block blk+1 (mn, nn).
    auto step = [&](int blk, int e, f32x16 (&mc)[NCT], f32x16 (&nc)[NCT], f32x16 (&mn)[NCT], f32x16 (&nn)[NCT]) {
        wait_vmcnt<FILL>();   // blocks <= blk+1 have landed (only block blk+2's loads may be in flight)
        __syncthreads();      // ... for every wave; and every wave is done with the stage about to be refilled
        issue_block(blk + 3);

        float r[NCT];
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct)
            r[ct] = blk < nblk ? sR[(e < p.E ? e : p.E - 1) * BT + wave * (32 * NCT) + ct * 32 + l32] : 0.0f;

        const unsigned char* st_next = smem + ((blk + 1) % FWD_NST) * FWD_STAGE_B;
        const unsigned char* st_cur = smem + (blk % FWD_NST) * FWD_STAGE_B;
        gemm1(st_next, mn, nn);

        bf16x8 pt[NCT][2];
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
            for (int s = 0; s < 2; ++s)
#pragma unroll
                for (int kk = 0; kk < 8; ++kk) {
                    const float x = mc[ct][8 * s + kk];
                    const float val = (x * nc[ct][8 * s + kk]) * (r[ct] * fast_sigmoid(x));
                    pt[ct][s][kk] = (bf16_t)val;
                }

#pragma unroll
        for (int i = 0; i < CT; ++i)
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                TrOperand avo = s == 0 ? tile_read_cols_async<0>(lds_addr(st_cur + 2 * TILE_B), trl, i)
                                       : tile_read_cols_async<4096>(lds_addr(st_cur + 2 * TILE_B), trl, i);
                lds_tr_wait(avo);
                const bf16x8 av = tr_value(avo);
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct) oacc[i][ct] = mfma32(av, pt[ct][s], oacc[i][ct]);
            }
    };

    if constexpr (!PIPE) {
        // Two waves per SIMD (waves w and w+4 share one).  Every wave runs, per block: first products (MFMA), element-wise
        // (VALU), second product (MFMA).  The one barrier per block would keep all waves in the same phase, so the upper
        // half of the workgroup runs half a block behind -- it finishes block b-1 (element-wise + second product) before
        // its first products of block b -- and each SIMD always has one wave feeding the MFMA pipe while the other one
        // is on the VALU.
        // Each phase first issues all of its LDS operand reads (their latency is covered by the other wave of the
        // SIMD), then its MFMAs; sched_barrier keeps the compiler from sinking the reads back next to their uses.
        auto phase_g1 = [&](int blk, f32x16 (&m)[NCT], f32x16 (&n)[NCT]) {
            const unsigned char* st = smem + (blk % FWD_NST) * FWD_STAGE_B;
            bf16x8 ak[KS], au[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                ak[ks] = tile_read_rows(st, krow, ks, g);
                au[ks] = tile_read_rows(st + TILE_B, krow, ks, g);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                for (int x = 0; x < 16; ++x) { m[ct][x] = 0.0f; n[ct][x] = 0.0f; }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct) {
                    m[ct] = mfma32(ak[ks], q[ct][ks], m[ct]);
                    n[ct] = mfma32(au[ks], q[ct][ks], n[ct]);
                }
            __builtin_amdgcn_sched_barrier(0);
        };
        auto phase_ew_g2 = [&](int blk, int e, f32x16 (&m)[NCT], f32x16 (&n)[NCT]) {
            const unsigned char* sV = smem + (blk % FWD_NST) * FWD_STAGE_B + 2 * TILE_B;
            float r[NCT];
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) r[ct] = sR[e * BT + wave * (32 * NCT) + ct * 32 + l32];
            TrOperand av[CT][2];
#pragma unroll
            for (int i = 0; i < CT; ++i)
#pragma unroll
                for (int s = 0; s < 2; ++s)
                    av[i][s] = s == 0 ? tile_read_cols_async<0>(lds_addr(sV), trl, i)
                                      : tile_read_cols_async<4096>(lds_addr(sV), trl, i);
            __builtin_amdgcn_sched_barrier(0);
            bf16x8 pt[NCT][2];
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                for (int s = 0; s < 2; ++s)
#pragma unroll
                    for (int kk = 0; kk < 8; ++kk) {
                        const float x = m[ct][8 * s + kk];
                        pt[ct][s][kk] = (bf16_t)((x * n[ct][8 * s + kk]) * (r[ct] * fast_sigmoid(x)));
                    }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < CT; ++i) lds_tr_wait(av[i][0], av[i][1]);
#pragma unroll
            for (int i = 0; i < CT; ++i)
#pragma unroll
                for (int s = 0; s < 2; ++s)
#pragma unroll
                    for (int ct = 0; ct < NCT; ++ct) oacc[i][ct] = mfma32(tr_value(av[i][s]), pt[ct][s], oacc[i][ct]);
            __builtin_amdgcn_sched_barrier(0);
        };
        f32x16 m[NCT], n[NCT];
        int e = 0, jb = 0;
        if (!FWD_SKEW || wave < NW / 2) {
            for (int blk = 0; blk < nblk; ++blk) {
                wait_vmcnt<FILL>();       // block blk has landed (block blk+1 may be in flight)
                __syncthreads();
                issue_block(blk + 2);
                phase_g1(blk, m, n);
                phase_ew_g2(blk, e, m, n);
                if (++jb == p.nbe) { jb = 0; ++e; }
            }
        } else {
            for (int blk = 0; blk < nblk; ++blk) {
                wait_vmcnt<FILL>();
                __syncthreads();
                issue_block(blk + 2);
                if (blk > 0) {
                    phase_ew_g2(blk - 1, e, m, n);
                    if (++jb == p.nbe) { jb = 0; ++e; }
                }
                phase_g1(blk, m, n);
            }
            phase_ew_g2(nblk - 1, e, m, n);
        }
    } else {
    f32x16 mA[NCT], nA[NCT], mB[NCT], nB[NCT];
    wait_vmcnt<2 * FILL>();   // block 0 (and the Q / R loads before it) have landed
    __syncthreads();
    gemm1(smem, mA, nA);

    // Blocks are consumed in pairs so the two M/N register sets alternate without copies; an odd block count is
    // rounded up with a phantom block whose gate value is 0.
    int e = 0, jb = 0;
    for (int blk = 0; blk < nblk; blk += 2) {
        step(blk, e, mA, nA, mB, nB);
        if (++jb == p.nbe) { jb = 0; ++e; }
        step(blk + 1, e, mB, nB, mA, nA);
        if (++jb == p.nbe) { jb = 0; ++e; }
    }
    }
    wait_vmcnt<0>();      // drain the phantom prefetches before the workgroup's LDS is released

    // O^T registers -> O[t][c]: register 4a+b of row tile i is c = 32i + 8a + 4g + b, so each lane owns runs of 4 c.
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) {
        const int t = tok0 + ct * 32 + l32;
        if (t < p.S) {
            bf16_t* orow = p.O + (rowbase + t) * DH;
#pragma unroll
            for (int i = 0; i < CT; ++i)
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    bf16x4 v;
#pragma unroll
                    for (int x = 0; x < 4; ++x) v[x] = (bf16_t)oacc[i][ct][4 * a + x];
                    *reinterpret_cast<bf16x4*>(orow + 32 * i + 8 * a + 4 * g) = v;
                }
        }
    }
}

size_t fwd_workspace_bytes_bf16(const Dims&) { return 0; }

template <int DH, int NCT, int NW, bool PIPE>
static hipError_t launch_fwd_t(const FwdArgs& a, const Dims& d, hipStream_t st)
{
    const int tokw = NW * 32 * NCT;
    const int smem = FWD_NST * FWD_STAGE_B + d.E * tokw * (int)sizeof(float);
    if (smem > 160 * 1024) return hipErrorInvalidValue;
    static int attr_smem = 0;   // dynamic LDS above 64 KB must be opted into, per kernel
    if (smem > attr_smem) {
        hipError_t e = hipFuncSetAttribute((const void*)mhffn_fwd_kernel<DH, NCT, NW, PIPE>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return e;
        attr_smem = smem;
    }
    dim3 grid((unsigned)d.H, (unsigned)((d.S + tokw - 1) / tokw), (unsigned)d.B);   // head fastest: one head per XCD
    hipLaunchKernelGGL((mhffn_fwd_kernel<DH, NCT, NW, PIPE>), grid, dim3(NW * 64), smem, st, a);
    return hipGetLastError();
}

hipError_t launch_fwd_bf16(const void* Q, const void* K, const void* U, const void* V, const float* R, void* O,
                           void* ws, const Dims& d, hipStream_t st, int phases)
{
    (void)ws;
    if (!(phases & 2)) return hipSuccess;
    FwdArgs a{(const bf16_t*)Q, (const bf16_t*)K, (const bf16_t*)U, (const bf16_t*)V, R, (bf16_t*)O,
              d.H,              d.H / d.Hkuv,     d.S,              d.E,              d.d_e / JB};
    switch (d.d_h) {
#ifndef FWD_VARIANT
#define FWD_VARIANT 1, 8, false
#endif
        case 64: return launch_fwd_t<64, FWD_VARIANT>(a, d, st);
        case 96: return launch_fwd_t<96, FWD_VARIANT>(a, d, st);
        case 128: return launch_fwd_t<128, FWD_VARIANT>(a, d, st);
    }
    return hipErrorInvalidValue;
}

}  // namespace mhffn
