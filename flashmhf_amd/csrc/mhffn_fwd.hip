// Fused multi-head FFN forward for gfx950 (bf16 MFMA, fp32 accumulation).
//
// One workgroup (4 waves) owns TOKW*4 tokens of one (batch, q-head); wave w owns NCT column tiles of 32 tokens.
// The workgroup streams the packed weight stage images (Kn | Un | Vt, one per 32-row block of the E*d_e axis)
// through a double-buffered LDS ring.  Per block and wave:
//     M^T = Kn Q^T, N^T = Un Q^T            (A from LDS, B = Q^T held in registers for the whole kernel)
//     P^T = silu(M^T) * N^T * r_e            (fp32 in the accumulator registers, rounded once to bf16)
//     O^T += Vt P^T                          (A from LDS, B = P^T straight from registers)
// so the [tokens, E*d_e] intermediate lives only in registers.  Reference semantics: flash_mlp_moe.py:243-266.
#include "mhffn_common.hpp"

namespace mhffn {

struct FwdArgs {
    const bf16_t* Q;
    const bf16_t* W;   // packed stage images [Hkuv][E * d_e/32][FWD_STAGE]
    const float* R;
    bf16_t* O;
    int H, G, S, E, nbe;  // G = H / Hkuv, nbe = d_e / 32 blocks per expert
};

template <int DH, int NCT>
__global__ __launch_bounds__(256) void mhffn_fwd_kernel(FwdArgs p)
{
    using Ge = Geo<DH>;
    constexpr int KS = DH / 16;   // k-steps of the first products
    constexpr int CT = DH / 32;   // row tiles of O^T
    constexpr int STAGE = Ge::FWD_STAGE;
    constexpr int CHUNKS = STAGE / 8;                 // 16-byte chunks per stage
    constexpr int NCH = (CHUNKS + 255) / 256;         // chunks per thread
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    bf16_t* lds = reinterpret_cast<bf16_t*>(smem_raw);
    constexpr int BT = 128 * NCT;                      // tokens per workgroup
    float* sR = reinterpret_cast<float*>(smem_raw + 2 * STAGE * sizeof(bf16_t));   // [E][BT]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int h = blockIdx.x, tb = blockIdx.y, b = blockIdx.z;
    const int hk = h / p.G;
    const long rowbase = ((long)b * p.H + h) * p.S;
    const int tok0 = tb * (128 * NCT) + wave * (32 * NCT);
    const int nblk = p.E * p.nbe;
    const bf16_t* img = p.W + (long)hk * nblk * STAGE;

    // Q^T B operands: lane holds token column l32 of each column tile, 8 consecutive c per k-step.
    bf16x8 q[NCT][KS];
    long trow[NCT];
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) {
        int t = tok0 + ct * 32 + l32;
        t = t < p.S ? t : p.S - 1;   // tail tokens read the last valid row; their stores are masked
        trow[ct] = rowbase + t;
        const bf16_t* qr = p.Q + trow[ct] * DH + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) q[ct][ks] = *reinterpret_cast<const bf16x8*>(qr + ks * 16);
    }

    f32x16 oacc[CT][NCT];
#pragma unroll
    for (int i = 0; i < CT; ++i)
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
            for (int x = 0; x < 16; ++x) oacc[i][ct][x] = 0.0f;

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
    // gate values of this workgroup's tokens, [E][BT] in LDS (read once per expert; keeps the main loop free of
    // global loads other than the stage prefetch)
    for (int idx = tid; idx < BT * p.E; idx += 256) {
        int t = tb * BT + idx / p.E;
        t = t < p.S ? t : p.S - 1;
        sR[(idx % p.E) * BT + idx / p.E] = p.R[(rowbase + t) * p.E + idx % p.E];
    }
    lstore(0);
    __syncthreads();

    float r[NCT];
    int blk = 0;
    for (int e = 0; e < p.E; ++e) {
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) r[ct] = sR[e * BT + wave * (32 * NCT) + ct * 32 + l32];
        for (int jb = 0; jb < p.nbe; ++jb, ++blk) {
            if (blk + 1 < nblk) gload(blk + 1);

            const bf16_t* sK = lds + (blk & 1) * STAGE;
            const bf16_t* sU = sK + Ge::NAT_ELEMS;
            const bf16_t* sV = sU + Ge::NAT_ELEMS;

            f32x16 m[NCT], n[NCT];
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                for (int x = 0; x < 16; ++x) { m[ct][x] = 0.0f; n[ct][x] = 0.0f; }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const bf16x8 ak = *reinterpret_cast<const bf16x8*>(sK + l32 * Ge::NAT_LD + ks * 16 + 8 * g);
                const bf16x8 au = *reinterpret_cast<const bf16x8*>(sU + l32 * Ge::NAT_LD + ks * 16 + 8 * g);
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct) {
                    m[ct] = mfma32(ak, q[ct][ks], m[ct]);
                    n[ct] = mfma32(au, q[ct][ks], n[ct]);
                }
            }

            bf16x8 pt[NCT][2];
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                for (int s = 0; s < 2; ++s)
#pragma unroll
                    for (int kk = 0; kk < 8; ++kk) {
                        const float x = m[ct][8 * s + kk];
                        const float val = (x * n[ct][8 * s + kk]) * (r[ct] * fast_sigmoid(x));
                        pt[ct][s][kk] = (bf16_t)val;
                    }

#pragma unroll
            for (int i = 0; i < CT; ++i)
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const bf16x8 av =
                        *reinterpret_cast<const bf16x8*>(sV + (i * 32 + l32) * Ge::TR_LD + 16 * s + 8 * g);
#pragma unroll
                    for (int ct = 0; ct < NCT; ++ct) oacc[i][ct] = mfma32(av, pt[ct][s], oacc[i][ct]);
                }
            if (blk + 1 < nblk) lstore((blk + 1) & 1);   // the other stage: last read before the previous barrier
            __syncthreads();
        }
    }

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

size_t fwd_workspace_bytes_bf16(const Dims& d) { return packed_weights_bytes(d, 0); }

template <int DH, int NCT>
static hipError_t launch_fwd_t(const FwdArgs& a, const Dims& d, hipStream_t st)
{
    const int tokw = 128 * NCT;
    const int smem = 2 * Geo<DH>::FWD_STAGE * (int)sizeof(bf16_t) + d.E * tokw * (int)sizeof(float);
    if (smem > 160 * 1024) return hipErrorInvalidValue;
    static int attr_smem = 0;   // dynamic LDS above 64 KB must be opted into, per kernel
    if (smem > 64 * 1024 && smem > attr_smem) {
        hipError_t e = hipFuncSetAttribute((const void*)mhffn_fwd_kernel<DH, NCT>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return e;
        attr_smem = smem;
    }
    dim3 grid((unsigned)d.H, (unsigned)((d.S + tokw - 1) / tokw), (unsigned)d.B);   // head fastest: one head per XCD
    hipLaunchKernelGGL((mhffn_fwd_kernel<DH, NCT>), grid, dim3(256), smem, st, a);
    return hipGetLastError();
}

hipError_t launch_fwd_bf16(const void* Q, const void* K, const void* U, const void* V, const float* R, void* O,
                           void* ws, const Dims& d, hipStream_t st, int phases)
{
    if (phases & 1) {
        hipError_t err = launch_pack_weights(K, U, V, ws, 0, d, st);
        if (err != hipSuccess) return err;
    }
    if (!(phases & 2)) return hipSuccess;
    FwdArgs a{(const bf16_t*)Q, (const bf16_t*)ws, R, (bf16_t*)O, d.H, d.H / d.Hkuv, d.S, d.E, d.d_e / JB};
    switch (d.d_h) {
        case 64: return launch_fwd_t<64, 2>(a, d, st);
        case 96: return launch_fwd_t<96, 2>(a, d, st);
        case 128: return launch_fwd_t<128, 2>(a, d, st);
    }
    return hipErrorInvalidValue;
}

}  // namespace mhffn
