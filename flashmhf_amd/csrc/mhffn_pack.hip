// Weight re-layout ("pack") kernel: one workgroup per (kuv-head, 32-row block of the E*d_e axis).
// HBM-bound byte shuffling: reads 3 tiles of 32 x d_h bf16 coalesced, writes the padded natural (row-permuted) and
// transposed tiles the main kernels stream into LDS.  Traffic is ~2.3x the weight bytes, microseconds per call.
#include "mhffn_common.hpp"

namespace mhffn {

template <int DH>
__global__ __launch_bounds__(256) void pack_weights_kernel(const bf16_t* __restrict__ K, const bf16_t* __restrict__ U,
                                                           const bf16_t* __restrict__ V, bf16_t* __restrict__ dst,
                                                           int bundle)
{
    using G = Geo<DH>;
    constexpr int LD = DH + 2;  // odd dword stride: column reads for the transposed tiles spread over banks
    __shared__ bf16_t tile[3][JB * LD];
    const int tid = threadIdx.x;
    const long blk = blockIdx.x;  // flattened (hk, e, jb): the 32 rows are contiguous in K/U/V
    const bf16_t* src[3] = {K + blk * JB * DH, U + blk * JB * DH, V + blk * JB * DH};

    constexpr int CH = JB * DH / 8;  // 16-byte chunks per tile
    for (int w = 0; w < 3; ++w)
        for (int i = tid; i < CH; i += 256) {
            const int row = i / (DH / 8), c8 = (i % (DH / 8)) * 8;
            bf16x8 v = *reinterpret_cast<const bf16x8*>(src[w] + row * DH + c8);
            for (int x = 0; x < 8; ++x) tile[w][row * LD + c8 + x] = v[x];
        }
    __syncthreads();

    const int stage = bundle == 0 ? G::FWD_STAGE : G::DQ_STAGE;
    bf16_t* out = dst + blk * stage;
    const int n_nat = bundle == 0 ? 2 : 3;             // natural tiles come first: K, U(, V)
    const int n_tr = bundle == 0 ? 1 : 2;               // bundle 0: Vt ; bundle 1: Kt, Ut
    constexpr int NAT_CH = G::NAT_ELEMS / 8, TR_CH = G::TR_ELEMS / 8;

    for (int w = 0; w < n_nat; ++w)
        for (int i = tid; i < NAT_CH; i += 256) {
            const int rho = i / (G::NAT_LD / 8), c8 = (i % (G::NAT_LD / 8)) * 8;
            bf16x8 v;
            for (int x = 0; x < 8; ++x)
                v[x] = (c8 + x < DH) ? tile[w][row_perm32(rho) * LD + c8 + x] : (bf16_t)0.0f;
            *reinterpret_cast<bf16x8*>(out + w * G::NAT_ELEMS + rho * G::NAT_LD + c8) = v;
        }
    for (int w = 0; w < n_tr; ++w) {
        const int srcw = bundle == 0 ? 2 : w;  // forward: V ; dQ/dR: K then U
        bf16_t* o = out + n_nat * G::NAT_ELEMS + w * G::TR_ELEMS;
        for (int i = tid; i < TR_CH; i += 256) {
            const int c = i / (G::TR_LD / 8), j8 = (i % (G::TR_LD / 8)) * 8;
            bf16x8 v;
            for (int x = 0; x < 8; ++x) v[x] = (j8 + x < JB) ? tile[srcw][(j8 + x) * LD + c] : (bf16_t)0.0f;
            *reinterpret_cast<bf16x8*>(o + c * G::TR_LD + j8) = v;
        }
    }
}

size_t packed_weights_bytes(const Dims& d, int bundle)
{
    const size_t nblk = (size_t)d.Hkuv * d.E * (d.d_e / JB);
    size_t stage = 0;
    switch (d.d_h) {
        case 64: stage = bundle == 0 ? Geo<64>::FWD_STAGE : Geo<64>::DQ_STAGE; break;
        case 96: stage = bundle == 0 ? Geo<96>::FWD_STAGE : Geo<96>::DQ_STAGE; break;
        case 128: stage = bundle == 0 ? Geo<128>::FWD_STAGE : Geo<128>::DQ_STAGE; break;
    }
    return nblk * stage * sizeof(bf16_t);
}

hipError_t launch_pack_weights(const void* K, const void* U, const void* V, void* dst, int bundle, const Dims& d,
                               hipStream_t st)
{
    const unsigned nblk = (unsigned)((size_t)d.Hkuv * d.E * (d.d_e / JB));
    const bf16_t *k = (const bf16_t*)K, *u = (const bf16_t*)U, *v = (const bf16_t*)V;
    bf16_t* o = (bf16_t*)dst;
    switch (d.d_h) {
        case 64: hipLaunchKernelGGL(pack_weights_kernel<64>, dim3(nblk), dim3(256), 0, st, k, u, v, o, bundle); break;
        case 96: hipLaunchKernelGGL(pack_weights_kernel<96>, dim3(nblk), dim3(256), 0, st, k, u, v, o, bundle); break;
        case 128: hipLaunchKernelGGL(pack_weights_kernel<128>, dim3(nblk), dim3(256), 0, st, k, u, v, o, bundle); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace mhffn
