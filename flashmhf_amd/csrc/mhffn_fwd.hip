// Fused multi-head FFN forward for gfx950 (bf16 MFMA, fp32 accumulation).
//
// One workgroup (4 waves, one per SIMD, 512 registers each) owns 256 tokens of one (batch, q-head); a wave owns 64 tokens
// (two column tiles of 32).  The workgroup streams the K, U, V blocks (32 rows of the E*d_e axis at a time) straight
// from the weight tensors into a ring of LDS stages with asynchronous LDS-direct loads.  Per block and wave:
//     M^T = K Q^T, N^T = U Q^T               (A = rows of the K/U tiles, B = Q^T held in AGPRs for the whole kernel)
//     P^T = silu(M^T) * N^T * r_e             (fp32 in the accumulator registers, rounded once to bf16)
//     O^T += V^T P^T                          (A = columns of the V tile via transposing LDS reads, B = P^T registers)
// so the [tokens, E*d_e] intermediate lives only in registers.  Reference semantics:
// kernels/triton/flash_mlp_moe.py:243-266.
//
// Why this shape.  A wave that is alone on its SIMD issues about one instruction every five cycles whatever its type,
// and a 32x32x16 MFMA occupies the matrix pipe for 32 cycles: the kernel runs at MFMA speed only if every MFMA is
// followed by about five other instructions that do not depend on it.  With 64 tokens per wave every K/U/V operand
// read from LDS feeds two MFMAs (32 tokens per wave and two waves per SIMD needs the full LDS bandwidth to feed the
// matrix pipe), and the loop is software-pipelined by hand: the first-product MFMAs of block i+1 and the
// second-product MFMAs of block i form the slots of one step; the element-wise work of block i (16 element pairs per
// lane) is cut into 48 chunks of five VALU instructions that are spread over the slots, as are the LDS operand reads.
// First products use the VGPR form of the instruction (inline assembly) so the element-wise code reads them without
// v_accvgpr_read; the O^T accumulators live in AGPRs.
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
    int tokmaj;           // Q, O token-major ([B, S, H, d_h]) instead of [B, H, S, d_h]
};

// LDS ring of FWD_NST stages, laid out as three regions (all V tiles, all K tiles, all U tiles).  The block loop is
// unrolled over the four stages, so the stage of every LDS access is a compile-time constant and goes into the
// instruction's 16-bit offset field: the per-lane parts of the addresses (row, swizzled chunk) are computed once before the
// loop and no step spends VALU instructions on addresses.  V and K regions lie below 64 KB; the U reads use a second set
// of per-lane bases that already contains the U region's start.
constexpr int FWD_NST = 4;
constexpr int FWD_REGION_B = FWD_NST * TILE_B;   // 32 KB
constexpr int FWD_V0 = 0, FWD_K0 = FWD_REGION_B, FWD_U0 = 2 * FWD_REGION_B;
constexpr int FWD_RING_B = 3 * FWD_REGION_B;     // 96 KB

// LDS operations issued behind the K/U reads of k-step ks up to the wait in front of that k-step's matrix instructions,
// for the issue order of the block step (K/U of k-steps 0 and 1 up front; in k-step j first the four V^T reads of row
// tile j - 1 while 1 <= j <= CT, then the two K/U reads of k-step j + 2).
__host__ __device__ constexpr int fwd_younger_reads(int ks, int KS, int CT)
{
    int n = ks == 0 ? 2 : 0;                       // k-step 1's reads follow k-step 0's up front
    for (int j = ks < 2 ? 0 : ks - 1; j <= ks; ++j) n += (j >= 1 && j <= CT ? 4 : 0) + (j + 2 < KS ? 2 : 0);
    return n;
}

template <int DH>
__global__ __launch_bounds__(256) void mhffn_fwd_kernel(FwdArgs p)
{
    constexpr int KS = DH / 16, CT = DH / 32, NW = 4, BT = NW * 64;
    constexpr int FILL = 24 / NW;
    constexpr int NG1 = 4 * KS, NG2 = 4 * CT, NSLOT = NG1 + NG2;   // MFMAs per step
    // The first products of a step are written by inline-assembly MFMAs whose results the next step's element-wise code
    // reads without a fence of its own: the NG2 second-product MFMAs issued in between (32 matrix-pipe cycles each) are
    // what covers the 18 wait states an MFMA result needs before a VALU read.
    static_assert(NG2 >= 8, "the second-product MFMAs of a step must cover the hazard window of its first products");
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    float* sR = reinterpret_cast<float*>(smem + FWD_RING_B);   // [min(E, GATE_WIN)][BT]: gate values of one expert window

    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = blockIdx.x, tb = blockIdx.y, b = blockIdx.z;
    const int hk = h / p.G;
    const long rowbase = ((long)b * p.H + h) * p.S;          // rows of R
    const TokRows qrows = tok_rows(p.tokmaj, b, h, p.H, p.S);   // rows of Q and O
    const int tok0 = tb * BT + wave * 64;
    const int nblk = p.E * p.nbe;
    const long wbase = (long)hk * nblk * JB * DH;
    const bf16_t* Kh = p.K + wbase;
    const long offU = p.U - p.K, offV = p.V - p.K;

    auto issue_block = [&](int blk, int stage) {
        const int bc = blk < nblk ? blk : nblk - 1;
        const long roff = (long)bc * JB * DH;
#pragma unroll
        for (int k = 0; k < FILL; ++k) {
            const int id = wave + NW * k;
            const int which = id >> 3;
            const long toff = which == 0 ? 0 : (which == 1 ? offU : offV);
            const int region = which == 0 ? FWD_K0 : (which == 1 ? FWD_U0 : FWD_V0);
            tile_fill_ins<DH>(Kh + toff + roff, DH, smem + region + stage * TILE_B, id & 7, lane);
        }
    };
    // The Q rows come from HBM and are the longest wait of the prologue: request them before anything else.
    bf16x8 q[2][KS];
#pragma unroll
    for (int ct = 0; ct < 2; ++ct) {
        int t = tok0 + ct * 32 + l32;
        t = t < p.S ? t : p.S - 1;
        const bf16_t* qr = p.Q + (qrows.base + (long)t * qrows.stride) * DH + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) q[ct][ks] = *reinterpret_cast<const bf16x8*>(qr + ks * 16);
    }
    issue_block(0, 0);
    // Gate values of the workgroup's 256 tokens, expert-major [E][BT]: one asynchronous 4-byte LDS-direct load per expert
    // and wave (lane = token, so the 64 values of an instruction are contiguous in LDS).  LDS holds a window of GATE_WIN
    // experts at a time; the first window is issued between block 0 and block 1, so that the wait for block 0 below
    // covers it too, and a layer with more experts restages the tile between two steps of the block loop.
    const float* rrow;
    {
        int t = tok0 + lane;
        t = t < p.S ? t : p.S - 1;
        rrow = p.R + (rowbase + t) * p.E;
    }
    auto stage_gates = [&](int e0) {
        const int e1 = e0 + GATE_WIN < p.E ? e0 + GATE_WIN : p.E;
        for (int e = e0; e < e1; ++e)
            __builtin_amdgcn_global_load_lds((gptr_t)(rrow + e), (lptr_t)(sR + (e - e0) * BT + wave * 64), 4, 0, 0);
    };
    stage_gates(0);
    issue_block(1, 1);
    issue_block(2, 2);

    f32x16 oacc[CT][2];
#pragma unroll
    for (int i = 0; i < CT; ++i)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
#pragma unroll
            for (int x = 0; x < 16; ++x) oacc[i][ct][x] = 0.0f;

    const int krow = row_perm32(l32);
    const TrLane<CT> trl = make_tr_lane<CT, 8, 4>(lane);
    // per-lane LDS addresses of the K row reads for every k-step (stage 0); the stage, and the distance to the U region,
    // go into the instruction's immediate offset
    unsigned kaddr[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
        kaddr[ks] = lds_addr(smem) + FWD_K0 + krow * TILE_ROW_B + (((2 * ks + g) ^ swz16(krow)) << 4);
    const unsigned smem0 = lds_addr(smem);

    // consumes M/N of block blk (mc, nc), produces M/N of block blk+1 (mn, nn); ST = blk % FWD_NST
    auto step = [&](auto st_, int blk, int e, f32x16 (&mc)[2], f32x16 (&nc)[2], f32x16 (&mn)[2], f32x16 (&nn)[2]) {
        constexpr int ST = decltype(st_)::value, STN = (ST + 1) % FWD_NST;
        wait_vmcnt<FILL>();   // blocks <= blk+1 have landed (only block blk+2's loads may be in flight)
        __syncthreads();      // ... for every wave; and every wave is done with the stage about to be refilled

        // LDS reads of the step, all issued from inline assembly and waited for by count (the compiler's own waits are
        // full ones: behind a group of reads in flight it waits for the youngest along with the one it needs).  Issue
        // order: the two gate values, the K/U operands of k-steps 0 and 1, then per k-step ks the V^T operands of row tile
        // ks - 1 (for the second product, long after) and the K/U operands of k-step ks + 2.  LDS operations complete in
        // order, so "at most younger(ks) outstanding" means the operands of k-step ks have arrived; the V^T operands
        // have a full wait of their own in front of the second product, by when they have long landed.
        u32x2 rvu = lds_read2x4_async(lds_addr(sR + (e & (GATE_WIN - 1)) * BT + wave * 64 + l32));
        TrOperand av[CT][2];
        u32x4 ak[3], au[3];   // K/U operand ring, two k-steps ahead
        auto request = [&](auto kc) {
            constexpr int ks = decltype(kc)::value;
            ak[ks % 3] = lds_read16_async<STN * TILE_B>(kaddr[ks]);
            au[ks % 3] = lds_read16_async<FWD_U0 - FWD_K0 + STN * TILE_B>(kaddr[ks]);
        };
        auto request_v = [&](auto ic) {
            constexpr int i = decltype(ic)::value;
            av[i][0] = tile_read_cols_async<FWD_V0 + ST * TILE_B>(smem0, trl, i);
            av[i][1] = tile_read_cols_async<FWD_V0 + ST * TILE_B + 4096>(smem0, trl, i);
        };
        request(std::integral_constant<int, 0>{});
        request(std::integral_constant<int, 1>{});
        // the fill of the stage that has just come free is issued behind the first reads: its address arithmetic and six
        // instructions pass while those reads are on their way
        __builtin_amdgcn_sched_barrier(0);
        issue_block(blk + 3, (ST + 3) % FWD_NST);
        float rinv[2];
        bf16x8 pt[2][2];
        float e0 = 0, e1 = 0, xn0 = 0, xn1 = 0;   // carried between the chunks of one element pair
        __builtin_amdgcn_sched_barrier(0);

        // chunk c: third c%3 of element pair c/3; pairs ordered (tile 0, s 0), (tile 1, s 0), (tile 0, s 1), (tile 1, s 1)
        // so that each second-product operand P^T[ct][s] is complete well before the slot that consumes it.  The thirds
        // are cut so that their issue times are about equal (a transcendental instruction costs a lone wave about 10
        // cycles, a plain one about 6): 3 plain + 1 transcendental, 2 + 2, 4 + 1.
        float t1 = 0, s0 = 0;
        auto chunk = [&](auto c_) {
            constexpr int c = decltype(c_)::value;
            constexpr int pi = c / 3, third = c % 3;
            constexpr int ct = (pi / 4) % 2, pp = (pi % 4) + 4 * (pi / 8), i0 = 2 * pp, i1 = i0 + 1;
            if constexpr (third == 0) {
                const float t0 = -LOG2E * mc[ct][i0];
                t1 = -LOG2E * mc[ct][i1];
                e0 = __builtin_amdgcn_exp2f(t0);
                xn0 = mc[ct][i0] * nc[ct][i0];
            } else if constexpr (third == 1) {
                e1 = __builtin_amdgcn_exp2f(t1);
                s0 = __builtin_amdgcn_rcpf(__builtin_fmaf(e0, rinv[ct], rinv[ct]));
                xn1 = mc[ct][i1] * nc[ct][i1];
            } else {
                const float s1 = __builtin_amdgcn_rcpf(__builtin_fmaf(e1, rinv[ct], rinv[ct]));
                pt[ct][i0 >> 3][i0 & 7] = (bf16_t)(xn0 * s0);
                pt[ct][i0 >> 3][i1 & 7] = (bf16_t)(xn1 * s1);
            }
        };

        static_for<NSLOT>([&](auto k_) {
            constexpr int k = decltype(k_)::value;
            if constexpr (k < NG1) {
                constexpr int ks = k / 4, w = k % 4, ct = w >> 1;
                if constexpr (w == 0) {
                    if constexpr (ks >= 1 && ks <= CT) request_v(std::integral_constant<int, ks - 1>{});
                    if constexpr (ks + 2 < KS) request(std::integral_constant<int, ks + 2>{});
                    if constexpr (ks == 0) {
                        lds_wait_n<fwd_younger_reads(0, KS, CT)>(ak[0], au[0], rvu);     // (the gate values are older)
                        // The gate value enters through its reciprocal: r / (1 + e) = 1 / fma(e, 1/r, 1/r), one multiply
                        // fewer per element.  1/r is clamped to the largest finite float, so a zero gate makes the
                        // denominator at least FLT_MAX, whose reciprocal the hardware flushes to exactly 0.
#pragma unroll
                        for (int c2 = 0; c2 < 2; ++c2) {
                            const unsigned bits = rvu[c2];    // (a scalar copy: the cast below must not see a vector element)
                            rinv[c2] = __builtin_amdgcn_fmed3f(__builtin_amdgcn_rcpf(__builtin_bit_cast(float, bits)),
                                                               -FLT_MAX_F, FLT_MAX_F);
                        }
                    } else {
                        lds_wait_n<fwd_younger_reads(ks, KS, CT)>();     // (consumed by asm matrix instructions only)
                    }
                }
                if constexpr ((w & 1) == 0) {
                    if constexpr (ks == 0) mfma32_vgpr_first_bacc(mn[ct], __builtin_bit_cast(bf16x8, ak[0]), q[ct][0]);
                    else mfma32_vgpr_acc_bacc(mn[ct], __builtin_bit_cast(bf16x8, ak[ks % 3]), q[ct][ks]);
                } else {
                    if constexpr (ks == 0) mfma32_vgpr_first_bacc(nn[ct], __builtin_bit_cast(bf16x8, au[0]), q[ct][0]);
                    else mfma32_vgpr_acc_bacc(nn[ct], __builtin_bit_cast(bf16x8, au[ks % 3]), q[ct][ks]);
                }
            } else {
                constexpr int g2 = k - NG1, s = g2 / (2 * CT), ct = (g2 / CT) % 2, i = g2 % CT;
                if constexpr (g2 == 0) {
#pragma unroll
                    for (int ii = 0; ii < CT; ++ii) lds_tr_wait(av[ii][0], av[ii][1]);
                }
                oacc[i][ct] = mfma32(tr_value(av[i][s]), pt[ct][s], oacc[i][ct]);
            }
            // element-wise chunks: chunk c goes behind slot c * (NSLOT - CT) / 48, so the last one is done before the
            // CT slots that consume P^T[1][1]
            static_for<48>([&](auto c_) {
                if constexpr (decltype(c_)::value * (NSLOT - CT) / 48 == k) chunk(c_);
            });
            __builtin_amdgcn_sched_barrier(0);
        });
        // The first products are written by the matrix pipe long after their instruction has issued.  Keep their
        // registers allocated to the end of the step even when nothing reads them (the phantom block behind an odd
        // count): otherwise the compiler hands them to other values, which the late write then overwrites.
        asm volatile("" :: "v"(mn[0]), "v"(mn[1]), "v"(nn[0]), "v"(nn[1]));
    };

    f32x16 mA[2], nA[2], mB[2], nB[2];
    wait_vmcnt<2 * FILL>();   // all but the fills of blocks 1 and 2: block 0 and the gate values have landed
    __syncthreads();
    {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const bf16x8 a = tile_read_rows(smem + FWD_K0, krow, ks, g), u = tile_read_rows(smem + FWD_U0, krow, ks, g);
#pragma unroll
            for (int ct = 0; ct < 2; ++ct) {
                if (ks == 0) { mfma32_vgpr_first_bacc(mA[ct], a, q[ct][0]); mfma32_vgpr_first_bacc(nA[ct], u, q[ct][0]); }
                else { mfma32_vgpr_acc_bacc(mA[ct], a, q[ct][ks]); mfma32_vgpr_acc_bacc(nA[ct], u, q[ct][ks]); }
            }
        }
        mfma_result_fence(mA[0], nA[0], mA[1]);   // the element-wise code of step 0 reads these results
        mfma_result_fence(nA[1]);
    }
    // Four blocks per trip (one per LDS stage; the two M/N register sets alternate), then the last one to three.  (The
    // step of the last block still computes first products, of the block its prefetch clamped to; nothing reads them.)
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    using S2 = std::integral_constant<int, 2>;
    using S3 = std::integral_constant<int, 3>;
    int e = 0, jb = 0, blk = 0;
    auto advance = [&]() {
        if (++jb == p.nbe) { jb = 0; ++e; }
    };
    // (A window of GATE_WIN experts is a multiple of four blocks, so every window starts on stage 0 and register set A.)
    for (int e0 = 0; e0 < p.E; e0 += GATE_WIN) {
        if (e0 > 0) {
            __syncthreads();      // every wave has read its gate values of the window before
            stage_gates(e0);
            wait_vmcnt<0>();      // (also lands the two blocks in flight; the next step's wait then passes at once)
            __syncthreads();
        }
        const int wend = (e0 + GATE_WIN) * p.nbe < nblk ? (e0 + GATE_WIN) * p.nbe : nblk;
        for (; blk + 4 <= wend; blk += 4) {
            step(S0{}, blk, e, mA, nA, mB, nB);
            advance();
            step(S1{}, blk + 1, e, mB, nB, mA, nA);
            advance();
            step(S2{}, blk + 2, e, mA, nA, mB, nB);
            advance();
            step(S3{}, blk + 3, e, mB, nB, mA, nA);
            advance();
        }
    }
    if (blk < nblk) {
        step(S0{}, blk, e, mA, nA, mB, nB);
        advance();
        if (blk + 1 < nblk) {
            step(S1{}, blk + 1, e, mB, nB, mA, nA);
            advance();
            if (blk + 2 < nblk) step(S2{}, blk + 2, e, mA, nA, mB, nB);
        }
    }
    wait_vmcnt<0>();      // drain the phantom prefetches: they write the ring, which the epilogue reuses
    __syncthreads();      // every wave is done reading the ring

    // O^T registers -> O[t][c].  Register 4a+b of row tile i is c = 32i + 8a + 4g + b: a lane owns runs of 4 c of one
    // token, which stored directly would be 8-byte pieces scattered over 32 rows per instruction.  Instead each wave
    // writes its 64 x d_h tile into a private 16 KB region of the ring (rows of 256 bytes, 16-byte chunk c16 of row r at
    // chunk c16 ^ (r & 15)), reads it back row-wise and stores whole rows: 16 lanes x 16 bytes per row, 4 rows per
    // instruction.  Only this wave touches the region, and LDS operations of one wave complete in order.
    {
        unsigned char* otile = smem + wave * (64 * TILE_ROW_B);
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
#pragma unroll
            for (int i = 0; i < CT; ++i)
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    bf16x4 v;
#pragma unroll
                    for (int x = 0; x < 4; ++x) v[x] = (bf16_t)oacc[i][ct][4 * a + x];
                    *reinterpret_cast<bf16x4*>(otile + (ct * 32 + l32) * TILE_ROW_B + (((4 * i + a) ^ (l32 & 15)) << 4) + 8 * g) = v;
                }
        const int c16 = lane & 15;
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const int row = 4 * k + (lane >> 4);
            const int t = tok0 + row;
            if (c16 < DH / 8 && t < p.S) {
                const u32x4 v = *reinterpret_cast<const u32x4*>(otile + row * TILE_ROW_B + ((c16 ^ (row & 15)) << 4));
                *reinterpret_cast<u32x4*>(p.O + (qrows.base + (long)t * qrows.stride) * DH + c16 * 8) = v;
            }
        }
    }
}

template <int DH>
static hipError_t launch_fwd_t(const FwdArgs& a, const Dims& d, hipStream_t st)
{
    const int tokw = 256;
    const int smem = FWD_RING_B + (d.E < GATE_WIN ? d.E : GATE_WIN) * tokw * (int)sizeof(float);
    if (smem > 160 * 1024) return hipErrorInvalidValue;
    static LdsOptIn optin;
    const hipError_t e = ensure_dynamic_lds(optin, (const void*)mhffn_fwd_kernel<DH>, smem);
    if (e != hipSuccess) return e;
    dim3 grid((unsigned)d.H, (unsigned)((d.S + tokw - 1) / tokw), (unsigned)d.B);
    hipLaunchKernelGGL((mhffn_fwd_kernel<DH>), grid, dim3(256), smem, st, a);
    return hipGetLastError();
}

size_t fwd_workspace_bytes_bf16(const Dims&) { return 0; }

hipError_t launch_fwd_bf16(const void* Q, const void* K, const void* U, const void* V, const float* R, void* O,
                           void* ws, const Dims& d, hipStream_t st, int phases)
{
    (void)ws;
    if (!(phases & PH_FWD_MAIN)) return hipSuccess;
    FwdArgs a{(const bf16_t*)Q, (const bf16_t*)K, (const bf16_t*)U, (const bf16_t*)V, R, (bf16_t*)O,
              d.H,              d.H / d.Hkuv,     d.S,              d.E,              d.d_e / JB,
              d.tokmaj};
    switch (d.d_h) {
        case 64: return launch_fwd_t<64>(a, d, st);
        case 96: return launch_fwd_t<96>(a, d, st);
        case 128: return launch_fwd_t<128>(a, d, st);
    }
    return hipErrorInvalidValue;
}

}  // namespace mhffn
