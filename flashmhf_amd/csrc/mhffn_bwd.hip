// Fused multi-head FFN backward for gfx950 (bf16 MFMA, fp32 accumulation), two kernels:
//
//  (1) dQ/dR kernel -- a workgroup of 8 waves (two per SIMD) owns 256 tokens of one (batch, q-head), 32 per wave, and
//      streams the K, U, V blocks (32 rows at a time) through a ring of LDS stages with LDS-direct loads.  Per block:
//          M^T = K Q^T, N^T = U Q^T, dA^T = V dO^T            (recomputed, registers only)
//          dR_e += sum_j dA * silu(M) * N                      (fp32, before any rounding)
//          dN^T = r_e dA^T silu(M^T),  dM^T = r_e dA^T N^T silu'(M^T)      (rounded once to bf16)
//          dQ^T += K^T dM^T + U^T dN^T                         (K^T, U^T: transposing reads of the same K, U tiles)
//      The two waves of a SIMD work half a block apart (one's element-wise phase under the other's matrix phases),
//      the later one at a higher wave priority.
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
    int tokmaj;   // Q, dO, dQ token-major ([B, S, H, d_h]) instead of [B, H, S, d_h]
};

constexpr int DQ_NST = 4;                  // LDS stages (K | U | V tiles each)
constexpr int DQ_STAGE_B = 3 * TILE_B;

template <int DH>
__global__ __launch_bounds__(512) void mhffn_bwd_dqdr_kernel(DqArgs p)
{
    constexpr int KS = DH / 16, CT = DH / 32, NW = 8;
    constexpr int BT = NW * 32;
    constexpr int FILL = 24 / NW;          // tile-fill wave-instructions per wave and block (3 tiles x 8 / NW waves)
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    float* sR = reinterpret_cast<float*>(smem + DQ_NST * DQ_STAGE_B);   // [min(E, 64)][BT]: expert e in slot e % 64

    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = blockIdx.x, tb = blockIdx.y, b = blockIdx.z;
    const int hk = h / p.G;
    const long rowbase = ((long)b * p.H + h) * p.S;          // rows of R, dR
    const TokRows qrows = tok_rows(p.tokmaj, b, h, p.H, p.S);   // rows of Q, dO, dQ
    const int tok0 = tb * BT + wave * 32;
    const int nblk = p.E * p.nbe;
    const bf16_t* Kh = p.K + (long)hk * nblk * JB * DH;
    const long offU = p.U - p.K, offV = p.V - p.K;

    auto issue_block = [&](int blk) {
        const int bc = blk < nblk ? blk : nblk - 1;
        unsigned char* st = smem + (blk % DQ_NST) * DQ_STAGE_B;
        const long roff = (long)bc * JB * DH;
#pragma unroll
        for (int k = 0; k < FILL; ++k) {
            const int id = wave + NW * k;            // 0..23: tile id/8 (K, U, V), 4-row group id%8
            const int which = id >> 3;
            const long toff = which == 0 ? 0 : (which == 1 ? offU : offV);
            tile_fill_ins<DH>(Kh + toff + roff, DH, st + which * TILE_B, id & 7, lane);
        }
    };
    // The Q and dO rows come from HBM and are the longest wait of the prologue: request them before anything else.
    bf16x8 q[KS], go[KS];
    {
        int t = tok0 + l32;
        t = t < p.S ? t : p.S - 1;
        const bf16_t* qr = p.Q + (qrows.base + (long)t * qrows.stride) * DH + 8 * g;
        const bf16_t* gr = p.dO + (qrows.base + (long)t * qrows.stride) * DH + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            q[ks] = *reinterpret_cast<const bf16x8*>(qr + ks * 16);
            go[ks] = *reinterpret_cast<const bf16x8*>(gr + ks * 16);
        }
    }
    issue_block(0);
    // Gate values of the workgroup's 256 tokens, expert-major [E][BT]: asynchronous 4-byte LDS-direct loads, lane = token;
    // a pair of waves shares a group of 64 tokens and takes the even and the odd experts.  LDS holds 64 experts, expert e
    // in slot e % 64; the first 64 are issued between block 0 and block 1, so that the first wait for block 0 covers
    // them too, and a layer with more experts refills the slots 32 at a time as the block loop leaves them behind.
    const float* rrow;
    {
        int t = tb * BT + (wave >> 1) * 64 + lane;
        t = t < p.S ? t : p.S - 1;
        rrow = p.R + (rowbase + t) * p.E;
    }
    auto stage_gates = [&](int e0, int e1) {
        e1 = e1 < p.E ? e1 : p.E;
        for (int e = e0 + (wave & 1); e < e1; e += 2)
            __builtin_amdgcn_global_load_lds((gptr_t)(rrow + e), (lptr_t)(sR + (e & 63) * BT + (wave >> 1) * 64), 4, 0, 0);
    };
    stage_gates(0, 64);
    issue_block(1);

    f32x16 dq[CT];
#pragma unroll
    for (int i = 0; i < CT; ++i)
#pragma unroll
        for (int x = 0; x < 16; ++x) dq[i][x] = 0.0f;

    const int krow = row_perm32(l32);
    const TrLane<CT> trl = make_tr_lane<CT, 8, 4>(lane);
    // One block takes three phases per wave: first products (24 matrix instructions for d_h = 128), element-wise work
    // (VALU only), second products (16 matrix instructions).  The two waves that share a SIMD run them in opposite phase
    // between two barriers -- waves 0..3: first(b), element-wise(b), second(b); waves 4..7: element-wise(b-1),
    // second(b-1), first(b) -- so that one wave's VALU phase lies under the other's matrix phases.  Left to the
    // hardware's oldest-first arbitration the early waves win every conflict and then idle at the barrier while the late
    // waves catch up alone; the late waves therefore run at a higher wave priority, which evens the two out.  The late
    // waves carry M, N, dA of block b across the barrier and need one more trip at the end; the ring keeps block b-1
    // alive that long (the refill behind barrier b targets the stage of block b-2).
    f32x16 m, n, da;
    bf16x8 dmt[2], dnt[2];
    float dr = 0.0f;
    auto first_products = [&](int blk) {
        const unsigned char* sK = smem + (blk % DQ_NST) * DQ_STAGE_B;
        const unsigned char* sU = sK + TILE_B;
        const unsigned char* sV = sU + TILE_B;
#pragma unroll
        for (int x = 0; x < 16; ++x) { m[x] = 0.0f; n[x] = 0.0f; da[x] = 0.0f; }
        // The K/U/V operands come from LDS through a ring of three register sets, read two k-steps ahead of the
        // matrix instructions that use them; the fence after each k-step keeps the compiler from gathering the
        // reads back to the front (which costs their whole latency once per block).
        bf16x8 ak[3], au[3], av[3];
#pragma unroll
        for (int k0 = 0; k0 < 2; ++k0) {
            ak[k0] = tile_read_rows(sK, krow, k0, g);
            au[k0] = tile_read_rows(sU, krow, k0, g);
            av[k0] = tile_read_rows(sV, krow, k0, g);
        }
        static_for<KS>([&](auto kc) {
            constexpr int ks = decltype(kc)::value;
            if constexpr (ks + 2 < KS) {
                ak[(ks + 2) % 3] = tile_read_rows(sK, krow, ks + 2, g);
                au[(ks + 2) % 3] = tile_read_rows(sU, krow, ks + 2, g);
                av[(ks + 2) % 3] = tile_read_rows(sV, krow, ks + 2, g);
            }
            m = mfma32(ak[ks % 3], q[ks], m);
            n = mfma32(au[ks % 3], q[ks], n);
            da = mfma32(av[ks % 3], go[ks], da);
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    auto element_wise = [&](float r) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) {
                const int i = 8 * s + kk;
                const float x = m[i], nn = n[i], a = da[i];
                const float sg = fast_sigmoid(x);
                const float sl = x * sg;                 // silu(m)
                const float as = a * sl;
                dr = __builtin_fmaf(as, nn, dr);
                const float w = __builtin_fmaf(sl, 1.0f - sg, sg);    // silu'(m)
                dnt[s][kk] = (bf16_t)(r * as);
                dmt[s][kk] = (bf16_t)((r * a) * (nn * w));
            }
    };
    // second products: operand pairs (Kt, Ut) are requested two steps ahead of the MFMAs that consume them; the region is
    // fenced so that the partial LDS waits count exactly these reads
    auto second_products = [&](int blk) {
        const unsigned sK = lds_addr(smem + (blk % DQ_NST) * DQ_STAGE_B);
        __builtin_amdgcn_sched_barrier(0);
        {
            constexpr int NSET = 2 * CT;          // (s, i) in s-major order
            TrOperand tk[3], tu[3];
            auto request = [&](auto ic) {
                constexpr int idx = decltype(ic)::value;
                constexpr int s = idx / CT, i = idx % CT;
                tk[idx % 3] = tile_read_cols_async<4096 * s>(sK, trl, i);
                tu[idx % 3] = tile_read_cols_async<4096 * s + TILE_B>(sK, trl, i);
            };
            request(std::integral_constant<int, 0>{});
            request(std::integral_constant<int, 1>{});
            static_for<NSET>([&](auto ic) {
                constexpr int idx = decltype(ic)::value;
                constexpr int s = idx / CT, i = idx % CT;
                if constexpr (idx + 2 < NSET) request(std::integral_constant<int, idx + 2>{});
                constexpr int ahead = (NSET - 1 - idx) < 2 ? (NSET - 1 - idx) : 2;
                lds_tr_wait_n<4 * ahead>(tk[idx % 3], tu[idx % 3]);
                dq[i] = mfma32(tr_value(tk[idx % 3]), dmt[s], dq[i]);
                dq[i] = mfma32(tr_value(tu[idx % 3]), dnt[s], dq[i]);
            });
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    int e = 0, jb = 0;          // expert and block-in-expert of the block whose element-wise work comes next
    auto finish_block = [&](int blk) {
        element_wise(sR[(e & 63) * BT + wave * 32 + l32]);
        second_products(blk);
        if (++jb == p.nbe) {
            // dR[t, e]: the two lane halves hold disjoint j rows of the same token column.
            const float tot = dr + __shfl_xor(dr, 32);
            const int t = tok0 + l32;
            if (g == 0 && t < p.S) p.dR[(rowbase + t) * p.E + e] = tot;
            dr = 0.0f;
            jb = 0;
            ++e;
            // More than 64 experts: with expert 32k behind it (k >= 1), this pair of waves refills the slots of experts
            // 32k-32 .. 32k-1 with experts 32k+32 .. 32k+63 of its own 64 tokens.  Its partner is in the same interval
            // between two barriers, so at a block of expert 32k or later; the values are first read 31 experts on, and
            // every barrier's wait on the way leaves at most three of this wave's loads outstanding.
            if (e > 1 && (e & 31) == 1 && e + 31 < p.E) stage_gates(e + 31, e + 63);
        }
    };
    // Barrier b: block b has landed for every wave, and every wave is done with block b - 2, whose stage the fill of
    // block b + 2 takes.
    auto next_interval = [&](int b) {
        wait_vmcnt<FILL>();       // block b has landed (block b+1 may be in flight)
        __syncthreads();
        issue_block(b + 2);
    };
    if (wave < NW / 2) {
        for (int b = 0; b < nblk; ++b) {
            next_interval(b);
            first_products(b);
            finish_block(b);
        }
        next_interval(nblk);      // the barrier of the late waves' extra trip
    } else {
        __builtin_amdgcn_s_setprio(2);
        next_interval(0);
        first_products(0);
        for (int b = 1; b < nblk; ++b) {
            next_interval(b);
            finish_block(b - 1);
            first_products(b);
        }
        next_interval(nblk);
        finish_block(nblk - 1);
        __builtin_amdgcn_s_setprio(0);
    }
    wait_vmcnt<0>();   // drain the phantom prefetches: they write the ring, which the epilogue reuses
    __syncthreads();   // every wave is done reading the ring

    // dQ^T registers -> dQ[t][c] through a private 8 KB region of the ring per wave (rows of 256 bytes, 16-byte chunk c16
    // of row r at chunk c16 ^ (r & 15)), so that the stores are whole rows (16 lanes x 16 bytes, 4 rows per instruction)
    // instead of 8-byte pieces scattered over 32 rows.  Register 4a+x of row tile i is c = 32i + 8a + 4g + x.
    {
        unsigned char* otile = smem + wave * (32 * TILE_ROW_B);
#pragma unroll
        for (int i = 0; i < CT; ++i)
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                bf16x4 v;
#pragma unroll
                for (int x = 0; x < 4; ++x) v[x] = (bf16_t)dq[i][4 * a + x];
                *reinterpret_cast<bf16x4*>(otile + l32 * TILE_ROW_B + (((4 * i + a) ^ (l32 & 15)) << 4) + 8 * g) = v;
            }
        const int c16 = lane & 15;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int row = 4 * k + (lane >> 4);
            const int t = tok0 + row;
            if (c16 < DH / 8 && t < p.S) {
                const u32x4 v = *reinterpret_cast<const u32x4*>(otile + row * TILE_ROW_B + ((c16 ^ (row & 15)) << 4));
                *reinterpret_cast<u32x4*>(p.dQ + (qrows.base + (long)t * qrows.stride) * DH + c16 * 8) = v;
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
    float* part;        // [nslice][3][Hkuv][E*d_e][DH] fp32 partial sums (nslice > 1)
    void* out[3];       // dK, dU, dV: written directly when there is one token slice
    int out_f32;        // element type of out: 1 = float32, 0 = bfloat16
    int B, H, G, S, E, nbe, nslice;
    int tokmaj;         // Q, dO token-major ([B, S, H, d_h]) instead of [B, H, S, d_h]
};

constexpr int DW_NST = 4;                              // LDS stages of the token-tile ring
constexpr int DW_RTILE_B = 1024;                       // staged gate values: [4 waves][64 lanes] fp32 (each wave: its expert)
constexpr int DW_STAGE_B = 2 * TILE_B + DW_RTILE_B;    // Q tile | dO tile | gate values

template <int DH, bool TAIL>
__global__ __launch_bounds__(256) void mhffn_bwd_dkdudv_kernel(DwArgs p)
{
    constexpr int KS = DH / 16, CT = DH / 32;
    constexpr int NCHUNK = DH / 8;                    // 16-byte chunks per token row
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];

    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hk = blockIdx.x, z = blockIdx.z;   // head index fastest: all columns of a head run on one XCD and share its L2
    const int nblk = p.E * p.nbe;
    const int jblk = blockIdx.y * 4 + wave;
    const bool active = jblk < nblk;
    const int jb_c = active ? jblk : nblk - 1;        // waves of the last column without a block: addresses stay valid
    const int e_w = jb_c / p.nbe;
    const long wrow = ((long)hk * nblk + jb_c) * JB + l32;      // this lane's row of K/U/V (column j of the products)

    float* sZero = reinterpret_cast<float*>(smem_raw + DW_NST * DW_STAGE_B);   // 32 zero gate values
    if (tid < 32) sZero[tid] = 0.0f;
    // The first step contracts a tile that does not exist (zero gate values) out of the last stage, which no load has
    // filled yet: clear its Q and dO tiles, or whatever bit patterns the previous kernel left there (possibly NaN or
    // Inf as bf16) would be multiplied by those zeros.
    {
        u32x4 z = {0u, 0u, 0u, 0u};
        u32x4* last_stage = reinterpret_cast<u32x4*>(smem_raw + (DW_NST - 1) * DW_STAGE_B);
        for (int i = tid; i < 2 * TILE_B / 16; i += 256) last_stage[i] = z;
    }
    // These clears are ordinary LDS stores that other waves read in step 0, and the barriers of the token loop are bare
    // (no wait on this wave's own LDS stores): one fenced barrier here publishes them, once per workgroup.
    __syncthreads();
    const int nS = (p.S + 31) / 32;
    const int ntile = p.G * p.B * nS;
    const int t_begin = (int)((long)ntile * z / p.nslice), t_end = (int)((long)ntile * (z + 1) / p.nslice);
    const int nt = t_end - t_begin;

    // Tile cursor of the prefetcher: tile index -> (q-head of the group, batch, 32-token tile).  It is kept as a running
    // token-row index that advances by one of three precomputed strides (next tile of the sequence, next
    // batch, next q-head of the group), so a step spends a handful of scalar instructions on it.
    int pf_st = t_begin % nS, pf_bb = (t_begin / nS) % p.B;
    int pf_left = nt;                                 // tiles not yet requested
    // (token rows are counted in 32 bits: B * H * S < 2^31 is checked on the host)
    const int pf_h0 = hk * p.G + t_begin / (nS * p.B);                        // q-head of the first tile
    int pf_row = (pf_bb * p.H + pf_h0) * p.S + pf_st * 32;                     // row of R ([B, H, S, E])
    const int drow_s = p.H * p.S - (nS - 1) * 32;                              // last tile of a sequence -> next batch
    const int drow_b = p.S - (p.B - 1) * p.H * p.S - (nS - 1) * 32;            // ... of the last batch -> next q-head
    // The same walk in rows of Q/dO, whose token stride is qs rows (1, or H when token-major).
    const int qs = p.tokmaj ? p.H : 1;
    int pf_qrow = p.tokmaj ? (pf_bb * p.S + pf_st * 32) * p.H + pf_h0 : pf_row;
    const int dqrow_s = p.H * p.S - (nS - 1) * 32 * qs;
    const int dqrow_b = (p.tokmaj ? 1 : p.S) - (p.B - 1) * p.H * p.S - (nS - 1) * 32 * qs;

    // per-lane constants of the tile fill: this wave's two 4-row groups of the Q/dO tiles (swizzled source chunk)
    int fill_row[2], fill_coff[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int ins = wave + 4 * k;
        const int r = 4 * ins + (lane >> 4);
        int c = (lane & 15) ^ swz16(r);
        c = c < NCHUNK ? c : 0;                       // unused chunk positions of narrow rows load a dummy chunk
        fill_row[k] = r;
        fill_coff[k] = c * 16;                        // bytes
    }

    // Asynchronous fill of a stage with the tile under the cursor (the last tile again once all are requested); every wave
    // issues its share of LDS-direct loads (no staging registers).  Addresses are a wave-uniform 64-bit base plus a
    // 32-bit lane offset.  Rows past the end of a sequence are clamped to its last row and their gate value is zeroed
    // afterwards (zero_tail), which removes them from all three products.
    // The work is split: prepare_tile computes the uniform bases of the tile under the cursor and advances the cursor
    // (some forty scalar instructions; called under the last matrix instructions of a step, where the wave has issue
    // slots to spare), fire_tile issues the loads (right behind the barrier) and returns the tile's valid rows.
    const char* nx_qb = nullptr;
    const char* nx_gb = nullptr;
    const char* nx_rbp = nullptr;
    int nx_last = 31;
    auto prepare_tile = [&]() {
        nx_last = p.S - pf_st * 32 - 1;                                       // last valid row of the tile (>= 0)
        nx_qb = reinterpret_cast<const char*>(p.Q) + (long)pf_qrow * (DH * 2);
        nx_gb = reinterpret_cast<const char*>(p.dO) + (long)pf_qrow * (DH * 2);
        nx_rbp = reinterpret_cast<const char*>(p.R) + (long)pf_row * (p.E * 4);
        // advance unless this was the last tile of the slice (then later requests reload it, harmlessly)
        // (0/1 flags and multiplies: selects here were turned into branches inside the hot loop)
        const int more = pf_left > 1 ? 1 : 0;
        const int ws = (pf_st + 1 == nS ? 1 : 0) * more;
        const int wb = (pf_bb + 1 == p.B ? 1 : 0) * ws;
        pf_left -= more;
        pf_row += more * 32 + ws * (drow_s - 32) + wb * (drow_b - drow_s);
        pf_qrow += more * 32 * qs + ws * (dqrow_s - 32 * qs) + wb * (dqrow_b - dqrow_s);
        pf_st = (pf_st + more) * (1 - ws);
        pf_bb = (pf_bb + ws) * (1 - wb);
    };
    auto fire_tile = [&](int sidx) -> int {
        const int last = nx_last;
        unsigned char* sbase = smem_raw + sidx * DW_STAGE_B;
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const int row = TAIL ? (fill_row[k] < last ? fill_row[k] : last) : fill_row[k];
            const unsigned off = (unsigned)(row * qs * (DH * 2) + fill_coff[k]);
            const int ins = wave + 4 * k;
            __builtin_amdgcn_global_load_lds((gptr_t)(nx_qb + off), (lptr_t)(sbase + ins * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((gptr_t)(nx_gb + off), (lptr_t)(sbase + TILE_B + ins * 1024), 16, 0, 0);
        }
        // gate values of this wave's expert for the 32 token rows (lanes 32..63 repeat them): one 4-byte element per lane
        const int trow = TAIL ? (l32 < last ? l32 : last) : l32;
        __builtin_amdgcn_global_load_lds((gptr_t)(nx_rbp + (unsigned)((trow * p.E + e_w) * 4)),
                                         (lptr_t)(sbase + 2 * TILE_B + wave * 256), 4, 0, 0);
        return last + 1;
    };
    // Called by every wave after its own loads of stage `sidx` have landed and before the barrier that publishes
    // the stage: zeroes the gate values of the rows a tail tile does not have.
    auto zero_tail = [&](int sidx, int nvalid) {
        float* sR = reinterpret_cast<float*>(smem_raw + sidx * DW_STAGE_B + 2 * TILE_B);
        if (l32 >= nvalid) sR[wave * 64 + lane] = 0.0f;
    };

    // First two tiles of the slice; the third is fired behind the first barrier of the loop.
    prepare_tile();
    int nv0 = fire_tile(0);
    prepare_tile();
    int nv1 = fire_tile(1), nv2 = 32, nv3 = 32;        // valid rows of the tile in each stage
    if constexpr (!TAIL) prepare_tile();

    if (!active) {
        // A wave of a head's last column that has no block: it keeps up its share of the tile fills and the barriers
        // (as many as the working waves pass, nt + 1) and issues no matrix instruction.
        for (int k = 0; k <= nt; ++k) {
            const int st = k & 3;
            wait_vmcnt<0>();
            if constexpr (TAIL) {
                const int nvalid = st == 0 ? nv0 : (st == 1 ? nv1 : (st == 2 ? nv2 : nv3));
                if (nvalid < 32) zero_tail(st, nvalid);
            }
            __builtin_amdgcn_s_barrier();
            if constexpr (TAIL) prepare_tile();
            const int nvn = fire_tile((st + 2) & 3);
            if constexpr (!TAIL) prepare_tile();
            if constexpr (TAIL) {
                if (st == 0) nv2 = nvn; else if (st == 1) nv3 = nvn; else if (st == 2) nv0 = nvn; else nv1 = nvn;
            }
        }
        wait_vmcnt<0>();
        __syncthreads();   // the barrier the working waves pass before their epilogue reuses the ring
        return;
    }

    // The K, U and V blocks stay in registers as MFMA B operands for the whole kernel (K, U in accumulation registers).
    bf16x8 kB[KS], uB[KS];
    bf16x8 vR[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        kB[ks] = *reinterpret_cast<const bf16x8*>(p.K + wrow * DH + ks * 16 + 8 * g);
        uB[ks] = *reinterpret_cast<const bf16x8*>(p.U + wrow * DH + ks * 16 + 8 * g);
        vR[ks] = *reinterpret_cast<const bf16x8*>(p.V + wrow * DH + ks * 16 + 8 * g);
    }

    f32x16 dk[CT], du[CT], dv[CT];
#pragma unroll
    for (int i = 0; i < CT; ++i)
#pragma unroll
        for (int x = 0; x < 16; ++x) { dk[i][x] = 0.0f; du[i][x] = 0.0f; dv[i][x] = 0.0f; }

    const int fr = swz16(l32);
    const TrLane<CT> trl = make_tr_lane<CT, 4, 8>(lane);
    // LDS address of this lane's 16 bytes of k-step 0 in the Q tile of stage 0 (row l32, chunk g ^ swizzle); k-step ks is
    // this address ^ (ks << 5): the ring starts on a 1 KB boundary, so the exclusive-or commutes with the sum
    const unsigned qaddr = lds_addr(smem_raw) + l32 * 256 + ((g ^ fr) << 4);

    // B operands of the token contraction (P, dM, dN of one tile, bf16).  They live across steps: the element pairs 0 and 1
    // of a tile are converted under the last matrix instructions of the step that computed its first products, the other
    // six under the next step's first 36.  Zero for the tile that does not exist before the first one.
    bf16x8 pB[2], dmB[2], dnB[2];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) { pB[s][kk] = (bf16_t)0.0f; dmB[s][kk] = (bf16_t)0.0f; dnB[s][kk] = (bf16_t)0.0f; }

    // first products of the tile in stage ST -> (m, n, da) in architectural VGPRs, element-wise work of the PREVIOUS
    // tile (registers pm, pn, pda; gate values from stage SP) dealt out between the matrix instructions so that the VALU
    // works under them; then the token contraction of the previous tile, with the first element pairs of THIS tile's
    // element-wise work under its last matrix instructions.
    //   registers 4a+b of m/n/da: token 8a + 4g + b (rows), column j = l32.
    auto step = [&](auto st_c, auto sp_c, f32x16& m, f32x16& n, f32x16& da, const f32x16& pm, const f32x16& pn,
                    const f32x16& pda, bool live, int& nv_next) {
        constexpr int ST = decltype(st_c)::value, SP = decltype(sp_c)::value;
        const unsigned char* sQ = smem_raw + ST * DW_STAGE_B;
        const unsigned char* sG = sQ + TILE_B;
        const unsigned char* pQ = smem_raw + SP * DW_STAGE_B;
        const unsigned char* pG = pQ + TILE_B;
        // the previous tile's gate values, or zeros when there is no previous tile to contract (first step of a slice,
        // phantom steps that pad the loop): a zero gate makes P, dM and dN exactly zero
        const float* pR = live ? reinterpret_cast<const float*>(pG + TILE_B) + wave * 64 : sZero;

        // LDS reads of the first products: the gate values of this tile's first four token rows (for the element pairs
        // converted at the end of this step) and of the previous tile for this lane's 16 token rows (4
        // consecutive rows per 16-byte read), then the operand ring (k-step ks + 2 is requested while ks is consumed).
        // All are issued from inline assembly and waited for by count; the element-wise slices in between are VALU only.
        __builtin_amdgcn_sched_barrier(0);
        u32x4 rvn = lds_read16_async<0>(lds_addr(smem_raw) + (ST * DW_STAGE_B + 2 * TILE_B) + wave * 256 + 16 * g);
        u32x4 rvu[4];
        {
            const unsigned ra = lds_addr(pR) + 16 * g;
            rvu[0] = lds_read16_async<0>(ra);
            rvu[1] = lds_read16_async<32>(ra);
            rvu[2] = lds_read16_async<64>(ra);
            rvu[3] = lds_read16_async<96>(ra);
        }
        u32x4 aq[3], ag[3];
        auto request = [&](auto kc) {
            constexpr int ks = decltype(kc)::value;
            const unsigned a = qaddr ^ (ks << 5);     // the stage goes into the instruction's immediate offset
            aq[ks % 3] = lds_read16_async<ST * DW_STAGE_B>(a);
            ag[ks % 3] = lds_read16_async<ST * DW_STAGE_B + TILE_B>(a);
        };
        request(std::integral_constant<int, 0>{});
        request(std::integral_constant<int, 1>{});
        // The fill of the stage that came free at the barrier (tile k + 2) is issued behind the first reads: its five
        // instructions and their address arithmetic pass while those reads are on their way.
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (TAIL) prepare_tile();     // (the tail instantiation has no registers to spare for the early call)
        nv_next = fire_tile((ST + 2) % DW_NST);
        f32x4 rv[4];
        // Transposed operands of the token contraction (phases 2 and 3 below), in (s, ct) order.  They come from the
        // previous tile, so the first two sets are requested under the last two k-steps of the first products, in the
        // ring slots those no longer need, and have arrived when the contraction starts.
        constexpr int NSET = 2 * CT;
        TrOperand tq[3], tg[3];
        auto request_tr = [&](auto ic) {
            constexpr int idx = decltype(ic)::value;
            constexpr int s = idx / CT, ct = idx % CT;
            tq[idx % 3] = tile_read_cols_async<4096 * s>(lds_addr(pQ), trl, ct);
            tg[idx % 3] = tile_read_cols_async<4096 * s + TILE_B>(lds_addr(pQ), trl, ct);
        };

        // Element-wise work of the previous tile, two elements (register indices 2pr, 2pr+1 of pm/pn/pda) at a time so
        // that no instruction waits on the one just before it, in five slices of at most six VALU instructions; one slice
        // fits under one MFMA (32 cycles).  With sigma = 1/(1+2^(-m log2 e)), B = r sigma, A = m B (= r silu(m)):
        //     P = A n,   dN = A dA,   dM = (B + A (1 - sigma)) (n dA)         [silu'(m) = sigma + silu(m) (1 - sigma)]
        float ex[8][2], sg[8][2], nda[8][2], Av[8][2], Bv[8][2], s1[8][2];
        f32x4 rvn4;                                   // gate values of THIS tile's token rows 4g .. 4g+3 (elements 0..3)
        auto slice_on = [&](auto pc, auto kc, const f32x16& sm, const f32x16& sn, const f32x16& sda, auto gate) {
            constexpr int pr = decltype(pc)::value, k = decltype(kc)::value;
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int i = 2 * pr + u;
                if constexpr (k == 0) {
                    ex[pr][u] = __builtin_amdgcn_exp2f(-LOG2E * sm[i]);
                } else if constexpr (k == 1) {
                    sg[pr][u] = __builtin_amdgcn_rcpf(1.0f + ex[pr][u]);
                    nda[pr][u] = sn[i] * sda[i];
                } else if constexpr (k == 2) {
                    Bv[pr][u] = gate(i) * sg[pr][u];
                    Av[pr][u] = sm[i] * Bv[pr][u];
                    s1[pr][u] = 1.0f - sg[pr][u];
                } else if constexpr (k == 3) {
                    pB[i >> 3][i & 7] = (bf16_t)(Av[pr][u] * sn[i]);
                    dnB[i >> 3][i & 7] = (bf16_t)(Av[pr][u] * sda[i]);
                } else {
                    dmB[i >> 3][i & 7] = (bf16_t)(__builtin_fmaf(Av[pr][u], s1[pr][u], Bv[pr][u]) * nda[pr][u]);
                }
            }
        };
        // The 40 slices of a tile (8 element pairs x 5) are spread over 48 consecutive matrix instructions for d_h = 128
        // (NSL in general): pairs 0 and 1 of THIS tile behind the last 3 CT of this step (the s = 1 half of the
        // contraction, which reads only the operand halves of elements 8..15), pairs 2..7 of the PREVIOUS tile behind
        // this step's first NSL - 3 CT.  Pairs 2 and 3 are done long before the s = 0 half starts, pairs 4..7 before the
        // s = 1 half.  Each matrix instruction so has about one slice behind it; two slices behind one cost the wave
        // more issue time than the instruction's 32 cycles, none leaves the matrix pipe's shadow unused.
        constexpr int NS1 = 3 * KS, NSL = NS1 + 6 * CT, NLATE = 3 * CT, NEARLY = NSL - NLATE;
        static_assert(9 * NEARLY / 30 < NS1, "pairs 2 and 3 must be converted before the s = 0 half of the contraction");
        auto ew_slot = [&](auto kc) {
            constexpr int k = decltype(kc)::value;
            if constexpr (k < NEARLY) {
                static_for<30>([&](auto qc) {
                    constexpr int q = decltype(qc)::value;
                    if constexpr (q * NEARLY / 30 == k)
                        slice_on(std::integral_constant<int, 2 + q / 5>{}, std::integral_constant<int, q % 5>{}, pm, pn, pda,
                                 [&](int i) { return rv[i >> 2][i & 3]; });
                });
            } else {
                static_for<10>([&](auto qc) {
                    constexpr int q = decltype(qc)::value;
                    if constexpr (NEARLY + q * NLATE / 10 == k)
                        slice_on(std::integral_constant<int, q / 5>{}, std::integral_constant<int, q % 5>{}, m, n, da,
                                 [&](int i) { return rvn4[i & 3]; });
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        auto after_slot1 = [&](auto kc) { ew_slot(kc); };

        static_for<KS>([&](auto kc) {
            constexpr int ks = decltype(kc)::value;
            if constexpr (ks + 2 < KS) request(std::integral_constant<int, ks + 2>{});
            if constexpr (ks == KS - 2) request_tr(std::integral_constant<int, 0>{});
            if constexpr (ks == KS - 1) request_tr(std::integral_constant<int, 1>{});
            // reads younger than this k-step's operands: two per later k-step of the ring, four per transposed set
            constexpr int younger = ks + 2 < KS ? 4 : (ks == KS - 2 ? 2 + 4 : 4 + 4);
            if constexpr (ks == 0) {
                lds_wait_n<younger>(aq[0], ag[0], rvu[0], rvu[1], rvu[2], rvu[3]);       // (the gate values are older)
#pragma unroll
                for (int a = 0; a < 4; ++a) rv[a] = __builtin_bit_cast(f32x4, rvu[a]);
                asm volatile("" : "+v"(rvn));     // (older than the reads just waited for; no use of it may move above)
                rvn4 = __builtin_bit_cast(f32x4, rvn);
            } else {
                lds_wait_n<younger>();        // (consumed by asm matrix instructions only)
            }
            const bf16x8 aqv = __builtin_bit_cast(bf16x8, aq[ks % 3]), agv = __builtin_bit_cast(bf16x8, ag[ks % 3]);
            if constexpr (ks == 0) mfma32_vgpr_first_bacc(m, aqv, kB[0]);
            else mfma32_vgpr_acc_bacc(m, aqv, kB[ks]);
            after_slot1(std::integral_constant<int, 3 * ks>{});
            if constexpr (ks == 0) mfma32_vgpr_first_bacc(n, aqv, uB[0]);
            else mfma32_vgpr_acc_bacc(n, aqv, uB[ks]);
            after_slot1(std::integral_constant<int, 3 * ks + 1>{});
            if constexpr (ks == 0) mfma32_vgpr_first(da, agv, vR[0]);
            else mfma32_vgpr_acc(da, agv, vR[ks]);
            after_slot1(std::integral_constant<int, 3 * ks + 2>{});
        });

        // Phases 2 and 3: token contraction of the previous tile, s-major.  A = Q^T / dO^T gathered from the row-major
        // tiles with transposing LDS reads (k-slot (s, g, kk) of the B operands is token 16s + 8(kk/4) + 4g + kk%4; a
        // 16-lane group covers 16 columns c), requested two operand sets ahead.  The s = 0 MFMAs only need the operands
        // phase 1 produced, so elements 8..15 are converted between them.  The region is fenced and contains no other
        // LDS instruction, so the partial LDS waits count exactly the asynchronous reads.
        __builtin_amdgcn_sched_barrier(0);
        {
            static_for<NSET>([&](auto ic) {
                constexpr int idx = decltype(ic)::value;
                constexpr int s = idx / CT, ct = idx % CT;
                if constexpr (idx + 2 < NSET) request_tr(std::integral_constant<int, idx + 2>{});
                constexpr int ahead = (NSET - 1 - idx) < 2 ? (NSET - 1 - idx) : 2;
                lds_tr_wait_n<4 * ahead>(tq[idx % 3], tg[idx % 3]);
                // (element-wise slices behind each matrix instruction: see ew_slot)
                auto after_slot2 = [&](auto kc) {
                    ew_slot(std::integral_constant<int, NS1 + 3 * idx + decltype(kc)::value>{});
                };
                dk[ct] = mfma32(tr_value(tq[idx % 3]), dmB[s], dk[ct]);
                if constexpr (idx == NSET - 1 && !TAIL) prepare_tile();     // scalar work of the next fill, under this MFMA
                after_slot2(std::integral_constant<int, 0>{});
                du[ct] = mfma32(tr_value(tq[idx % 3]), dnB[s], du[ct]);
                after_slot2(std::integral_constant<int, 1>{});
                dv[ct] = mfma32(tr_value(tg[idx % 3]), pB[s], dv[ct]);
                after_slot2(std::integral_constant<int, 2>{});
            });
        }
        __builtin_amdgcn_sched_barrier(0);
        // The first products were written by inline-assembly MFMAs the compiler cannot see.  The 6 CT contraction MFMAs
        // issued since then cover the wait states before the next step's element-wise code reads them; what is still
        // needed is that their registers stay allocated to the end of the step even when nothing reads them (the
        // phantom steps), or the compiler hands them to other values that the late write would overwrite.
        static_assert(KS >= 2 && NSET >= 2 && 6 * CT >= 8, "the contraction MFMAs of a step must cover the hazard window of its first products");
        asm volatile("" :: "v"(m), "v"(n), "v"(da));
    };

    // Pipeline over tiles k = 0 .. nt (step k: first products of tile k, element-wise + contraction of tile k-1).
    // Stage of tile k is k % 4; the two (m, n, da) register sets alternate with the parity of k.  Before step k every
    // wave waits for its own outstanding loads (tiles <= k), then the barrier publishes tile k and retires the stage
    // that tile k+2 is about to overwrite (last read by the contraction of tile k-2 in step k-1).
    f32x16 mA, nA, dA_, mB, nB, dB_;
#pragma unroll
    for (int x = 0; x < 16; ++x) { mA[x] = 0.0f; nA[x] = 0.0f; dA_[x] = 0.0f; mB[x] = 0.0f; nB[x] = 0.0f; dB_[x] = 0.0f; }
    auto sync_step = [&](auto st_c, int nvalid) {
        constexpr int ST = decltype(st_c)::value;
        // All of this wave's loads, not only the older tile's: a partial count (the next tile's loads still in flight)
        // measured no faster.
        wait_vmcnt<0>();
        if constexpr (TAIL) {
            if (nvalid < 32) zero_tail(ST, nvalid);
        }
        // (a bare barrier: the LDS-direct loads were waited for just above, and this wave's LDS reads of the stage that
        // is refilled next were consumed by the matrix instructions of the step before)
        __builtin_amdgcn_s_barrier();
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    // nt + 1 steps (step k contracts tile k-1), in trips of four (one per LDS stage) and a remainder of up to three.
    {
        int k = 0;
        for (; k + 3 <= nt; k += 4) {
            sync_step(I0{}, nv0);
            step(I0{}, I3{}, mA, nA, dA_, mB, nB, dB_, k > 0, nv2);
            sync_step(I1{}, nv1);
            step(I1{}, I0{}, mB, nB, dB_, mA, nA, dA_, true, nv3);
            sync_step(I2{}, nv2);
            step(I2{}, I1{}, mA, nA, dA_, mB, nB, dB_, true, nv0);
            sync_step(I3{}, nv3);
            step(I3{}, I2{}, mB, nB, dB_, mA, nA, dA_, true, nv1);
        }
        if (k <= nt) {
            sync_step(I0{}, nv0);
            step(I0{}, I3{}, mA, nA, dA_, mB, nB, dB_, k > 0, nv2);
            if (k + 1 <= nt) {
                sync_step(I1{}, nv1);
                step(I1{}, I0{}, mB, nB, dB_, mA, nA, dA_, true, nv3);
                if (k + 2 <= nt) {
                    sync_step(I2{}, nv2);
                    step(I2{}, I1{}, mA, nA, dA_, mB, nB, dB_, true, nv0);
                }
            }
        }
    }
    wait_vmcnt<0>();
    __syncthreads();      // every wave is done reading the tile ring, which the epilogue reuses

    // dK^T registers 4a+x of row tile ct: c = 32ct + 8a + 4g + x, column j = l32, i.e. a lane owns runs of 4 c of weight row
    // j.  Stored directly these are 8- or 16-byte pieces scattered over 32 rows per instruction; instead each wave passes
    // one gradient block at a time through a private 16 KB region of the ring (16-byte chunk c16 of row r at chunk
    // c16 ^ r), reads it back row-wise and stores whole rows.  Only this wave touches the region, and LDS operations of
    // one wave complete in order, so no barrier is needed between the three blocks.
    {
        unsigned char* region = smem_raw + wave * 16384;
        const long wsz = (long)gridDim.x * nblk * JB * DH;   // elements of one weight tensor
        const long row0 = (wrow - l32) * DH;                 // first element of this wave's block of rows
        auto store_f32 = [&](const f32x16 (&acc)[CT], float* dst) {      // rows of DH floats, 512-byte rows in LDS
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    f32x4 v;
#pragma unroll
                    for (int x = 0; x < 4; ++x) v[x] = acc[ct][4 * a + x];
                    *reinterpret_cast<f32x4*>(region + l32 * 512 + (((8 * ct + 2 * a + g) ^ l32) << 4)) = v;
                }
            const int c16 = lane & 31;
#pragma unroll
            for (int k = 0; k < 16; ++k) {
                const int row = 2 * k + (lane >> 5);
                if (c16 < DH / 4) {
                    const u32x4 v = *reinterpret_cast<const u32x4*>(region + row * 512 + ((c16 ^ row) << 4));
                    *reinterpret_cast<u32x4*>(dst + row0 + row * DH + c16 * 4) = v;
                }
            }
        };
        auto store_bf16 = [&](const f32x16 (&acc)[CT], bf16_t* dst) {    // rows of DH bf16, 256-byte rows in LDS
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    bf16x4 v;
#pragma unroll
                    for (int x = 0; x < 4; ++x) v[x] = (bf16_t)acc[ct][4 * a + x];
                    *reinterpret_cast<bf16x4*>(region + l32 * 256 + (((4 * ct + a) ^ (l32 & 15)) << 4) + 8 * g) = v;
                }
            const int c16 = lane & 15;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int row = 4 * k + (lane >> 4);
                if (c16 < DH / 8) {
                    const u32x4 v = *reinterpret_cast<const u32x4*>(region + row * 256 + ((c16 ^ (row & 15)) << 4));
                    *reinterpret_cast<u32x4*>(dst + row0 + row * DH + c16 * 8) = v;
                }
            }
        };
        if (p.nslice > 1) {                                  // fp32 partial sums of this token slice
            float* base = p.part + (long)z * 3 * wsz;
            store_f32(dk, base);
            store_f32(du, base + wsz);
            store_f32(dv, base + 2 * wsz);
        } else if (p.out_f32) {                              // one slice: the sums are the gradients
            store_f32(dk, static_cast<float*>(p.out[0]));
            store_f32(du, static_cast<float*>(p.out[1]));
            store_f32(dv, static_cast<float*>(p.out[2]));
        } else {
            store_bf16(dk, static_cast<bf16_t*>(p.out[0]));
            store_bf16(du, static_cast<bf16_t*>(p.out[1]));
            store_bf16(dv, static_cast<bf16_t*>(p.out[2]));
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
static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// Token slices of the dK/dU/dV kernel for a workspace of `ws_bytes`.  One workgroup fits a CU at a time, so a launch
// runs in rounds of CUs workgroups; a workgroup costs its share of the token tiles plus a fixed prologue and epilogue
// (loading its K/U/V blocks, storing 3 x 64 accumulator registers per lane: about 9 tiles' worth).  More slices than
// one are worth it only where one slice leaves CUs idle; with one slice the kernel writes dK, dU, dV itself and neither
// partial sums nor the summing pass exist.  Every further slice adds a set of fp32 partial sums that is written and
// read back once (priced at the time of a token tile per 2.5 MB: about 4 TB/s against 1.25 us per tile).
constexpr int DW_CUS = 256;             // compute units of an MI355X
constexpr long DW_FIXED_TILES = 9;      // prologue + epilogue of a workgroup, in token tiles
constexpr long DW_BYTES_PER_TILE_TIME = 2500000;
static int pick_nslice(const Dims& d, size_t ws_bytes)
{
    const int nblk = d.E * (d.d_e / JB);
    const long cols = (long)((nblk + 3) / 4) * d.Hkuv;
    const long ntile = (long)(d.H / d.Hkuv) * d.B * ((d.S + 31) / 32);
    const size_t slice_b = (size_t)3 * d.Hkuv * d.E * d.d_e * d.d_h * sizeof(float);
    long best = 1, best_cost = -1;
    for (long ns = 1; ns <= 64 && (ns == 1 || ns <= ntile / 8); ++ns) {
        if (ns > 1 && align256((size_t)ns * slice_b) > ws_bytes) break;
        const long rounds = (cols * ns + DW_CUS - 1) / DW_CUS;
        const long cost = rounds * ((ntile + ns - 1) / ns + DW_FIXED_TILES) +
                          (ns > 1 ? ns * (long)(slice_b / DW_BYTES_PER_TILE_TIME) : 0);
        if (best_cost < 0 || cost < best_cost) { best = ns; best_cost = cost; }
    }
    return (int)best;
}

size_t bwd_workspace_bytes_bf16(const Dims& d)
{
    const size_t wsz = (size_t)d.Hkuv * d.E * d.d_e * d.d_h;
    const int ns = pick_nslice(d, ~(size_t)0);
    return ns > 1 ? align256((size_t)ns * 3 * wsz * sizeof(float)) : 0;
}

template <int DH>
static hipError_t launch_bwd_t(const void* Q, const void* K, const void* U, const void* V, const float* R,
                               const void* dO, void* dQ, void* dK, void* dU, void* dV, float* dR, int grad_w_f32,
                               void* ws, size_t ws_bytes, const Dims& d, hipStream_t st, int phases)
{
    hipError_t err = hipSuccess;
    float* part = reinterpret_cast<float*>(ws);
    const int nbe = d.d_e / JB, G = d.H / d.Hkuv;

    if (phases & PH_BWD_DQDR) {
        DqArgs a{(const bf16_t*)Q, (const bf16_t*)dO, (const bf16_t*)K, (const bf16_t*)U, (const bf16_t*)V, R,
                 (bf16_t*)dQ, dR, d.H, G, d.S, d.E, nbe, d.tokmaj};
        const int tokw = 256;
        const int smem = DQ_NST * DQ_STAGE_B + (d.E < GATE_WIN ? d.E : GATE_WIN) * tokw * (int)sizeof(float);
        if (smem > 160 * 1024) return hipErrorInvalidValue;
        static LdsOptIn optin;
        err = ensure_dynamic_lds(optin, (const void*)mhffn_bwd_dqdr_kernel<DH>, smem);
        if (err != hipSuccess) return err;
        dim3 grid((unsigned)d.H, (unsigned)((d.S + tokw - 1) / tokw), (unsigned)d.B);
        hipLaunchKernelGGL((mhffn_bwd_dqdr_kernel<DH>), grid, dim3(512), smem, st, a);
        err = hipGetLastError();
        if (err != hipSuccess) return err;
    }
    const int nslice = pick_nslice(d, ws_bytes);
    if (phases & PH_BWD_DKDUDV) {
        DwArgs a{(const bf16_t*)Q, (const bf16_t*)dO, (const bf16_t*)K, (const bf16_t*)U, (const bf16_t*)V, R, part,
                 {dK, dU, dV}, grad_w_f32, d.B, d.H, G, d.S, d.E, nbe, nslice, d.tokmaj};
        const int smem = DW_NST * DW_STAGE_B + 128;
        static LdsOptIn optin_full, optin_tail;
        err = d.S % 32 == 0 ? ensure_dynamic_lds(optin_full, (const void*)mhffn_bwd_dkdudv_kernel<DH, false>, smem)
                            : ensure_dynamic_lds(optin_tail, (const void*)mhffn_bwd_dkdudv_kernel<DH, true>, smem);
        if (err != hipSuccess) return err;
        const int nblk = d.E * nbe;
        dim3 grid((unsigned)d.Hkuv, (unsigned)((nblk + 3) / 4), (unsigned)nslice);
        if (d.S % 32 == 0)
            hipLaunchKernelGGL((mhffn_bwd_dkdudv_kernel<DH, false>), grid, dim3(256), smem, st, a);
        else
            hipLaunchKernelGGL((mhffn_bwd_dkdudv_kernel<DH, true>), grid, dim3(256), smem, st, a);
        err = hipGetLastError();
        if (err != hipSuccess) return err;
    }
    if ((phases & PH_BWD_REDUCE) && nslice > 1) {
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
                           void* dQ, void* dK, void* dU, void* dV, float* dR, int grad_w_f32, void* ws, size_t ws_bytes,
                           const Dims& d, hipStream_t st, int phases)
{
    switch (d.d_h) {
        case 64: return launch_bwd_t<64>(Q, K, U, V, R, dO, dQ, dK, dU, dV, dR, grad_w_f32, ws, ws_bytes, d, st, phases);
        case 96: return launch_bwd_t<96>(Q, K, U, V, R, dO, dQ, dK, dU, dV, dR, grad_w_f32, ws, ws_bytes, d, st, phases);
        case 128: return launch_bwd_t<128>(Q, K, U, V, R, dO, dQ, dK, dU, dV, dR, grad_w_f32, ws, ws_bytes, d, st, phases);
    }
    return hipErrorInvalidValue;
}

}  // namespace mhffn
