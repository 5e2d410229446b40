/* C ABI of the MI355X (gfx950) fused multi-head FFN library, libmhffn_hip.so.
 *
 *   O[b,h,t,:] = sum_e R[b,h,t,e] * ( (silu(Q[b,h,t,:] K[hk,e]^T) * (Q[b,h,t,:] U[hk,e]^T)) V[hk,e] ),   hk = h / (H/Hkuv)
 *
 * These entry points are what the reference's Python operator boundary binds for this path:
 *   - kernels/triton/flash_mlp_moe.py:739-868   FlashMLPFunction.forward / .backward (Triton launches)
 *   - kernels/thunderkittens/flash_ffn_moe.cu:938-1007, 1012-1133  flashffn_moe_forward / flashffn_moe_backward
 *     (the pybind11 launchers, exported at :1135-1138)
 *
 * Conventions for every call:
 *   - all tensor pointers are DEVICE pointers to contiguous row-major buffers owned by the caller, 16-byte aligned:
 *       Q, O, dO, dQ   [B, H, S, d_h]
 *       K, U, V        [Hkuv, E, d_e, d_h]        dK, dU, dV same shape
 *       R, dR          [B, H, S, E]   always float32 (models/flashmhf/modeling_mhffnmoe.py:384-386)
 *   - `dtype` is the element type of Q, K, U, V, O, dO, dQ (MHFFN_DTYPE_*).
 *   - the library never allocates, never synchronises and never throws; work is enqueued on `stream`
 *     (a hipStream_t passed as void*, NULL = the default stream).
 *   - return value: MHFFN_OK or a negative MHFFN_ERR_* code; all argument checks happen before any launch.
 *   - `workspace` is caller-provided device scratch of at least the size the matching *_workspace_bytes()
 *     call reports (16-byte aligned).  Its contents are undefined after the call.
 */
#ifndef MHFFN_H_
#define MHFFN_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    MHFFN_DTYPE_BF16 = 0,
    MHFFN_DTYPE_F32  = 1
};

enum {
    MHFFN_OK               =  0,
    MHFFN_ERR_NULL_POINTER = -1,
    MHFFN_ERR_DTYPE        = -2,  /* reference: TypeError, flash_mlp_moe.py:761-766; TORCH_CHECK flash_ffn_moe.cu:943-945 */
    MHFFN_ERR_HEAD_DIM     = -3,  /* reference: assert head_dim == 128, flash_ffn_moe.cu:956 */
    MHFFN_ERR_EXPERT_DIM   = -4,  /* reference: ValueError, flash_mlp_moe.py:758-759; assert flash_ffn_moe.cu:958 */
    MHFFN_ERR_SHAPE        = -5,  /* non-positive extent, H not a multiple of Hkuv, gate kernels with E > 64 */
    MHFFN_ERR_WORKSPACE    = -6,  /* workspace missing or smaller than *_workspace_bytes() */
    MHFFN_ERR_LAUNCH       = -7,  /* hipGetLastError() after a launch */
    MHFFN_ERR_ALIGNMENT    = -8,  /* a tensor or workspace pointer is not 16-byte aligned */
    MHFFN_ERR_STATIC_SCRATCH = -9 /* mhffn_bwd_static only: the problem needs more than MHFFN_STATIC_SCRATCH_BYTES */
};

/* Problem extents, shared by every call. */
typedef struct mhffn_dims {
    int B;      /* batch */
    int H;      /* q heads */
    int Hkuv;   /* K/U/V heads; H % Hkuv == 0 (grouped "GQ-FFN", flash_mlp_moe.py:194,222) */
    int S;      /* tokens per (batch, head) */
    int d_h;    /* head dim */
    int E;      /* experts (sub-networks) per head (bf16: at most 64) */
    int d_e;    /* rows of K/U/V per expert */
} mhffn_dims;

/* Human-readable text for a return code (static storage). */
const char* mhffn_strerror(int code);

/* 1 if kernels exist for (d_h, d_e, dtype), else 0.  bf16 (MFMA kernels): d_h in {64, 96, 128}, d_e % 32 == 0, any E.
 * float32 (correctness instantiation, plain FMA): d_h a multiple of 8 up to 128, any d_e, any E.
 * Replaces the reference's shape gates (flash_mlp_moe.py:758, flash_ffn_moe.cu:956-958, 1037). */
int mhffn_is_supported(int d_h, int d_e, int dtype);

/* Checks extents and dtype only (no pointers, no GPU).  Returns MHFFN_OK or the error the launch would return. */
int mhffn_check_dims(const mhffn_dims* dims, int dtype);

/* Scratch bytes needed by mhffn_fwd / mhffn_bwd for these extents.  0 is a valid answer, not only the answer for invalid
 * extents (ask mhffn_check_dims for those): the forward never needs scratch, and the bfloat16 backward needs none where
 * its dK/dU/dV kernel runs as one token slice (e.g. the 370M and 1.3B layers); `workspace` may then be NULL. */
size_t mhffn_fwd_workspace_bytes(const mhffn_dims* dims, int dtype);
size_t mhffn_bwd_workspace_bytes(const mhffn_dims* dims, int dtype);

/* Forward.  Replaces the launch in FlashMLPFunction.forward (flash_mlp_moe.py:777-790) and
 * flashffn_moe_forward (flash_ffn_moe.cu:938-1007).  O is written, nothing else. */
int mhffn_fwd(const void* Q, const void* K, const void* U, const void* V, const float* R,
              void* O,
              void* workspace, size_t workspace_bytes,
              const mhffn_dims* dims, int dtype, void* stream);

/* Backward.  Replaces the two launches in FlashMLPFunction.backward (flash_mlp_moe.py:832-866) and
 * flashffn_moe_backward (flash_ffn_moe.cu:1012-1133).
 *   dQ has `dtype`; dR is float32 (flash_mlp_moe.py:811).
 *   dK, dU, dV have `grad_w_dtype`: MHFFN_DTYPE_BF16 as the Triton wrapper allocates them
 *   (flash_mlp_moe.py:808-810) or MHFFN_DTYPE_F32 as the ThunderKittens wrapper does
 *   (flash_ffn_moe_torch.py:18-20).  They are overwritten (no need to zero them first). */
int mhffn_bwd(const void* Q, const void* K, const void* U, const void* V, const float* R,
              const void* dO,
              void* dQ, void* dK, void* dU, void* dV, float* dR,
              int grad_w_dtype,
              void* workspace, size_t workspace_bytes,
              const mhffn_dims* dims, int dtype, void* stream);

/* Phase-selectable variants for profiling: run only the kernels whose bit is set in `phases`, on a workspace that an
 * earlier full call with the same arguments has filled.  mhffn_fwd == mhffn_fwd_phases(..., MHFFN_FWD_ALL) and
 * mhffn_bwd == mhffn_bwd_phases(..., MHFFN_BWD_ALL).  They exist so a benchmark can bracket one kernel with HIP
 * events on the launch stream; the reference has no counterpart (its kernels are launched one per Python call,
 * flash_mlp_moe.py:832-866).  A mask with a bit outside MHFFN_FWD_ALL / MHFFN_BWD_ALL returns MHFFN_ERR_SHAPE (the bit
 * values are not stable across versions of this header: pass the names, not numbers). */
enum {
    MHFFN_FWD_MAIN = 1, MHFFN_FWD_ALL = 1,
    MHFFN_BWD_DQDR = 1, MHFFN_BWD_DKDUDV = 2, MHFFN_BWD_REDUCE = 4, MHFFN_BWD_ALL = 7
};
int mhffn_fwd_phases(const void* Q, const void* K, const void* U, const void* V, const float* R,
                     void* O, void* workspace, size_t workspace_bytes,
                     const mhffn_dims* dims, int dtype, void* stream, int phases);
int mhffn_bwd_phases(const void* Q, const void* K, const void* U, const void* V, const float* R,
                     const void* dO,
                     void* dQ, void* dK, void* dU, void* dV, float* dR,
                     int grad_w_dtype,
                     void* workspace, size_t workspace_bytes,
                     const mhffn_dims* dims, int dtype, void* stream, int phases);

/* Token-major variants: Q, O, dO, dQ are [B, S, H, d_h] (MHFFN_TOKENS_BSHD) -- the layout the caller's projections
 * produce and consume -- instead of [B, H, S, d_h] (MHFFN_TOKENS_BHSD, what the calls above use).  K, U, V, R, dR and all
 * other conventions are unchanged; results are identical to the [B, H, S, d_h] calls on the transposed tensors.
 * With them the caller drops the two transposes-with-copy around the operator
 * (models/flashmhf/modeling_mhffnmoe.py:374 `Q_multihead.transpose(1, 2).contiguous()` and
 * :408 `.transpose(1, 2).contiguous().view(batch_size, seq_len, hidden_size)`).  `phases` as in the *_phases calls. */
enum {
    MHFFN_TOKENS_BHSD = 0,
    MHFFN_TOKENS_BSHD = 1
};
int mhffn_fwd_layout(const void* Q, const void* K, const void* U, const void* V, const float* R,
                     void* O, void* workspace, size_t workspace_bytes,
                     const mhffn_dims* dims, int dtype, int token_layout, void* stream, int phases);
int mhffn_bwd_layout(const void* Q, const void* K, const void* U, const void* V, const float* R,
                     const void* dO,
                     void* dQ, void* dK, void* dU, void* dV, float* dR,
                     int grad_w_dtype,
                     void* workspace, size_t workspace_bytes,
                     const mhffn_dims* dims, int dtype, int token_layout, void* stream, int phases);

/* Backward for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc) and so have no workspace to hand to mhffn_bwd.  It has no counterpart in the reference, whose
 * wrappers allocate with torch on every call (flash_mlp_moe.py:806-811, flash_ffn_moe_torch.py:17-21).
 * Same arguments, kernels and results as mhffn_bwd_layout(..., MHFFN_BWD_ALL) without the workspace pair: the token-slice
 * partial sums of dK, dU, dV live in a fixed array of MHFFN_STATIC_SCRATCH_BYTES that is part of the library's device
 * code (each GPU the library runs on holds one copy until the process ends).  The call allocates nothing and frees
 * nothing; its first call on a device looks the array's address up once.
 *   - bfloat16: the dK/dU/dV kernel runs with as many token slices as the array holds partial sums for (fewer than
 *     mhffn_bwd would use on some problems: dK, dU, dV then differ from mhffn_bwd's in the last float32 bits of the
 *     partial sums' order, and the kernel fills the GPU less well); with a single slice it needs no partial sums, so
 *     no bfloat16 problem is refused.
 *   - float32 (the correctness instantiation): problems whose mhffn_bwd_workspace_bytes() exceed the array return
 *     MHFFN_ERR_STATIC_SCRATCH before any launch.
 *   - all calls on one GPU share the array: calls that overlap in time on one GPU (two streams, two threads) race.
 *     Nothing in it has to start at zero (every element read was written by the same call), so it is never cleared. */
#define MHFFN_STATIC_SCRATCH_BYTES (96u << 20)
int mhffn_bwd_static(const void* Q, const void* K, const void* U, const void* V, const float* R,
                     const void* dO,
                     void* dQ, void* dK, void* dU, void* dV, float* dR,
                     int grad_w_dtype,
                     const mhffn_dims* dims, int dtype, int token_layout, void* stream);

/* Head prologue of the block: what the caller does between its projection and the operator
 * (models/flashmhf/modeling_mhffnmoe.py:371-372 per-head RMSNorm, class at :97-135; :384-386 expert gate), in one pass
 * over the projected heads instead of a dozen element-wise passes plus a float32 copy of Q:
 *
 *     u = X * rsqrt(mean(X^2 over d_h) + eps)        y = bf16(u * norm_weight[h])          (skipped when norm_weight is NULL)
 *     z = y . router[h]  (float32)                   s = sigmoid(z)       R = s / max(sum_e s, 1e-20)
 *
 *   X, Qn, dX       [B, S, H, d_h] bfloat16: the projection's own memory layout; Qn is the Q to hand to
 *                   mhffn_fwd_layout(..., MHFFN_TOKENS_BSHD, ...).  With norm_weight NULL, Q is X itself and Qn is not
 *                   touched (may be NULL).
 *   norm_weight     [H, d_h] float32 or NULL;  router [H, d_h, E] float32;  R, dR [B, H, S, E] float32.
 *   dQ              gradient with respect to y, bfloat16, in the layout named by dq_token_layout (MHFFN_TOKENS_*).
 *   d_norm_weight   [H, d_h] float32 (ignored when norm_weight is NULL), d_router [H, d_h, E] float32: the kernel ADDS
 *                   its sums over all tokens to what the buffers hold (atomic float adds, so the last bits depend on
 *                   the order waves finish in); the caller zero-fills them for a plain gradient.
 * Only dims->B, H, S, d_h, E are read (d_h 64, 96 or 128; E <= 64; B and H at most 65535).  No workspace. */
int mhffn_gate_fwd(const void* X, const float* norm_weight, float eps, const float* router,
                   void* Qn, float* R, const mhffn_dims* dims, void* stream);
int mhffn_gate_bwd(const void* X, const float* norm_weight, float eps, const float* router,
                   const void* dQ, int dq_token_layout, const float* dR,
                   void* dX, float* d_norm_weight, float* d_router, const mhffn_dims* dims, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MHFFN_H_ */
