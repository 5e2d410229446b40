"""Drop-in for the reference's ``kernels/triton/flash_mlp_moe.py`` operator boundary
(``FlashMLPFunction`` :739-868, ``FlashMLPMoE`` :871-903), backed by hand-written gfx950 HIP kernels.

    from flashmhf_amd.flash_mlp_moe import FlashMLPMoE
    O = FlashMLPMoE()(Q, K, U, V, R)      # Q [B,H,S,d_h] bf16; K,U,V [Hkuv,E,d_e,d_h] bf16; R [B,H,S,E] fp32

Same call signature, tensor contract, saved tensors (Q, K, U, V, R only -- no activations) and exception types.
Differences, all widening: d_e may be any multiple of 32 (the reference needs 64, :758), the sequence length is
free, R's gradient is exact fp32 instead of bf16-rounded (:542), and all-float32 tensors are accepted (slow exact path).

Q may also be the transposed view of a contiguous [B,S,H,d_h] tensor -- what ``w_self(x).view(B,S,H,d_h).transpose(1,2)``
is before the caller's ``.contiguous()`` (models/flashmhf/modeling_mhffnmoe.py:362,374).  The kernels then read it in place
and O (and dQ) come back in the same token-major layout, so ``O.transpose(1,2).contiguous().view(B,S,hid)`` (:408) copies
nothing.
"""
import contextlib
import functools

import torch

from . import _capi


@functools.lru_cache(maxsize=512)
def _plan(B, H, Hk, S, dh, E, de, code):
    """(extents struct, forward workspace bytes, backward workspace bytes) of one problem shape, validated once by the
    library (raises the reference's exception types); later calls with the same shape cost a dictionary lookup."""
    L = _capi.lib()
    dims = _capi.Dims(B, H, Hk, S, dh, E, de)
    _capi.raise_for_code(L.mhffn_check_dims(dims, code), "mhffn")
    return dims, L.mhffn_fwd_workspace_bytes(dims, code), L.mhffn_bwd_workspace_bytes(dims, code)


def _plan_for(Q, K):
    B, H, S, dh = Q.shape
    Hk, E, de, dh2 = K.shape
    if dh2 != dh:
        raise RuntimeError(f"head dim mismatch: Q has {dh}, K has {dh2}")
    return _plan(B, H, Hk, S, dh, E, de, _capi.torch_dtype_code(Q.dtype))


def _check_inputs(Q, K, U, V, R):
    if Q.dim() != 4 or K.dim() != 4 or R.dim() != 4:
        raise RuntimeError("expected Q [B,H,S,d_h], K/U/V [Hkuv,E,d_e,d_h], R [B,H,S,E]")
    expected = (torch.bfloat16, torch.float32)     # float32 = the correctness instantiation (a widening over the reference)
    if Q.dtype not in expected or K.dtype != Q.dtype or V.dtype != Q.dtype or U.dtype != Q.dtype:
        raise TypeError(
            f"FlashMLPFunction expects all inputs in {expected[0]} (or all in {expected[1]}), got"
            f" Q={Q.dtype}, K={K.dtype}, V={V.dtype}, U={U.dtype}")
    if R.dtype != torch.float32:
        raise TypeError(f"R must be float32 (the router gate is computed in fp32), got {R.dtype}")
    if U.shape != K.shape or V.shape != K.shape:
        raise RuntimeError(f"K, U, V must share one shape, got {tuple(K.shape)}, {tuple(U.shape)}, {tuple(V.shape)}")
    if R.shape != (*Q.shape[:3], K.shape[1]):
        raise RuntimeError(f"R must be [B,H,S,E] = {(*Q.shape[:3], K.shape[1])}, got {tuple(R.shape)}")
    if Q.dtype == torch.bfloat16 and K.shape[2] % 32 != 0:
        raise ValueError(f"Expert dimension {K.shape[2]} must be divisible by 32")
    if not Q.is_cuda:
        raise RuntimeError("flashmhf_amd runs on the GPU only; there is no CPU path")
    for name, t in (("Q", Q), ("K", K), ("U", U), ("V", V), ("R", R)):
        if t.device != Q.device:
            raise RuntimeError(f"{name} is on {t.device}, Q on {Q.device}")


def _token_layout(Q):
    """(layout code, tensor to pass): [B,H,S,d_h] contiguous, or the transposed view of a contiguous [B,S,H,d_h]."""
    if Q.is_contiguous():
        return _capi.TOKENS_BHSD, Q
    if Q.transpose(1, 2).is_contiguous():
        return _capi.TOKENS_BSHD, Q
    return _capi.TOKENS_BHSD, Q.contiguous()


def _as_layout(t, layout):
    """`t` ([B,H,S,d_h] logical shape) with the memory layout `layout`, copying only if it has another one."""
    if layout == _capi.TOKENS_BSHD:
        return t if t.transpose(1, 2).is_contiguous() else t.transpose(1, 2).contiguous().transpose(1, 2)
    return t.contiguous()


_NO_GUARD = contextlib.nullcontext()


def _ws(nbytes, device):
    """(pointer, size) of a workspace: a null pointer where the launch needs none."""
    if nbytes == 0:
        return None, 0
    return torch.empty(nbytes, dtype=torch.uint8, device=device), nbytes


def _device_guard(device):
    """The library launches on the current device: switch only when the tensors live on another one."""
    return _NO_GUARD if device.index == torch.cuda.current_device() else torch.cuda.device(device)


def mhffn_forward(Q, K, U, V, R):
    """Launches the fused forward on the current stream and returns O (same shape and dtype as Q)."""
    _check_inputs(Q, K, U, V, R)
    layout, Q = _token_layout(Q)
    K, U, V, R = (t.contiguous() for t in (K, U, V, R))
    dims, fwd_bytes, _ = _plan_for(Q, K)
    O = torch.empty_strided(Q.shape, Q.stride(), dtype=Q.dtype, device=Q.device)
    ws, ws_bytes = _ws(fwd_bytes, Q.device)
    with _device_guard(Q.device):
        rc = _capi.lib().mhffn_fwd_layout(Q.data_ptr(), K.data_ptr(), U.data_ptr(), V.data_ptr(), R.data_ptr(),
                                          O.data_ptr(), ws.data_ptr() if ws is not None else None, ws_bytes, dims,
                                          _capi.torch_dtype_code(Q.dtype), layout,
                                          torch.cuda.current_stream().cuda_stream, _capi.FWD_ALL)
    _capi.raise_for_code(rc, "mhffn_fwd")
    return O


def mhffn_backward(Q, K, U, V, R, dO, grad_w_dtype=torch.bfloat16):
    """Launches the fused backward; returns (dQ, dK, dU, dV, dR).  dQ has Q's dtype, dR is fp32,
    dK/dU/dV have ``grad_w_dtype`` (bf16 as flash_mlp_moe.py:808-810, or fp32 as flash_ffn_moe_torch.py:18-20)."""
    _check_inputs(Q, K, U, V, R)
    assert dO.shape == Q.shape, "grad_output shape should be the same as Q"
    layout, Q = _token_layout(Q)
    K, U, V, R = (t.contiguous() for t in (K, U, V, R))
    dO = _as_layout(dO.to(Q.dtype), layout)
    dims, _, bwd_bytes = _plan_for(Q, K)
    dQ = torch.empty_strided(Q.shape, Q.stride(), dtype=Q.dtype, device=Q.device)
    dK, dU, dV = (torch.empty(K.shape, dtype=grad_w_dtype, device=K.device) for _ in range(3))
    dR = torch.empty_like(R)
    ws, ws_bytes = _ws(bwd_bytes, Q.device)
    with _device_guard(Q.device):
        rc = _capi.lib().mhffn_bwd_layout(Q.data_ptr(), K.data_ptr(), U.data_ptr(), V.data_ptr(), R.data_ptr(),
                                          dO.data_ptr(), dQ.data_ptr(), dK.data_ptr(), dU.data_ptr(), dV.data_ptr(),
                                          dR.data_ptr(), _capi.torch_dtype_code(grad_w_dtype),
                                          ws.data_ptr() if ws is not None else None, ws_bytes, dims,
                                          _capi.torch_dtype_code(Q.dtype), layout,
                                          torch.cuda.current_stream().cuda_stream, _capi.BWD_ALL)
    _capi.raise_for_code(rc, "mhffn_bwd")
    return dQ, dK, dU, dV, dR


class FlashMLPFunction(torch.autograd.Function):
    """forward(ctx, Q, K, U, V, R) -> O ; backward(ctx, dO) -> (dQ, dK, dU, dV, dR).
    Mirrors kernels/triton/flash_mlp_moe.py:739-868."""

    @staticmethod
    def forward(ctx, Q, K, U, V, R):
        O = mhffn_forward(Q, K, U, V, R)
        ctx.save_for_backward(Q, K, U, V, R)
        return O

    @staticmethod
    def backward(ctx, grad_output):
        Q, K, U, V, R = ctx.saved_tensors
        assert grad_output.shape == Q.shape, "grad_output shape should be the same as Q"
        return mhffn_backward(Q, K, U, V, R, grad_output, grad_w_dtype=K.dtype)


class FlashMLPMoE(torch.nn.Module):
    """Stateless module, ``forward(Q, K, U, V, R) -> O``.  Mirrors kernels/triton/flash_mlp_moe.py:871-903."""

    def __init__(self):
        super().__init__()

    def forward(self, Q, K, U, V, R):
        return FlashMLPFunction.apply(Q, K, U, V, R)
