"""Head prologue of the MH-FFN block as one HIP pass each way: per-head RMSNorm of the projected heads
(models/flashmhf/modeling_mhffnmoe.py:97-135, applied at :371-372) and the expert gate
``R = sigmoid(Q router) / max(sum_e, 1e-20)`` (:384-386).

    Q, R = head_norm_gate(x4, norm_weight, router, eps)      # x4 [B,S,H,d_h] bf16 contiguous

``Q`` is the [B,H,S,d_h] *view* of a [B,S,H,d_h] buffer -- the token-major layout the fused operator reads in place --
and ``R`` is [B,H,S,E] float32.  With ``norm_weight=None`` no normalisation happens and Q is a view of ``x4`` itself.
The backward takes dQ (either layout) and dR and returns dx4, d_norm_weight and d_router, recomputing the forward from
``x4``: nothing but the inputs is saved.  bfloat16 only, d_h in {64, 96, 128}, E <= 64; no CPU path.
"""
import torch

from . import _capi


def _check(x4, norm_weight, router):
    if x4.dim() != 4 or router.dim() != 3:
        raise RuntimeError("expected x [B,S,H,d_h] and router [H,d_h,E]")
    if x4.dtype != torch.bfloat16:
        raise TypeError(f"head_norm_gate expects bfloat16 heads, got {x4.dtype}")
    B, S, H, dh = x4.shape
    if router.shape[:2] != (H, dh):
        raise RuntimeError(f"router must be [H,d_h,E] = [{H},{dh},E], got {tuple(router.shape)}")
    if norm_weight is not None and norm_weight.shape != (H, dh):
        raise RuntimeError(f"norm_weight must be [H,d_h] = [{H},{dh}], got {tuple(norm_weight.shape)}")
    if not x4.is_cuda:
        raise RuntimeError("flashmhf_amd runs on the GPU only; there is no CPU path")
    return _capi.Dims(B, H, H, S, dh, router.shape[2], 32)


def _ptr(t):
    return None if t is None else t.data_ptr()


class HeadNormGateFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x4, norm_weight, router, eps):
        dims = _check(x4, norm_weight, router)
        x4 = x4.contiguous()
        wn = None if norm_weight is None else norm_weight.detach().float().contiguous()
        wr = router.detach().float().contiguous()
        qn = torch.empty_like(x4) if wn is not None else None
        R = torch.empty(dims.B, dims.H, dims.S, dims.E, dtype=torch.float32, device=x4.device)
        rc = _capi.lib().mhffn_gate_fwd(x4.data_ptr(), _ptr(wn), float(eps), wr.data_ptr(), _ptr(qn), R.data_ptr(),
                                        dims, torch.cuda.current_stream(x4.device).cuda_stream)
        _capi.raise_for_code(rc, "mhffn_gate_fwd")
        ctx.save_for_backward(x4, norm_weight, router, wn, wr)
        ctx.eps = float(eps)
        Q = (qn if qn is not None else x4).transpose(1, 2)
        return Q, R

    @staticmethod
    def backward(ctx, dQ, dR):
        x4, norm_weight, router, wn, wr = ctx.saved_tensors
        dims = _check(x4, norm_weight, router)
        if dQ is None:
            dQ = torch.zeros_like(x4).transpose(1, 2)
        if dR is None:
            dR = torch.zeros(dims.B, dims.H, dims.S, dims.E, dtype=torch.float32, device=x4.device)
        if dQ.transpose(1, 2).is_contiguous():
            layout = _capi.TOKENS_BSHD
        else:
            layout, dQ = _capi.TOKENS_BHSD, dQ.contiguous()
        dR = dR.float().contiguous()
        dx = torch.empty_like(x4)
        dwn = None if wn is None else torch.zeros_like(wn)
        dwr = torch.zeros_like(wr)
        rc = _capi.lib().mhffn_gate_bwd(x4.data_ptr(), _ptr(wn), ctx.eps, wr.data_ptr(), dQ.data_ptr(), layout,
                                        dR.data_ptr(), dx.data_ptr(), _ptr(dwn), dwr.data_ptr(), dims,
                                        torch.cuda.current_stream(x4.device).cuda_stream)
        _capi.raise_for_code(rc, "mhffn_gate_bwd")
        return (dx, None if dwn is None else dwn.to(norm_weight.dtype), dwr.to(router.dtype), None)


def head_norm_gate(x4, norm_weight, router, eps=1e-6):
    return HeadNormGateFunction.apply(x4, norm_weight, router, eps)
