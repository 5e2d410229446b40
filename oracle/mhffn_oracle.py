"""CPU restatement of the reference's eager multi-head FFN.  TEST INFRASTRUCTURE ONLY.

This file is the checker the HIP kernels are compared against; it is never the thing
measured or shipped.  Every function cites the reference lines it restates.

    forward, per (b, h, t), q = Q[b,h,t,:], expert e, kuv-head hk = h // G:
        m_e = K[hk,e] q ; n_e = U[hk,e] q ; a_e = silu(m_e) * n_e ; o_e = V[hk,e]^T a_e
        O[b,h,t,:] = sum_e R[b,h,t,e] * o_e

Pinning status (what fixes each function independently of this file's own formulas):
  * mhffn_forward            -- library routines (torch.matmul, F.silu); the E=1, R=1 case equals
                                F.linear(silu(F.linear(q,K)) * F.linear(q,U), V^T); scalar C loops in
                                oracle/mhffn_scalar.c; pure-Python brute force on tiny shapes.
  * mhffn_backward (analytic)-- torch.autograd of mhffn_forward in fp64, torch.autograd.gradcheck,
                                central finite differences, and the scalar C backward.
  * tk_ground_truth          -- equals mhffn_forward up to rounding (same closed form).
  * bf16_eager_autograd      -- torch.autograd of mhffn_forward (pinned above) on bf16 leaves; its gradients stay within
                                the bf16 bar of the fp64 analytic backward on the reference script's shapes.
  * router_gate              -- hand-computed rows (logits (0, ln 3) -> (0.4, 0.6), which a softmax misses by 0.15), the
                                zero-router and all-saturated (clamp) cases, per-head routers with swapped experts.
  * mhffn_layer_forward      -- an independent per-head, per-expert F.linear / torch.sigmoid / F.silu composition with
                                E > 1 and a W_r whose columns all differ, so a swapped [H,E] view, a softmax gate or a
                                transposed projection fails.
  * mhffn_block_forward      -- library routines around mhffn_forward; with E = 1 (gate identically 1) and no
                                RMSNorm it equals F.linear -> per-head SwiGLU via F.linear -> F.linear; the per-head
                                RMSNorm equals F.rms_norm over d_h times the per-head weight; and it agrees with the
                                independently written flashmhf_amd.mhffn_layer.MHFFNLayer (einsum gate, module
                                projections) run on the same eager operator.
  * head_norm_gate           -- F.rms_norm over d_h times the per-head weight, torch.sigmoid and a plain sum (library
                                routines); rows of R sum to 1; a zero router gives R = 1/E; its gradients are
                                torch.autograd's and are checked by gradcheck in fp64.
The reference holds no golden vectors for this path (it has no tests with stored data), so the
vectors under tests/golden/ are produced by this oracle after it passed the checks above.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def repeat_kuv(w: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[H_kuv,E,d_e,d_h] -> [H_kuv*n_rep,E,d_e,d_h]; q-head i uses kuv-head i // n_rep.

    Restates models/flashmhf/modeling_mhffnmoe.py:224-253 (the 4-D branch, :246-251).
    """
    if n_rep == 1:
        return w
    return torch.repeat_interleave(w, n_rep, dim=0)


def mhffn_forward(Q, K, U, V, R, *, compute_dtype=None, out_dtype=None):
    """Eager expert loop, models/flashmhf/modeling_mhffnmoe.py:412-431 with s0=s1=s2=1 (:270-279).

    Q [B,H,S,d_h]; K,U,V [H_kuv,E,d_e,d_h]; R [B,H,S,E].  ``compute_dtype`` is the dtype the matmuls
    and the activation run in (the reference runs them in x.dtype); each expert's result is cast to
    fp32 (fp64 when compute_dtype is fp64) before the multiplication by R and the sum over experts
    (:425), and the sum is cast to ``out_dtype`` at the end (:427).
    """
    compute_dtype = compute_dtype or Q.dtype
    out_dtype = out_dtype or compute_dtype
    acc_dtype = torch.float64 if compute_dtype == torch.float64 else torch.float32
    H, Hk = Q.shape[1], K.shape[0]
    assert H % Hk == 0
    G = H // Hk
    q = Q.to(compute_dtype)
    k = repeat_kuv(K.to(compute_dtype), G)
    u = repeat_kuv(U.to(compute_dtype), G)
    v = repeat_kuv(V.to(compute_dtype), G)
    r = R.to(acc_dtype)
    out = torch.zeros(Q.shape, dtype=acc_dtype, device=Q.device)
    for e in range(K.shape[1]):
        w = q @ k[:, e].transpose(1, 2)                 # [B,H,S,d_e]   (:418)
        w = F.silu(w)                                    # (:419)
        w = w * (q @ u[:, e].transpose(1, 2))            # (:420)
        out += (w @ v[:, e]).to(acc_dtype) * r[..., e:e + 1]   # (:425)
    return out.to(out_dtype)


def tk_ground_truth(Q, K, U, V, R):
    """kernels/thunderkittens/run_from_python.py:19-24 -- the reference's own 5-line check (H == H_kuv)."""
    O = torch.zeros_like(Q)
    for e in range(K.shape[1]):
        oi = (F.silu(Q @ K[:, e].transpose(1, 2)) * (Q @ U[:, e].transpose(1, 2))) @ V[:, e]
        O = O + (oi * R[..., e:e + 1]).to(O.dtype)
    return O


def mhffn_backward(Q, K, U, V, R, dO, *, compute_dtype=torch.float64):
    """Analytic backward, kernels/triton/flash_mlp_moe.py:401-414 extended by the R factor
    (:534-536 for dR/dM/dN, :720-729 for dV/dK/dU).

        dA = dO V^T ; dR_e = sum_j dA*silu(M)*N ; dN = R_e*dA*silu(M)
        dM = R_e*dA*N*silu'(M), silu'(x) = sig(x) + x*sig(x)*(1-sig(x))      (:531)
        dQ = sum_e dM K_e + dN U_e ; dK_e = dM^T Q ; dU_e = dN^T Q ; dV_e = (R_e*silu(M)*N)^T dO
    dK/dU/dV are summed over batch, tokens and the G q-heads that share a kuv-head.
    Returns (dQ, dK, dU, dV, dR) in ``compute_dtype``.
    """
    cd = compute_dtype
    B, H, S, dh = Q.shape
    Hk, E, de, _ = K.shape
    G = H // Hk
    q, g, r = Q.to(cd), dO.to(cd), R.to(cd)
    k, u, v = (repeat_kuv(w.to(cd), G) for w in (K, U, V))
    dQ = torch.zeros_like(q)
    dK = torch.zeros((H, E, de, dh), dtype=cd)
    dU = torch.zeros_like(dK)
    dV = torch.zeros_like(dK)
    dR = torch.zeros_like(r)
    for e in range(E):
        m = q @ k[:, e].transpose(1, 2)
        n = q @ u[:, e].transpose(1, 2)
        sig = torch.sigmoid(m)
        s = m * sig
        dA = g @ v[:, e].transpose(1, 2)
        re = r[..., e:e + 1]
        dR[..., e] = (dA * s * n).sum(-1)
        dN = re * dA * s
        dM = re * dA * n * (sig + s * (1 - sig))
        dQ += dM @ k[:, e] + dN @ u[:, e]
        dK[:, e] = (dM.transpose(2, 3) @ q).sum(0)
        dU[:, e] = (dN.transpose(2, 3) @ q).sum(0)
        dV[:, e] = ((re * s * n).transpose(2, 3) @ g).sum(0)
    fold = lambda w: w.view(Hk, G, E, de, dh).sum(1)
    return dQ, fold(dK), fold(dU), fold(dV), dR


def mhffn_autograd(Q, K, U, V, R, dO, *, compute_dtype=torch.float64):
    """Gradients of mhffn_forward by torch.autograd (the cross-check for mhffn_backward)."""
    leaves = [t.detach().to(compute_dtype).requires_grad_(True) for t in (Q, K, U, V, R)]
    out = mhffn_forward(*leaves, compute_dtype=compute_dtype)
    grads = torch.autograd.grad(out, leaves, dO.to(out.dtype))
    return out.detach(), grads


def bf16_eager_autograd(Q, K, U, V, R, dO):
    """The gradients the reference's eager path itself produces in bf16: the expert loop of
    models/flashmhf/modeling_mhffnmoe.py:412-431 on bf16 tensors (R fp32, fp32 sum over experts, bf16 result) under
    torch.autograd.  Used only to show that the HIP backward is at least as close to the fp64 gradients as this is."""
    leaves = [t.detach().to(torch.bfloat16).requires_grad_(True) for t in (Q, K, U, V)]
    leaves.append(R.detach().to(torch.float32).requires_grad_(True))
    out = mhffn_forward(*leaves, compute_dtype=torch.bfloat16, out_dtype=torch.bfloat16)
    return torch.autograd.grad(out, leaves, dO.to(torch.bfloat16))


def router_gate(Qh, router):
    """R = sigmoid(Q.float() @ router.float()), divided by its sum over experts clamped at 1e-20.
    models/flashmhf/modeling_mhffnmoe.py:384-386.  Qh [B,H,S,d_h], router [d_h,E] or [H,d_h,E]."""
    R = (Qh.to(torch.float32) @ router.to(torch.float32)).contiguous().sigmoid()
    return R / R.sum(dim=-1, keepdim=True).clamp(min=1e-20)


def head_norm_gate(x4, norm_weight, router, eps=1e-6, out_dtype=None):
    """The block's head prologue, differentiable: per-head RMSNorm in fp32 with the result cast back to the input
    dtype (models/flashmhf/modeling_mhffnmoe.py:124-133; skipped when norm_weight is None, :371), then the gate from
    the *rounded* Q in fp32 (:384-386).  x4 [B,S,H,d_h], norm_weight [H,d_h], router [H,d_h,E].
    Returns Q [B,H,S,d_h] (dtype of x4 unless out_dtype) and R [B,H,S,E] fp32 (or fp64 if x4 is fp64)."""
    out_dtype = out_dtype or x4.dtype
    acc = torch.float64 if x4.dtype == torch.float64 else torch.float32
    q = x4
    if norm_weight is not None:
        xf = x4.to(acc)
        xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
        q = (xf * norm_weight.to(acc).unsqueeze(0).unsqueeze(0)).to(out_dtype)
    Qh = q.transpose(1, 2)
    Rs = (Qh.to(acc) @ router.to(acc)).sigmoid()
    return Qh, Rs / Rs.sum(dim=-1, keepdim=True).clamp(min=1e-20)


def mhffn_layer_forward(X, Wq, Wr, K, U, V, Wo, *, num_heads, compute_dtype=torch.float32):
    """The benchmark's CPU layer: Q = X Wq split into heads, R = sigmoid(X Wr) normalised over E,
    the eager expert loop, heads merged, output projection Wo.

    Follows models/flashmhf/modeling_mhffnmoe.py:352-431 with RMSNorm off (the 128M config) and the gate
    logits taken from X through Wr [hid, H*E] as the benchmark configuration states.
    X [B,S,hid]; Wq, Wo [hid,hid] used as x @ W.
    """
    B, S, hid = X.shape
    H = num_heads
    E = K.shape[1]
    x = X.to(compute_dtype)
    Qh = (x @ Wq.to(compute_dtype)).view(B, S, H, hid // H).transpose(1, 2).contiguous()
    Rl = (X.to(torch.float32) @ Wr.to(torch.float32)).view(B, S, H, E).transpose(1, 2).sigmoid()
    R = (Rl / Rl.sum(-1, keepdim=True).clamp(min=1e-20)).contiguous()
    Oh = mhffn_forward(Qh, K, U, V, R, compute_dtype=compute_dtype)
    O = Oh.transpose(1, 2).contiguous().view(B, S, hid)
    return O @ Wo.to(compute_dtype), Qh, R, Oh


def error_metrics(x, ref):
    """max-abs, max-abs normalised by max|ref| (kernels/thunderkittens/run_from_python.py:54-58 prints this
    as a percentage) and mean relative error sum|x-ref| / sum|ref|."""
    x = x.detach().double().cpu()
    ref = ref.detach().double().cpu()
    d = (x - ref).abs()
    return {
        "max_abs": d.max().item(),
        "norm_max": (d.max() / ref.abs().max().clamp(min=1e-30)).item(),
        "mean_rel": (d.sum() / ref.abs().sum().clamp(min=1e-30)).item(),
    }


def mhffn_block_forward(x, w_self, w_self_2, K, U, V, *, num_heads, router=None, w_router=None, q_norm_weight=None,
                        eps=1e-6, compute_dtype=torch.float32):
    """One MH-FFN block as the reference module computes it (models/flashmhf/modeling_mhffnmoe.py:352-431, eager
    branch), differentiable in every argument: Q = x w_self^T split into heads, optional per-head RMSNorm in fp32
    (:97-135), gate from the per-head Q through ``router`` [H,d_h,E] (:384-386) or, if ``w_router`` [hid, H*E] is given,
    from x; the eager expert loop; heads merged; w_self_2.  Linear weights are [out, in] as nn.Linear stores them."""
    B, S, hid = x.shape
    H = num_heads
    E = K.shape[1]
    xc = x.to(compute_dtype)
    q = (xc @ w_self.to(compute_dtype).t()).view(B, S, H, hid // H)
    if q_norm_weight is not None:
        qf = q.float()
        q = (qf * torch.rsqrt(qf.pow(2).mean(-1, keepdim=True) + eps) * q_norm_weight.float()).to(compute_dtype)
    Qh = q.transpose(1, 2)
    if w_router is not None:
        logits = (x.float() @ w_router.float()).view(B, S, H, E).transpose(1, 2)
    else:
        logits = Qh.float() @ router.float()
    Rs = logits.sigmoid()
    R = Rs / Rs.sum(-1, keepdim=True).clamp(min=1e-20)
    Oh = mhffn_forward(Qh, K, U, V, R, compute_dtype=compute_dtype)
    return Oh.transpose(1, 2).reshape(B, S, hid) @ w_self_2.to(compute_dtype).t()
