"""Host side of one multi-head FFN block around the fused operator, and a minimal decoder that stacks it.

``MHFFNLayer`` computes what the reference's ``MHFFNMoEMultiHeadFFNFlash.forward`` computes
(models/flashmhf/modeling_mhffnmoe.py:352-431, fused branch :406-410):

    Q = w_self(x) -> heads -> optional per-head RMSNorm (:97-135) -> R = sigmoid(Q router) / sum_e (:384-386)
      -> O = fused(Q, K, U, V, R) -> heads merged -> w_self_2

but laid out for the HIP kernels instead of for the Triton ones:

* the gate/up/down parameters are stored as ``[Hkuv, E, d_e, d_h]``, the layout the kernels read, so no weight is
  re-laid-out per forward (the reference copies all three every call, :363-365, :375-382);
  ``load_reference_weights`` converts from the reference's ``[E*d_e, Hkuv*d_h]`` parameters;
* Q stays in the ``[B, S, H, d_h]`` memory the projection wrote and O comes back in it, so neither of the two
  transposes-with-copy around the operator (:374, :408) happens.

* with bfloat16 activations and ``router_input="q"`` the per-head RMSNorm and the gate run as one HIP pass over the
  projection's output (``head_gate.head_norm_gate``) instead of a dozen element-wise kernels and a float32 copy of Q;
  ``fused_prologue=False`` keeps the plain torch operations (the only path for float32 activations).

``router_input="q"`` takes the gate logits from the per-head Q through ``router [H, d_h, E]`` as the reference model
does; ``router_input="x"`` takes them from the block input through ``w_router [hid, H*E]``, which is how the layer
benchmark configurations state the gate.

``MHFFNDecoder`` is a plain pre-norm decoder (token embedding, N x [RMSNorm, causal multi-head attention with rotary
positions, RMSNorm, MHFFNLayer], final RMSNorm, untied output head, cross-entropy) with the residual structure of
modeling_mhffnmoe.py:612-652; it exists to time one training step of a whole model built on the operator and carries
none of the reference's transformers plumbing.
"""
import math

import torch
import torch.nn.functional as F
from torch import nn

from .flash_mlp_moe import FlashMLPMoE
from .head_gate import head_norm_gate


class RMSNorm(nn.Module):
    """x * rsqrt(mean(x^2) + eps) in fp32, cast back, times weight (modeling_mhffnmoe.py:73-89).
    ``shape`` = (hidden,) for a whole-row norm, (H, d_h) for the per-head norm applied to [B, S, H, d_h] (:97-135)."""

    def __init__(self, shape, eps=1e-6):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(shape))
        self.eps = eps

    def forward(self, x):
        if self.weight.dim() == 1 and x.is_cuda:
            # whole-row norm of the decoder blocks: torch's fused kernel (fp32 inside, one rounding at the end instead of
            # the two of `weight * normed.to(dtype)`)
            return F.rms_norm(x, (x.shape[-1],), self.weight.to(x.dtype), self.eps)
        xf = x.float()
        xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps)
        if self.weight.dim() == 1:
            return self.weight * xf.to(x.dtype)
        return (xf * self.weight).to(x.dtype)


def router_gate(logits):
    """sigmoid, then divide by the sum over experts clamped at 1e-20 (modeling_mhffnmoe.py:384-386); fp32 in and out."""
    R = logits.sigmoid()
    return R / R.sum(dim=-1, keepdim=True).clamp(min=1e-20)


class MHFFNLayer(nn.Module):
    def __init__(self, hidden_size, num_heads, num_experts, expert_dim, num_kuv_heads=None, *, apply_rmsnorm=False,
                 rms_norm_eps=1e-6, bias=False, router_input="q", op=None, fused_prologue=True):
        super().__init__()
        if hidden_size % num_heads:
            raise ValueError("hidden_size must be a multiple of num_heads")
        if router_input not in ("q", "x"):
            raise ValueError("router_input is 'q' (per-head Q through router) or 'x' (block input through w_router)")
        self.hidden_size, self.num_heads = hidden_size, num_heads
        self.num_kuv_heads = num_kuv_heads or num_heads
        self.head_dim = hidden_size // num_heads
        self.num_experts, self.expert_dim = num_experts, expert_dim
        self.router_input = router_input
        self.fused_prologue = fused_prologue
        self.rms_norm_eps = rms_norm_eps
        self.w_self = nn.Linear(hidden_size, hidden_size, bias=bias)
        self.w_self_2 = nn.Linear(hidden_size, hidden_size, bias=bias)
        wshape = (self.num_kuv_heads, num_experts, expert_dim, self.head_dim)
        std = self.head_dim ** -0.5
        self.K = nn.Parameter(torch.randn(wshape) * std)
        self.U = nn.Parameter(torch.randn(wshape) * std)
        self.V = nn.Parameter(torch.randn(wshape) * std)
        if router_input == "q":
            self.router = nn.Parameter(torch.randn(num_heads, self.head_dim, num_experts) * 0.02)
        else:
            self.w_router = nn.Parameter(torch.randn(hidden_size, num_heads * num_experts) * 0.02)
        self.q_norm = RMSNorm((num_heads, self.head_dim), rms_norm_eps) if apply_rmsnorm else None
        self.op = op if op is not None else FlashMLPMoE()

    @torch.no_grad()
    def load_reference_weights(self, gate_weight, up_weight, down_weight):
        """From the reference's parameters, each [E*d_e, Hkuv*d_h] (modeling_mhffnmoe.py:343-345), following its own
        view/transpose/view chain (:363-365, :375-382)."""
        for dst, src in ((self.K, gate_weight), (self.U, up_weight), (self.V, down_weight)):
            w = src.view(self.num_experts * self.expert_dim, self.num_kuv_heads, self.head_dim).transpose(0, 1)
            dst.copy_(w.reshape(self.num_kuv_heads, self.num_experts, self.expert_dim, self.head_dim))

    @torch.no_grad()
    def export_reference_weights(self):
        """The inverse of load_reference_weights: (gate_weight, up_weight, down_weight), each [E*d_e, Hkuv*d_h] as the
        reference stores them (modeling_mhffnmoe.py:343-345), so a model trained here can be saved in its format."""
        rows = self.num_experts * self.expert_dim
        return tuple(w.detach().reshape(self.num_kuv_heads, rows, self.head_dim).transpose(0, 1)
                     .reshape(rows, self.num_kuv_heads * self.head_dim).clone() for w in (self.K, self.U, self.V))

    def heads_and_gate(self, x):
        """Q as the [B, H, S, d_h] view of the projection's [B, S, H, d_h] memory, and R [B, H, S, E] fp32."""
        B, S, _ = x.shape
        H, dh, E = self.num_heads, self.head_dim, self.num_experts
        q = self.w_self(x).view(B, S, H, dh)
        # (d_h = 128 with more than 32 experts and RMSNorm is left to torch: that instantiation of the prologue's backward
        # kernel does not fit the register file and runs several times slower than it should)
        if (self.fused_prologue and self.router_input == "q" and q.dtype == torch.bfloat16 and q.is_cuda
                and E <= 64 and dh in (64, 96, 128) and not (dh == 128 and E > 32 and self.q_norm is not None)):
            return head_norm_gate(q, None if self.q_norm is None else self.q_norm.weight, self.router,
                                  self.rms_norm_eps)
        if self.q_norm is not None:
            q = self.q_norm(q)
        Q = q.transpose(1, 2)                                       # a view: the kernels read token-major rows
        if self.router_input == "q":
            logits = torch.einsum("bshd,hde->bhse", q.float(), self.router.float())
        else:
            logits = (x.float() @ self.w_router.float()).view(B, S, H, E).transpose(1, 2)
        return Q, router_gate(logits).contiguous()

    def forward(self, x):
        B, S, hid = x.shape
        Q, R = self.heads_and_gate(x)
        O = self.op(Q, self.K.to(Q.dtype), self.U.to(Q.dtype), self.V.to(Q.dtype), R)
        return self.w_self_2(O.transpose(1, 2).reshape(B, S, hid))  # token-major O: the reshape is a view


def _rotary(seq_len, head_dim, base, device, dtype):
    """cos/sin tables [S, head_dim] in the activations' dtype (computed in fp32)."""
    inv = 1.0 / (base ** (torch.arange(0, head_dim, 2, device=device, dtype=torch.float32) / head_dim))
    ang = torch.outer(torch.arange(seq_len, device=device, dtype=torch.float32), inv)
    ang = torch.cat((ang, ang), dim=-1)
    return ang.cos().to(dtype), ang.sin().to(dtype)


def _apply_rotary(x, cos, sin):
    half = x.shape[-1] // 2
    rot = torch.cat((-x[..., half:], x[..., :half]), dim=-1)
    return x * cos + rot * sin


class CausalSelfAttention(nn.Module):
    def __init__(self, hidden_size, num_heads, rope_base=10000.0):
        super().__init__()
        self.num_heads, self.head_dim, self.rope_base = num_heads, hidden_size // num_heads, rope_base
        self.qkv = nn.Linear(hidden_size, 3 * hidden_size, bias=False)
        self.out = nn.Linear(hidden_size, hidden_size, bias=False)

    def forward(self, x, rope=None):
        B, S, hid = x.shape
        q, k, v = self.qkv(x).view(B, S, 3, self.num_heads, self.head_dim).permute(2, 0, 3, 1, 4)
        cos, sin = rope if rope is not None else _rotary(S, self.head_dim, self.rope_base, x.device, x.dtype)
        q, k = _apply_rotary(q, cos, sin), _apply_rotary(k, cos, sin)
        y = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        return self.out(y.transpose(1, 2).reshape(B, S, hid))


class MHFFNDecoderBlock(nn.Module):
    def __init__(self, hidden_size, attn_heads, ffn_heads, num_experts, expert_dim, eps=1e-6, **layer_kw):
        super().__init__()
        self.input_norm = RMSNorm((hidden_size,), eps)
        self.attn = CausalSelfAttention(hidden_size, attn_heads)
        self.post_attn_norm = RMSNorm((hidden_size,), eps)
        self.mlp = MHFFNLayer(hidden_size, ffn_heads, num_experts, expert_dim, rms_norm_eps=eps, **layer_kw)

    def forward(self, x, rope=None):
        x = x + self.attn(self.input_norm(x), rope)
        return x + self.mlp(self.post_attn_norm(x))


class MHFFNDecoder(nn.Module):
    def __init__(self, vocab_size, hidden_size, num_layers, attn_heads, ffn_heads, num_experts, expert_dim, eps=1e-6,
                 **layer_kw):
        super().__init__()
        self.embed = nn.Embedding(vocab_size, hidden_size)
        self.blocks = nn.ModuleList(
            MHFFNDecoderBlock(hidden_size, attn_heads, ffn_heads, num_experts, expert_dim, eps, **layer_kw)
            for _ in range(num_layers))
        self.norm = RMSNorm((hidden_size,), eps)
        self.lm_head = nn.Linear(hidden_size, vocab_size, bias=False)
        nn.init.normal_(self.embed.weight, std=0.02)
        for m in self.modules():
            if isinstance(m, nn.Linear):
                nn.init.normal_(m.weight, std=0.02 if m is not self.lm_head else 1.0 / math.sqrt(hidden_size))

    def forward(self, ids, labels=None):
        x = self.embed(ids)
        attn = self.blocks[0].attn
        rope = _rotary(ids.shape[1], attn.head_dim, attn.rope_base, x.device, x.dtype)   # one table for every block
        for blk in self.blocks:
            x = blk(x, rope)
        logits = self.lm_head(self.norm(x))
        if labels is None:
            return logits
        # next-token loss: position t predicts token t + 1 (the causal-LM loss the reference calls at
        # modeling_mhffnmoe.py:1162-1164)
        return F.cross_entropy(logits[:, :-1].reshape(-1, logits.shape[-1]).float(), labels[:, 1:].reshape(-1))
