"""Drop-in for the reference's legacy single-expert operator ``kernels/triton/flash_mlp.py`` (``FlashMLP`` :1021-1064):

    O = FlashMLP()(Q, K, U, V, apply_dot_scaling, head_scaling, up_scaling, activation_fn)
    Q [B,H,S,d_h], K/U/V [Hkuv, I, d_h] bf16   ->   O[b,h] = (silu(Q K^T) * (Q U^T)) V

It is the E = 1, R = 1 case of the fused MoE operator (which is what runs), with the reference's argument checks
(:1050-1058): only SiLU, no dot scaling, U required.  The model calls it once per expert when
``mhffnmoe_use_legacy_flash`` is set (models/flashmhf/modeling_mhffnmoe.py:394-404).
"""
import torch

from .flash_mlp_moe import FlashMLPFunction


class FlashMLP(torch.nn.Module):
    def __init__(self):
        super().__init__()

    def forward(self, Q, K, U, V, apply_dot_scaling=False, head_scaling=1.0, up_scaling=1.0, activation_fn="silu"):
        if activation_fn != "silu":
            raise ValueError("FlashMLP currently supports only SiLU activation")
        if apply_dot_scaling or head_scaling != 1.0 or up_scaling != 1.0:
            raise ValueError("FlashMLP does not support dot scaling")
        if U is None:
            raise ValueError("FlashMLP SiLU variant requires up-projection tensor U (got None)")
        if K.dim() != 3:
            raise RuntimeError("expected K/U/V [Hkuv, intermediate, d_h]")
        ones = torch.ones(*Q.shape[:3], 1, dtype=torch.float32, device=Q.device)
        return FlashMLPFunction.apply(Q, K.unsqueeze(1), U.unsqueeze(1), V.unsqueeze(1), ones)
