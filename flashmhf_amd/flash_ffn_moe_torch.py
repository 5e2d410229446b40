"""Drop-in for the reference's ``kernels/thunderkittens/flash_ffn_moe_torch.py`` (``FlashFFNMoEFunction`` :5-24,
``FlashFFNMoE`` :27-31): same call signature, and -- as that wrapper does (:17-21) -- gradients of the bf16
weights and of Q are returned in float32.  The R transpose the ThunderKittens kernel needs (:9, :23) is not
needed here: the HIP kernels read R as [B,H,S,E].
"""
import torch

from .flash_mlp_moe import mhffn_backward, mhffn_forward


class FlashFFNMoEFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, Q, K, U, V, R):
        O = mhffn_forward(Q, K, U, V, R)
        ctx.save_for_backward(Q, K, U, V, R)
        return O

    @staticmethod
    def backward(ctx, grad_output):
        Q, K, U, V, R = ctx.saved_tensors
        dQ, dK, dU, dV, dR = mhffn_backward(Q, K, U, V, R, grad_output, grad_w_dtype=torch.float32)
        return dQ.float(), dK, dU, dV, dR


class FlashFFNMoE(torch.nn.Module):
    def __init__(self):
        super().__init__()

    def forward(self, Q, K, U, V, R):
        return FlashFFNMoEFunction.apply(Q, K, U, V, R)
