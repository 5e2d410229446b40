"""GPU parity of the float32 instantiation (through the C ABI): outputs and all five gradients within 1e-4 (max-abs,
relative to max(1, max|ref|)) of the fp64 oracle on identical seeded inputs."""
import pytest
import torch

from oracle import mhffn_oracle as orc
from tests.helpers import make_inputs

pytestmark = pytest.mark.gpu
TOL = 1e-4

CASES = [
    (2, 8, 128, 96, 8, 256, 8),     # the CPU-runnable reference configuration (128M layer dims, B2 x S128)
    (1, 2, 70, 128, 3, 352, 2),     # d_e = 352, tail tokens
    (2, 4, 45, 40, 2, 21, 2),       # generic d_h / d_e, grouped K/U/V heads
]


@pytest.mark.parametrize("B,H,S,dh,E,de,Hk", CASES)
def test_fp32_forward_backward_within_1e4(B, H, S, dh, E, de, Hk):
    from flashmhf_amd import FlashMLPMoE, mhffn_backward
    print(f"case B={B} H={H} S={S} dh={dh} E={E} de={de} Hk={Hk}", flush=True)
    Q, K, U, V, R, dO = make_inputs(B, H, S, dh, E, de, Hk, seed=300 + S, dtype=torch.float32)
    ref_O = orc.mhffn_forward(Q, K, U, V, R, compute_dtype=torch.float64)
    ref_g = orc.mhffn_backward(Q, K, U, V, R, dO, compute_dtype=torch.float64)
    dev = "cuda:0"
    ins = [t.to(dev) for t in (Q, K, U, V, R)]
    O = FlashMLPMoE()(*ins)
    grads = mhffn_backward(*ins, dO.to(dev), grad_w_dtype=torch.float32)
    torch.cuda.synchronize()
    assert O.dtype == torch.float32
    for name, got, ref in zip(("O", "dQ", "dK", "dU", "dV", "dR"), (O, *grads), (ref_O, *ref_g)):
        m = orc.error_metrics(got.cpu(), ref)
        scale = max(1.0, ref.abs().max().item())
        print(name, m, flush=True)
        assert m["max_abs"] <= TOL * scale, (name, m)


def test_fp32_autograd_path():
    from flashmhf_amd import FlashMLPMoE
    dev = "cuda:0"
    Q, K, U, V, R, dO = make_inputs(1, 2, 33, 64, 2, 48, seed=5, dtype=torch.float32)
    leaves = [t.to(dev).requires_grad_(True) for t in (Q, K, U, V, R)]
    out = FlashMLPMoE()(*leaves)
    out.backward(dO.to(dev))
    ref = orc.mhffn_backward(Q, K, U, V, R, dO)
    for leaf, r in zip(leaves, ref):
        m = orc.error_metrics(leaf.grad.cpu(), r)
        assert m["max_abs"] <= TOL * max(1.0, r.abs().max().item()), m
