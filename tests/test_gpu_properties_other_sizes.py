"""The token-subset oracle comparison and the batch-additivity property at the other two layer sizes the benchmark names:
the 128M layer (B8 x S2048, H8, d_h96, E8, d_e256, forward) and the 1.3B layer (B4 x S8192, H16, d_h128, E22, d_e352,
forward + backward), both far too large for a CPU oracle of the whole problem."""
import pytest
import torch

from oracle import mhffn_oracle as orc
from tests.helpers import assert_bf16_parity

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(B, H, S, dh, E, de, seed):
    g = torch.Generator().manual_seed(seed)
    Q = torch.randn(B, H, S, dh, generator=g).bfloat16()
    K, U, V = ((torch.randn(H, E, de, dh, generator=g) * dh ** -0.5).bfloat16() for _ in range(3))
    R = torch.sigmoid(torch.randn(B, H, S, E, generator=g) * 0.64)
    R = R / R.sum(-1, keepdim=True)
    dO = torch.randn(B, H, S, dh, generator=g).bfloat16()
    return [t.to(DEV) for t in (Q, K, U, V, R, dO)]


def test_128m_layer_forward_rows_match_oracle_on_a_token_subset():
    from flashmhf_amd import mhffn_forward
    Q, K, U, V, R, _ = _inputs(8, 8, 2048, 96, 8, 256, seed=21)
    O = mhffn_forward(Q, K, U, V, R)
    torch.cuda.synchronize()
    idx = torch.tensor([0, 31, 32, 63, 64, 1000, 2046, 2047])
    sub = lambda t: t[::3, :, idx].cpu()
    ref = orc.mhffn_forward(sub(Q), K.cpu(), U.cpu(), V.cpu(), sub(R), compute_dtype=torch.float32)
    m = orc.error_metrics(sub(O).float(), ref)
    assert m["max_abs"] <= 2e-2 and m["mean_rel"] <= 1e-2, m


def test_1p3b_layer_rows_match_oracle_and_weight_gradients_add_over_batch():
    from flashmhf_amd import mhffn_backward, mhffn_forward
    Q, K, U, V, R, dO = _inputs(4, 16, 8192, 128, 22, 352, seed=22)
    O = mhffn_forward(Q, K, U, V, R)
    dQ, dK, dU, dV, dR = mhffn_backward(Q, K, U, V, R, dO, grad_w_dtype=torch.float32)
    torch.cuda.synchronize()
    idx = torch.tensor([0, 1, 63, 64, 4095, 4096, 8190, 8191])
    sub = lambda t: t[1:3, :, idx].cpu()
    Kc, Uc, Vc = K.cpu(), U.cpu(), V.cpu()
    ref_O = orc.mhffn_forward(sub(Q), Kc, Uc, Vc, sub(R), compute_dtype=torch.float32)
    ref = orc.mhffn_backward(sub(Q), Kc, Uc, Vc, sub(R), sub(dO), compute_dtype=torch.float64)
    for name, got, r in (("O", sub(O), ref_O), ("dQ", sub(dQ), ref[0]), ("dR", sub(dR), ref[4])):
        assert_bf16_parity(name, got.float(), r)          # raw max-abs 2e-2, mean-rel 1e-2
    # dK, dU, dV are sums over tokens: the whole batch equals the sum of its elements run one by one (fp32 partial sums
    # are added in a different order, hence a tolerance instead of equality)
    acc = [torch.zeros_like(dK) for _ in range(3)]
    for b in range(4):
        one = lambda t: t[b:b + 1].contiguous()
        _, k1, u1, v1, _ = mhffn_backward(one(Q), K, U, V, one(R), one(dO), grad_w_dtype=torch.float32)
        for a, t in zip(acc, (k1, u1, v1)):
            a += t
    torch.cuda.synchronize()
    for name, whole, parts in zip(("dK", "dU", "dV"), (dK, dU, dV), acc):
        scale = whole.abs().max().item()
        assert (whole - parts).abs().max().item() <= 1e-4 * scale, name
