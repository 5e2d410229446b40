"""Seeded random shapes through the C ABI (both token layouts), forward and backward against the fp64 oracle: ragged
sequence lengths, grouped heads, every supported head dim, odd and even block counts."""
import random

import pytest
import torch

from oracle import mhffn_oracle as orc
from tests.helpers import make_inputs

pytestmark = pytest.mark.gpu


def _shapes(n, seed):
    rng = random.Random(seed)
    out = []
    while len(out) < n:
        H = rng.choice([1, 2, 3, 4, 6, 8])
        Hk = rng.choice([d for d in (1, 2, 3, 4, 6, 8) if H % d == 0])
        out.append((rng.randint(1, 3), H, rng.randint(1, 600), rng.choice([64, 96, 128]), rng.randint(1, 6),
                    32 * rng.randint(1, 5), Hk, rng.random() < 0.5))
    return out


@pytest.mark.parametrize("B,H,S,dh,E,de,Hk,token_major", _shapes(14, seed=2024))
def test_random_shapes_match_oracle(B, H, S, dh, E, de, Hk, token_major):
    from flashmhf_amd import mhffn_backward, mhffn_forward
    print(f"case B={B} H={H} S={S} dh={dh} E={E} de={de} Hk={Hk} token_major={token_major}", flush=True)
    Q, K, U, V, R, dO = make_inputs(B, H, S, dh, E, de, Hk, seed=S * 7 + H, dtype=torch.bfloat16)
    ref_O = orc.mhffn_forward(Q, K, U, V, R, compute_dtype=torch.float64)
    ref_g = orc.mhffn_backward(Q, K, U, V, R, dO, compute_dtype=torch.float64)
    dev = "cuda:0"
    Qd, dOd = Q.to(dev), dO.to(dev)
    if token_major:
        Qd = Qd.transpose(1, 2).contiguous().transpose(1, 2)
        dOd = dOd.transpose(1, 2).contiguous().transpose(1, 2)
    ins = [Qd] + [t.to(dev) for t in (K, U, V, R)]
    O = mhffn_forward(*ins)
    g = mhffn_backward(*ins, dOd, grad_w_dtype=torch.float32)
    torch.cuda.synchronize()
    for name, got, ref in zip(("O", "dQ", "dK", "dU", "dV", "dR"), (O,) + tuple(g), (ref_O,) + tuple(ref_g)):
        assert torch.isfinite(got).all(), name
        m = orc.error_metrics(got.float().cpu(), ref.float())
        scale = max(1.0, ref.abs().max().item())
        assert m["max_abs"] <= 2e-2 * scale, (name, m)
        assert m["mean_rel"] <= 1e-2, (name, m)
