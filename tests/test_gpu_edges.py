"""Edge shapes through the C ABI, forward and backward against the fp64 oracle: a single token, sequences shorter than
one 32-token tile, one expert of one block, the largest expert count the bf16 kernels accept (E = 64), odd block
counts (phantom pipeline steps), more K/U/V rows than tokens, several batches with a ragged last tile."""
import pytest
import torch

from oracle import mhffn_oracle as orc
from tests.helpers import assert_bf16_parity, make_inputs

pytestmark = pytest.mark.gpu

CASES = [
    # B, H, S, dh, E, de, Hk
    (1, 1, 1, 64, 1, 32, 1),        # one token, one block
    (1, 2, 31, 96, 1, 32, 1),       # less than a tile
    (3, 2, 33, 128, 5, 32, 2),      # 5 blocks (odd), one token in the second tile, grouped heads, 3 batches
    (1, 1, 255, 128, 1, 96, 1),     # 3 blocks, one token short of a workgroup tile
    (1, 4, 256, 64, 64, 32, 1),     # E = 64 (the limit), all four q-heads share one K/U/V head
    (2, 2, 40, 128, 3, 160, 2),     # 15 blocks for 40 tokens: the dK/dU/dV token loop is shorter than its pipeline depth
]


@pytest.mark.parametrize("B,H,S,dh,E,de,Hk", CASES)
def test_edge_shapes_match_oracle(B, H, S, dh, E, de, Hk):
    from flashmhf_amd import mhffn_backward, mhffn_forward
    print(f"case B={B} H={H} S={S} dh={dh} E={E} de={de} Hk={Hk}", flush=True)
    Q, K, U, V, R, dO = make_inputs(B, H, S, dh, E, de, Hk, seed=77 + S, dtype=torch.bfloat16)
    ref_O = orc.mhffn_forward(Q, K, U, V, R, compute_dtype=torch.float64)
    ref_g = orc.mhffn_backward(Q, K, U, V, R, dO, compute_dtype=torch.float64)
    dev = "cuda:0"
    ins = [t.to(dev) for t in (Q, K, U, V, R)]
    O = mhffn_forward(*ins)
    g = mhffn_backward(*ins, dO.to(dev), grad_w_dtype=torch.float32)
    torch.cuda.synchronize()
    for name, got, ref in zip(("O", "dQ", "dK", "dU", "dV", "dR"), (O,) + tuple(g), (ref_O,) + tuple(ref_g)):
        print(name, assert_bf16_parity(name, got.float().cpu(), ref.float()), flush=True)
