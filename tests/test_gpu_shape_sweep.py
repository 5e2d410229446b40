"""Seeded sweep over shapes the fixed cases do not visit: ragged sequence lengths around the 32/64/256-token tile
boundaries, odd and even counts of 32-row blocks per expert (the forward's phantom block, the dK/dU/dV tail
instantiation), grouped K/U/V heads with every divisor, expert counts up to and beyond one LDS gate window of 64, all three head widths,
both token layouts and both weight-gradient dtypes.  Every case: forward and all five gradients against the fp64 oracle
on the same bf16-rounded inputs, at the bars of the fixed cases (mean-rel 1e-2; max-abs 2e-2 raw for O, dQ, dR and relative to
max(1, max|ref|) for dK, dU, dV: tests/helpers.py)."""
import random

import pytest
import torch

from oracle import mhffn_oracle as orc
from tests.helpers import assert_bf16_parity, make_inputs

pytestmark = pytest.mark.gpu

def _cases(n=64, seed=20240607):
    rnd = random.Random(seed)
    out = []
    while len(out) < n:
        dh = rnd.choice([64, 96, 128])
        H = rnd.choice([1, 2, 3, 4, 6, 8])
        Hk = rnd.choice([d for d in range(1, H + 1) if H % d == 0])
        E = rnd.choice([1, 2, 3, 5, 8, 11, 22, 33, 64])
        de = 32 * rnd.choice([1, 2, 3, 4, 5, 8, 11])
        S = rnd.choice([1, 31, 32, 33, 63, 65, 127, 255, 256, 257, 300, 511, 513, 777, 1024, 1100])
        B = rnd.choice([1, 2, 3])
        work = B * H * S * E * de * dh
        if work > 3e9 or E * de > 4096:       # keeps the fp64 oracle of the whole sweep within a few seconds
            continue
        out.append((B, H, S, dh, E, de, Hk, rnd.choice([False, True]), rnd.choice(["bf16", "f32"])))
    return out


CASES = _cases()


def _check(got, ref, name, case):
    assert_bf16_parity(name, got, ref, case)


@pytest.mark.parametrize("case", CASES, ids=["B{}H{}S{}dh{}E{}de{}Hk{}{}{}".format(*c[:7], "tm" if c[7] else "hm", c[8]) for c in CASES])
def test_forward_and_backward_match_the_oracle_over_the_sweep(case):
    from flashmhf_amd import mhffn_backward, mhffn_forward
    B, H, S, dh, E, de, Hk, token_major, wd = case
    print("case", case, flush=True)
    Q, K, U, V, R, dO = make_inputs(B, H, S, dh, E, de, Hk, seed=(B * 7 + H * 13 + S * 17 + dh * 19 + E * 23 + de * 29 + Hk * 31) % 100000, dtype=torch.bfloat16)
    ref_O = orc.mhffn_forward(Q, K, U, V, R, compute_dtype=torch.float64)
    ref_g = orc.mhffn_backward(Q, K, U, V, R, dO, compute_dtype=torch.float64)
    dev = "cuda:0"
    Qd, dOd = Q.to(dev), dO.to(dev)
    if token_major:      # the same values seen through the transposed view of a [B,S,H,d_h] tensor
        Qd = Qd.transpose(1, 2).contiguous().transpose(1, 2)
        dOd = dOd.transpose(1, 2).contiguous().transpose(1, 2)
    ins = [Qd] + [t.to(dev) for t in (K, U, V, R)]
    O = mhffn_forward(*ins)
    g = mhffn_backward(*ins, dOd, grad_w_dtype=torch.bfloat16 if wd == "bf16" else torch.float32)
    torch.cuda.synchronize()
    for name, got, ref in zip(("O", "dQ", "dK", "dU", "dV", "dR"), (O,) + tuple(g), (ref_O,) + tuple(ref_g)):
        assert got.shape == ref.shape, (name, case)
        _check(got.float().cpu(), ref, name, case)


# More experts than the 64 whose gate values the forward and the dQ/dR kernel hold in LDS at a time (the forward restages
# the tile every 64 experts, the dQ/dR kernel refills it as a ring, 32 slots at a time): one expert past 64, exactly 128,
# counts that end inside the four-block trips of the forward (d_e = 64: two blocks per expert), 200 with one block per
# expert, 97 with three.
CASES_MANY_EXPERTS = [
    (1, 2, 300, 128, 65, 32, 1, False, "bf16"),
    (2, 1, 257, 64, 128, 32, 1, True, "f32"),
    (1, 2, 513, 96, 130, 64, 2, False, "bf16"),
    (1, 1, 64, 128, 200, 32, 1, True, "bf16"),
    (1, 1, 200, 64, 97, 96, 1, False, "bf16"),       # three blocks per expert, the ring refilled twice
]


@pytest.mark.parametrize("case", CASES_MANY_EXPERTS, ids=["B{}H{}S{}dh{}E{}de{}Hk{}{}{}".format(*c[:7], "tm" if c[7] else "hm", c[8]) for c in CASES_MANY_EXPERTS])
def test_more_experts_than_one_gate_window(case):
    test_forward_and_backward_match_the_oracle_over_the_sweep(case)


def _cases_f32(n=20, seed=77):
    rnd = random.Random(seed)
    out = []
    while len(out) < n:
        dh = rnd.choice([8, 24, 64, 96, 120, 128])
        H = rnd.choice([1, 2, 4, 6])
        Hk = rnd.choice([d for d in range(1, H + 1) if H % d == 0])
        E = rnd.choice([1, 2, 3, 7, 11, 70])
        de = rnd.choice([1, 8, 40, 72, 100, 256, 352])
        S = rnd.choice([1, 31, 33, 64, 100, 257, 400])
        B = rnd.choice([1, 2])
        if B * H * S * E * de * dh > 3e8:
            continue
        out.append((B, H, S, dh, E, de, Hk, rnd.choice([False, True])))
    return out


CASES_F32 = _cases_f32()


@pytest.mark.parametrize("case", CASES_F32, ids=["B{}H{}S{}dh{}E{}de{}Hk{}{}".format(*c[:7], "tm" if c[7] else "hm") for c in CASES_F32])
def test_float32_instantiation_matches_the_oracle_over_the_sweep(case):
    """The all-float32 kernels take any expert width and count and any head width that is a multiple of 8 up to 128;
    bar 1e-4 (max-abs relative to max(1, max|ref|), and mean-rel)."""
    from flashmhf_amd import mhffn_backward, mhffn_forward
    B, H, S, dh, E, de, Hk, token_major = case
    print("case", case, flush=True)
    Q, K, U, V, R, dO = make_inputs(B, H, S, dh, E, de, Hk, seed=(B * 7 + H * 13 + S * 17 + dh * 19 + E * 23 + de * 29 + Hk * 31) % 100000,
                                    dtype=torch.float32)
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
        m = orc.error_metrics(got.double().cpu(), ref)
        scale = max(1.0, ref.abs().max().item())
        assert m["max_abs"] <= 1e-4 * scale and m["mean_rel"] <= 1e-4, (name, case, m)
