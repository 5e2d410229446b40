"""Saturated activations: pre-activations far outside the range where exp stays finite (|m| up to a few hundred), gates
that are exactly zero, and rows that are exactly zero.  sigma must go to exactly 0 or 1 without producing inf * 0, in the
forward and in every gradient; results are still held to the oracle."""
import pytest
import torch

from oracle import mhffn_oracle as orc
from tests.helpers import make_inputs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("token_major", [False, True])
def test_saturated_preactivations_and_zero_gates(token_major):
    from flashmhf_amd import mhffn_backward, mhffn_forward
    B, H, S, dh, E, de = 2, 2, 96, 128, 3, 64
    Q, K, U, V, R, dO = make_inputs(B, H, S, dh, E, de, H, seed=5, dtype=torch.bfloat16)
    Q = (Q.float() * 12.0).bfloat16()          # |Q K^T| reaches a few hundred: exp2 overflows / underflows
    K = (K.float() * 4.0).bfloat16()
    Q[:, :, 5] = 0                             # an all-zero token row
    R = R.clone()
    R[:, :, ::3, 1] = 0.0                      # gates that are exactly zero
    R[:, :, 7] = 0.0                           # a token with every gate zero
    m = torch.einsum("bhsd,hejd->bhsej", Q.float(), K.float())
    assert m.abs().max() > 150
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
    assert torch.equal(O[:, :, 7].cpu().float(), torch.zeros(B, H, dh))       # all gates zero: exactly zero output
    for name, got, ref in zip(("O", "dQ", "dK", "dU", "dV", "dR"), (O,) + tuple(g), (ref_O,) + tuple(ref_g)):
        assert torch.isfinite(got).all(), name
        e = orc.error_metrics(got.float().cpu(), ref.float())
        assert e["norm_max"] <= 2e-2 and e["mean_rel"] <= 1e-2, (name, e)


def test_forward_with_special_gate_values():
    """The forward folds the gate into the sigmoid's denominator (r / (1 + e) = 1 / fma(e, 1/r, 1/r), the reciprocal
    clamped to the largest finite float).  Gates of +0, -0, denormal size, tiny, negative and huge magnitude must give:
    exactly zero for a zero gate (either sign) and for gates whose reciprocal overflows, and the oracle's value
    (relative to the row's scale) everywhere else -- with saturated pre-activations in the mix, where e is 0 or inf."""
    from flashmhf_amd import mhffn_forward
    B, H, S, dh, E, de = 1, 2, 64, 128, 2, 64
    Q, K, U, V, R, _ = make_inputs(B, H, S, dh, E, de, H, seed=11, dtype=torch.bfloat16)
    Q[:, :, 32:] = (Q[:, :, 32:].float() * 12.0).bfloat16()      # second half of the tokens: |m| up to a few hundred
    K = (K.float() * 2.0).bfloat16()
    gates = [0.0, -0.0, 1e-39, -1e-39, 1e-30, -3.5, 0.25, 1e30]
    R = R.clone()
    for t in range(S):
        R[:, :, t, :] = gates[t % len(gates)]
    R[:, :, :, 1] *= 0.5
    ref = orc.mhffn_forward(Q, K, U, V, R, compute_dtype=torch.float64)
    dev = "cuda:0"
    O = mhffn_forward(*(x.to(dev) for x in (Q, K, U, V, R))).float().cpu()
    assert torch.isfinite(O).all()
    for t in range(S):
        gv = gates[t % len(gates)]
        if abs(gv) < 1e-38:                       # zero and denormal gates: exactly zero
            assert torch.equal(O[:, :, t], torch.zeros(B, H, dh)), (t, gv)
        else:
            scale = ref[:, :, t].abs().max().item()
            err = (O[:, :, t].double() - ref[:, :, t]).abs().max().item()
            assert err <= 2e-2 * scale, (t, gv, err, scale)
