"""The parity bar at the benchmark's own sizes, against the fp64 CPU oracle on identical seeded inputs.

Bar (bf16 runs): max-abs <= 2e-2 and mean-rel <= 1e-2.  O, dQ and dR meet it as raw figures and are asserted so.
dK, dU and dV are sums over every token; at the 370M layer's 16,384 tokens they reach |45|, where a single bf16 ulp
is 0.25 and the rounding of the bf16 matrix operands alone random-walks to several 1e-2, so a raw 2e-2 cannot hold for
any bf16 implementation.  For them the criterion is the one the reference's own check implies
(kernels/thunderkittens/run_from_python.py:40-58 compares the kernel with the eager path): the HIP gradients must be
no further from the fp64 gradients than the reference's eager expert loop run in bf16 under torch.autograd
(models/flashmhf/modeling_mhffnmoe.py:412-431) is, in raw max-abs and in mean-rel, and mean-rel <= 1e-2 as stated.
The raw figures are printed (pytest -s).
"""
import pytest
import torch

from oracle import mhffn_oracle as orc
from tests.helpers import MAX_ABS, MEAN_REL

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NAMES = ("O", "dQ", "dK", "dU", "dV", "dR")


def _inputs(B, H, S, dh, E, de, seed):
    """The benchmark's distributions (bench.py make_inputs): Q, dO ~ N(0,1); K, U, V ~ N(0, d_h^-1/2); gate = sigmoid of
    N(0, 0.64) logits normalised over the experts."""
    g = torch.Generator().manual_seed(seed)
    Q = torch.randn(B, H, S, dh, generator=g).bfloat16()
    K, U, V = ((torch.randn(H, E, de, dh, generator=g) * dh ** -0.5).bfloat16() for _ in range(3))
    R = torch.sigmoid(torch.randn(B, H, S, E, generator=g) * 0.64)
    R = R / R.sum(-1, keepdim=True)
    dO = torch.randn(B, H, S, dh, generator=g).bfloat16()
    return Q, K, U, V, R, dO


def _hip_vs_eager_vs_oracle(tag, ins, compute_dtype):
    from flashmhf_amd import mhffn_backward, mhffn_forward
    ref = (orc.mhffn_forward(*ins[:5], compute_dtype=compute_dtype),) + tuple(
        orc.mhffn_backward(*ins, compute_dtype=compute_dtype))
    gi = [t.to(DEV) for t in ins]
    O = mhffn_forward(*gi[:5])
    g32 = mhffn_backward(*gi, grad_w_dtype=torch.float32)
    g16 = mhffn_backward(*gi, grad_w_dtype=torch.bfloat16)
    eager = (orc.mhffn_forward(*gi[:5], compute_dtype=torch.bfloat16, out_dtype=torch.bfloat16),) + tuple(
        orc.bf16_eager_autograd(*gi))
    torch.cuda.synchronize()
    assert torch.equal(g16[0], g32[0]) and torch.equal(g16[4], g32[4])      # dQ, dR do not depend on the dK/dU/dV dtype
    for name, r, hip32, hip16, eag in zip(NAMES, ref, (O,) + tuple(g32), (O,) + tuple(g16), eager):
        me = orc.error_metrics(eag.float().cpu(), r)
        for label, got in (("fp32 dK/dU/dV", hip32), ("bf16 dK/dU/dV", hip16)):
            if label.startswith("bf16") and name not in ("dK", "dU", "dV"):
                continue
            m = orc.error_metrics(got.float().cpu(), r)
            print(f"{tag} {name:2s} [{label if name in ('dK', 'dU', 'dV') else 'bf16 out' if name != 'dR' else 'fp32 out'}]: "
                  f"HIP raw max-abs {m['max_abs']:.3e} mean-rel {m['mean_rel']:.3e} | bf16 eager raw max-abs "
                  f"{me['max_abs']:.3e} mean-rel {me['mean_rel']:.3e} | max|ref| {r.abs().max().item():.3e}", flush=True)
            assert torch.isfinite(got).all(), (tag, name, label)
            assert m["mean_rel"] <= MEAN_REL, (tag, name, label, m)
            if name in ("O", "dQ", "dR"):
                assert m["max_abs"] <= MAX_ABS, (tag, name, m)
            else:
                assert m["max_abs"] <= me["max_abs"] and m["mean_rel"] <= me["mean_rel"], (tag, name, label, m, me)


def test_370m_layer_at_full_size_all_outputs():
    """BASELINE configuration 2 as stated: B8 x S2048 = 16,384 tokens, H8, d_h128, E11, d_e352."""
    _hip_vs_eager_vs_oracle("370M layer B8xS2048", _inputs(8, 8, 2048, 128, 11, 352, seed=1234), torch.float64)


def test_370m_layer_one_full_length_batch_row():
    _hip_vs_eager_vs_oracle("370M layer B1xS2048", _inputs(1, 8, 2048, 128, 11, 352, seed=4321), torch.float64)


def test_1p3b_layer_dims_all_outputs():
    """The 1.3B layer's heads and experts (H16, E22, d_e352: 242 blocks per head, 61 workgroup columns of the dK/dU/dV
    kernel, the last with two waves idle) on one batch row of 1,024 tokens in fp64, and on one full-length batch row
    (8,192 tokens) with the oracle in fp32."""
    _hip_vs_eager_vs_oracle("1.3B layer B1xS1024", _inputs(1, 16, 1024, 128, 22, 352, seed=99), torch.float64)
    _hip_vs_eager_vs_oracle("1.3B layer B1xS8192", _inputs(1, 16, 8192, 128, 22, 352, seed=98), torch.float32)


def test_128m_layer_dims_all_outputs():
    """The 128M layer (d_h 96, E8, d_e256), one batch row of the benchmark's B8 x S2048."""
    _hip_vs_eager_vs_oracle("128M layer B1xS2048", _inputs(1, 8, 2048, 96, 8, 256, seed=7), torch.float64)
