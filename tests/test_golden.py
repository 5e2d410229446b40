"""Golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py from the fp64 oracle).
CPU: the oracle and the scalar C restatement still reproduce them.  GPU: the HIP kernels match them."""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import mhffn_oracle as orc
from tests.helpers import assert_bf16_parity

HERE = os.path.dirname(os.path.abspath(__file__))
FILES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))
NAMES = ("dQ", "dK", "dU", "dV", "dR")


def _load(path):
    z = np.load(path, allow_pickle=False)
    return {k: torch.from_numpy(z[k]) for k in z.files}


def test_fixtures_exist():
    assert len(FILES) >= 3


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f) for f in FILES])
def test_oracle_reproduces_golden(path, scalar_oracle):
    g = _load(path)
    ins = [g[k].double() for k in ("Q", "K", "U", "V", "R")]
    O = orc.mhffn_forward(*ins, compute_dtype=torch.float64)
    assert (O - g["O"].double()).abs().max().item() <= 1e-6 * max(1.0, g["O"].abs().max().item())
    grads = orc.mhffn_backward(*ins, g["dO"].double())
    for name, got in zip(NAMES, grads):
        ref = g[name].double()
        assert (got - ref).abs().max().item() <= 2e-6 * max(1.0, ref.abs().max().item()), name
    O_c = scalar_oracle.forward(*(t.numpy() for t in ins))
    assert np.abs(O_c - g["O"].numpy()).max() <= 1e-6 * max(1.0, float(g["O"].abs().max()))


@pytest.mark.gpu
@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f) for f in FILES])
def test_hip_kernels_match_golden(path):
    from flashmhf_amd import mhffn_backward, mhffn_forward
    g = _load(path)
    dev = "cuda:0"
    ins = [g[k].to(torch.bfloat16).to(dev) for k in ("Q", "K", "U", "V")] + [g["R"].to(dev)]
    O = mhffn_forward(*ins)
    grads = mhffn_backward(*ins, g["dO"].to(torch.bfloat16).to(dev), grad_w_dtype=torch.float32)
    torch.cuda.synchronize()
    for name, got in zip(("O",) + NAMES, (O,) + tuple(grads)):
        assert_bf16_parity(name, got.float().cpu(), g[name], os.path.basename(path))
