"""Writes the golden vectors under tests/golden/ from the CPU oracle (oracle/mhffn_oracle.py, fp64).

The reference repository holds no stored vectors, fixtures or asserts for this path (its only check,
kernels/thunderkittens/run_from_python.py, prints differences on a CUDA GPU), and nothing of the reference is imported
or executed here: the vectors pin this repository's own oracle against accidental change, after that oracle passed the
independent checks in tests/test_oracle.py.  Inputs are bf16-representable so GPU runs can consume them exactly.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import mhffn_oracle as orc  # noqa: E402
from tests.helpers import make_inputs  # noqa: E402

CASES = {
    # name: (B, H, S, dh, E, de, Hk, r_mode)
    "tiny_gq": (1, 4, 37, 64, 2, 32, 2, "gate"),
    "tk_script_shape_small": (1, 2, 48, 128, 2, 64, 2, "randn"),
    "de352": (1, 1, 33, 128, 1, 352, 1, "gate"),
}


def main():
    for name, (B, H, S, dh, E, de, Hk, r_mode) in CASES.items():
        Q, K, U, V, R, dO = make_inputs(B, H, S, dh, E, de, Hk, seed=4242, dtype=torch.bfloat16, r_mode=r_mode)
        O = orc.mhffn_forward(Q, K, U, V, R, compute_dtype=torch.float64)
        dQ, dK, dU, dV, dR = orc.mhffn_backward(Q, K, U, V, R, dO, compute_dtype=torch.float64)
        np.savez_compressed(
            os.path.join(HERE, f"{name}.npz"),
            Q=Q.float().numpy(), K=K.float().numpy(), U=U.float().numpy(), V=V.float().numpy(), R=R.numpy(),
            dO=dO.float().numpy(), O=O.numpy().astype(np.float32), dQ=dQ.numpy().astype(np.float32),
            dK=dK.numpy().astype(np.float32), dU=dU.numpy().astype(np.float32), dV=dV.numpy().astype(np.float32),
            dR=dR.numpy().astype(np.float32))
        print(name, "written")


if __name__ == "__main__":
    main()
