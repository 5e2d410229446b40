"""Seeded synthetic inputs shared by the tests (distributions of the benchmark configurations)."""
import torch


def make_inputs(B, H, S, dh, E, de, Hk=None, *, seed=0, dtype=torch.float32, r_mode="gate", device="cpu"):
    """Q ~ N(0,1); K,U,V ~ N(0, dh^-1/2); R = sigmoid(N(0,~0.6)) normalised over E ("gate") or N(0,1) ("randn",
    the reference script's choice, kernels/thunderkittens/run_from_python.py:31); dO ~ N(0,1).
    Values are generated in fp32 on the CPU, rounded once to ``dtype`` and returned in ``dtype`` (R stays fp32, fp64 when dtype is fp64)."""
    Hk = Hk or H
    g = torch.Generator().manual_seed(seed)
    Q = torch.randn(B, H, S, dh, generator=g)
    K, U, V = (torch.randn(Hk, E, de, dh, generator=g) * dh ** -0.5 for _ in range(3))
    if r_mode == "gate":
        R = torch.sigmoid(torch.randn(B, H, S, E, generator=g) * 0.6)
        R = R / R.sum(-1, keepdim=True)
    else:
        R = torch.randn(B, H, S, E, generator=g)
    dO = torch.randn(B, H, S, dh, generator=g)
    cast = lambda t: t.to(dtype).to(device)
    R = R.to(torch.float64 if dtype == torch.float64 else torch.float32)
    return cast(Q), cast(K), cast(U), cast(V), R.to(device), cast(dO)
