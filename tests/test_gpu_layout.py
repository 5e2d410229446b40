"""Token-major Q/O/dO/dQ ([B,S,H,d_h] memory, passed as its [B,H,S,d_h] transposed view) through the C ABI's
*_layout entry points: the kernels run the same arithmetic in the same order as on [B,H,S,d_h] tensors, so every
result must be bit-identical to the contiguous call, and O / dQ must come back token-major
(what models/flashmhf/modeling_mhffnmoe.py:408 then merges without a copy)."""
import pytest
import torch

from tests.helpers import make_inputs

pytestmark = pytest.mark.gpu

CASES = [
    # B, H, S, dh, E, de, Hk
    (2, 4, 300, 128, 2, 64, 2),     # tail tokens, grouped K/U/V heads
    (2, 3, 70, 96, 3, 96, 3),
    (1, 2, 257, 64, 2, 32, 2),
    (3, 8, 512, 128, 11, 352, 8),   # 370M layer dims, several batches (the dK/dU/dV tile walk crosses batches and heads)
]


def _token_major(t):
    return t.transpose(1, 2).contiguous().transpose(1, 2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,H,S,dh,E,de,Hk", CASES)
def test_token_major_matches_contiguous_bit_for_bit(B, H, S, dh, E, de, Hk, dtype):
    from flashmhf_amd import mhffn_backward, mhffn_forward
    print(f"case B={B} H={H} S={S} dh={dh} E={E} de={de} Hk={Hk} {dtype}", flush=True)
    dev = "cuda:0"
    Q, K, U, V, R, dO = (t.to(dev) for t in make_inputs(B, H, S, dh, E, de, Hk, seed=31 + S, dtype=dtype))
    O_ref = mhffn_forward(Q, K, U, V, R)
    g_ref = mhffn_backward(Q, K, U, V, R, dO, grad_w_dtype=torch.float32)
    Qt, dOt = _token_major(Q), _token_major(dO)
    assert not Qt.is_contiguous() and Qt.transpose(1, 2).is_contiguous()
    O = mhffn_forward(Qt, K, U, V, R)
    assert O.transpose(1, 2).is_contiguous(), "O must come back token-major"
    assert torch.equal(O, O_ref)
    for dO_in in (dOt, dO):                       # upstream gradient in either layout
        g = mhffn_backward(Qt, K, U, V, R, dO_in, grad_w_dtype=torch.float32)
        assert g[0].transpose(1, 2).is_contiguous(), "dQ must come back token-major"
        for name, a, b in zip(("dQ", "dK", "dU", "dV", "dR"), g, g_ref):
            assert torch.equal(a, b), name


def test_autograd_with_the_callers_views_copies_nothing_on_the_way_out():
    """The caller's own sequence (modeling_mhffnmoe.py:362, 374 without its .contiguous(), 406-408)."""
    from flashmhf_amd import FlashMLPMoE
    dev = "cuda:0"
    B, H, S, dh, E, de = 2, 4, 200, 128, 2, 64
    Q, K, U, V, R, _ = (t.to(dev) for t in make_inputs(B, H, S, dh, E, de, seed=5, dtype=torch.bfloat16))
    x = Q.transpose(1, 2).contiguous().view(B, S, H * dh).requires_grad_(True)      # [B,S,hid], as w_self(x) returns
    Qv = x.view(B, S, H, dh).transpose(1, 2)
    Kp, Up, Vp = (t.clone().requires_grad_(True) for t in (K, U, V))
    out = FlashMLPMoE()(Qv, Kp, Up, Vp, R)
    merged = out.transpose(1, 2).contiguous().view(B, S, H * dh)
    assert merged.data_ptr() == out.data_ptr(), "merging heads must not copy"
    merged.float().sum().backward()
    xr = Q.clone().requires_grad_(True)
    Kr, Ur, Vr = (t.clone().requires_grad_(True) for t in (K, U, V))
    FlashMLPMoE()(xr, Kr, Ur, Vr, R).float().sum().backward()
    assert torch.equal(x.grad.view(B, S, H, dh).transpose(1, 2), xr.grad)
    for a, b in ((Kp, Kr), (Up, Ur), (Vp, Vr)):
        assert torch.equal(a.grad, b.grad)
