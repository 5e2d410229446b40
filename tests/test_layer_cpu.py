"""Host logic of the MH-FFN block (flashmhf_amd/mhffn_layer.py) on the CPU, with the fused operator replaced by the
oracle's eager loop: prologue (projection, head split, per-head RMSNorm, router gate), epilogue (head merge, output
projection) and the conversion from the reference's weight layout.  No GPU, no HIP call."""
import pytest
import torch

from flashmhf_amd.mhffn_layer import MHFFNDecoder, MHFFNLayer, RMSNorm, router_gate
from oracle import mhffn_oracle as orc


def _eager_op(Q, K, U, V, R):
    return orc.mhffn_forward(Q, K, U, V, R, compute_dtype=torch.float32)


@pytest.mark.parametrize("router_input,rms,Hk", [("q", False, 4), ("q", True, 2), ("x", False, 4)])
def test_block_matches_the_reference_module_arithmetic(router_input, rms, Hk):
    torch.manual_seed(0)
    B, S, hid, H, E, de = 2, 9, 32, 4, 3, 5
    layer = MHFFNLayer(hid, H, E, de, Hk, apply_rmsnorm=rms, router_input=router_input, op=_eager_op)
    if rms:
        with torch.no_grad():
            layer.q_norm.weight.uniform_(0.5, 1.5)
    x = torch.randn(B, S, hid, requires_grad=True)
    y = layer(x)
    kw = dict(router=layer.router) if router_input == "q" else dict(w_router=layer.w_router)
    x2 = x.detach().clone().requires_grad_(True)
    y_ref = orc.mhffn_block_forward(x2, layer.w_self.weight, layer.w_self_2.weight, layer.K, layer.U, layer.V,
                                    num_heads=H, q_norm_weight=layer.q_norm.weight if rms else None, **kw)
    assert torch.allclose(y, y_ref, atol=1e-5, rtol=1e-5)
    g = torch.randn_like(y)
    (gx,) = torch.autograd.grad(y, x, g)
    (gx_ref,) = torch.autograd.grad(y_ref, x2, g)
    assert torch.allclose(gx, gx_ref, atol=1e-5, rtol=1e-4)


def test_queries_reach_the_operator_token_major_and_merge_is_a_view():
    seen = {}

    def op(Q, K, U, V, R):
        seen["Q"], seen["R"] = Q, R
        return Q.clone(memory_format=torch.preserve_format)

    layer = MHFFNLayer(32, 4, 2, 4, op=op)
    layer(torch.randn(2, 7, 32))
    Q, R = seen["Q"], seen["R"]
    assert Q.shape == (2, 4, 7, 8) and Q.transpose(1, 2).is_contiguous() and not Q.is_contiguous()
    assert R.shape == (2, 4, 7, 2) and R.dtype == torch.float32 and R.is_contiguous()
    assert torch.allclose(R.sum(-1), torch.ones(2, 4, 7))


def test_load_reference_weights_puts_each_head_and_expert_where_the_kernels_expect_it():
    H, Hk, dh, E, de = 4, 2, 8, 3, 5
    layer = MHFFNLayer(H * dh, H, E, de, Hk, op=_eager_op)
    gate, up, down = (torch.randn(E * de, Hk * dh) for _ in range(3))      # modeling_mhffnmoe.py:343-345
    layer.load_reference_weights(gate, up, down)
    for hk in range(Hk):
        for e in range(E):
            # row i of the reference parameter is row i % d_e of expert i // d_e; columns hk*d_h.. belong to kuv-head hk
            assert torch.equal(layer.K[hk, e], gate[e * de:(e + 1) * de, hk * dh:(hk + 1) * dh])
            assert torch.equal(layer.U[hk, e], up[e * de:(e + 1) * de, hk * dh:(hk + 1) * dh])
            assert torch.equal(layer.V[hk, e], down[e * de:(e + 1) * de, hk * dh:(hk + 1) * dh])


def test_export_reference_weights_inverts_the_load():
    H, Hk, dh, E, de = 4, 2, 8, 3, 5
    layer = MHFFNLayer(H * dh, H, E, de, Hk, op=_eager_op)
    gate, up, down = (torch.randn(E * de, Hk * dh) for _ in range(3))
    layer.load_reference_weights(gate, up, down)
    for got, want in zip(layer.export_reference_weights(), (gate, up, down)):
        assert got.shape == want.shape and got.is_contiguous() and torch.equal(got, want)


def test_rmsnorm_and_gate_closed_forms():
    x = torch.tensor([[3.0, 4.0]])
    assert torch.allclose(RMSNorm((2,), eps=0.0)(x), x / (12.5 ** 0.5))
    ph = RMSNorm((2, 2), eps=0.0)
    with torch.no_grad():
        ph.weight.copy_(torch.tensor([[1.0, 1.0], [2.0, 0.5]]))
    xh = torch.tensor([[[[3.0, 4.0], [1.0, 1.0]]]])          # [B=1, S=1, H=2, d_h=2]
    assert torch.allclose(ph(xh), torch.tensor([[[[3.0, 4.0], [2.0, 0.5]]]]) / torch.tensor([[12.5 ** 0.5], [1.0]]))
    assert torch.allclose(router_gate(torch.zeros(2, 3)), torch.full((2, 3), 1 / 3))
    big = router_gate(torch.tensor([[-200.0, -200.0]]))       # sigmoid underflows to 0: the clamp keeps it finite
    assert torch.isfinite(big).all()


def test_decoder_runs_and_trains_on_cpu_with_the_eager_operator():
    torch.manual_seed(1)
    model = MHFFNDecoder(vocab_size=50, hidden_size=32, num_layers=2, attn_heads=4, ffn_heads=4, num_experts=2,
                         expert_dim=8, op=_eager_op)
    ids = torch.randint(0, 50, (2, 12))
    opt = torch.optim.SGD(model.parameters(), lr=0.5)
    losses = []
    for _ in range(8):
        loss = model(ids, labels=ids)
        opt.zero_grad()
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert all(map(lambda v: v == v, losses)) and losses[-1] < losses[0]
    # causality: changing a later token leaves earlier logits unchanged
    with torch.no_grad():
        a = model(ids)
        ids2 = ids.clone()
        ids2[:, -1] = (ids2[:, -1] + 1) % 50
        b = model(ids2)
    assert torch.allclose(a[:, :-1], b[:, :-1], atol=1e-6)
