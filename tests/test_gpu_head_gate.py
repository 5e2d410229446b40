"""Head prologue kernels (per-head RMSNorm + expert gate) through the C ABI against the CPU restatement
(oracle.head_norm_gate, following models/flashmhf/modeling_mhffnmoe.py:97-135 and :384-386)."""
import pytest
import torch

from oracle import mhffn_oracle as orc

pytestmark = pytest.mark.gpu

CASES = [
    # B, S, H, dh, E, norm
    (2, 128, 4, 128, 11, True),
    (1, 77, 3, 96, 8, True),
    (2, 200, 2, 64, 5, False),
    (1, 33, 2, 128, 40, True),      # two expert tiles
    (3, 1, 5, 96, 1, True),         # one token, one expert
    (1, 2048, 8, 128, 22, True),    # several tiles per wave
    (1, 31, 1, 64, 64, False),
]


def _inputs(B, S, H, dh, E, norm, seed=0, router_bf16=True):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(B, S, H, dh, generator=g) * 1.5).bfloat16()
    w = (torch.rand(H, dh, generator=g) + 0.5).bfloat16() if norm else None
    router = torch.randn(H, dh, E, generator=g) * 0.1
    router = router.bfloat16() if router_bf16 else router
    return x, w, router


def _bf16_ulps(a, b):
    """Largest difference between two bf16 tensors in units of the larger magnitude's ulp."""
    a, b = a.float(), b.float()
    ulp = torch.maximum(a.abs(), b.abs()).clamp(min=1e-30).log2().floor().exp2() * 2.0 ** -7
    return ((a - b).abs() / ulp).max().item()


@pytest.mark.parametrize("B,S,H,dh,E,norm", CASES)
@pytest.mark.parametrize("router_bf16", [True, False])
def test_gate_forward_matches_oracle(B, S, H, dh, E, norm, router_bf16):
    from flashmhf_amd.head_gate import head_norm_gate
    print(f"case B={B} S={S} H={H} dh={dh} E={E} norm={norm} router_bf16={router_bf16}", flush=True)
    x, w, router = _inputs(B, S, H, dh, E, norm, router_bf16=router_bf16)
    ref_Q, _ = orc.head_norm_gate(x, w, router, eps=1e-6)
    dev = "cuda:0"
    Q, R = head_norm_gate(x.to(dev), None if w is None else w.to(dev), router.to(dev), 1e-6)
    torch.cuda.synchronize()
    assert Q.shape == (B, H, S, dh) and Q.transpose(1, 2).is_contiguous() and R.shape == (B, H, S, E)
    Qc = Q.cpu()
    if norm:
        # same fp32 operations in the same order; only the reduction order of the mean and a 1-ulp rsqrt differ, which
        # can move a product across a bf16 rounding boundary: at most one bf16 ulp, on few elements
        assert _bf16_ulps(Qc, ref_Q) <= 1.0
        assert (Qc != ref_Q).float().mean().item() < 5e-3
    else:
        assert torch.equal(Qc, ref_Q)
    # the gate is checked on the Q the kernel produced: products of bf16 values are exact in fp32, so only the
    # accumulation order and the sigmoid's last bits differ
    _, ref_R = orc.head_norm_gate(Qc.transpose(1, 2), None, router)
    torch.testing.assert_close(R.cpu(), ref_R, rtol=2e-5, atol=2e-6)
    torch.testing.assert_close(R.sum(-1).cpu(), torch.ones(B, H, S), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("B,S,H,dh,E,norm", CASES)
@pytest.mark.parametrize("token_major_dq", [True, False])
def test_gate_backward_matches_autograd_of_oracle(B, S, H, dh, E, norm, token_major_dq):
    from flashmhf_amd.head_gate import head_norm_gate
    print(f"case B={B} S={S} H={H} dh={dh} E={E} norm={norm} token_major_dq={token_major_dq}", flush=True)
    x, w, router = _inputs(B, S, H, dh, E, norm, seed=1)
    g = torch.Generator().manual_seed(2)
    dQ = torch.randn(B, H, S, dh, generator=g).bfloat16()
    dR = torch.randn(B, H, S, E, generator=g)
    # reference: fp32 autograd of the restatement on the same bf16 inputs (the cast of Q to bf16 passes gradients through)
    leaves = [x.float().requires_grad_(True), None if w is None else w.float().requires_grad_(True),
              router.float().requires_grad_(True)]
    rq, rR = orc.head_norm_gate(leaves[0], leaves[1], leaves[2], eps=1e-6)
    (rq * dQ.float()).sum().add((rR * dR).sum()).backward()
    dev = "cuda:0"
    xd = x.to(dev).requires_grad_(True)
    wd = None if w is None else w.to(dev).requires_grad_(True)
    rd = router.to(dev).requires_grad_(True)
    Q, R = head_norm_gate(xd, wd, rd, 1e-6)
    dQd = dQ.to(dev)
    if token_major_dq:
        dQd = dQd.transpose(1, 2).contiguous().transpose(1, 2)
    torch.autograd.backward([Q, R], [dQd, dR.to(dev)])
    torch.cuda.synchronize()
    pairs = [("dx", xd.grad, leaves[0].grad), ("d_router", rd.grad, leaves[2].grad)]
    if norm:
        pairs.append(("d_norm_weight", wd.grad, leaves[1].grad))
    for name, got, ref in pairs:
        assert torch.isfinite(got).all(), name
        m = orc.error_metrics(got.float().cpu(), ref)
        scale = max(1.0, ref.abs().max().item())
        assert m["max_abs"] <= 2e-2 * scale, (name, m)
        if ref.abs().max().item() > 1e-4:      # E = 1 makes the gate identically 1: its gradients are rounding noise
            assert m["mean_rel"] <= 1e-2, (name, m)


def test_gate_backward_accumulates_into_weight_gradients():
    """d_router and d_norm_weight are added to what the buffers hold: a second call doubles them; dx is overwritten."""
    from flashmhf_amd import _capi
    B, S, H, dh, E = 2, 100, 3, 96, 7
    x, w, router = _inputs(B, S, H, dh, E, True, seed=3)
    dev = "cuda:0"
    g = torch.Generator().manual_seed(4)
    xd, wd, rd = x.to(dev), w.float().to(dev), router.float().to(dev)
    dQ = torch.randn(B, S, H, dh, generator=g).bfloat16().to(dev)
    dR = torch.randn(B, H, S, E, generator=g).to(dev)
    dx = torch.empty_like(xd)
    dwn, dwr = torch.zeros_like(wd), torch.zeros_like(rd)
    L, dims, st = _capi.lib(), _capi.Dims(B, H, H, S, dh, E, 32), torch.cuda.current_stream().cuda_stream

    def call():
        rc = L.mhffn_gate_bwd(xd.data_ptr(), wd.data_ptr(), 1e-6, rd.data_ptr(), dQ.data_ptr(), _capi.TOKENS_BSHD,
                              dR.data_ptr(), dx.data_ptr(), dwn.data_ptr(), dwr.data_ptr(), dims, st)
        assert rc == 0, rc
        torch.cuda.synchronize()

    call()
    dx1, dwn1, dwr1 = dx.clone(), dwn.clone(), dwr.clone()
    call()
    assert torch.equal(dx, dx1)
    torch.testing.assert_close(dwn, 2 * dwn1, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(dwr, 2 * dwr1, rtol=1e-5, atol=1e-6)


def test_layer_with_and_without_the_fused_prologue_agree():
    from flashmhf_amd import MHFFNLayer
    torch.manual_seed(0)
    dev = "cuda:0"
    layer = MHFFNLayer(256, 2, 4, 64, apply_rmsnorm=True).to(dev).bfloat16()
    with torch.no_grad():
        layer.q_norm.weight.uniform_(0.5, 1.5)
        layer.router.normal_(0, 0.2)
    x = torch.randn(2, 70, 256, device=dev).bfloat16()
    outs = []
    for fused in (True, False):
        layer.fused_prologue = fused
        layer.zero_grad(set_to_none=True)
        xi = x.clone().requires_grad_(True)
        y = layer(xi)
        y.float().square().mean().backward()
        outs.append((y.detach().float(), xi.grad.float(), layer.router.grad.float(), layer.q_norm.weight.grad.float(),
                     layer.w_self.weight.grad.float()))
    for name, a, b in zip(("y", "dx", "d_router", "d_q_norm", "d_w_self"), *outs):
        scale = max(b.abs().max().item(), 1e-6)
        assert (a - b).abs().max().item() <= 3e-2 * scale, (name, (a - b).abs().max().item(), scale)


def test_gate_saturation_and_zero_rows():
    """Zero rows (rsqrt of eps alone), logits far beyond the sigmoid's range in both directions, and a head whose every
    logit underflows (sum of sigmoids below the clamp): forward and backward stay finite and on the oracle."""
    from flashmhf_amd.head_gate import head_norm_gate
    B, S, H, dh, E = 1, 64, 3, 128, 6
    x, w, router = _inputs(B, S, H, dh, E, True, seed=9)
    x[:, 3] = 0                                   # a token whose every head row is zero
    router = router.float()
    router[0] *= 400.0                            # head 0: logits of a few hundred, both signs
    router[1] = -3.0 * w[1].float().sign().unsqueeze(-1) * torch.ones(dh, E)   # head 1: strongly negative for most rows
    router = router.bfloat16()
    g = torch.Generator().manual_seed(10)
    dQ = torch.randn(B, H, S, dh, generator=g).bfloat16()
    dR = torch.randn(B, H, S, E, generator=g)
    leaves = [x.float().requires_grad_(True), w.float().requires_grad_(True), router.float().requires_grad_(True)]
    rq, rR = orc.head_norm_gate(leaves[0], leaves[1], leaves[2], eps=1e-6)
    (rq * dQ.float()).sum().add((rR * dR).sum()).backward()
    dev = "cuda:0"
    xd, wd, rd = (t.to(dev).requires_grad_(True) for t in (x, w, router))
    Q, R = head_norm_gate(xd, wd, rd, 1e-6)
    torch.autograd.backward([Q, R], [dQ.to(dev), dR.to(dev)])
    torch.cuda.synchronize()
    assert torch.equal(Q[:, :, 3].cpu().float(), torch.zeros(B, H, dh))
    torch.testing.assert_close(R[:, :, 3].cpu(), torch.full((B, H, E), 1.0 / E))
    _, ref_R = orc.head_norm_gate(Q.detach().cpu().transpose(1, 2), None, router)
    assert torch.isfinite(R).all()
    torch.testing.assert_close(R.detach().cpu(), ref_R, rtol=1e-4, atol=1e-6)
    for name, got, ref in (("dx", xd.grad, leaves[0].grad), ("d_router", rd.grad, leaves[2].grad),
                           ("d_norm_weight", wd.grad, leaves[1].grad)):
        assert torch.isfinite(got).all(), name
        m = orc.error_metrics(got.float().cpu(), ref)
        assert m["norm_max"] <= 2e-2 and m["mean_rel"] <= 2e-2, (name, m)
