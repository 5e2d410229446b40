"""The C-ABI calls only enqueue kernels on the stream they are given (no allocation, no synchronisation, no memset), so a
caller may record them into a HIP graph.  One graph holds the head prologue, the fused forward and the fused backward; it
is replayed several times with eager work and synchronisations in between, and every replay must reproduce the eager
results bit for bit (the weight-gradient sums of the prologue use float atomics and are compared with a tolerance)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_fused_calls_replay_from_a_graph():
    from flashmhf_amd import _capi
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(11)
    B, S, H, dh, E, de = 2, 150, 4, 128, 5, 96
    x = torch.randn(B, S, H, dh, generator=g).bfloat16().to(dev)
    wn = (torch.rand(H, dh, generator=g) + 0.5).to(dev)
    wr = (torch.randn(H, dh, E, generator=g) * 0.1).to(dev)
    K, U, V = ((torch.randn(H, E, de, dh, generator=g) * dh ** -0.5).bfloat16().to(dev) for _ in range(3))
    dO = torch.randn(B, S, H, dh, generator=g).bfloat16().to(dev)
    L = _capi.lib()
    dims = _capi.Dims(B, H, H, S, dh, E, de)
    Qn, O, dQ, dX = (torch.empty_like(x) for _ in range(4))
    R = torch.empty(B, H, S, E, device=dev)
    dR = torch.empty_like(R)
    dK, dU, dV = (torch.empty(H, E, de, dh, device=dev) for _ in range(3))
    dwn, dwr = torch.zeros_like(wn), torch.zeros_like(wr)
    ws = torch.empty(max(16, L.mhffn_bwd_workspace_bytes(dims, 0)), dtype=torch.uint8, device=dev)
    BSHD = _capi.TOKENS_BSHD

    def enqueue():
        st = torch.cuda.current_stream().cuda_stream
        rcs = [
            L.mhffn_gate_fwd(x.data_ptr(), wn.data_ptr(), 1e-6, wr.data_ptr(), Qn.data_ptr(), R.data_ptr(), dims, st),
            L.mhffn_fwd_layout(Qn.data_ptr(), K.data_ptr(), U.data_ptr(), V.data_ptr(), R.data_ptr(), O.data_ptr(),
                               None, 0, dims, 0, BSHD, st, _capi.FWD_ALL),
            L.mhffn_bwd_layout(Qn.data_ptr(), K.data_ptr(), U.data_ptr(), V.data_ptr(), R.data_ptr(), dO.data_ptr(),
                               dQ.data_ptr(), dK.data_ptr(), dU.data_ptr(), dV.data_ptr(), dR.data_ptr(), 1,
                               ws.data_ptr(), ws.numel(), dims, 0, BSHD, st, _capi.BWD_ALL),
            L.mhffn_gate_bwd(x.data_ptr(), wn.data_ptr(), 1e-6, wr.data_ptr(), dQ.data_ptr(), BSHD, dR.data_ptr(),
                             dX.data_ptr(), dwn.data_ptr(), dwr.data_ptr(), dims, st),
        ]
        assert rcs == [0, 0, 0, 0], rcs

    outs = (Qn, R, O, dQ, dK, dU, dV, dR, dX)
    enqueue()                       # eager reference; also performs the one-time per-kernel LDS opt-in outside capture
    torch.cuda.synchronize()
    ref = [t.clone() for t in outs]
    ref_dwn, ref_dwr = dwn.clone(), dwr.clone()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            enqueue()
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(3):
        for t in outs:
            t.fill_(float("nan")) if t.is_floating_point() else t.zero_()
        dwn.zero_()                  # a fill kernel, eager, between replays
        dwr.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, got, want in zip(("Qn", "R", "O", "dQ", "dK", "dU", "dV", "dR", "dX"), outs, ref):
            assert torch.equal(got, want), (replay, name)
        torch.testing.assert_close(dwn, ref_dwn, rtol=1e-4, atol=1e-5)
        torch.testing.assert_close(dwr, ref_dwr, rtol=1e-4, atol=1e-5)
        _ = (x.float() @ x.float().transpose(-1, -2)).sum().item()   # unrelated eager work + sync between replays
