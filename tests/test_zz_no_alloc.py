"""mhffn_bwd_static (the backward that allocates nothing: its dK/dU/dV partial sums live in a fixed device array inside the
library) against mhffn_bwd_layout on the same inputs, through the C ABI.  Two calls in a row share the array, the second
on a smaller problem, so stale partials of the first call would show up in the second.  Where both entry points run the
same number of token slices every output must be bit-identical; on a problem for which mhffn_bwd asks for more
workspace than the fixed array has, the static call runs fewer slices, so dK, dU, dV are sums of the same float32 terms
in another order (bar: 1e-5 of the tensor's largest value; dQ and dR stay bit-identical)."""
import ctypes

import pytest
import torch

from tests.helpers import make_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _run_both(shape, seed, dtype, wdtype, layout=0):
    from flashmhf_amd import _capi
    L = _capi.lib()
    B, H, S, dh, E, de, Hk = shape
    Q, K, U, V, R, dO = (t.to(DEV) for t in make_inputs(B, H, S, dh, E, de, Hk, seed=seed, dtype=dtype))
    if layout == _capi.TOKENS_BSHD:
        Q, dO = (t.transpose(1, 2).contiguous() for t in (Q, dO))     # memory [B,S,H,d_h]
    dims = _capi.Dims(B, H, Hk, S, dh, E, de)
    code, wcode = _capi.torch_dtype_code(dtype), _capi.torch_dtype_code(wdtype)
    st = torch.cuda.current_stream().cuda_stream

    def outputs():
        return [torch.full_like(Q, float("nan")), *(torch.full(K.shape, float("nan"), dtype=wdtype, device=DEV) for _ in range(3)),
                torch.full_like(R, float("nan"))]

    ref = outputs()
    ws = torch.empty(max(16, L.mhffn_bwd_workspace_bytes(dims, code)), dtype=torch.uint8, device=DEV)
    rc = L.mhffn_bwd_layout(*(t.data_ptr() for t in (Q, K, U, V, R, dO)), *(t.data_ptr() for t in ref), wcode,
                            ws.data_ptr(), ws.numel(), dims, code, layout, st, _capi.BWD_ALL)
    assert rc == 0, _capi.strerror(rc)
    got = outputs()
    rc = L.mhffn_bwd_static(*(t.data_ptr() for t in (Q, K, U, V, R, dO)), *(t.data_ptr() for t in got), wcode,
                            dims, code, layout, st)
    assert rc == 0, _capi.strerror(rc)
    torch.cuda.synchronize()
    return ref, got, ws.numel()


def test_static_scratch_backward_matches_the_workspace_backward_on_two_calls_in_a_row():
    from flashmhf_amd import _capi
    # first a problem whose partial sums fill half the array (4 slices of 12 MiB), then smaller ones, then float32
    calls = [((2, 4, 1024, 128, 8, 256, 4), 41, torch.bfloat16, torch.bfloat16, _capi.TOKENS_BHSD),
             ((1, 4, 300, 128, 2, 64, 2), 42, torch.bfloat16, torch.float32, _capi.TOKENS_BSHD),
             ((2, 3, 70, 96, 3, 96, 3), 43, torch.bfloat16, torch.bfloat16, _capi.TOKENS_BHSD),
             ((1, 2, 45, 40, 3, 24, 1), 44, torch.float32, torch.float32, _capi.TOKENS_BHSD)]
    for shape, seed, dtype, wdtype, layout in calls:
        print("case", shape, dtype, wdtype, layout, flush=True)
        ref, got, ws_bytes = _run_both(shape, seed, dtype, wdtype, layout)
        assert ws_bytes <= _capi.STATIC_SCRATCH_BYTES, "these cases are meant to run the same token slices in both calls"
        for name, a, b in zip(("dQ", "dK", "dU", "dV", "dR"), got, ref):
            assert not torch.isnan(a.float()).any(), name
            assert torch.equal(a, b), name


def test_static_scratch_backward_with_fewer_token_slices_than_the_workspace_backward():
    from flashmhf_amd import _capi
    # 6 heads of the 370M layer: mhffn_bwd asks for 4 slices of 34 MiB, the fixed 96 MiB array holds 2
    ref, got, ws_bytes = _run_both((8, 6, 2048, 128, 11, 352, 6), 45, torch.bfloat16, torch.float32)
    assert ws_bytes > _capi.STATIC_SCRATCH_BYTES, "this case is meant to need fewer token slices than mhffn_bwd uses"
    assert torch.equal(got[0], ref[0]) and torch.equal(got[4], ref[4])
    for name, a, b in zip(("dK", "dU", "dV"), got[1:4], ref[1:4]):
        err = (a - b).abs().max().item()
        assert err <= 1e-5 * b.abs().max().item(), (name, err)
    # and once more on a small problem right after the large one
    ref, got, _ = _run_both((1, 2, 257, 64, 2, 32, 2), 46, torch.bfloat16, torch.bfloat16)
    for name, a, b in zip(("dQ", "dK", "dU", "dV", "dR"), got, ref):
        assert torch.equal(a, b), name


def test_static_scratch_backward_rejects_what_does_not_fit_before_any_launch():
    from flashmhf_amd import _capi
    L = _capi.lib()
    dims = _capi.Dims(1, 16, 16, 64, 128, 22, 352)       # float32 partial sums: 3 * 16*22*352*128 * 4 B = 190 MB
    buf = torch.zeros(1024, device=DEV)
    p = buf.data_ptr()
    rc = L.mhffn_bwd_static(p, p, p, p, p, p, p, p, p, p, p, _capi.DTYPE_F32, dims, _capi.DTYPE_F32, 0, None)
    assert rc == _capi.ERR_STATIC_SCRATCH
    assert "mhffn_bwd_static" in _capi.strerror(rc)
    assert L.mhffn_bwd_workspace_bytes(dims, _capi.DTYPE_F32) > _capi.STATIC_SCRATCH_BYTES


def test_static_scratch_backward_allocates_no_device_memory():
    """The property the entry point exists for: after one warm-up call (address look-up, LDS opt-in) a call changes
    neither the device's free memory nor torch's allocator statistics.  Problem with several token slices, so the fixed
    array is really used."""
    from flashmhf_amd import _capi
    L = _capi.lib()
    B, H, S, dh, E, de, Hk = 2, 4, 1024, 128, 8, 256, 4
    Q, K, U, V, R, dO = (t.to(DEV) for t in make_inputs(B, H, S, dh, E, de, Hk, seed=5, dtype=torch.bfloat16))
    dims = _capi.Dims(B, H, Hk, S, dh, E, de)
    assert L.mhffn_bwd_workspace_bytes(dims, 0) > 0
    outs = [torch.empty_like(Q), *(torch.empty_like(K) for _ in range(3)), torch.empty_like(R)]
    st = torch.cuda.current_stream().cuda_stream
    args = (*(t.data_ptr() for t in (Q, K, U, V, R, dO)), *(t.data_ptr() for t in outs), 0, dims, 0, 0, st)
    assert L.mhffn_bwd_static(*args) == 0
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    reserved0, allocated0 = torch.cuda.memory_reserved(), torch.cuda.memory_allocated()
    for _ in range(3):
        assert L.mhffn_bwd_static(*args) == 0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    assert (torch.cuda.memory_reserved(), torch.cuda.memory_allocated()) == (reserved0, allocated0)
