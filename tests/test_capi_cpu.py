"""CPU-side checks of the C-ABI library and the Python operator boundary: the library loads, exports every symbol
include/mhffn.h declares, and rejects bad arguments with the documented codes / the reference's exception types.
No compute call is made (no GPU here)."""
import ctypes
import os
import re

import pytest
import torch

from flashmhf_amd import _capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def L():
    if not os.path.exists(_capi.LIB_PATH):
        from flashmhf_amd.build import build_lib
        build_lib()
    return _capi.lib()


def test_every_declared_symbol_is_exported(L):
    header = open(os.path.join(ROOT, "include", "mhffn.h")).read()
    declared = set(re.findall(r"\b(mhffn_[a-z_]+)\s*\(", header))
    assert declared == set(_capi.EXPORTS)
    for name in declared:
        assert getattr(L, name) is not None


def test_strerror_and_is_supported(L):
    assert _capi.strerror(0) == "ok"
    for code in range(-8, 0):
        assert "unknown" not in _capi.strerror(code)
    assert "unknown" in _capi.strerror(-99)
    assert L.mhffn_is_supported(128, 352, 0) == 1      # the 370M / 1.3B benchmark shape the reference kernels reject
    assert L.mhffn_is_supported(96, 256, 0) == 1
    assert L.mhffn_is_supported(64, 32, 0) == 1
    assert L.mhffn_is_supported(128, 48, 0) == 0
    assert L.mhffn_is_supported(80, 64, 0) == 0
    assert L.mhffn_is_supported(128, 64, 1) == 1       # fp32 correctness instantiation
    assert L.mhffn_is_supported(40, 7, 1) == 1         # ... generic in d_h (multiple of 8) and d_e
    assert L.mhffn_is_supported(132, 64, 1) == 0
    assert L.mhffn_is_supported(128, 64, 2) == 0


@pytest.mark.parametrize("dims,dtype,code", [
    ((8, 8, 8, 2048, 128, 11, 352), 0, 0),
    ((8, 8, 8, 2048, 128, 11, 350), 0, _capi.ERR_EXPERT_DIM),
    ((8, 8, 8, 2048, 100, 11, 352), 0, _capi.ERR_HEAD_DIM),
    ((8, 8, 3, 2048, 128, 11, 352), 0, _capi.ERR_SHAPE),
    ((0, 8, 8, 2048, 128, 11, 352), 0, _capi.ERR_SHAPE),
    ((8, 8, 8, 2048, 128, 65, 352), 0, _capi.OK),            # more experts than one LDS gate window holds
    ((8, 8, 8, 2048, 128, 11, 352), 1, 0),
    ((8, 8, 8, 2048, 100, 11, 352), 1, _capi.ERR_HEAD_DIM),
    ((8, 8, 8, 2048, 128, 11, 352), 7, _capi.ERR_DTYPE),
])
def test_check_dims_codes(L, dims, dtype, code):
    d = _capi.Dims(*dims)
    assert L.mhffn_check_dims(d, dtype) == code
    if code != 0:
        assert L.mhffn_fwd_workspace_bytes(d, dtype) == 0 and L.mhffn_bwd_workspace_bytes(d, dtype) == 0
    elif dtype == _capi.DTYPE_F32:
        assert L.mhffn_bwd_workspace_bytes(d, dtype) > 0     # float32 kernels: partial sums of dK/dU/dV
    else:
        # 11 * 11 * 8 = 968 weight-block columns fill the chip without slicing the tokens: no partial sums
        assert L.mhffn_bwd_workspace_bytes(d, dtype) == 0


def test_backward_workspace_follows_the_token_slice_policy(L):
    """bfloat16 dK/dU/dV: the tokens are cut into slices only where the weight-block columns alone leave compute units
    idle; each slice beyond the first costs one float32 copy of dK, dU, dV in the workspace (256-byte aligned)."""
    one = 3 * 4 * 128                                        # bytes per weight row over dK, dU, dV
    for dims, slices in (((8, 8, 8, 2048, 128, 11, 352), 1), ((4, 16, 16, 8192, 128, 22, 352), 1),
                         ((8, 6, 6, 2048, 128, 11, 352), 4), ((2, 4, 4, 1024, 128, 8, 256), 4)):
        d = _capi.Dims(*dims)
        rows = dims[2] * dims[5] * dims[6]
        want = 0 if slices == 1 else -(-slices * rows * one // 256) * 256
        assert L.mhffn_bwd_workspace_bytes(d, _capi.DTYPE_BF16) == want, (dims, slices)


def test_entry_points_validate_before_touching_the_gpu(L):
    d = _capi.Dims(1, 2, 2, 64, 128, 2, 64)
    null = ctypes.c_void_p(0)
    assert L.mhffn_fwd(null, null, null, null, null, null, null, 0, d, 0, null) == _capi.ERR_NULL_POINTER
    assert L.mhffn_bwd(*([null] * 11), 0, null, 0, d, 0, null) == _capi.ERR_NULL_POINTER
    odd = ctypes.c_void_p(0x1008)
    ok = ctypes.c_void_p(0x1000)
    assert L.mhffn_fwd(odd, ok, ok, ok, ok, ok, ok, 1 << 30, d, 0, null) == _capi.ERR_ALIGNMENT
    sliced = _capi.Dims(2, 4, 4, 1024, 128, 8, 256)          # a shape whose backward keeps partial sums (4 token slices)
    assert L.mhffn_bwd(*([ok] * 11), 0, ok, 16, sliced, 0, null) == _capi.ERR_WORKSPACE
    assert L.mhffn_bwd(*([ok] * 11), 0, null, 1 << 30, sliced, 0, null) == _capi.ERR_WORKSPACE
    assert L.mhffn_bwd(*([ok] * 11), 5, ok, 1 << 30, d, 0, null) == _capi.ERR_DTYPE
    bad = _capi.Dims(1, 2, 2, 64, 128, 2, 65)
    assert L.mhffn_fwd(ok, ok, ok, ok, ok, ok, ok, 1 << 30, bad, 0, null) == _capi.ERR_EXPERT_DIM
    # token-layout variants: same checks, plus the layout code itself
    assert L.mhffn_fwd_layout(null, null, null, null, null, null, null, 0, d, 0, _capi.TOKENS_BSHD, null, _capi.FWD_ALL) == _capi.ERR_NULL_POINTER
    assert L.mhffn_fwd_layout(ok, ok, ok, ok, ok, ok, ok, 1 << 30, d, 0, 7, null, _capi.FWD_ALL) == _capi.ERR_SHAPE
    assert L.mhffn_bwd_layout(*([ok] * 11), 0, ok, 1 << 30, d, 0, -1, null, _capi.BWD_ALL) == _capi.ERR_SHAPE
    assert L.mhffn_bwd_layout(*([ok] * 11), 0, ok, 16, sliced, 0, _capi.TOKENS_BSHD, null, _capi.BWD_ALL) == _capi.ERR_WORKSPACE
    # phase masks with a bit the header does not define are refused, not ignored (the bit values have changed before)
    assert L.mhffn_fwd_layout(ok, ok, ok, ok, ok, ok, ok, 1 << 30, d, 0, 0, null, 2) == _capi.ERR_SHAPE
    assert L.mhffn_fwd_phases(ok, ok, ok, ok, ok, ok, ok, 1 << 30, d, 0, null, 3) == _capi.ERR_SHAPE
    assert L.mhffn_bwd_layout(*([ok] * 11), 0, ok, 1 << 30, d, 0, 0, null, 8) == _capi.ERR_SHAPE
    assert L.mhffn_bwd_phases(*([ok] * 11), 0, ok, 1 << 30, d, 0, null, 15) == _capi.ERR_SHAPE
    # more than 2^31 token rows are rejected (row indices are 32-bit inside the kernels)
    huge = _capi.Dims(4096, 64, 64, 1 << 14, 128, 2, 64)
    assert L.mhffn_check_dims(huge, 0) == _capi.ERR_SHAPE


def test_gate_entry_points_validate_before_touching_the_gpu(L):
    d = _capi.Dims(1, 2, 2, 64, 128, 2, 32)
    null, ok, odd = ctypes.c_void_p(0), ctypes.c_void_p(0x1000), ctypes.c_void_p(0x1004)
    assert L.mhffn_gate_fwd(null, null, 1e-6, null, null, null, d, null) == _capi.ERR_NULL_POINTER
    assert L.mhffn_gate_fwd(ok, ok, 1e-6, ok, null, ok, d, null) == _capi.ERR_NULL_POINTER     # norm weight without Qn
    assert L.mhffn_gate_fwd(ok, ok, 1e-6, ok, odd, ok, d, null) == _capi.ERR_ALIGNMENT
    assert L.mhffn_gate_fwd(ok, ok, 1e-6, ok, ok, ok, _capi.Dims(1, 2, 2, 64, 100, 2, 32), null) == _capi.ERR_HEAD_DIM
    assert L.mhffn_gate_fwd(ok, ok, 1e-6, ok, ok, ok, _capi.Dims(1, 2, 2, 64, 128, 65, 32), null) == _capi.ERR_SHAPE
    assert L.mhffn_gate_fwd(ok, ok, 1e-6, ok, ok, ok, _capi.Dims(1, 70000, 2, 64, 128, 2, 32), null) == _capi.ERR_SHAPE
    assert L.mhffn_gate_bwd(ok, ok, 1e-6, ok, ok, 0, ok, ok, null, ok, d, null) == _capi.ERR_NULL_POINTER   # norm without its grad
    assert L.mhffn_gate_bwd(ok, ok, 1e-6, ok, ok, 5, ok, ok, ok, ok, d, null) == _capi.ERR_SHAPE
    assert L.mhffn_gate_bwd(ok, ok, 1e-6, ok, ok, 1, ok, odd, ok, ok, d, null) == _capi.ERR_ALIGNMENT
    assert L.mhffn_gate_bwd(ok, ok, 1e-6, ok, ok, 1, ok, ok, ok, ok, None, null) == _capi.ERR_NULL_POINTER


def test_head_gate_python_boundary_checks():
    import torch
    from flashmhf_amd.head_gate import head_norm_gate
    x = torch.zeros(1, 4, 2, 128, dtype=torch.bfloat16)
    router = torch.zeros(2, 128, 3)
    with pytest.raises(RuntimeError, match="GPU only"):
        head_norm_gate(x, None, router)
    with pytest.raises(TypeError):
        head_norm_gate(x.float(), None, router)
    with pytest.raises(RuntimeError, match="router must be"):
        head_norm_gate(x, None, torch.zeros(3, 128, 3))
    with pytest.raises(RuntimeError, match="norm_weight must be"):
        head_norm_gate(x, torch.zeros(2, 64), router)


def test_python_boundary_raises_reference_exception_types():
    from flashmhf_amd import FlashFFNMoE, FlashMLPMoE
    Q = torch.zeros(1, 2, 8, 128, dtype=torch.bfloat16)
    K = torch.zeros(2, 2, 64, 128, dtype=torch.bfloat16)
    R = torch.zeros(1, 2, 8, 2)
    for mod in (FlashMLPMoE(), FlashFFNMoE()):
        with pytest.raises(TypeError):                     # flash_mlp_moe.py:761-766 (mixed dtypes)
            mod(Q.float(), K, K, K, R)
        with pytest.raises(TypeError):
            mod(Q.half(), K.half(), K.half(), K.half(), R)
        with pytest.raises(TypeError):
            mod(Q, K, K, K, R.bfloat16())
        with pytest.raises(ValueError):                    # flash_mlp_moe.py:758-759
            mod(Q, K[:, :, :40], K[:, :, :40], K[:, :, :40], R)
        with pytest.raises(RuntimeError):                  # no CPU path: must fail loudly, never fall back
            mod(Q, K, K, K, R)
        with pytest.raises(RuntimeError):
            mod(Q, K, K, K, R[..., :1])


def test_legacy_single_expert_signature_checks():
    """flash_mlp.py:1050-1058: only SiLU, no dot scaling, U required -- all ValueError, before any GPU work."""
    from flashmhf_amd import FlashMLP
    Q = torch.zeros(1, 2, 8, 64, dtype=torch.bfloat16)
    W = torch.zeros(2, 32, 64, dtype=torch.bfloat16)
    op = FlashMLP()
    with pytest.raises(ValueError):
        op(Q, W, W, W, False, 1.0, 1.0, "gelu")
    with pytest.raises(ValueError):
        op(Q, W, W, W, True, 1.0, 1.0, "silu")
    with pytest.raises(ValueError):
        op(Q, W, W, W, False, 2.0, 1.0, "silu")
    with pytest.raises(ValueError):
        op(Q, W, None, W, False, 1.0, 1.0, "silu")
    with pytest.raises(RuntimeError):          # CPU tensors: there is no CPU path
        op(Q, W, W, W, False, 1.0, 1.0, "silu")


def test_raise_for_code_mapping():
    with pytest.raises(TypeError):
        _capi.raise_for_code(_capi.ERR_DTYPE, "x")
    with pytest.raises(ValueError):
        _capi.raise_for_code(_capi.ERR_EXPERT_DIM, "x")
    with pytest.raises(ValueError):
        _capi.raise_for_code(_capi.ERR_HEAD_DIM, "x")
    with pytest.raises(RuntimeError):
        _capi.raise_for_code(_capi.ERR_LAUNCH, "x")
    _capi.raise_for_code(0, "x")


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_capi, "_lib", None)
    monkeypatch.setattr(_capi, "LIB_PATH", "/nonexistent/libmhffn_hip.so")
    with pytest.raises(ImportError):
        _capi.lib()


def test_tile_permutations_are_bijections():
    """The two index permutations baked into the packed tiles (mirrors of the constexpr functions in
    csrc/mhffn_common.hpp) must be bijections on 0..31 that realise the documented register/slot mapping."""
    row_perm = lambda r: 16 * ((r >> 3) >> 1) + 8 * ((r >> 2) & 1) + 4 * ((r >> 3) & 1) + (r & 3)
    tok_perm = lambda p: (p & 16) + 8 * ((p >> 2) & 1) + 4 * ((p >> 3) & 1) + (p & 3)
    assert sorted(map(row_perm, range(32))) == list(range(32))
    assert sorted(map(tok_perm, range(32))) == list(range(32))
    for g in range(2):
        for i in range(16):                     # C register i of lane group g is MFMA output row 8(i/4)+4g+i%4
            rho = 8 * (i // 4) + 4 * g + i % 4
            s, kk = divmod(i, 8)
            assert row_perm(rho) == 16 * s + 8 * g + kk      # ... and must be B-operand k-slot (s, g, kk)
            assert tok_perm(16 * s + 8 * g + kk) == rho
