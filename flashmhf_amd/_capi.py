"""ctypes binding of libmhffn_hip.so (declared in include/mhffn.h).

torch only supplies device memory and the current stream: tensors are passed as raw device pointers, the
stream as ``torch.cuda.current_stream().cuda_stream`` -- the same launch discipline as the reference's
launcher (kernels/thunderkittens/flash_ffn_moe.cu:991).  There is no CPU fallback: if the library has not
been built, loading raises and every operator that needs it fails loudly.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "_lib", "libmhffn_hip.so")

DTYPE_BF16, DTYPE_F32 = 0, 1
OK = 0
(ERR_NULL_POINTER, ERR_DTYPE, ERR_HEAD_DIM, ERR_EXPERT_DIM, ERR_SHAPE, ERR_WORKSPACE, ERR_LAUNCH, ERR_ALIGNMENT,
 ERR_STATIC_SCRATCH) = range(-1, -10, -1)
STATIC_SCRATCH_BYTES = 96 << 20

EXPORTS = (
    "mhffn_strerror", "mhffn_is_supported", "mhffn_check_dims", "mhffn_fwd_workspace_bytes",
    "mhffn_bwd_workspace_bytes", "mhffn_fwd", "mhffn_bwd", "mhffn_fwd_phases", "mhffn_bwd_phases",
    "mhffn_fwd_layout", "mhffn_bwd_layout", "mhffn_bwd_static", "mhffn_gate_fwd", "mhffn_gate_bwd",
)
TOKENS_BHSD, TOKENS_BSHD = 0, 1     # layout of Q, O, dO, dQ
FWD_MAIN, FWD_ALL = 1, 1
BWD_DQDR, BWD_DKDUDV, BWD_REDUCE, BWD_ALL = 1, 2, 4, 7


class Dims(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in ("B", "H", "Hkuv", "S", "d_h", "E", "d_e")]


_lib = None


def lib():
    """Loads the library once.  Raises ImportError (never falls back) when it is missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} not found: build it with `python -m flashmhf_amd.build` (hipcc, gfx950). "
                "flashmhf_amd has no CPU or eager fallback.")
        L = ctypes.CDLL(LIB_PATH)
        vp, dp = ctypes.c_void_p, ctypes.POINTER(Dims)
        L.mhffn_strerror.restype = ctypes.c_char_p
        L.mhffn_strerror.argtypes = [ctypes.c_int]
        L.mhffn_is_supported.argtypes = [ctypes.c_int] * 3
        L.mhffn_check_dims.argtypes = [dp, ctypes.c_int]
        for f in (L.mhffn_fwd_workspace_bytes, L.mhffn_bwd_workspace_bytes):
            f.restype = ctypes.c_size_t
            f.argtypes = [dp, ctypes.c_int]
        L.mhffn_fwd.argtypes = [vp] * 6 + [vp, ctypes.c_size_t, dp, ctypes.c_int, vp]
        L.mhffn_bwd.argtypes = [vp] * 6 + [vp] * 5 + [ctypes.c_int, vp, ctypes.c_size_t, dp, ctypes.c_int, vp]
        L.mhffn_fwd_phases.argtypes = L.mhffn_fwd.argtypes + [ctypes.c_int]
        L.mhffn_bwd_phases.argtypes = L.mhffn_bwd.argtypes + [ctypes.c_int]
        L.mhffn_fwd_layout.argtypes = [vp] * 6 + [vp, ctypes.c_size_t, dp, ctypes.c_int, ctypes.c_int, vp, ctypes.c_int]
        L.mhffn_bwd_layout.argtypes = ([vp] * 6 + [vp] * 5 + [ctypes.c_int, vp, ctypes.c_size_t, dp, ctypes.c_int,
                                                              ctypes.c_int, vp, ctypes.c_int])
        L.mhffn_bwd_static.argtypes = [vp] * 6 + [vp] * 5 + [ctypes.c_int, dp, ctypes.c_int, ctypes.c_int, vp]
        L.mhffn_gate_fwd.argtypes = [vp, vp, ctypes.c_float, vp, vp, vp, dp, vp]
        L.mhffn_gate_bwd.argtypes = [vp, vp, ctypes.c_float, vp, vp, ctypes.c_int, vp, vp, vp, vp, dp, vp]
        _lib = L
    return _lib


def strerror(code):
    return lib().mhffn_strerror(code).decode()


def raise_for_code(code, what):
    """Maps return codes to the exception types the reference raises for the same condition:
    TypeError for dtypes (kernels/triton/flash_mlp_moe.py:761-766), ValueError for the expert dim (:758-759),
    RuntimeError for everything a TORCH_CHECK would catch (kernels/thunderkittens/flash_ffn_moe.cu:943-958)."""
    if code == OK:
        return
    msg = f"{what}: {strerror(code)} (code {code})"
    if code == ERR_DTYPE:
        raise TypeError(msg)
    if code in (ERR_EXPERT_DIM, ERR_HEAD_DIM):
        raise ValueError(msg)
    raise RuntimeError(msg)


def torch_dtype_code(dt):
    if dt == torch.bfloat16:
        return DTYPE_BF16
    if dt == torch.float32:
        return DTYPE_F32
    return -1
