"""MI355X-native fused multi-head FFN (FlashMHF hot path): hand-written gfx950 HIP kernels behind the
reference's operator boundary.  See ``flash_mlp_moe`` (Triton-path signature) and ``flash_ffn_moe_torch``
(ThunderKittens-path signature); ``mhffn_layer`` holds the host side of one MH-FFN block and a minimal decoder."""
from .flash_mlp_moe import FlashMLPFunction, FlashMLPMoE, mhffn_backward, mhffn_forward  # noqa: F401
from .flash_ffn_moe_torch import FlashFFNMoE, FlashFFNMoEFunction  # noqa: F401
from .mhffn_layer import MHFFNDecoder, MHFFNLayer  # noqa: F401
from .flash_mlp import FlashMLP  # noqa: F401
