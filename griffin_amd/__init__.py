"""MI355X-native RG-LRU: the reference's RG_LRU / RecurrentBlock interface over hand-written
gfx950 HIP kernels (``scan_mode="hip"``)."""

from .hip_scan import (
    PreparedParams,
    hip_rglru,
    hip_rglru_scan,
    hip_rglru_step,
    hip_rglru_steps,
    hip_scan_available,
    hip_scan_is_usable,
    set_chain_forward,
    set_reproducible,
)
from .hip_block_ops import (hip_block_forward, hip_causal_conv, hip_causal_conv_padded, hip_gelu_gate, hip_linear,
                            hip_linear_pair, hip_rmsnorm)
from .modules import (
    BlockDiagonalLinear,
    RG_LRU,
    RMSNorm,
    RecurrentBlock,
    RecurrentBlockCache,
)

__all__ = [
    "BlockDiagonalLinear",
    "PreparedParams",
    "RG_LRU",
    "RMSNorm",
    "RecurrentBlock",
    "RecurrentBlockCache",
    "hip_block_forward",
    "hip_causal_conv",
    "hip_causal_conv_padded",
    "hip_gelu_gate",
    "hip_linear",
    "hip_linear_pair",
    "hip_rmsnorm",
    "hip_rglru",
    "hip_rglru_scan",
    "hip_rglru_step",
    "hip_rglru_steps",
    "hip_scan_available",
    "hip_scan_is_usable",
    "set_chain_forward",
    "set_reproducible",
]
