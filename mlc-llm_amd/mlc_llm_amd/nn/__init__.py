"""Layer-level mirror: the quantized Mixtral MoE block."""
from .mixtral_moe import MixtralMoE  # noqa: F401
