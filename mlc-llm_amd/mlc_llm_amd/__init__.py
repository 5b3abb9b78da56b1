"""MI355X-native group-quantized linear path for MLC-LLM weights (q4f16_1 / q3f16_1).

Host-side mirror of the reference interface (`quantization`, `op.moe_matmul`,
`op.moe_misc`, `nn.MixtralMoE`) over a C-ABI HIP library (`_lib`, `ops`).
Importing the package does not load the library; the first operator call does,
and raises if it has not been built.
"""

from . import _lib, ops  # noqa: F401
from .quantization import (  # noqa: F401
    QUANTIZATION,
    GroupQuantize,
    GroupQuantizeEmbedding,
    GroupQuantizeLinear,
    GroupQuantizeMixtralExperts,
    MixtralExperts,
    QuantizeMapping,
)

__version__ = "0.1.0"
