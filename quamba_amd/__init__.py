"""quamba_amd: MI355X-native (gfx950) kernels behind the Quamba quantized Mamba mixer modules."""
from .chunk_scan import Quamba2ChunkScan  # noqa: F401
from .conv import QCausalConv1D, Quamb2Conv1D  # noqa: F401
from .hadamard import QHadamard  # noqa: F401
from .mixer import W4A8QMamba, W4A8QMamba2, W8A8QMamba, W8A8QMamba2  # noqa: F401
from .norm import QRMSNormGated  # noqa: F401
from .linear import (W4A8B8O8Linear, W4A8B8O8LinearParallel, W4A8B16O16Linear, W8A8B8O8Linear,  # noqa: F401
                     W8A8B8O8LinearParallel, W8A8B16O16Linear)
from .sscan import QSScan, quant_selective_scan_fn  # noqa: F401
