"""
MI355X-native TurboQuant V3 KV-cache compress / decompress path.

The directory name contains a hyphen, so import it through the `turboquant_amd`
alias module at the repository root (or `importlib.import_module("turboquant-pytorch_amd")`):

    from turboquant_amd import TurboQuantV3, MSECompressor
"""
from .lloyd_max import LloydMaxCodebook, solve_lloyd_max
from .rotation import generate_rotation_matrix
from .compressors_v3 import MSECompressor, TurboQuantV3
from .compressors import TurboQuantCompressorV2, TurboQuantCompressorMSE
from .kv_cache import V3Cache, hf_cache_class, packed_attention_forward, register_packed_attention
from .metrics import attention_scores, compute_metrics
from .serialize import save_cache, load_cache, save_compressed, load_compressed, codec_digest, FormatError
from . import _native

__all__ = [
    "MSECompressor", "TurboQuantV3", "TurboQuantCompressorV2", "TurboQuantCompressorMSE", "V3Cache", "hf_cache_class", "packed_attention_forward", "register_packed_attention", "attention_scores", "compute_metrics",
    "LloydMaxCodebook", "solve_lloyd_max",
    "generate_rotation_matrix", "_native",
    "save_cache", "load_cache", "save_compressed", "load_compressed", "codec_digest", "FormatError",
]
