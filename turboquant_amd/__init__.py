"""MI355X-native TurboQuant KV-cache engine (drop-in for the `turboquant` hot path)."""

from .codebook import compute_lloyd_max_codebook, get_codebook
from .quantizer import TurboQuantMSE, TurboQuantProd
from .kv_cache import TurboQuantKVCache

from .capture import RingBuffer, KVCaptureEngine
from .store import CompressedKVStore
from .score import compute_hybrid_attention

__version__ = "0.2.0"
