"""gaac_amd: the GAAC compressed-KV decode path (lossless BF16 KV codec, block encoder, fused split-K decode attention,
slot cache) for AMD MI355X, with the Python surface of the reference's `gaac` package."""
from .codec import Codec, Page
from .encoder import TileEncoder
from .kernel import attention, choose_nsplit
from .kv_cache import CompressedKVCache
from .calibration import BaseCollector

__all__ = ["Codec", "Page", "TileEncoder", "attention", "choose_nsplit", "CompressedKVCache", "BaseCollector"]
