"""TurboQuant+ KV-cache codec and compressed-KV attention on MI355X (gfx950).

Same public names as the reference package (turboquant/__init__.py:17-22);
the per-vector arithmetic runs in hand-written HIP kernels behind the C ABI
declared in include/tq.h.  `turbo` holds the production block format and the
attention entry points, which the reference only describes in prose.
"""
from .polar_quant import PolarQuant
from .qjl import QJL
from .turboquant import TurboQuant, TurboQuantMSE, CompressedVector
from .kv_cache import KVCacheCompressor, CompressedKVCache
from .outlier import OutlierTurboQuant, OutlierCompressedVector
from .policy import LayerFormat, LayerKV, layer_formats, effective_bits
from .turbo import (TurboCodec, DecodeAttention, q8_0_store, q8_0_unpack, q8_0_append, packed_bytes, PRODUCTION_CENTROIDS,
                    sparse_bias_from_dense, rows_of_256)

__all__ = ["PolarQuant", "QJL", "TurboQuant", "TurboQuantMSE", "CompressedVector", "KVCacheCompressor",
           "OutlierTurboQuant", "OutlierCompressedVector",
           "CompressedKVCache", "TurboCodec", "DecodeAttention", "q8_0_store", "q8_0_unpack", "q8_0_append", "packed_bytes",
           "PRODUCTION_CENTROIDS", "sparse_bias_from_dense", "rows_of_256", "LayerFormat", "LayerKV", "layer_formats",
           "effective_bits"]
