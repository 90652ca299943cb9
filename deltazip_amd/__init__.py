"""MI355X-native multi-delta linear layer (the hot path of DeltaZip-style serving).

    y = x @ W_base^T + x @ dequant(delta[id(x)])^T

Python keeps the reference's operator and layer API; all arithmetic runs in hand-written HIP
kernels for gfx950 behind the C ABI declared in include/dz_amd.h.  There is no CPU fallback.
"""
from .checkpoint import (CompressionConfig, DeltaLayerWeights, DeltaModel, compress_model, convert_model,
                         save_compressed, save_converted)
from .calibrate import lossy_compress
from .config import DeltaConfig
from .layers import (BaseLayerWithDelta, ColumnParallelLinearWithDelta, DeltaMapping, LogitsProcessorWithDelta,
                     MergedColumnParallelLinearWithDelta, MergedQKVParallelLinearWithDelta,
                     RowParallelLinearWithDelta, VocabParallelEmbeddingWithDelta, convert_mapping, from_layer,
                     from_layer_logits_processor)
from .manager import DeltaModelManager, LRUCacheDeltaModelManager, create_delta_manager
from .ops import (add_delta, add_delta_slice, apply_delta, apply_delta_batch, apply_delta_into, apply_delta_packed_nslice, apply_delta_embed, apply_delta_uncompressed, compress_delta, dequant, merge, multi_delta_linear,
                  native_sizes, repack_gptq_to_native, unrepack_native_to_gptq, segment, stacked_shapes, tile_base, token_order)
from .quant_linear import QuantLinear
from .sparsegpt import Quantizer, SparseGPT

__all__ = [
    "DeltaConfig", "BaseLayerWithDelta", "ColumnParallelLinearWithDelta", "DeltaMapping",
    "MergedColumnParallelLinearWithDelta", "MergedQKVParallelLinearWithDelta",
    "RowParallelLinearWithDelta", "convert_mapping", "from_layer", "add_delta", "add_delta_slice",
    "apply_delta", "dequant", "merge", "multi_delta_linear", "native_sizes",
    "repack_gptq_to_native", "unrepack_native_to_gptq", "segment", "stacked_shapes", "QuantLinear", "CompressionConfig",
    "DeltaLayerWeights", "DeltaModel", "convert_model", "compress_model", "save_compressed", "save_converted", "DeltaModelManager", "LRUCacheDeltaModelManager",
    "create_delta_manager", "LogitsProcessorWithDelta", "VocabParallelEmbeddingWithDelta",
    "from_layer_logits_processor", "apply_delta_embed", "apply_delta_uncompressed", "compress_delta", "apply_delta_batch", "token_order", "apply_delta_into", "apply_delta_packed_nslice",
    "Quantizer", "SparseGPT", "lossy_compress", "tile_base",
]
