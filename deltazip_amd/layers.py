"""Delta layers: the state holders that wrap a base linear layer and apply per-token deltas.

Mirrors the layer protocol of serving/vllm/delta/layers_marlin.py (eth-easl/deltazip):
`BaseLayerWithDelta.{create_delta_weights, reset_delta, set_delta, set_mapping}` (:61-95), the
stacked tensors each linear variant allocates (:311-333, 407-429, 510-534), `apply_weights` ->
`apply_delta` (:362-373, 461-472, 559-571), `forward` returning (output, output_bias) (:251-260,
573-597) and the `from_layer` factory (:736-750).

The reference has one class per tensor-parallel linear type of its vLLM fork.  On a single GPU all
of them compute the same thing, so the classes below share one implementation and differ only in
what `can_replace_layer` accepts.  A base layer is any module with a fp16 `weight` of shape
[out_features, in_features] (torch.nn.Linear fits); optional attributes `bias`, `skip_bias_add`
and `output_sizes` are honoured as the reference honours them.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
import torch.nn as nn

from . import ops
from .config import DeltaConfig

ASYNC_COPY = True


@dataclass
class DeltaMapping:
    """serving/vllm/delta/layers_marlin.py:46-58."""
    # Per every token in input_ids:
    index_mapping: Tuple[int, ...]
    # Per sampled token:
    prompt_mapping: Tuple[int, ...]

    def __post_init__(self):
        self.index_mapping = tuple(self.index_mapping)
        self.prompt_mapping = tuple(self.prompt_mapping)

    def __str__(self):
        return f"index_mapping: {self.index_mapping}, prompt_mapping: {self.prompt_mapping}"


class BaseLayerWithDelta(nn.Module):
    def create_delta_weights(self, max_deltas: int, delta_config: DeltaConfig, model_config=None) -> None:
        """Initializes delta matrices."""
        ...

    def reset_delta(self, index: int):
        """Resets the delta weights at index back to 0."""
        ...

    def set_delta(self, index: int, bitwidth: int, qweight, qzeros, scales, g_idx, meta):
        """Overwrites delta tensors at index."""
        ...

    def set_mapping(self, base_indices, sampler_indices, sampler_indices_padded, embeddings_indices,
                    indices_len: List[int]):
        """Sets the mapping indices."""
        ...


class LinearWithDelta(BaseLayerWithDelta):
    """Shared implementation of the four linear variants."""

    def __init__(self, base_layer: nn.Module) -> None:
        super().__init__()
        self.base_layer = base_layer
        self.indices: Optional[torch.Tensor] = None
        self.indices_len: Optional[List[int]] = None
        self.token_order: Optional[torch.Tensor] = None
        self.row_blocks: Optional[list] = None

    # -- state ---------------------------------------------------------------------------------
    def create_delta_weights(self, max_deltas: int, delta_config: DeltaConfig, model_config=None) -> None:
        w = self.base_layer.weight
        if w.dtype != torch.float16 or w.dim() != 2:
            raise ValueError("base layer weight must be float16 [out_features, in_features]")
        N, K = w.shape
        self.base_shape = (N, K)      # stays when the row-major weight is freed (keep_row_major_base=False)
        self.bits = delta_config.max_bitwidth
        self.pack_factor = delta_config.pack_factor
        self.group_size = delta_config.group_size
        qs, ms, ss = ops.stacked_shapes(K, N, self.bits, self.group_size)
        self.bitwidth = [0] * max_deltas
        self.qweight_stacked = torch.zeros((max_deltas,) + qs, dtype=torch.int32, device=w.device)
        self.meta_stacked = torch.zeros((max_deltas,) + ms, dtype=torch.int16, device=w.device)
        self.scales_stacked = torch.zeros((max_deltas,) + ss, dtype=torch.float16, device=w.device)
        self._tile_base = bool(delta_config.tile_base_weights) and w.is_cuda
        self._drop_row_major = self._tile_base and not delta_config.keep_row_major_base
        self._row_major_dropped = False
        self.base_tiled = None
        self.refresh_base_tiles()
        self._wrap_weight_loader()

    def refresh_base_tiles(self) -> None:
        """(Re)makes the tiled copy of the base weight that calls of up to 128 tokens read.  It runs
        when the delta weights are created; again, by itself, when the weight tensor has been
        replaced or written in place through autograd-visible ops (`weight.mul_()`, `weight.copy_()`
        under no_grad: the tensor's version counter moves); and after every call of the parameter's
        `weight_loader`, the way the serving engine loads and swaps base weights
        (model_executor/layers/linear.py:231, 305, 442, 616).  A write that bypasses all three --
        `weight.data.copy_()` from user code leaves the version counter where it was -- cannot be seen
        from here: call this method after it (or `DeltaModelManager.refresh_base_weights()`)."""
        if not self._tile_base or self._row_major_dropped:
            return
        w = self.base_layer.weight
        self.base_tiled = ops.tile_base(w.detach().contiguous())
        self._tiled_of = (w.data_ptr(), w._version)
        if self._drop_row_major:
            # one copy of the base weight: the tiles.  The parameter stays (empty) so that the
            # module tree and the loader hooks keep their shape.
            w.data = torch.empty(0, dtype=w.dtype, device=w.device)
            self._row_major_dropped = True

    def restore_row_major_base(self) -> torch.Tensor:
        """Rebuilds `base_layer.weight` from the tiled copy (keep_row_major_base=False frees it);
        `refresh_base_tiles()` afterwards tiles and frees it again."""
        if self._row_major_dropped:
            self.base_layer.weight.data = ops.untile_base(self.base_tiled)
            self._row_major_dropped = False
        return self.base_layer.weight

    def _wrap_weight_loader(self) -> None:
        """The engine's loaders write `param.data` (no version bump): a loader that a base parameter
        carries is wrapped so that the tiled copy follows every load."""
        w = self.base_layer.weight
        loader = getattr(w, "weight_loader", None)
        if loader is None or getattr(loader, "_refreshes_base_tiles", False):
            return

        def weight_loader(*args, **kwargs):
            self.restore_row_major_base()
            out = loader(*args, **kwargs)
            self.refresh_base_tiles()
            return out
        weight_loader._refreshes_base_tiles = True
        w.weight_loader = weight_loader

    def reset_delta(self, index: int):
        # all-zero scales make the slot contribute exactly 0 whatever the packed words hold
        self.bitwidth[index] = 0
        self.qweight_stacked[index] = 0
        self.scales_stacked[index] = 0
        self.meta_stacked[index] = 0x4444  # valid positions (0, 1) in every group

    def set_delta(self, index: int, bitwidth: int, qweight: torch.Tensor, qzeros, scales: torch.Tensor,
                  g_idx, meta: Optional[torch.Tensor]):
        """With `meta` given, (qweight, scales, meta) are in the native layout (as
        ops.repack_gptq_to_native returns them) and are copied into slot `index`, asynchronously
        when they sit in pinned host memory.  With meta=None the GPTQ-style (qweight, qzeros, scales,
        g_idx) are converted on the host first."""
        if bitwidth != self.bits:
            raise ValueError(f"layer was created for {self.bits}-bit deltas, got {bitwidth}")
        if meta is None:
            qweight, meta, scales = ops.repack_gptq_to_native(qweight, qzeros, scales, g_idx, bitwidth)
        self.reset_delta(index)
        self.bitwidth[index] = bitwidth
        self.qweight_stacked[index].copy_(qweight.view(self.qweight_stacked[index].shape), non_blocking=ASYNC_COPY)
        self.scales_stacked[index].copy_(scales.view(self.scales_stacked[index].shape), non_blocking=ASYNC_COPY)
        self.meta_stacked[index].copy_(meta.view(self.meta_stacked[index].shape), non_blocking=ASYNC_COPY)

    def set_mapping(self, base_indices: torch.Tensor, sampler_indices=None, sampler_indices_padded=None,
                    embeddings_indices=None, indices_len: Optional[List[int]] = None,
                    token_order: Optional[torch.Tensor] = None, row_blocks: Optional[list] = None):
        # a view of the manager's buffer, re-read on the device at every call
        self.indices = base_indices
        self.indices_len = indices_len if indices_len is not None else [base_indices.numel()]
        # optional: the manager's buffer with the order in which the kernel takes the tokens of a
        # 33..128-token batch (the manager refreshes it with the mapping; None: computed per call)
        self.token_order = token_order
        # optional: the manager's one-element list holding ops.row_blocks() of the current batch when
        # it has more than 128 tokens (None inside: made per call)
        self.row_blocks = row_blocks

    # -- compute -------------------------------------------------------------------------------
    def apply_weights(self, x: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        T = self.indices_len[0]
        order = self.token_order[:T] if self.token_order is not None and 32 < T <= ops.MAX_TOKENS_FUSED else None
        if T > ops.MAX_TOKENS_FUSED and self.row_blocks is not None:
            order = self.row_blocks[0]
        w = self.base_layer.weight
        if self._row_major_dropped:
            w = None
        elif self.base_tiled is not None and self._tiled_of != (w.data_ptr(), w._version):
            self.refresh_base_tiles()
            w = None if self._row_major_dropped else w
        return ops.apply_delta(x, self.qweight_stacked, self.scales_stacked, self.meta_stacked,
                               self.indices[:T], w, order=order, base_tiled=self.base_tiled)

    def forward(self, input_):
        skip_bias_add = getattr(self.base_layer, "skip_bias_add", False)
        base_bias = getattr(self.base_layer, "bias", None)
        bias = base_bias if not skip_bias_add else None
        output = self.apply_weights(input_, bias)
        if bias is not None:
            output = output + bias
        output_bias = base_bias if skip_bias_add else None
        return output, output_bias

    @property
    def weight(self):
        return self.base_layer.weight

    @property
    def linear_weights(self):
        return {"weight": self.base_layer.weight}

    @classmethod
    def can_replace_layer(cls, source_layer: nn.Module, delta_config: DeltaConfig, packed_modules_list: List,
                          model_config=None) -> bool:
        w = getattr(source_layer, "weight", None)
        if isinstance(source_layer, (nn.Embedding, BaseLayerWithDelta)):
            return False
        return isinstance(w, torch.Tensor) and w.dim() == 2 and len(packed_modules_list) == cls._n_packed


class ColumnParallelLinearWithDelta(LinearWithDelta):
    """layers_marlin.py:174-278."""
    _n_packed = 1


class MergedColumnParallelLinearWithDelta(LinearWithDelta):
    """gate_proj + up_proj fused along the output dimension (layers_marlin.py:281-388)."""
    _n_packed = 2

    def create_delta_weights(self, max_deltas, delta_config, model_config=None) -> None:
        sizes = getattr(self.base_layer, "output_sizes", None)
        if sizes is not None and not (len(sizes) == 2 and sizes[0] == sizes[1]):
            raise ValueError("DeltaColumnParallelLinear2Slice requires 2 slices with the same size.")
        super().create_delta_weights(max_deltas, delta_config, model_config)


class MergedQKVParallelLinearWithDelta(LinearWithDelta):
    """q, k and v projections fused along the output dimension (layers_marlin.py:391-487)."""
    _n_packed = 3


class RowParallelLinearWithDelta(LinearWithDelta):
    """o_proj / down_proj (layers_marlin.py:490-611)."""
    _n_packed = 0

    def apply_weights(self, x: torch.Tensor, bias=None) -> torch.Tensor:
        if getattr(self.base_layer, "bias", None) is not None:
            raise ValueError("RowParallelLinearWithDelta does not support bias yet.")
        return super().apply_weights(x, None)


class VocabParallelEmbeddingWithDelta(BaseLayerWithDelta):
    """Embedding whose table is replaced, per token, by the token's delta's own table
    (layers_marlin.py:97-171).  The base layer is any module with a fp16 `weight` [vocab, hidden]
    (torch.nn.Embedding fits)."""

    def __init__(self, base_layer: nn.Module) -> None:
        super().__init__()
        self.base_layer = base_layer
        self.indices: Optional[torch.Tensor] = None
        self.indices_len: Optional[List[int]] = None

    def create_delta_weights(self, max_deltas: int, delta_config: DeltaConfig, model_config=None) -> None:
        w = self.base_layer.weight
        if w.dtype != torch.float16 or w.dim() != 2:
            raise ValueError("base embedding weight must be float16 [vocab, hidden]")
        vocab = getattr(self.base_layer, "org_vocab_size", w.shape[0])
        self.delta_weights = torch.zeros((max_deltas, vocab, w.shape[1]), dtype=w.dtype, device=w.device)
        self.bitwidth = [0] * max_deltas

    def reset_delta(self, index: int):
        self.bitwidth[index] = 0
        self.delta_weights[index] = 0

    def set_delta(self, index: int, bitwidth: int, weight: torch.Tensor, *unused):
        self.bitwidth[index] = bitwidth
        self.delta_weights[index].copy_(weight, non_blocking=ASYNC_COPY)

    def set_mapping(self, base_indices: torch.Tensor, sampler_indices=None, sampler_indices_padded=None,
                    embeddings_indices=None, indices_len: Optional[List[int]] = None):
        self.indices = base_indices
        self.embeddings_indices = embeddings_indices
        self.indices_len = indices_len if indices_len is not None else [base_indices.numel()]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.apply_delta_embed(x, self.delta_weights, self.indices[: self.indices_len[0]],
                                     self.base_layer.weight)

    @classmethod
    def can_replace_layer(cls, source_layer: nn.Module, delta_config: DeltaConfig, packed_modules_list: List,
                          model_config=None) -> bool:
        return type(source_layer) is nn.Embedding


class LogitsProcessorWithDelta(BaseLayerWithDelta):
    """Output projection with one full [vocab, hidden] weight per delta (layers_marlin.py:614-725):
    a sampled row multiplies its delta's weight, or the base `embedding` passed to `_get_logits`
    when it has none.  `base_layer` only has to provide `vocab_size`; when it has a `forward` of
    its own (the serving engine's LogitsProcessor), `forward` defers to it with this object in
    place of `self`, as the reference does."""

    def __init__(self, base_layer, hidden_size: int, dtype: torch.dtype, device: torch.device) -> None:
        super().__init__()
        self.base_layer = base_layer
        self.hidden_size = hidden_size
        self.dtype = dtype
        self.device = device

    @property
    def vocab_size(self):
        return self.base_layer.vocab_size

    def __getattr__(self, name):
        # logits_as_input, scale, org_vocab_size, include_gpu_probs_tensor, ...: the base layer's
        try:
            return super().__getattr__(name)
        except AttributeError:
            if name == "base_layer":
                raise
            return getattr(self.base_layer, name)

    def create_delta_weights(self, max_deltas: int, delta_config: DeltaConfig, model_config=None) -> None:
        self.weight_stacked = torch.zeros((max_deltas, self.base_layer.vocab_size, self.hidden_size),
                                          dtype=self.dtype, device=self.device)
        self.indices = None
        self.indices_padded = None
        self.indices_len = None
        self.bitwidth = [0] * max_deltas

    def reset_delta(self, index: int):
        self.weight_stacked[index] = 0
        self.bitwidth[index] = 0

    def set_delta(self, index: int, bitwidth: int, weight: torch.Tensor, *unused):
        self.reset_delta(index)
        self.bitwidth[index] = bitwidth
        self.weight_stacked[index, :, :].copy_(weight, non_blocking=ASYNC_COPY)

    def set_mapping(self, base_indices, sampler_indices, sampler_indices_padded=None, embeddings_indices=None,
                    indices_len: Optional[List[int]] = None):
        self.indices = sampler_indices
        self.indices_padded = sampler_indices_padded
        self.indices_len = indices_len

    def _get_logits(self, hidden_states: torch.Tensor, embedding: torch.Tensor,
                    embedding_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.apply_delta_uncompressed(hidden_states, self.weight_stacked,
                                            self.indices[: self.indices_len[1]], base_embedding=embedding)

    def forward(self, *args, **kwargs):
        base_forward = getattr(type(self.base_layer), "forward", None)
        if base_forward is None or base_forward is nn.Module.forward:
            return self._get_logits(*args, **kwargs)
        return base_forward(self, *args, **kwargs)

    @classmethod
    def can_replace_layer(cls, source_layer, delta_config, packed_modules_list, model_config=None) -> bool:
        return False      # special handling: see from_layer_logits_processor


_all_delta_classes = (VocabParallelEmbeddingWithDelta, ColumnParallelLinearWithDelta,
                      MergedColumnParallelLinearWithDelta,
                      MergedQKVParallelLinearWithDelta, RowParallelLinearWithDelta)


def from_layer_logits_processor(layer, lm_head: nn.Module, max_deltas: int, delta_config: DeltaConfig,
                                model_config=None) -> LogitsProcessorWithDelta:
    """layers_marlin.py:753-768."""
    w = lm_head.weight
    ret = LogitsProcessorWithDelta(layer, w.shape[1], w.dtype, w.device)
    ret.create_delta_weights(max_deltas, delta_config, model_config)
    return ret


def from_layer(layer: nn.Module, max_deltas: int, delta_config: DeltaConfig, packed_modules_list: List,
               model_config=None) -> nn.Module:
    """layers_marlin.py:736-750: wrap `layer` in the first delta class that accepts it."""
    for delta_cls in _all_delta_classes:
        if delta_cls.can_replace_layer(layer, delta_config, packed_modules_list, model_config):
            ret = delta_cls(layer)
            ret.create_delta_weights(max_deltas, delta_config, model_config)
            return ret
    return layer


def convert_mapping(index_mapping, delta_index_to_id: List[Optional[int]], out: Optional[torch.Tensor] = None,
                    device=None) -> torch.Tensor:
    """Per-token delta id (0 or None = base) -> slot index (-1 = base), the part of
    serving/vllm/delta/models.py:69-145 that feeds `set_mapping`.  Writes into `out[:T]` when given
    (the manager's persistent buffer) and returns the [T] view."""
    slots = [(-1 if (i is None or i <= 0) else delta_index_to_id.index(i)) for i in index_mapping]
    t = torch.tensor(slots, dtype=torch.int64)
    if out is not None:
        out[: len(slots)].copy_(t, non_blocking=True)
        return out[: len(slots)]
    return t.to(device) if device is not None else t
