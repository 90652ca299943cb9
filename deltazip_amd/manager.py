"""Slot manager: which delta sits in which GPU slot, and the per-batch index tensors.

Mirrors serving/vllm/delta/models.py of eth-easl/deltazip:
  :69-145    convert_mapping          (here: one H2D copy of the raw ids + one kernel, dz_map_ids,
                                       instead of a Python loop doing list.index per token)
  :266-503   DeltaModelManager        activate / deactivate / add / remove / set_delta_mapping,
                                       module replacement through `from_layer`
  :533-603   DeltaLRUCache, LRUCacheDeltaModelManager, create_delta_manager

The manager owns the index buffers; the layers hold views of them (`set_mapping`), and the kernels
read them on the device when a layer runs.  `activate_delta` copies a delta's native-layout
tensors from (pinned) host memory into slot `index` of every wrapped layer on the current stream:
the compressed triples of the linear layers and the uncompressed per-delta tables of the embedding
and of the output projection (the latter held by the model's `logits_processor` sub-module, when
it has one).
"""
from __future__ import annotations

import copy
import math
import re
from collections import OrderedDict
from typing import Any, Callable, Dict, Hashable, List, Optional, Type

import torch
import torch.nn as nn

from . import ops
from .checkpoint import DeltaModel
from .config import DeltaConfig
from .layers import BaseLayerWithDelta, DeltaMapping, LinearWithDelta, from_layer, from_layer_logits_processor


class LRUCache:
    """serving/vllm/utils.py:62-130."""

    def __init__(self, capacity: int):
        self.cache: "OrderedDict[Hashable, Any]" = OrderedDict()
        self.capacity = capacity

    def __contains__(self, key: Hashable) -> bool:
        return key in self.cache

    def __len__(self) -> int:
        return len(self.cache)

    def __getitem__(self, key: Hashable):
        return self.get(key)

    def __setitem__(self, key: Hashable, value) -> None:
        self.put(key, value)

    def __delitem__(self, key: Hashable) -> None:
        self.pop(key)

    def keys(self):
        return self.cache.keys()

    def touch(self, key: Hashable) -> None:
        self.cache.move_to_end(key)

    def get(self, key: Hashable, default_value=None):
        if key in self.cache:
            self.cache.move_to_end(key)
            return self.cache[key]
        return default_value

    def put(self, key: Hashable, value) -> None:
        self.cache[key] = value
        self.cache.move_to_end(key)
        while len(self.cache) > self.capacity:
            self.remove_oldest()

    def _on_remove(self, key: Hashable, value) -> None:
        pass

    def remove_oldest(self) -> None:
        if not self.cache:
            return
        key, value = self.cache.popitem(last=False)
        self._on_remove(key, value)

    def pop(self, key: Hashable, default_value=None):
        run_on_remove = key in self.cache
        value = self.cache.pop(key, default_value)
        if run_on_remove:
            self._on_remove(key, value)
        return value

    def clear(self) -> None:
        while len(self.cache) > 0:
            self.remove_oldest()
        self.cache.clear()


def replace_submodule(model: nn.Module, module_name: str, new_module: nn.Module) -> nn.Module:
    """serving/vllm/delta/utils.py: swap a sub-module by dotted name."""
    parent = model.get_submodule(".".join(module_name.split(".")[:-1]))
    setattr(parent, module_name.split(".")[-1], new_module)
    return new_module


class DeltaModelManager:
    """A manager that manages multiple full-fine-tuned models (delta/models.py:266-503)."""

    def __init__(self, model: nn.Module, max_num_seqs: int, max_num_batched_tokens: int, vocab_size: int,
                 delta_config: DeltaConfig, device: Optional[torch.device] = None) -> None:
        self.delta_config = delta_config
        self.max_num_seqs = max_num_seqs
        assert self.capacity >= self.delta_slots, "capacity must be greater than delta_slots"
        self.max_num_batched_tokens = math.ceil(max_num_batched_tokens / 8) * 8
        self.delta_index_to_id: List[Optional[int]] = [None] * self.delta_slots
        self.vocab_size = vocab_size
        if device is None:
            device = next(model.parameters()).device
        self.device = torch.device(device)
        n = self.max_num_batched_tokens
        self.base_indices = torch.empty(n, dtype=torch.long, device=self.device)
        self.sampler_indices = torch.empty(n, dtype=torch.long, device=self.device)
        self.sampler_indices_padded = torch.empty(n, dtype=torch.long, device=self.device)
        self.embeddings_indices = torch.empty(2, n, dtype=torch.long, device=self.device)
        # order in which the fused kernel takes the tokens of a 33..128-token batch; refreshed with
        # the mapping, shared by every linear layer
        self.token_order = torch.zeros(ops.MAX_TOKENS_FUSED, dtype=torch.int32, device=self.device)
        # larger batches: the tokens ordered by delta and cut into row blocks, made once per batch
        # (the layers keep a reference to this list)
        self.row_blocks = [None]
        # raw delta ids of the batch ([tokens | sampled rows]) and the id resident in each slot:
        # staged in pinned host memory, copied with one transfer each
        pin = self.device.type == "cuda"
        self._ids_host = torch.zeros(2 * n, dtype=torch.long, pin_memory=pin)
        self._ids_dev = torch.zeros(2 * n, dtype=torch.long, device=self.device)
        self._slots_host = torch.zeros(self.delta_slots, dtype=torch.long, pin_memory=pin)
        self._slots_dev = torch.zeros(self.delta_slots, dtype=torch.long, device=self.device)
        self._slots_dirty = True
        self._staged = torch.cuda.Event() if pin else None    # last copy out of the pinned buffers
        self.indices_len: List[int] = []
        self.model = model
        self.supported_delta_modules: List[str] = []
        self.packed_modules_mapping: Dict[str, List[str]] = {}
        if hasattr(self.model, "supported_delta_modules"):
            self.supported_delta_modules = copy.deepcopy(self.model.supported_delta_modules)
            self.packed_modules_mapping = copy.deepcopy(getattr(self.model, "packed_modules_mapping", {}))
        # llama.py:336-339 of the serving model
        self.embedding_modules = dict(getattr(self.model, "embedding_modules",
                                              {"embed_tokens": "input_embeddings", "lm_head": "output_embeddings"}))
        self.packed_modules: Dict[str, List[str]] = {}
        self.modules: Dict[str, BaseLayerWithDelta] = {}
        self._registered_deltas: Dict[int, DeltaModel] = {}
        self._active_deltas: Dict[int, None] = {}
        self._last_mapping: Optional[DeltaMapping] = None
        self._create_delta_modules()
        self.model.delta_manager = self

    # -- bookkeeping -----------------------------------------------------------------------
    @property
    def capacity(self) -> int:
        return self.delta_config.max_cpu_deltas

    @property
    def delta_slots(self) -> int:
        return self.delta_config.max_deltas

    def __len__(self) -> int:
        return len(self._registered_deltas)

    def activate_delta(self, delta_id: int) -> bool:
        """Move a delta into the GPU slots to be used in the forward pass."""
        if delta_id in self._active_deltas:
            return False
        index = next((i for i, d in enumerate(self.delta_index_to_id) if d is None), None)
        if index is None:
            raise ValueError("No free delta slots")
        self._active_deltas[delta_id] = None
        delta_model = self._registered_deltas[delta_id]
        self.delta_index_to_id[index] = delta_model.id
        self._slots_dirty = True
        self._last_mapping = None     # slot numbers may have changed under an unchanged mapping
        for module_name, module in self.modules.items():
            module_delta = delta_model.get_delta(module_name)
            if module_delta is None:
                module.reset_delta(index)
            elif module_delta._compressed:
                module.set_delta(index, delta_model.bitwidth, module_delta.qweight, module_delta.qzeros,
                                 module_delta.scales, module_delta.g_idx, module_delta.meta)
            else:
                module.set_delta(index, delta_model.bitwidth, module_delta.weight)
        return True

    def _deactivate_delta(self, delta_id: int) -> None:
        try:
            index = self.delta_index_to_id.index(delta_id)
            self.delta_index_to_id[index] = None
            self._slots_dirty = True
            self._last_mapping = None
        except ValueError:
            pass

    def deactivate_delta(self, delta_id: int) -> bool:
        """Remove a delta from its GPU slot."""
        if delta_id in self._active_deltas:
            self._deactivate_delta(delta_id)
            self._active_deltas.pop(delta_id)
            return True
        return False

    def _add_delta(self, delta: DeltaModel) -> None:
        self._registered_deltas[delta.id] = delta

    def add_delta(self, delta: DeltaModel) -> bool:
        """Add a DeltaModel to the manager's host cache."""
        if delta.id not in self._registered_deltas:
            if len(self._registered_deltas) >= self.capacity:
                raise RuntimeError("No free Delta slots.")
            self._add_delta(delta)
            return True
        return False

    def remove_delta(self, delta_id: int) -> bool:
        """Remove a DeltaModel from the manager's host cache."""
        self.deactivate_delta(delta_id)
        return bool(self._registered_deltas.pop(delta_id, None))

    def list_deltas(self) -> Dict[int, DeltaModel]:
        return dict(self._registered_deltas)

    def get_delta(self, delta_id: int) -> Optional[DeltaModel]:
        return self._registered_deltas.get(delta_id, None)

    def remove_all_deltas(self) -> None:
        self._registered_deltas.clear()
        self.delta_index_to_id = [None] * self.delta_slots
        self._active_deltas.clear()
        self._slots_dirty = True
        self._last_mapping = None

    # -- the per-batch mapping -------------------------------------------------------------
    def _set_delta_mapping(self, mapping: DeltaMapping) -> None:
        T, P = len(mapping.index_mapping), len(mapping.prompt_mapping)
        n = self.max_num_batched_tokens
        if T < 1 or T > n or P > n:
            raise ValueError(f"batch of {T} tokens / {P} sampled rows does not fit the index buffers ({n})")
        resident = {d for d in self.delta_index_to_id if d is not None}
        for ids in (mapping.index_mapping, mapping.prompt_mapping):
            for x in set(ids):
                if x > 0 and x not in resident:
                    raise ValueError(f"{x} is not in list")     # what list.index raises in the reference
        if self._staged is not None:
            self._staged.synchronize()      # the previous transfer has read the staging buffers
        # the kernels' status words (a delta id out of range; a partial sum that did not arrive): the
        # copy started at the previous batch is looked at, the next one is started -- no wait of its own
        ops.poll_status(self.device)
        if self._slots_dirty:
            self._slots_host.copy_(torch.tensor([d if d is not None else 0 for d in self.delta_index_to_id],
                                                dtype=torch.long))
            self._slots_dev.copy_(self._slots_host, non_blocking=True)
            self._slots_dirty = False
        self._ids_host[:T] = torch.tensor(mapping.index_mapping, dtype=torch.long)
        if P:
            self._ids_host[T:T + P] = torch.tensor(mapping.prompt_mapping, dtype=torch.long)
        self._ids_dev[:T + P].copy_(self._ids_host[:T + P], non_blocking=True)
        if self._staged is not None:
            self._staged.record()
        ops.map_ids(self._ids_dev[:T], self._ids_dev[T:T + P] if P else None, self._slots_dev,
                    self.delta_slots + 1, self.vocab_size, self.delta_config.delta_extra_vocab_size,
                    self.base_indices, self.sampler_indices, self.sampler_indices_padded,
                    self.embeddings_indices)
        if 32 < T <= ops.MAX_TOKENS_FUSED:
            ops.token_order(self.base_indices[:T], self.delta_slots, out=self.token_order)
        self.row_blocks[0] = None
        if T > ops.MAX_TOKENS_FUSED and not ops.takes_fused_chunks(T, self.delta_slots):
            self.row_blocks[0] = ops.row_blocks(self.base_indices[:T], self.delta_slots)
        # the layers keep a reference to this list
        self.indices_len[:] = (T, P, P, T)

    def refresh_base_weights(self) -> None:
        """Re-tiles the base weight of every delta layer: for callers that have written base weights
        in a way the layers cannot see (`weight.data.copy_()`), e.g. after swapping the base model."""
        for module in self.modules.values():
            if isinstance(module, LinearWithDelta):
                module.refresh_base_tiles()

    def check_status(self) -> None:
        """Looks at the kernels' status words now (synchronises with the stream the layers run on):
        raises `ops.DeltaKernelError` if a launch since the last look reported an invalid output, warns
        once about delta ids out of range.  `set_delta_mapping` does the same for the previous batch
        without waiting; this is for a point of the caller's choosing (end of a step, shutdown)."""
        ops.poll_status(self.device, wait=True)

    def set_delta_mapping(self, delta_mapping: DeltaMapping) -> None:
        if self._last_mapping != delta_mapping:
            self._set_delta_mapping(delta_mapping)
        self._last_mapping = delta_mapping

    # -- module replacement ----------------------------------------------------------------
    def _create_delta_modules(self) -> None:
        for module_name, module in list(self.model.named_modules()):
            if not self._match_target_modules(module_name):
                continue
            last = module_name.split(".")[-1]
            model_config = getattr(self.model, "config", None)
            if self.embedding_modules.get(last) == "output_embeddings":
                # the output projection's delta lives in the logits processor (models.py:467-479)
                try:
                    logits_processor = self.model.get_submodule("logits_processor")
                except AttributeError:
                    continue
                new_module = replace_submodule(
                    self.model, "logits_processor",
                    from_layer_logits_processor(logits_processor, module, self.delta_slots, self.delta_config,
                                                model_config))
            else:
                packed = self.packed_modules_mapping.get(last, [])
                new_module = from_layer(module, self.delta_slots, self.delta_config, packed, model_config)
                if not isinstance(new_module, BaseLayerWithDelta):
                    continue
                replace_submodule(self.model, module_name, new_module)
            self.register_module(module_name, new_module)
            self._register_packed_modules(module_name)
            if isinstance(new_module, LinearWithDelta):
                new_module.set_mapping(self.base_indices, self.sampler_indices, self.sampler_indices_padded,
                                       self.embeddings_indices, self.indices_len, token_order=self.token_order,
                                       row_blocks=self.row_blocks)
            else:
                new_module.set_mapping(self.base_indices, self.sampler_indices, self.sampler_indices_padded,
                                       self.embeddings_indices, self.indices_len)

    def register_module(self, module_name: str, module: BaseLayerWithDelta) -> None:
        assert isinstance(module, BaseLayerWithDelta)
        self.modules[module_name] = module

    def _match_target_modules(self, module_name: str) -> bool:
        return any(re.match(r".*\.{target_module}$".format(target_module=t), module_name) or t == module_name
                   for t in self.supported_delta_modules)

    def _register_packed_modules(self, module_full_name: str) -> None:
        parts = module_full_name.split(".")
        replacements = self.packed_modules_mapping.get(parts[-1])
        if not replacements:
            return
        prefix = ".".join(parts[:-1])
        self.packed_modules[module_full_name] = [prefix + "." + r if prefix else r for r in replacements]


class DeltaLRUCache(LRUCache):
    def __init__(self, capacity: int, deactivate_delta_fn: Callable[[Hashable], None]):
        super().__init__(capacity)
        self.deactivate_delta_fn = deactivate_delta_fn

    def _on_remove(self, key: Hashable, value) -> None:
        self.deactivate_delta_fn(key)
        return super()._on_remove(key, value)


class LRUCacheDeltaModelManager(DeltaModelManager):
    """A manager that evicts the least recently used delta (delta/models.py:546-603)."""

    def __init__(self, model: nn.Module, max_num_seqs: int, max_num_batched_tokens: int, vocab_size: int,
                 delta_config: DeltaConfig, device: Optional[torch.device] = None):
        super().__init__(model, max_num_seqs, max_num_batched_tokens, vocab_size, delta_config, device)
        self._registered_deltas = DeltaLRUCache(self.capacity, self.deactivate_delta)
        self._active_deltas = DeltaLRUCache(self.delta_slots, self._deactivate_delta)

    def list_deltas(self) -> Dict[int, DeltaModel]:
        return dict(self._registered_deltas.cache)

    def add_delta(self, delta: DeltaModel) -> bool:
        if delta.id not in self._registered_deltas:
            self._add_delta(delta)
            return True
        self._registered_deltas.touch(delta.id)   # always touch to update the LRU order
        return False

    def activate_delta(self, delta_id: int) -> bool:
        if delta_id not in self._active_deltas and len(self._active_deltas) >= self.delta_slots:
            self._active_deltas.remove_oldest()
        result = super().activate_delta(delta_id)
        self._active_deltas.touch(delta_id)
        return result

    def remove_oldest_delta(self) -> bool:
        if len(self._registered_deltas) > 0:
            self._registered_deltas.remove_oldest()
            return True
        return False


def create_delta_manager(model: nn.Module, max_num_seqs: int, max_num_batched_tokens: int, vocab_size: int,
                         delta_config: DeltaConfig,
                         delta_manager_cls: Type[DeltaModelManager] = DeltaModelManager,
                         **kwargs) -> DeltaModelManager:
    """Create a delta manager for a given model (delta/models.py:606-626)."""
    if not hasattr(model, "supported_delta_modules"):
        raise ValueError(f"Model {type(model)} is not supported for Delta.")
    return delta_manager_cls(model=model, max_num_seqs=max_num_seqs,
                             max_num_batched_tokens=max_num_batched_tokens, vocab_size=vocab_size,
                             delta_config=delta_config, **kwargs)
