"""Slot manager: which delta sits in which GPU slot, and the per-batch index tensors.

Stands in for serving/vllm/delta/models.py of eth-easl/deltazip, with its public names:
  :69-145    convert_mapping          (here: one H2D copy of the raw ids + one kernel, dz_map_ids,
                                       instead of a Python loop doing list.index per token)
  :266-503   DeltaModelManager        activate / deactivate / add / remove / set_delta_mapping,
                                       module replacement through `from_layer`
  :533-603   LRUCacheDeltaModelManager, create_delta_manager
The bookkeeping is one class with two tiers (host, slots) of the same small container and an
eviction policy flag, rather than a base manager plus a subclass that swaps its dictionaries for
caches with removal callbacks.

The manager owns the index buffers; the layers hold views of them (`set_mapping`), and the kernels
read them on the device when a layer runs.  `activate_delta` copies a delta's native-layout
tensors from (pinned) host memory into slot `index` of every wrapped layer on the current stream:
the compressed triples of the linear layers and the uncompressed per-delta tables of the embedding
and of the output projection (the latter held by the model's `logits_processor` sub-module, when
it has one).
"""
from __future__ import annotations

from typing import Any, Dict, Hashable, List, Optional, Type

import torch
import torch.nn as nn

from . import ops
from .checkpoint import DeltaModel
from .config import DeltaConfig
from .layers import BaseLayerWithDelta, DeltaMapping, LinearWithDelta, from_layer, from_layer_logits_processor


class LRUCache:
    """Bounded mapping that forgets its least recently used entry; same interface as the helper the
    serving engine uses (serving/vllm/utils.py:62-130: `get` / `put` / `touch` / `pop` /
    `remove_oldest` / `clear`, `_on_remove(key, value)` as the hook for subclasses).  Built on the
    insertion order of a plain dict: the first key is the oldest, using a key re-inserts it."""

    def __init__(self, capacity: int):
        self.capacity = capacity
        self._entries: Dict[Hashable, Any] = {}

    # container protocol
    def __contains__(self, key: Hashable) -> bool:
        return key in self._entries

    def __len__(self) -> int:
        return len(self._entries)

    def __getitem__(self, key: Hashable):
        return self.get(key)

    def __setitem__(self, key: Hashable, value) -> None:
        self.put(key, value)

    def __delitem__(self, key: Hashable) -> None:
        self.pop(key)

    def keys(self):
        return self._entries.keys()

    @property
    def cache(self) -> Dict[Hashable, Any]:
        return self._entries

    # recency
    def touch(self, key: Hashable) -> None:
        self._entries[key] = self._entries.pop(key)

    def get(self, key: Hashable, default_value=None):
        if key not in self._entries:
            return default_value
        self.touch(key)
        return self._entries[key]

    def put(self, key: Hashable, value) -> None:
        self._entries.pop(key, None)
        self._entries[key] = value
        while len(self._entries) > self.capacity:
            self.remove_oldest()

    # removal: every entry that leaves passes through the hook exactly once
    def _on_remove(self, key: Hashable, value) -> None:
        pass

    def remove_oldest(self) -> None:
        for key in self._entries:
            self._on_remove(key, self._entries.pop(key))
            return

    def pop(self, key: Hashable, default_value=None):
        if key not in self._entries:
            return default_value
        value = self._entries.pop(key)
        self._on_remove(key, value)
        return value

    def clear(self) -> None:
        while self._entries:
            self.remove_oldest()


def replace_submodule(model: nn.Module, module_name: str, new_module: nn.Module) -> nn.Module:
    """Puts `new_module` where the dotted name points (serving/vllm/delta/utils.py)."""
    parent_name, _, leaf = module_name.rpartition(".")
    setattr(model.get_submodule(parent_name), leaf, new_module)
    return new_module


class _Recency:
    """id -> value, remembered in order of last use (oldest first).  The manager's two sets -- the
    deltas registered in host memory and the deltas resident in GPU slots -- are one of these each;
    whether the oldest entry may be pushed out to make room is the manager's policy, not the
    container's."""

    def __init__(self) -> None:
        self._d: Dict[int, Any] = {}

    def __contains__(self, key: int) -> bool:
        return key in self._d

    def __len__(self) -> int:
        return len(self._d)

    def __iter__(self):
        return iter(self._d)

    def peek(self, key: int, default=None):
        return self._d.get(key, default)

    def use(self, key: int):
        value = self._d[key] = self._d.pop(key)
        return value

    def add(self, key: int, value) -> None:
        self._d.pop(key, None)
        self._d[key] = value

    def drop(self, key: int, default=None):
        return self._d.pop(key, default)

    def oldest(self) -> Optional[int]:
        return next(iter(self._d), None)

    def snapshot(self) -> Dict[int, Any]:
        return dict(self._d)

    def clear(self) -> None:
        self._d.clear()


class DeltaModelManager:
    """Keeps fine-tuned deltas in two tiers -- registered in (pinned) host memory, resident in one of
    the GPU slots of every wrapped layer -- and turns a batch's delta ids into the index tensors the
    layers read (the role of serving/vllm/delta/models.py:266-503; same public methods).

    `evict_lru = False`: a full tier refuses (`add_delta` raises RuntimeError, `activate_delta`
    raises ValueError), as the reference's plain manager does.  `evict_lru = True`
    (`LRUCacheDeltaModelManager`): the least recently used entry of the full tier makes room; a
    delta that leaves the host tier also leaves its slot."""

    evict_lru = False

    def __init__(self, model: nn.Module, max_num_seqs: int, max_num_batched_tokens: int, vocab_size: int,
                 delta_config: DeltaConfig, device: Optional[torch.device] = None) -> None:
        self.delta_config = delta_config
        self.max_num_seqs = max_num_seqs
        if self.capacity < self.delta_slots:
            raise AssertionError("capacity must be greater than delta_slots")
        self.max_num_batched_tokens = -(-max_num_batched_tokens // 8) * 8
        self.vocab_size = vocab_size
        self.device = torch.device(device if device is not None else next(model.parameters()).device)
        # the two tiers; `_slot_ids[i]` = id of the delta resident in slot i (public name:
        # delta_index_to_id, as in the reference)
        self._host = _Recency()          # id -> DeltaModel
        self._resident = _Recency()      # id -> slot
        self._slot_ids: List[Optional[int]] = [None] * self.delta_slots
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
        # which sub-modules carry deltas: the model says so (llama.py:336-339 of the serving model)
        self.supported_delta_modules: List[str] = list(getattr(model, "supported_delta_modules", []))
        self.packed_modules_mapping: Dict[str, List[str]] = {
            k: list(v) for k, v in getattr(model, "packed_modules_mapping", {}).items()}
        self.embedding_modules = dict(getattr(model, "embedding_modules",
                                              {"embed_tokens": "input_embeddings", "lm_head": "output_embeddings"}))
        self.packed_modules: Dict[str, List[str]] = {}
        self.modules: Dict[str, BaseLayerWithDelta] = {}
        self._last_mapping: Optional[DeltaMapping] = None
        self._wrap_modules()
        self.model.delta_manager = self

    # -- the two tiers -----------------------------------------------------------------------
    @property
    def capacity(self) -> int:
        return self.delta_config.max_cpu_deltas

    @property
    def delta_slots(self) -> int:
        return self.delta_config.max_deltas

    @property
    def delta_index_to_id(self) -> List[Optional[int]]:
        return self._slot_ids

    @delta_index_to_id.setter
    def delta_index_to_id(self, ids) -> None:
        # for callers that fill the layers' slot stacks themselves (synthetic benchmarks)
        ids = list(ids)
        if len(ids) != self.delta_slots:
            raise ValueError("one entry per slot")
        self._slot_ids[:] = ids
        self._resident.clear()
        for slot, d in enumerate(ids):
            if d is not None:
                self._resident.add(d, slot)
        self._slots_changed()

    def __len__(self) -> int:
        return len(self._host)

    def _slots_changed(self) -> None:
        self._slots_dirty = True
        self._last_mapping = None     # slot numbers may have changed under an unchanged mapping

    def _vacate(self, delta_id: int) -> Optional[int]:
        """Takes a delta out of the resident tier; returns the slot it held.  The slot's tensors stay
        as they are: nothing points at them until the next delta is written there."""
        slot = self._resident.drop(delta_id)
        if slot is not None:
            self._slot_ids[slot] = None
            self._slots_changed()
        return slot

    def _write_slot(self, slot: int, delta_model: DeltaModel) -> None:
        for name, module in self.modules.items():
            part = delta_model.get_delta(name)
            if part is None:
                module.reset_delta(slot)
            elif part._compressed:
                module.set_delta(slot, delta_model.bitwidth, part.qweight, part.qzeros, part.scales, part.g_idx,
                                 part.meta)
            else:
                module.set_delta(slot, delta_model.bitwidth, part.weight)

    def activate_delta(self, delta_id: int) -> bool:
        """Makes a registered delta resident: picks a slot (the lowest free one; with `evict_lru` the
        least recently activated delta's when none is free) and copies the delta's tensors into that
        slot of every wrapped layer.  False if it was resident already."""
        if delta_id in self._resident:
            self._resident.use(delta_id)
            return False
        if None not in self._slot_ids and not self.evict_lru:
            raise ValueError("No free delta slots")
        delta_model = self._host.use(delta_id)       # KeyError for an id that was never added
        if None not in self._slot_ids:
            self._vacate(self._resident.oldest())
        slot = self._slot_ids.index(None)
        self._slot_ids[slot] = delta_model.id
        self._resident.add(delta_id, slot)
        self._slots_changed()
        self._write_slot(slot, delta_model)
        return True

    def _deactivate_delta(self, delta_id: int) -> None:
        self._vacate(delta_id)

    def deactivate_delta(self, delta_id: int) -> bool:
        """Takes a delta out of its GPU slot; False if it had none."""
        return self._vacate(delta_id) is not None

    def add_delta(self, delta: DeltaModel) -> bool:
        """Registers a DeltaModel in the host tier; False if its id is registered already."""
        if delta.id in self._host:
            if self.evict_lru:
                self._host.use(delta.id)
            return False
        if len(self._host) >= self.capacity:
            if not self.evict_lru:
                raise RuntimeError("No free Delta slots.")
            self.remove_oldest_delta()
        self._host.add(delta.id, delta)
        return True

    def remove_delta(self, delta_id: int) -> bool:
        """Forgets a delta: out of its slot, out of the host tier."""
        self._vacate(delta_id)
        return self._host.drop(delta_id) is not None

    def remove_oldest_delta(self) -> bool:
        """Forgets the registered delta that was used longest ago."""
        oldest = self._host.oldest()
        return oldest is not None and self.remove_delta(oldest)

    def list_deltas(self) -> Dict[int, DeltaModel]:
        return self._host.snapshot()

    def get_delta(self, delta_id: int) -> Optional[DeltaModel]:
        if delta_id not in self._host:
            return None
        return self._host.use(delta_id) if self.evict_lru else self._host.peek(delta_id)

    def remove_all_deltas(self) -> None:
        self._host.clear()
        self._resident.clear()
        self._slot_ids[:] = [None] * self.delta_slots
        self._slots_changed()

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
    def _is_target(self, module_name: str) -> bool:
        """A module carries deltas when its dotted name is, or ends in, one of the model's
        `supported_delta_modules`."""
        return any(module_name == t or module_name.endswith("." + t) for t in self.supported_delta_modules)

    def _wrap_modules(self) -> None:
        """Swaps every target sub-module for its delta-carrying counterpart and hands it the index
        buffers.  The output projection is special: its per-delta tables live in the model's
        `logits_processor` (delta/models.py:467-479), which is wrapped in its stead and registered
        under the projection's name."""
        model_config = getattr(self.model, "config", None)
        for name, module in list(self.model.named_modules()):
            if not self._is_target(name):
                continue
            leaf = name.rpartition(".")[2]
            if self.embedding_modules.get(leaf) == "output_embeddings":
                if not hasattr(self.model, "logits_processor"):
                    continue
                wrapped = from_layer_logits_processor(self.model.logits_processor, module, self.delta_slots,
                                                      self.delta_config, model_config)
                replace_submodule(self.model, "logits_processor", wrapped)
            else:
                wrapped = from_layer(module, self.delta_slots, self.delta_config,
                                     self.packed_modules_mapping.get(leaf, []), model_config)
                if not isinstance(wrapped, BaseLayerWithDelta):
                    continue        # from_layer hands back what it cannot wrap
                replace_submodule(self.model, name, wrapped)
            self.register_module(name, wrapped)
            extra = ({"token_order": self.token_order, "row_blocks": self.row_blocks}
                     if isinstance(wrapped, LinearWithDelta) else {})
            wrapped.set_mapping(self.base_indices, self.sampler_indices, self.sampler_indices_padded,
                                self.embeddings_indices, self.indices_len, **extra)

    def register_module(self, module_name: str, module: BaseLayerWithDelta) -> None:
        if not isinstance(module, BaseLayerWithDelta):
            raise TypeError("only delta-carrying layers are registered")
        self.modules[module_name] = module
        # a fused layer also answers for the projections it is made of (q/k/v, gate/up)
        parent, _, leaf = module_name.rpartition(".")
        parts = self.packed_modules_mapping.get(leaf)
        if parts:
            self.packed_modules[module_name] = [f"{parent}.{part}" if parent else part for part in parts]


class LRUCacheDeltaModelManager(DeltaModelManager):
    """The manager with both tiers evicting their least recently used delta
    (role of delta/models.py:546-603)."""

    evict_lru = True


def create_delta_manager(model: nn.Module, max_num_seqs: int, max_num_batched_tokens: int, vocab_size: int,
                         delta_config: DeltaConfig,
                         delta_manager_cls: Type[DeltaModelManager] = DeltaModelManager,
                         **kwargs) -> DeltaModelManager:
    """Wraps the model's delta modules and returns their manager (delta/models.py:606-626)."""
    if not hasattr(model, "supported_delta_modules"):
        raise ValueError(f"Model {type(model)} is not supported for Delta.")
    return delta_manager_cls(model, max_num_seqs, max_num_batched_tokens, vocab_size, delta_config, **kwargs)
