"""Configuration objects of the delta layers.

Mirrors serving/vllm/delta/config.py:78-104 (DeltaConfig) of eth-easl/deltazip: `pack_factor` is
32 / bits codes per 32-bit word and `sparse_factor` is 2 (2:4 sparsity keeps half the values).
The reference selects the bit width through the BITWIDTH environment variable at import time;
here it is an explicit field.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from fractions import Fraction
from typing import Optional

import torch


@dataclass
class DeltaConfig:
    max_deltas: int = 1
    max_bitwidth: int = 4
    delta_dtype: Optional[torch.dtype] = torch.int32
    max_cpu_deltas: Optional[int] = None
    delta_extra_vocab_size: int = 0
    pack_factor: Fraction = field(default=Fraction(32, 1))
    sparse_factor: Fraction = field(default=Fraction(2, 1))
    # group size of the fp16 scales along the input dimension; -1 = one scale per output channel
    group_size: int = -1
    # every delta layer keeps a second copy of its base weight in the tiled form the fused kernel
    # streams fastest (calls of up to 128 tokens read it, larger ones the row-major weight); off:
    # the base weight is held once and read row-major by every call
    tile_base_weights: bool = True
    # off (needs tile_base_weights): once the tiled copy is made the layer frees the row-major base
    # weight -- `base_layer.weight` becomes an empty tensor -- and serves every batch size from the
    # tiles: one copy of the base model in memory instead of two.  The parameter's weight_loader
    # still works (the row-major form is rebuilt for the load and dropped again).
    keep_row_major_base: bool = True

    def __post_init__(self):
        if self.max_cpu_deltas is None:
            self.max_cpu_deltas = self.max_deltas
        elif self.max_cpu_deltas < self.max_deltas:
            raise ValueError("max_cpu_deltas must be greater than max_deltas")
        if not self.keep_row_major_base and not self.tile_base_weights:
            raise ValueError("keep_row_major_base=False needs tile_base_weights=True")
        if self.max_bitwidth not in (2, 4):
            raise ValueError("max_bitwidth must be 2 or 4")
        if self.group_size != -1 and (self.group_size <= 0 or self.group_size % 64):
            raise ValueError("group_size must be -1 or a positive multiple of 64")
        self.pack_factor = Fraction(32, self.max_bitwidth)
