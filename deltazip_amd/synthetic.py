"""Synthetic deltas generated directly in the native layout, on the device.

For benchmarks and full-size tests, where compressing real fp32 deltas on the host (a few seconds
per 4096 x 4096 matrix) would dominate the run.  Every group of four input columns gets a valid,
uniformly chosen pair of kept positions; codes are uniform random bits; scales are uniform in
[2e-4, 1.2e-3), the range symmetric 2..4-bit quantisation of sigma = 1e-3 deltas produces.
"""
from __future__ import annotations

import torch

from . import ops

# the six ways of keeping 2 of 4 positions, as (second << 2 | first) with first < second
_PAIRS = (0b0100, 0b1000, 0b1100, 0b1001, 0b1101, 0b1110)


def random_native_stack(K: int, N: int, bits: int, group_size: int, num_deltas: int, device,
                        generator: torch.Generator):
    """(qweight_stacked, meta_stacked, scales_stacked) for `num_deltas` slots."""
    qs, ms, ss = ops.stacked_shapes(K, N, bits, group_size)
    q = torch.randint(-2 ** 31, 2 ** 31 - 1, (num_deltas,) + qs, dtype=torch.int32, device=device,
                      generator=generator)
    pairs = torch.tensor(_PAIRS, dtype=torch.int64, device=device)
    nwords = num_deltas * ms[0] * ms[1] // 2
    w = torch.zeros(nwords, dtype=torch.int64, device=device)
    for f in range(8):
        w |= pairs[torch.randint(0, 6, (nwords,), device=device, generator=generator)] << (4 * f)
    m = torch.where(w >= 2 ** 31, w - 2 ** 32, w).to(torch.int32).view(torch.int16).view((num_deltas,) + ms)
    s = (torch.rand((num_deltas,) + ss, device=device, generator=generator) * 1e-3 + 2e-4).half()
    return q, m, s
