"""Synthetic deltas in the native layout, made on the device.

`gaussian_native_stack` is the workload the benchmark configurations describe: every delta is
drawn from N(0, sigma), its scales come from the un-pruned values, it is pruned 2:4 by magnitude
and quantised (`ops.compress_delta`, byte-identical to the reference's pipeline followed by the
repacker).  Such deltas have most kept codes at or next to the zero-point and scales tied to the
row maximum.  The benchmark and the full-size parity tests use it.

`random_native_stack` fills the layout with uniformly random bits instead (every group of four
input columns gets a valid, uniformly chosen pair of kept positions; codes are uniform; scales
uniform in [2e-4, 1.2e-3)): every code and position value occurs equally often, which is what
the layout and arithmetic tests want, and it needs no fp32 delta (64 resident deltas of a whole
model are filled in seconds).
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


def gaussian_native_stack(K: int, N: int, bits: int, group_size: int, num_deltas: int, device,
                          generator: torch.Generator, sigma: float = 1e-3, keep_deltas=()):
    """(qweight_stacked, meta_stacked, scales_stacked) for `num_deltas` slots, each the compressed
    form of its own delta ~ N(0, sigma) [N, K] fp32 (drawn on the device from `generator`).
    keep_deltas: slot numbers whose fp32 delta is returned as well, as a dict slot -> tensor (for
    checks against the CPU restatement of the compression pipeline)."""
    qs, ms, ss = ops.stacked_shapes(K, N, bits, group_size)
    q = torch.empty((num_deltas,) + qs, dtype=torch.int32, device=device)
    m = torch.empty((num_deltas,) + ms, dtype=torch.int16, device=device)
    s = torch.empty((num_deltas,) + ss, dtype=torch.float16, device=device)
    deltas = {}
    for d in range(num_deltas):
        delta = torch.randn((N, K), device=device, dtype=torch.float32, generator=generator) * sigma
        q[d], m[d], s[d] = ops.compress_delta(delta, bits, group_size)
        if d in keep_deltas:
            deltas[d] = delta
    return (q, m, s, deltas) if keep_deltas else (q, m, s)
