"""Prefill-sized calls (T > 128): sort the tokens by delta id, dequantise the deltas that are
present (dz_dequant, bit-exact) and run one grouped matrix-core GEMM over base and delta together
(dz_gemm_f16_grouped): every block of 256 tokens multiplies the base weight and its own delta.

This is the strategy the reference's exllama backend switches to above 50 rows: reconstruct the
weight, then a dense half-precision GEMM (serving/csrc/quantization/deltazip/exllama/cuda/
q_gemm.cu:118-137).  Base and delta products share fp32 accumulators; they are not summed in
fp16 first, which would cost about 5e-5 of the output range in absolute error.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib


def gemm_f16(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
             accumulate: bool = False, w2: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[T, N] (+)= x[T, K] @ w[N, K]^T (+ x @ w2^T) on the matrix cores."""
    T, K = x.shape
    N = w.shape[0]
    if out is None:
        out = torch.empty((T, N), dtype=torch.float16, device=x.device)
    st = torch.cuda.current_stream().cuda_stream
    if w2 is None:
        rc = _lib.lib().dz_gemm_f16(x.data_ptr(), w.data_ptr(), out.data_ptr(), T, K, N,
                                    1 if accumulate else 0, out.stride(0), st)
    else:
        rc = _lib.lib().dz_gemm_f16_pair(x.data_ptr(), w.data_ptr(), w2.data_ptr(), out.data_ptr(), T, K, N,
                                         1 if accumulate else 0, out.stride(0), st)
    _lib.check(rc, "dz_gemm_f16")
    return out


SCRATCH_LIMIT_BYTES = 4 << 30   # dequantised deltas held at once


def multi_delta_linear_prefill(x2, base_weight, qweight_stacked, scales_stacked, meta_stacked, indices,
                               *, bits: int, out: torch.Tensor, accumulate: bool) -> torch.Tensor:
    from .ops import segment
    T, K = x2.shape
    N = scales_stacked.shape[-1]
    S = qweight_stacked.shape[0]
    G = scales_stacked[0].numel() // N
    group_size = -1 if G == 1 else K // G
    lib = _lib.lib()
    perm, seg_off = segment(indices, S)
    off = seg_off.cpu().tolist()          # segment sizes decide the launches: one host sync
    perm64 = perm.long()
    in_order = bool((perm64[1:] > perm64[:-1]).all().item()) if T > 1 else True
    xs = x2 if in_order else x2.index_select(0, perm64)
    ys = out if in_order else torch.empty((T, N), dtype=torch.float16, device=x2.device)
    if not in_order and accumulate:
        ys.copy_(out.index_select(0, perm64))
    stream = torch.cuda.current_stream().cuda_stream

    def blocks(lo, hi, group):
        return [(r, min(r + 256, hi), group, 0) for r in range(lo, hi, 256)]

    present = [d for d in range(S) if off[d + 2] > off[d + 1]]
    per_chunk = max(1, SCRATCH_LIMIT_BYTES // (N * K * 2))
    chunks = [present[i:i + per_chunk] for i in range(0, len(present), per_chunk)] or [[]]
    scratch = None
    for ci, chunk in enumerate(chunks):
        tiles = []
        if ci == 0 and off[1] > off[0]:               # tokens without a delta
            if base_weight is not None:
                tiles += blocks(off[0], off[1], -1)
            elif not accumulate:
                ys[off[0]:off[1]].zero_()
        if chunk and scratch is None:
            scratch = torch.empty((min(per_chunk, len(present)), N, K), dtype=torch.float16, device=x2.device)
        for j, d in enumerate(chunk):
            rc = lib.dz_dequant(qweight_stacked[d].data_ptr(), meta_stacked[d].data_ptr(),
                                scales_stacked[d].data_ptr(), K, N, bits, group_size,
                                scratch[j].data_ptr(), stream)
            _lib.check(rc, "dz_dequant")
            tiles += blocks(off[d + 1], off[d + 2], j)
        if not tiles:
            continue
        tt = torch.tensor(tiles, dtype=torch.int32, device=x2.device)
        rc = lib.dz_gemm_f16_grouped(xs.data_ptr(), base_weight.data_ptr() if base_weight is not None else None,
                                     scratch.data_ptr() if scratch is not None else None, N * K,
                                     tt.data_ptr(), len(tiles), ys.data_ptr(), T, K, N,
                                     1 if accumulate else 0, ys.stride(0), stream)
        _lib.check(rc, "dz_gemm_f16_grouped")
    if not in_order:
        out.index_copy_(0, perm64, ys)
    return out
