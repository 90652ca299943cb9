"""Prefill-sized calls (T > 128): per delta segment, dequantise the delta (dz_dequant, bit-exact)
and run the dense matrix-core GEMM over base and delta together (dz_gemm_f16_pair).

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


def multi_delta_linear_prefill(x2, base_weight, qweight_stacked, scales_stacked, meta_stacked, indices,
                               *, bits: int, out: torch.Tensor, accumulate: bool) -> torch.Tensor:
    from .ops import segment
    T, K = x2.shape
    N = scales_stacked.shape[-1]
    S = qweight_stacked.shape[0]
    G = scales_stacked[0].numel() // N
    group_size = -1 if G == 1 else K // G
    perm, seg_off = segment(indices, S)
    off = seg_off.cpu().tolist()          # segment sizes decide the launches: one host sync
    perm64 = perm.long()
    in_order = bool((perm64[1:] > perm64[:-1]).all().item()) if T > 1 else True
    xs = x2 if in_order else x2.index_select(0, perm64)
    ys = out if in_order else torch.empty((T, N), dtype=torch.float16, device=x2.device)
    if not in_order and accumulate:
        ys.copy_(out.index_select(0, perm64))
    stream = torch.cuda.current_stream().cuda_stream
    scratch = None
    for s in range(S + 1):
        lo, hi = off[s], off[s + 1]
        if hi == lo:
            continue
        w2 = None
        if s == 0:
            if base_weight is None:
                if not accumulate:
                    ys[lo:hi].zero_()
                continue
            w = base_weight
        else:
            d = s - 1
            if scratch is None:
                scratch = torch.empty((N, K), dtype=torch.float16, device=x2.device)
            rc = _lib.lib().dz_dequant(qweight_stacked[d].data_ptr(), meta_stacked[d].data_ptr(),
                                       scales_stacked[d].data_ptr(), K, N, bits, group_size,
                                       scratch.data_ptr(), stream)
            _lib.check(rc, "dz_dequant")
            if base_weight is not None:
                w, w2 = base_weight, scratch
            else:
                w = scratch
        gemm_f16(xs[lo:hi], w, ys[lo:hi], accumulate, w2)
    if not in_order:
        out.index_copy_(0, perm64, ys)
    return out
