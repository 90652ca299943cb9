"""Prefill-sized calls (T > 128) on the matrix cores.

The reference's exllama backend switches, above 50 rows, to "reconstruct the weight, then a dense
half-precision GEMM" (serving/csrc/quantization/deltazip/exllama/cuda/q_gemm.cu:118-137).  Here
the delta is never reconstructed in memory: dz_multi_delta_gemm multiplies the base weight on the
dense matrix-core instructions and each token block's delta, straight from its packed form, on
the 2:4-sparse ones, into the same fp32 accumulators (base and delta are not summed in fp16
first, which would cost about 5e-5 of the output range in absolute error).
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
                               *, bits: int, out: torch.Tensor, accumulate: bool, blocks=None,
                               base_tiled=None) -> torch.Tensor:
    """T > 128: tokens are ordered by delta id on the device (dz_segment), the order is cut into
    row blocks of one delta each (dz_build_tiles) and one launch of dz_multi_delta_gemm multiplies
    every block by the base weight and by its delta in packed form.  Nothing is read back to the
    host, gathered, scattered or dequantised to memory.  `blocks`: ops.row_blocks(indices, S) when
    the caller made it once for the batch (else made here, per call).  `base_tiled`: the base weight
    in tiles (ops.tile_base), read instead of base_weight when given."""
    from .ops import row_blocks
    T, K = x2.shape
    N = scales_stacked.shape[-1]
    S = qweight_stacked.shape[0]
    G = scales_stacked[0].numel() // N
    group_size = -1 if G == 1 else K // G
    # the kernel addresses an operand with 31-bit byte offsets: very long batches go in pieces
    max_rows = ((1 << 31) - 1) // (2 * K)
    if T > max_rows:
        step = max(256, max_rows // 256 * 256)
        for r in range(0, T, step):
            multi_delta_linear_prefill(x2[r:r + step], base_weight, qweight_stacked, scales_stacked, meta_stacked,
                                       indices[r:r + step].contiguous(), bits=bits, out=out[r:r + step],
                                       accumulate=accumulate, base_tiled=base_tiled)
        return out
    lib = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    if blocks is None:
        blocks = row_blocks(indices, S)
    fn, wptr = lib.dz_multi_delta_gemm, base_weight.data_ptr() if base_weight is not None else None
    if base_tiled is not None:
        fn, wptr = lib.dz_multi_delta_gemm_tiled, base_tiled.data_ptr()
    rc = fn(x2.data_ptr(), wptr,
                                 qweight_stacked.data_ptr(), meta_stacked.data_ptr(), scales_stacked.data_ptr(),
                                 S, bits, group_size, blocks.tiles.data_ptr(), blocks.max_tiles, blocks.perm.data_ptr(),
                                 out.data_ptr(), T, K, N, 1 if accumulate else 0, out.stride(0), stream)
    _lib.check(rc, "dz_multi_delta_gemm")
    return out
