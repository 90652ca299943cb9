"""The operator names of serving/vllm/delta/deltazip.py (the reference's non-fused delta ops),
so that `from vllm.delta.deltazip import add_delta, apply_delta, ...` can become
`from deltazip_amd.deltazip import ...`.

  add_delta                  deltazip.py:14-37     y += x @ dequant(W[indices])^T
  add_delta_slice            deltazip.py:40-77     the same into a column slice of y
  apply_delta                deltazip.py:78-100    in-place form over flattened leading dimensions
  apply_delta_packed_nslice  deltazip.py:103-153   several sublayers packed side by side

All of them take the 2:4 positions of the native layout as `meta` / `meta_stacked` (the reference's
add_delta has the same `meta` parameter, deltazip.py:22).  The fused base + delta form of
serving/vllm/delta/deltazip_marlin.py is `deltazip_amd.ops.apply_delta`.
"""
from .ops import add_delta, add_delta_slice, apply_delta_packed_nslice
from .ops import apply_delta_into as apply_delta

__all__ = ["add_delta", "add_delta_slice", "apply_delta", "apply_delta_packed_nslice"]
