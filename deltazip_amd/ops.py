"""Operator layer: the reference's delta ops, backed by the HIP kernels in libdz_amd.so.

Mirrors
  serving/vllm/delta/deltazip_marlin.py:10-19   apply_delta(x, qweight_stacked, scales_stacked,
                                                meta_stacked, indices, base_weight) -> y
  serving/vllm/delta/deltazip.py:14-77          add_delta / add_delta_slice (in-place y +=)
of eth-easl/deltazip.  Tensor names and roles are the reference's; the bit layout inside
`qweight`/`meta` is this project's native gfx950 layout (see csrc/dz_layout.h), produced from the
reference's GPTQ-style tensors by `repack_gptq_to_native`.

PyTorch is used for device memory and streams only; all arithmetic happens in the library.
"""
from __future__ import annotations

import ctypes as C
import math
from typing import Dict, Optional, Sequence, Tuple

import torch

from . import _lib

MAX_TOKENS_FUSED = 128

# ---------------------------------------------------------------------------------------------
# layout helpers
# ---------------------------------------------------------------------------------------------


def native_sizes(K: int, N: int, bits: int, group_size: int = -1) -> Tuple[int, int, int]:
    """(codes_bytes, meta_bytes, scales_bytes) of one delta in the native layout."""
    cb, mb, sb = C.c_size_t(), C.c_size_t(), C.c_size_t()
    _lib.check(_lib.lib().dz_native_sizes(K, N, bits, group_size, C.byref(cb), C.byref(mb), C.byref(sb)),
               "dz_native_sizes")
    return cb.value, mb.value, sb.value


def stacked_shapes(K: int, N: int, bits: int, group_size: int = -1):
    """Shapes (without the leading slot dimension) of the three stacked tensors, following
    layers_marlin.py:311-333: qweight [K/(pf*4), 2N] int32, meta [N, K/16] int16, scales [G, N]."""
    native_sizes(K, N, bits, group_size)  # validates
    pf = 32 // bits
    g = 1 if group_size in (-1, K) else K // group_size
    return (K // (pf * 4), 2 * N), (N, K // 16), (g, N)


def repack_gptq_to_native(qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor,
                          g_idx: Optional[torch.Tensor], bits: int):
    """GPTQ-style tensors of one delta (as QuantLinear.pack writes them,
    deltazip/nn_modules/qlinear_cuda.py:144-244) -> (qweight, meta, scales) CPU tensors in the
    native layout, shaped as `stacked_shapes` says.  Host work, done once per delta; stands where
    the reference calls its checkpoint converter (deltazip/utils/converter.py:13-101)."""
    if bits not in (2, 4):
        raise NotImplementedError("Only 2 and 4 bits are supported.")
    qweight = qweight.detach().cpu().contiguous()
    qzeros = qzeros.detach().cpu().contiguous()
    scales = scales.detach().cpu().contiguous()
    if qweight.dtype != torch.int32 or qzeros.dtype != torch.int32 or scales.dtype != torch.float16:
        raise ValueError("qweight/qzeros must be int32 and scales float16")
    pf = 32 // bits
    K, N = qweight.shape[0] * pf, qweight.shape[1]
    G = scales.shape[0]
    if scales.shape != (G, N) or qzeros.shape != (G, N // pf) or K % G:
        raise ValueError("inconsistent qzeros/scales shapes")
    group_size = -1 if G == 1 else K // G
    gi = None
    if g_idx is not None:
        gi = g_idx.detach().cpu().to(torch.int32).contiguous()
        if gi.numel() != K:
            raise ValueError("g_idx must have K entries")
    (qs, ms, ss) = stacked_shapes(K, N, bits, group_size)
    out_q = torch.empty(qs, dtype=torch.int32)
    out_m = torch.empty(ms, dtype=torch.int16)
    out_s = torch.empty(ss, dtype=torch.float16)
    rc = _lib.lib().dz_repack_2of4(qweight.data_ptr(), qzeros.data_ptr(), scales.data_ptr(),
                                   gi.data_ptr() if gi is not None else None, K, N, bits, group_size,
                                   out_q.data_ptr(), out_m.data_ptr(), out_s.data_ptr())
    _lib.check(rc, "dz_repack_2of4")
    return out_q, out_m, out_s


def unrepack_native_to_gptq(qweight: torch.Tensor, meta: torch.Tensor, scales: torch.Tensor, K: int, N: int,
                            bits: int):
    """One delta in the native layout -> (qweight, qzeros, scales, g_idx) CPU tensors in the
    reference's GPTQ-style format (QuantLinear.pack, deltazip/nn_modules/qlinear_cuda.py:144-244):
    qweight int32 [K*bits/32, N], qzeros int32 [G, N*bits/32], scales fp16 [G, N], g_idx int32 [K].
    The inverse of `repack_gptq_to_native`; host work."""
    if bits not in (2, 4):
        raise NotImplementedError("Only 2 and 4 bits are supported.")
    qweight = qweight.detach().cpu().contiguous()
    meta = meta.detach().cpu().contiguous()
    scales = scales.detach().cpu().contiguous()
    if scales.dtype != torch.float16 or scales.numel() % N:
        raise ValueError("scales must be float16 [G, N]")
    G = scales.numel() // N
    group_size = -1 if G == 1 else K // G
    cb, mb, sb = native_sizes(K, N, bits, group_size)
    if (qweight.numel() * qweight.element_size() != cb or meta.numel() * meta.element_size() != mb
            or scales.numel() * 2 != sb):
        raise ValueError("tensors do not match the native layout for these sizes")
    pf = 32 // bits
    out_q = torch.empty((K // pf, N), dtype=torch.int32)
    out_z = torch.empty((G, N // pf), dtype=torch.int32)
    out_s = torch.empty((G, N), dtype=torch.float16)
    out_g = torch.empty(K, dtype=torch.int32)
    rc = _lib.lib().dz_unrepack_2of4(qweight.data_ptr(), meta.data_ptr(), scales.data_ptr(), K, N, bits, group_size,
                                     out_q.data_ptr(), out_z.data_ptr(), out_s.data_ptr(), out_g.data_ptr())
    _lib.check(rc, "dz_unrepack_2of4")
    return out_q, out_z, out_s, out_g


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _need_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise ValueError("tensors must live on the GPU (there is no CPU implementation)")


def dequant(qweight: torch.Tensor, meta: torch.Tensor, scales: torch.Tensor, K: int, N: int,
            bits: int) -> torch.Tensor:
    """One native delta -> fp16 [N, K] on the GPU; bit-exact with QuantLinear.unpack
    (deltazip/nn_modules/qlinear_cuda.py:246-329)."""
    _need_cuda(qweight, meta, scales)
    G = scales.numel() // N
    out = torch.empty((N, K), dtype=torch.float16, device=qweight.device)
    rc = _lib.lib().dz_dequant(qweight.data_ptr(), meta.data_ptr(), scales.data_ptr(), K, N, bits,
                               -1 if G == 1 else K // G, out.data_ptr(), _stream())
    _lib.check(rc, "dz_dequant")
    return out


def merge(base_weight: torch.Tensor, qweight, meta, scales, bits: int) -> torch.Tensor:
    """W_base + dequant(delta) as fp16 [N, K] (deltazip/utils/generate.py:9-20 at fp16 storage)."""
    _need_cuda(base_weight, qweight, meta, scales)
    N, K = base_weight.shape
    G = scales.numel() // N
    out = torch.empty_like(base_weight)
    rc = _lib.lib().dz_merge(base_weight.data_ptr(), qweight.data_ptr(), meta.data_ptr(),
                             scales.data_ptr(), K, N, bits, -1 if G == 1 else K // G, out.data_ptr(),
                             _stream())
    _lib.check(rc, "dz_merge")
    return out


def segment(indices: torch.Tensor, num_slots: int):
    """(perm [T] int32, seg_off [S+2] int32): tokens grouped by delta id, id -1 first."""
    _need_cuda(indices)
    if indices.dtype != torch.int64:
        raise ValueError("indices must be int64")
    T = indices.numel()
    perm = torch.empty(T, dtype=torch.int32, device=indices.device)
    off = torch.empty(num_slots + 2, dtype=torch.int32, device=indices.device)
    _lib.check(_lib.lib().dz_segment(indices.data_ptr(), T, num_slots, perm.data_ptr(), off.data_ptr(),
                                     _stream()), "dz_segment")
    return perm, off


class RowBlocks:
    """A batch of more than 128 tokens ordered by delta id and cut into row blocks of one delta each
    (what dz_segment and dz_build_tiles write): depends on the indices only, so it can be made once
    per batch and passed to every layer call of the step (`order=`)."""
    __slots__ = ("perm", "tiles", "max_tiles", "T", "S")

    def __init__(self, perm, tiles, max_tiles, T, S):
        self.perm, self.tiles, self.max_tiles, self.T, self.S = perm, tiles, max_tiles, T, S


def row_blocks(indices: torch.Tensor, num_slots: int) -> RowBlocks:
    """Row blocks of a prefill-sized batch, as the reference converts its mapping once per batch
    (serving/vllm/delta/models.py:421-435).  Two small launches, nothing read back to the host."""
    indices = indices.reshape(-1)
    if not indices.is_contiguous():
        raise ValueError("indices must be contiguous")
    T = indices.numel()
    perm, seg_off = segment(indices, num_slots)
    max_tiles = (T + 255) // 256 + min(num_slots + 1, T)
    tiles = torch.empty((max_tiles, 4), dtype=torch.int32, device=indices.device)
    _lib.check(_lib.lib().dz_build_tiles(seg_off.data_ptr(), num_slots, tiles.data_ptr(), max_tiles, _stream()),
               "dz_build_tiles")
    return RowBlocks(perm, tiles, max_tiles, T, num_slots)


def apply_delta_embed(x: torch.Tensor, delta_weights: torch.Tensor, indices: torch.Tensor,
                      base_weight: torch.Tensor) -> torch.Tensor:
    """Embedding lookup where every token reads the table of its own delta
    (serving/vllm/delta/deltazip_marlin.py:56-86): out[t] = delta_weights[indices[t]][x[t]], or
    base_weight[x[t]] for indices[t] == -1.  x [T] int64 token ids, delta_weights [S, V, H] fp16,
    base_weight [V, H] fp16; returns [T, H] fp16."""
    _need_cuda(x, delta_weights, indices, base_weight)
    if x.dtype != torch.int64 or indices.dtype != torch.int64:
        raise ValueError("token ids and indices must be int64")
    if delta_weights.dtype != torch.float16 or base_weight.dtype != torch.float16:
        raise ValueError("embedding tables must be float16")
    S, V, H = delta_weights.shape
    if tuple(base_weight.shape) != (V, H) or not delta_weights.is_contiguous() or not base_weight.is_contiguous():
        raise ValueError("base_weight must be [V, H] like each delta table, all contiguous")
    T = x.numel()
    if indices.numel() != T:
        raise ValueError("one index per token is required")
    out = torch.empty((T, H), dtype=torch.float16, device=x.device)
    rc = _lib.lib().dz_embedding_select(x.reshape(-1).contiguous().data_ptr(), indices.contiguous().data_ptr(),
                                        base_weight.data_ptr(), delta_weights.data_ptr(), V * H, S,
                                        out.data_ptr(), T, V, H, H, _stream())
    _lib.check(rc, "dz_embedding_select")
    return out.view(*x.shape, H)


def apply_delta_uncompressed(x: torch.Tensor, delta_weights: torch.Tensor, indices: torch.Tensor,
                             base_embedding: torch.Tensor) -> torch.Tensor:
    """Per-row dense product against the row's own full weight
    (serving/vllm/delta/deltazip_marlin.py:21-53, the lm_head of LogitsProcessorWithDelta):
    out[t] = x[t] @ delta_weights[indices[t]]^T, or x[t] @ base_embedding^T for indices[t] == -1.
    Where the reference loops over torch.unique(indices) on the host, the rows are grouped by id
    and cut into row blocks on the device (dz_segment, dz_build_tiles) and one launch multiplies
    every block by its own table (dz_gemm_f16_select), reading and writing the rows in place
    through the token order: three launches, nothing gathered, scattered or read back to the
    host, so the call can be captured in a HIP graph."""
    _need_cuda(x, delta_weights, indices, base_embedding)
    if x.dtype != torch.float16 or delta_weights.dtype != torch.float16 or base_embedding.dtype != torch.float16:
        raise ValueError("x and the weights must be float16")
    S, N, K = delta_weights.shape
    T = x.shape[0]
    if x.dim() != 2 or x.shape[1] != K or tuple(base_embedding.shape) != (N, K) or indices.numel() != T:
        raise ValueError("shapes: x [T, K], delta_weights [S, N, K], base_embedding [N, K], indices [T]")
    if not (delta_weights.is_contiguous() and base_embedding.is_contiguous() and x.is_contiguous()):
        raise ValueError("x and the weights must be contiguous")
    blocks = row_blocks(indices, S)
    out = torch.empty((T, N), dtype=torch.float16, device=x.device)
    _lib.check(_lib.lib().dz_gemm_f16_select(x.data_ptr(), base_embedding.data_ptr(), delta_weights.data_ptr(), N * K,
                                             blocks.tiles.data_ptr(), blocks.max_tiles, blocks.perm.data_ptr(),
                                             out.data_ptr(), T, K, N, 0, N, _stream()), "dz_gemm_f16_select")
    return out


_minus_one_ids: Dict[int, torch.Tensor] = {}


def _minus_ones(device) -> torch.Tensor:
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if idx not in _minus_one_ids:
        _minus_one_ids[idx] = torch.full((MAX_TOKENS_FUSED,), -1, dtype=torch.int64, device=device)
    return _minus_one_ids[idx]


def compress_delta(delta: torch.Tensor, bits: int, group_size: int = -1):
    """fp32 delta [N, K] on the GPU -> (qweight, meta, scales) of one slot in the native layout:
    symmetric scales from the un-pruned values, 2:4 magnitude pruning, round-to-nearest codes
    (deltazip/core/quant.py:9-18, 48-130; core/sparsegpt.py:64-66, 123-135 with an identity
    Hessian).  The same bytes as compressing and packing the reference's way and converting with
    `repack_gptq_to_native`."""
    _need_cuda(delta)
    if bits not in (2, 4):
        raise NotImplementedError("Only 2 and 4 bits are supported.")
    if delta.dtype != torch.float32 or delta.dim() != 2 or not delta.is_contiguous():
        raise ValueError("delta must be a contiguous float32 [N, K] tensor")
    N, K = delta.shape
    qs, ms, ss = stacked_shapes(K, N, bits, group_size)
    q = torch.empty(qs, dtype=torch.int32, device=delta.device)
    m = torch.empty(ms, dtype=torch.int16, device=delta.device)
    s = torch.empty(ss, dtype=torch.float16, device=delta.device)
    ws = torch.empty(ss, dtype=torch.float32, device=delta.device)
    rc = _lib.lib().dz_compress_2of4(delta.data_ptr(), K, N, bits, group_size, q.data_ptr(), m.data_ptr(),
                                     s.data_ptr(), ws.data_ptr(), _stream())
    _lib.check(rc, "dz_compress_2of4")
    return q, m, s


def quant_scales(delta: torch.Tensor, bits: int, group_size: int = -1, mse: bool = False, norm: float = 2.4,
                 grid: int = 100, maxshrink: float = 0.8):
    """Symmetric scales of the reference's Quantizer.find_params (deltazip/core/quant.py:48-130,
    perchannel, sym) for an fp32 delta [N, K] on the GPU: (scale32 [G, N] fp32, scale16 [G, N] fp16).
    mse=True runs the reference's search over the clipping range (quant.py:85-101) with its
    `norm`, `grid` and `maxshrink`."""
    _need_cuda(delta)
    if delta.dtype != torch.float32 or delta.dim() != 2 or not delta.is_contiguous():
        raise ValueError("delta must be a contiguous float32 [N, K] tensor")
    N, K = delta.shape
    _, _, ss = stacked_shapes(K, N, bits, group_size)
    s32 = torch.empty(ss, dtype=torch.float32, device=delta.device)
    s16 = torch.empty(ss, dtype=torch.float16, device=delta.device)
    if mse:
        rc = _lib.lib().dz_quant_scales_mse(delta.data_ptr(), K, N, bits, group_size, float(norm), int(grid),
                                            float(maxshrink), s32.data_ptr(), s16.data_ptr(), _stream())
        _lib.check(rc, "dz_quant_scales_mse")
    else:
        rc = _lib.lib().dz_quant_scales(delta.data_ptr(), K, N, bits, group_size, s32.data_ptr(), s16.data_ptr(), _stream())
        _lib.check(rc, "dz_quant_scales")
    return s32, s16


def pack_2of4(w: torch.Tensor, scale32: torch.Tensor, bits: int, group_size: int = -1):
    """(qweight, meta) of one slot in the native layout from fp32 values [N, K] that are 2:4 sparse and
    on the grid of `scale32` [G, N] (what `obs_sweep` leaves behind)."""
    _need_cuda(w, scale32)
    if w.dtype != torch.float32 or w.dim() != 2 or not w.is_contiguous():
        raise ValueError("w must be a contiguous float32 [N, K] tensor")
    N, K = w.shape
    qs, ms, ss = stacked_shapes(K, N, bits, group_size)
    if scale32.dtype != torch.float32 or tuple(scale32.shape) != tuple(ss) or not scale32.is_contiguous():
        raise ValueError("scale32 must be a contiguous float32 [G, N] tensor")
    q = torch.empty(qs, dtype=torch.int32, device=w.device)
    m = torch.empty(ms, dtype=torch.int16, device=w.device)
    rc = _lib.lib().dz_pack_2of4(w.data_ptr(), scale32.data_ptr(), K, N, bits, group_size, q.data_ptr(), m.data_ptr(),
                                 _stream())
    _lib.check(rc, "dz_pack_2of4")
    return q, m


def hessian_add(H: torch.Tensor, x: torch.Tensor, nsamples: int, batch: int) -> int:
    """H <- H * n/(n+b) + (sqrt(2/(n+b)) x)^T (sqrt(2/(n+b)) x) in place for x [T, K] (fp16 or fp32),
    as SparseGPT.add_batch does for a linear layer (deltazip/core/sparsegpt.py:27-40); returns n + b."""
    _need_cuda(H, x)
    K = H.shape[0]
    if H.dtype != torch.float32 or tuple(H.shape) != (K, K) or not H.is_contiguous():
        raise ValueError("H must be a contiguous float32 [K, K] tensor")
    if x.dim() != 2 or x.shape[1] != K or x.dtype not in (torch.float16, torch.float32) or not x.is_contiguous():
        raise ValueError("x must be a contiguous [T, K] float16 or float32 tensor")
    n = nsamples + batch
    rc = _lib.lib().dz_hessian_add(H.data_ptr(), x.data_ptr(), int(x.dtype == torch.float16), x.shape[0], K,
                                   float(nsamples / n), math.sqrt(2.0 / n), _stream())
    _lib.check(rc, "dz_hessian_add")
    return n


def obs_sweep(W: torch.Tensor, hinv_upper: torch.Tensor, scale: Optional[torch.Tensor], bits: int = 4,
              prunen: int = 2, prunem: int = 4) -> torch.Tensor:
    """The column sweep of SparseGPT.fasterprune (deltazip/core/sparsegpt.py:92-146) over W [N, K] fp32
    in place: n:m pruning by w^2 / diag(hinv)^2, rounding to the grid of `scale` [N] (None: no
    rounding), error compensation along the rows of `hinv_upper`.  Returns the per-row losses [N]."""
    _need_cuda(W, hinv_upper, scale)
    N, K = W.shape
    if W.dtype != torch.float32 or not W.is_contiguous():
        raise ValueError("W must be a contiguous float32 [N, K] tensor")
    if hinv_upper.dtype != torch.float32 or tuple(hinv_upper.shape) != (K, K) or not hinv_upper.is_contiguous():
        raise ValueError("hinv_upper must be a contiguous float32 [K, K] tensor")
    if scale is not None and (scale.dtype != torch.float32 or scale.numel() != N or not scale.is_contiguous()):
        raise ValueError("scale must be a contiguous float32 tensor with one entry per row")
    err = torch.empty((N, 128), dtype=torch.float32, device=W.device)
    loss = torch.zeros(N, dtype=torch.float32, device=W.device)
    rc = _lib.lib().dz_obs_sweep(W.data_ptr(), hinv_upper.data_ptr(), scale.data_ptr() if scale is not None else None,
                                 N, K, bits, prunen, prunem, err.data_ptr(), loss.data_ptr(), _stream())
    _lib.check(rc, "dz_obs_sweep")
    return loss


def token_order(indices: torch.Tensor, num_slots: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Order in which the fused kernel takes the tokens of a batch of up to 128 tokens (int32 [T]):
    depends on the indices only, so it can be computed once per batch and passed to every layer
    call of the step (`order=`), as the reference converts its mapping once per batch
    (serving/vllm/delta/models.py:421-435)."""
    _need_cuda(indices, out)
    T = indices.numel()
    if indices.dtype != torch.int64 or not indices.is_contiguous():
        raise ValueError("indices must be a contiguous int64 tensor")
    if out is None:
        out = torch.empty(T, dtype=torch.int32, device=indices.device)
    elif out.dtype != torch.int32 or out.numel() < T or not out.is_contiguous():
        raise ValueError("out must be a contiguous int32 tensor with at least T entries")
    _lib.check(_lib.lib().dz_token_order(indices.data_ptr(), T, num_slots, out.data_ptr(), _stream()), "dz_token_order")
    return out[:T]


def map_ids(token_ids: torch.Tensor, prompt_ids: Optional[torch.Tensor], slot_ids: torch.Tensor,
            max_deltas: int, vocab_size: int, extra_vocab_size: int, base_indices: torch.Tensor,
            sampler_indices: Optional[torch.Tensor] = None,
            sampler_indices_padded: Optional[torch.Tensor] = None,
            embeddings_indices: Optional[torch.Tensor] = None,
            n_missing: Optional[torch.Tensor] = None) -> None:
    """Delta ids -> slot indices on the device, written into the given int64 tensors (the index
    tensors of convert_mapping, serving/vllm/delta/models.py:69-145).  token_ids [T], prompt_ids [P]
    or None, slot_ids [S]: int64 on the GPU; the outputs are the manager's persistent buffers
    (at least T resp. P long; embeddings_indices [2, >= T])."""
    _need_cuda(token_ids, prompt_ids, slot_ids, base_indices, sampler_indices, sampler_indices_padded,
               embeddings_indices, n_missing)
    for t in (token_ids, prompt_ids, slot_ids, base_indices, sampler_indices, sampler_indices_padded,
              embeddings_indices):
        if t is not None and t.dtype != torch.int64:
            raise ValueError("id and index tensors must be int64")
    T = token_ids.numel()
    P = 0 if prompt_ids is None else prompt_ids.numel()
    if base_indices.numel() < T or (P and (sampler_indices is None or sampler_indices.numel() < P)):
        raise ValueError("index buffers are shorter than the batch")
    if sampler_indices_padded is not None and sampler_indices_padded.numel() < P:
        raise ValueError("index buffers are shorter than the batch")
    ld = 0
    if embeddings_indices is not None:
        if embeddings_indices.dim() != 2 or embeddings_indices.shape[0] != 2 or embeddings_indices.stride(1) != 1:
            raise ValueError("embeddings_indices must be [2, n] with contiguous rows")
        ld = embeddings_indices.stride(0)
    ptr = lambda t: None if t is None else t.data_ptr()
    rc = _lib.lib().dz_map_ids(token_ids.data_ptr(), T, ptr(prompt_ids), P, slot_ids.data_ptr(),
                               slot_ids.numel(), max_deltas, vocab_size, extra_vocab_size,
                               base_indices.data_ptr(), ptr(sampler_indices), ptr(sampler_indices_padded),
                               ptr(embeddings_indices), ld, ptr(n_missing), _stream())
    _lib.check(rc, "dz_map_ids")


# ---------------------------------------------------------------------------------------------
# workspace: zero-filled once per device, reused by every call on that device
# ---------------------------------------------------------------------------------------------
# one per (device, stream): calls that share a workspace must be ordered on one stream
_workspaces: Dict[Tuple[int, int], torch.Tensor] = {}


WS_HEADER_BYTES = 256          # the status word sits in front of the token order and the partial sums

STATUS_BAD_ID = 1              # a delta id outside [-1, S) was met and treated as -1
STATUS_SUM_MISSING = 2         # a partial sum of a K-slice did not arrive: that call's output is invalid


def _workspace(device: torch.device, T: int, K: int, N: int) -> torch.Tensor:
    need = _lib.lib().dz_workspace_bytes(T, K, N)
    idx = device.index if device.index is not None else torch.cuda.current_device()
    key = (idx, _stream())
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        new = torch.zeros(max(need, 1 << 20), dtype=torch.uint8, device=device)
        if ws is not None:
            # the status word of the buffer that is left behind is carried over (same stream: after
            # the calls that may still set it)
            new[:WS_HEADER_BYTES].copy_(ws[:WS_HEADER_BYTES])
        _workspaces[key] = ws = new
        _status_polls.pop(key, None)
    return ws


def workspace_status(device=None) -> int:
    """Status words of the device's workspaces, OR-ed (bit 0: a delta id outside [-1, S) was seen
    and treated as -1; bit 1: a partial sum did not arrive).  Synchronises; meant for debugging
    and tests -- the serving path uses `poll_status`."""
    idx = torch.cuda.current_device() if device is None else torch.device(device).index
    status = 0
    for (i, _), ws in _workspaces.items():
        if i == idx:
            status |= int(ws[:4].view(torch.int32).item())
    return status


class DeltaKernelError(RuntimeError):
    """A launch of the fused kernel reported that its output is invalid."""


_warned_bad_id = False


def raise_for_status(word: int, where: str = "multi-delta linear") -> None:
    """What a status word means to the caller.  Bit 1 -> DeltaKernelError (a RuntimeError, as every
    failure of the reference's ops is a Python exception); bit 0 -> one warning per process."""
    global _warned_bad_id
    if word & STATUS_SUM_MISSING:
        raise DeltaKernelError(
            f"{where}: a partial sum of a K dimension split over workgroups did not arrive within the kernel's "
            "bounded wait; the outputs of the calls since the last check are invalid (status bit 1). The "
            "workspace has been cleared; repeat the step.")
    if word & STATUS_BAD_ID and not _warned_bad_id:
        _warned_bad_id = True
        import warnings
        warnings.warn(f"{where}: a delta id outside [-1, S) was met and served as -1 (base weight only; status bit 0)",
                      RuntimeWarning, stacklevel=3)


# (device, stream) -> (pinned int32[1], event of the copy that fills it)
_status_polls: Dict[Tuple[int, int], Tuple[torch.Tensor, "torch.cuda.Event"]] = {}


def _clear_workspace(ws: torch.Tensor, word: int) -> None:
    """After a reported failure: empty the partial-sum slots (late slices may have left values in
    them that later calls would take for ready) and drop the reported bits."""
    if word & STATUS_SUM_MISSING:
        ws[WS_HEADER_BYTES:].zero_()
    ws[:4].zero_()


def poll_status(device=None, wait: bool = False) -> None:
    """The serving path's look at the status words, without a synchronisation of its own: every call
    evaluates the copy the previous call started (if it has completed, or after waiting for it when
    `wait` is set) and starts the next one, a 4-byte device-to-host copy into pinned memory on the
    workspace's stream.  Raises DeltaKernelError / warns as `raise_for_status` says; a reported
    failure also clears the workspace.  With `wait` the current state is read as well (this
    synchronises with the workspace's stream)."""
    if not _workspaces:
        return                                        # no fused call has run yet (or no GPU at all)
    idx = None if device is None else torch.device(device).index
    if idx is None:
        idx = torch.cuda.current_device()
    found = 0
    for key, ws in list(_workspaces.items()):
        if key[0] != idx:
            continue
        stream = torch.cuda.ExternalStream(key[1], device=ws.device) if key[1] else torch.cuda.default_stream(ws.device)
        pending = _status_polls.pop(key, None)
        host = pending[0] if pending is not None else torch.zeros(1, dtype=torch.int32, pin_memory=True)
        word = 0
        if pending is not None:
            if wait:
                pending[1].synchronize()
            if pending[1].query():
                word = int(host[0])
            else:
                _status_polls[key] = pending          # not in yet: looked at by the next call
                continue
        with torch.cuda.stream(stream):
            if wait:
                # the state as of now, too
                host.copy_(ws[:4].view(torch.int32), non_blocking=True)
                stream.synchronize()
                word |= int(host[0])
            if word:
                _clear_workspace(ws, word)            # before the next copy is started
            if not wait:
                ev = torch.cuda.Event()
                host.copy_(ws[:4].view(torch.int32), non_blocking=True)
                ev.record()
                _status_polls[key] = (host, ev)
        found |= word
    if found:
        raise_for_status(found)


# ---------------------------------------------------------------------------------------------
# the ops
# ---------------------------------------------------------------------------------------------


def _infer(qweight_stacked, scales_stacked, N: int):
    """(K, bits, group_size, S) from the stacked tensors' shapes."""
    S = qweight_stacked.shape[0]
    words = qweight_stacked[0].numel()
    G = scales_stacked[0].numel() // N
    return S, words, G


def tile_base(weight: torch.Tensor) -> torch.Tensor:
    """The base weight [N, K] in the tiled form the fused kernel streams fastest (`dz_tile_base`):
    a tensor of the same shape and dtype whose bytes are the tiles.  A layer converts its base
    weight once and hands it to `multi_delta_linear` / `apply_delta_batch` (`base_tiled=`); calls of
    every size read the tiles when they are given."""
    _need_cuda(weight)
    if weight.dtype != torch.float16 or weight.dim() != 2 or not weight.is_contiguous():
        raise ValueError("weight must be a contiguous float16 [N, K] tensor")
    N, K = weight.shape
    out = torch.empty_like(weight)
    _lib.check(_lib.lib().dz_tile_base(weight.data_ptr(), K, N, out.data_ptr(), _stream()), "dz_tile_base")
    return out


def untile_base(tiled: torch.Tensor) -> torch.Tensor:
    """Inverse of `tile_base`: the row-major [N, K] weight from its tiles (plain tensor ops; not on
    any hot path).  Tile (np, kb) holds fragments (s, j, h); position 16*g + i of a fragment holds
    W[32*np + 16*s + i][256*kb + 64*j + 16*g + 8*h + e], e = 0..7."""
    if tiled.dtype != torch.float16 or tiled.dim() != 2 or not tiled.is_contiguous():
        raise ValueError("tiled must be a contiguous float16 [N, K] tensor")
    N, K = tiled.shape
    if N % 32 or K % 256:
        raise ValueError("N must be a multiple of 32 and K of 256")
    t = tiled.view(N // 32, K // 256, 2, 4, 2, 4, 16, 8)          # np kb s j h g i e
    return t.permute(0, 2, 6, 1, 3, 5, 4, 7).reshape(N, K).contiguous()   # np s i | kb j g h e


def _check_tiled(base_tiled, base_weight, N: int, K: int, device) -> None:
    if tuple(base_tiled.shape) != (N, K) or base_tiled.dtype != torch.float16 \
            or not base_tiled.is_contiguous() or base_tiled.device != device \
            or (base_weight is not None and base_weight.numel() and base_tiled.shape != base_weight.shape):
        raise ValueError("base_tiled must be tile_base(base_weight): float16 [N, K], contiguous, on x's device")


def takes_fused_chunks(T: int, S: int) -> bool:
    """Whether a batch above the fused kernel's 128 tokens goes through it in chunks of 128 rather than
    through the matrix-core kernel.  That kernel works on row blocks of up to 256 tokens of one delta
    and needs some 256 x (N / 256) of them to fill the GPU: a few hundred tokens, the more so when
    they are spread over many deltas, leave most of it idle (5120 x 5120, 2-bit, tiled base weight;
    chunks against the matrix-core kernel with 1 / 16 / 64 deltas in the batch: 384 tokens 0.15 / 0.16
    / 0.21 ms against 0.19 / 0.24 / 0.57 ms; 512 tokens 0.20 / 0.21 / 0.26 against 0.19 / 0.24 / 0.57;
    768 tokens 0.29 / 0.30 / 0.34 against 0.20 / 0.24 / 0.58).  The number of distinct deltas is
    known on the device only, so the number of slots stands in for it."""
    return T <= 3 * MAX_TOKENS_FUSED or (T <= 4 * MAX_TOKENS_FUSED and S >= 16)


def multi_delta_linear(x: torch.Tensor, base_weight: Optional[torch.Tensor], qweight_stacked,
                       scales_stacked, meta_stacked, indices: torch.Tensor, *, bits: int,
                       out: Optional[torch.Tensor] = None, accumulate: bool = False,
                       order: Optional[torch.Tensor] = None,
                       base_tiled: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x @ W_base^T + x @ dequant(delta[indices])^T.  `out` may be a column slice of a wider
    tensor (last-dim stride 1); with accumulate=True the result is added to it.  `order`: what the
    caller already has for this batch -- the result of `token_order(indices, S)` (up to 128
    tokens) or of `row_blocks(indices, S)` (more).
    `base_tiled`: `tile_base(base_weight)`, read instead of the row-major weight (the results are
    the same bit for bit); base_weight may then be None -- a layer that keeps only the tiled copy."""
    _need_cuda(x, base_weight, qweight_stacked, scales_stacked, meta_stacked, indices)
    if x.dtype != torch.float16:
        raise ValueError("x must be float16")
    if indices.dtype != torch.int64:
        raise ValueError("indices must be int64")
    if bits not in (2, 4):
        raise NotImplementedError("Only 2 and 4 bits are supported.")
    K = x.shape[-1]
    x2 = x.reshape(-1, K)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    T = x2.shape[0]
    indices = indices.reshape(-1)
    if indices.numel() != T or not indices.is_contiguous():
        raise ValueError("indices must be a contiguous vector with one entry per token")
    S = qweight_stacked.shape[0]
    N = scales_stacked.shape[-1]
    if base_tiled is not None:
        _check_tiled(base_tiled, base_weight, N, K, x.device)
        if base_weight is not None and base_weight.numel() == 0:
            base_weight = None
    if base_weight is not None:
        if base_weight.dtype != torch.float16 or tuple(base_weight.shape) != (N, K) or not base_weight.is_contiguous():
            raise ValueError("base_weight must be a contiguous float16 [N, K] tensor")
    G = scales_stacked[0].numel() // N
    group_size = -1 if G == 1 else K // G
    cb, mb, sb = native_sizes(K, N, bits, group_size)
    if (qweight_stacked[0].numel() * qweight_stacked.element_size() != cb
            or meta_stacked[0].numel() * meta_stacked.element_size() != mb
            or not qweight_stacked.is_contiguous() or not meta_stacked.is_contiguous()
            or not scales_stacked.is_contiguous() or scales_stacked.dtype != torch.float16):
        raise ValueError("stacked delta tensors do not match the native layout for these sizes")
    if out is None:
        if accumulate:
            raise ValueError("accumulate needs an output tensor")
        out = torch.empty((T, N), dtype=torch.float16, device=x.device)
    else:
        if out.dtype != torch.float16 or out.dim() != 2 or out.shape != (T, N) or out.stride(1) != 1:
            raise ValueError("out must be float16 [T, N] with unit column stride")
    ldy = out.stride(0)
    if T > MAX_TOKENS_FUSED:
        if takes_fused_chunks(T, S):
            for r in range(0, T, MAX_TOKENS_FUSED):
                multi_delta_linear(x2[r:r + MAX_TOKENS_FUSED], base_weight, qweight_stacked, scales_stacked,
                                   meta_stacked, indices[r:r + MAX_TOKENS_FUSED], bits=bits,
                                   out=out[r:r + MAX_TOKENS_FUSED], accumulate=accumulate, base_tiled=base_tiled)
            return out
        from .prefill import multi_delta_linear_prefill
        blocks = order if isinstance(order, RowBlocks) else None
        if blocks is not None and (blocks.T != T or blocks.S != S):
            raise ValueError("row blocks were made for another batch size or number of slots")
        return multi_delta_linear_prefill(x2, base_weight, qweight_stacked, scales_stacked, meta_stacked,
                                          indices, bits=bits, out=out, accumulate=accumulate, blocks=blocks,
                                          base_tiled=base_tiled)
    ws = _workspace(x.device, T, K, N)
    optr = _order_ptr(order, T, x.device)
    if base_tiled is not None:
        one = lambda p: (C.c_void_p * 1)(p)
        rc = _lib.lib().dz_multi_delta_linear_batch_tiled(
            1, one(x2.data_ptr()), one(base_tiled.data_ptr()), one(qweight_stacked.data_ptr()),
            one(meta_stacked.data_ptr()), one(scales_stacked.data_ptr()), indices.data_ptr(), one(out.data_ptr()),
            (C.c_int * 1)(N), (C.c_int * 1)(ldy), T, K, S, bits, group_size, 1 if accumulate else 0, optr,
            ws.data_ptr(), ws.numel(), _stream())
        _lib.check(rc, "dz_multi_delta_linear_batch_tiled")
        return out
    if optr is None:
        rc = _lib.lib().dz_multi_delta_linear(
            x2.data_ptr(), base_weight.data_ptr() if base_weight is not None else None,
            qweight_stacked.data_ptr(), meta_stacked.data_ptr(), scales_stacked.data_ptr(),
            indices.data_ptr(), out.data_ptr(), T, K, N, S, bits, group_size, 1 if accumulate else 0, ldy,
            ws.data_ptr(), ws.numel(), _stream())
    else:
        one = lambda p: (C.c_void_p * 1)(p)
        rc = _lib.lib().dz_multi_delta_linear_batch(
            1, one(x2.data_ptr()), one(base_weight.data_ptr() if base_weight is not None else None),
            one(qweight_stacked.data_ptr()), one(meta_stacked.data_ptr()), one(scales_stacked.data_ptr()),
            indices.data_ptr(), one(out.data_ptr()), (C.c_int * 1)(N), (C.c_int * 1)(ldy), T, K, S, bits, group_size,
            1 if accumulate else 0, optr, ws.data_ptr(), ws.numel(), _stream())
    _lib.check(rc, "dz_multi_delta_linear")
    return out


def _bits_from_shapes(qweight_stacked: torch.Tensor, K: int, N: int) -> int:
    words = qweight_stacked[0].numel()
    bits = words * 64 // (K * N)  # words = K*N*bits/64
    if bits not in (2, 4) or words * 64 != K * N * bits:
        raise ValueError("cannot infer the bit width from qweight_stacked")
    return bits


def apply_delta(x: torch.Tensor, qweight_stacked: torch.Tensor, scales_stacked: torch.Tensor,
                meta_stacked: torch.Tensor, indices: torch.Tensor, base_weight: torch.Tensor,
                order: Optional[torch.Tensor] = None, base_tiled: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Drop-in for serving/vllm/delta/deltazip_marlin.py:10-19.  Returns a new [T, N] tensor;
    indices == -1 selects the base weight only.  (`order`: optional, see `token_order`; `base_tiled`:
    optional, see `tile_base`.)"""
    N, K = base_tiled.shape if base_tiled is not None else base_weight.shape
    bits = _bits_from_shapes(qweight_stacked, K, N)
    y = multi_delta_linear(x, base_weight, qweight_stacked, scales_stacked, meta_stacked, indices, bits=bits,
                           order=order, base_tiled=base_tiled)
    return y.view(*x.shape[:-1], N)


def _order_ptr(order: Optional[torch.Tensor], T: int, device) -> Optional[int]:
    if isinstance(order, RowBlocks):
        raise ValueError("row blocks are for batches above %d tokens; pass token_order() here" % MAX_TOKENS_FUSED)
    if order is None or T <= 32:
        return None
    if (not order.is_cuda or order.device != device or order.dtype != torch.int32 or order.numel() < T
            or not order.is_contiguous()):
        raise ValueError("order must be a contiguous int32 GPU tensor with one entry per token")
    return order.data_ptr()


def apply_delta_batch(x, qweight_stacked: Sequence[torch.Tensor], scales_stacked: Sequence[torch.Tensor],
                      meta_stacked: Sequence[torch.Tensor], indices: torch.Tensor,
                      base_weight: Sequence[torch.Tensor], order: Optional[torch.Tensor] = None,
                      base_tiled: Optional[Sequence[torch.Tensor]] = None):
    """`apply_delta` for up to 4 projections that share the tokens -- q/k/v or gate/up held as
    separate weights, which the reference fuses into one layer
    (serving/vllm/delta/layers_marlin.py:281-487) -- in one launch.  `x` is one [T, K] tensor for
    all or a sequence with one per projection; `order` is what `token_order(indices, S)` returned
    for this batch, if the caller has it; returns the list of [T, N_j] outputs."""
    n = len(base_weight)
    xs = [x] * n if isinstance(x, torch.Tensor) else list(x)
    if not (len(xs) == len(qweight_stacked) == len(scales_stacked) == len(meta_stacked) == n) or not 1 <= n <= 4:
        raise ValueError("one x / qweight / scales / meta / base weight per projection, at most 4 projections")
    K = base_weight[0].shape[1]
    T = xs[0].reshape(-1, K).shape[0]
    bits = _bits_from_shapes(qweight_stacked[0], K, base_weight[0].shape[0])
    G = scales_stacked[0][0].numel() // base_weight[0].shape[0]
    S = qweight_stacked[0].shape[0]
    if T > MAX_TOKENS_FUSED:
        return [apply_delta(xs[j], qweight_stacked[j], scales_stacked[j], meta_stacked[j], indices, base_weight[j],
                            base_tiled=None if base_tiled is None else base_tiled[j])
                for j in range(n)]
    _need_cuda(indices, *xs, *qweight_stacked, *scales_stacked, *meta_stacked, *base_weight)
    if indices.dtype != torch.int64 or indices.numel() != T or not indices.is_contiguous():
        raise ValueError("indices must be a contiguous int64 tensor with one entry per token")
    group_size = -1 if G == 1 else K // G
    x2s, outs, Ns = [], [], []
    for j in range(n):
        N = base_weight[j].shape[0]
        x2 = xs[j].reshape(-1, K)
        if (x2.dtype != torch.float16 or base_weight[j].dtype != torch.float16 or base_weight[j].shape[1] != K
                or x2.shape[0] != T or not x2.is_contiguous() or not base_weight[j].is_contiguous()):
            raise ValueError("x and base weights must be contiguous float16 with the same K and T")
        cb, mb, sb = native_sizes(K, N, bits, group_size)
        q, m, sc = qweight_stacked[j], meta_stacked[j], scales_stacked[j]
        if (q.shape[0] != S or q[0].numel() * q.element_size() != cb or m[0].numel() * m.element_size() != mb
                or sc[0].numel() * sc.element_size() != sb or sc.dtype != torch.float16
                or not (q.is_contiguous() and m.is_contiguous() and sc.is_contiguous())):
            raise ValueError("stacked delta tensors do not match the native layout for these sizes")
        x2s.append(x2); Ns.append(N)
        outs.append(torch.empty((T, N), dtype=torch.float16, device=x2.device))
    vp = C.c_void_p * n
    ptrs = lambda ts: vp(*[t.data_ptr() for t in ts])
    ws = _workspace(x2s[0].device, T, K, sum(Ns))
    entry, bases = _lib.lib().dz_multi_delta_linear_batch, base_weight
    if base_tiled is not None:
        if len(base_tiled) != n:
            raise ValueError("one tiled base weight per projection")
        for j in range(n):
            _check_tiled(base_tiled[j], base_weight[j], Ns[j], K, x2s[j].device)
        entry, bases = _lib.lib().dz_multi_delta_linear_batch_tiled, base_tiled
    rc = entry(
        n, ptrs(x2s), ptrs(bases), ptrs(qweight_stacked), ptrs(meta_stacked), ptrs(scales_stacked),
        indices.data_ptr(), ptrs(outs), (C.c_int * n)(*Ns), (C.c_int * n)(*Ns), T, K, S, bits, group_size, 0,
        _order_ptr(order, T, indices.device), ws.data_ptr(), ws.numel(), _stream())
    _lib.check(rc, "dz_multi_delta_linear_batch")
    return [outs[j].view(*xs[j].shape[:-1], Ns[j]) for j in range(n)]


def add_delta(y: torch.Tensor, x: torch.Tensor, qweight: torch.Tensor, qzeros, scales: torch.Tensor,
              g_idx, indices: torch.Tensor, meta: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Drop-in for serving/vllm/delta/deltazip.py:14-37: y[i] += x[i] @ dequant(W[indices[i]])^T,
    in place.  `qzeros` and `g_idx` are accepted for signature compatibility and unused: the native
    layout is symmetric with g_idx = k // group_size (checked when the delta was repacked)."""
    if meta is None:
        raise ValueError("meta (2:4 positions) is required")
    K = x.shape[-1]
    N = scales.shape[-1]
    bits = _bits_from_shapes(qweight, K, N)
    y2 = y.view(-1, y.shape[-1])
    multi_delta_linear(x, None, qweight, scales, meta, indices, bits=bits, out=y2, accumulate=True)
    return y


def add_delta_slice(y: torch.Tensor, x: torch.Tensor, qweight, qzeros, scales, g_idx, indices,
                    scale: float, y_offset: int, y_slice_size: int, *, buffer=None,
                    meta: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Drop-in for serving/vllm/delta/deltazip.py:40-77: as add_delta, into the column slice
    y[:, y_offset : y_offset + y_slice_size].  `scale` is ignored, as it is by the reference."""
    if meta is None:
        raise ValueError("meta (2:4 positions) is required")
    K = x.shape[-1]
    N = scales.shape[-1]
    if N != y_slice_size:
        raise ValueError("y_slice_size must equal the delta's output features")
    bits = _bits_from_shapes(qweight, K, N)
    y2 = y.view(-1, y.shape[-1])[:, y_offset:y_offset + y_slice_size]
    multi_delta_linear(x, None, qweight, scales, meta, indices, bits=bits, out=y2, accumulate=True)
    return y


def apply_delta_into(x: torch.Tensor, qweight_stacked: torch.Tensor, qzeros_stacked, scales_stacked: torch.Tensor,
                     g_idx_stacked, indices: torch.Tensor, output: torch.Tensor, *,
                     meta_stacked: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Drop-in for the in-place, seven-argument apply_delta of serving/vllm/delta/deltazip.py:78-100:
    output[i] += x[i] @ dequant(W[indices[i]])^T for all leading dimensions flattened, returned with
    output's shape.  `meta_stacked` carries the 2:4 positions of the native layout (the reference's
    add_delta takes them as `meta`, deltazip.py:22); `qzeros_stacked` / `g_idx_stacked` are unused, as
    in `add_delta`."""
    x2 = x.view(-1, x.shape[-1])
    out2 = output.view(-1, output.shape[-1])
    add_delta(out2, x2, qweight_stacked, qzeros_stacked, scales_stacked, g_idx_stacked, indices.view(-1),
              meta=meta_stacked)
    return out2.view_as(output)


def apply_delta_packed_nslice(x: torch.Tensor, qweight_stacked: Sequence[torch.Tensor], qzeros_stacked,
                              scales_stacked: Sequence[torch.Tensor], g_idx_stacked, indices: torch.Tensor,
                              output: torch.Tensor, output_slices: Sequence[int], *,
                              meta_stacked: Optional[Sequence[torch.Tensor]] = None,
                              order: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Drop-in for serving/vllm/delta/deltazip.py:103-153: a layer made of several sublayers packed
    side by side (q/k/v, gate/up).  For slice j with n_j = output_slices[j] output features,
    output[:, off_j : off_j + n_j] += x @ dequant(W_j[indices])^T, off_j the sum of the slices before
    it; index -1 adds nothing.  Up to 128 tokens and 4 slices go in one launch (every slice a call
    of dz_multi_delta_linear_batch that adds into its columns of `output`); larger batches take one
    add_delta_slice per slice like the reference.  `meta_stacked[j]`: 2:4 positions of slice j."""
    n = len(output_slices)
    if meta_stacked is None:
        raise ValueError("meta_stacked (2:4 positions of every slice) is required")
    if not (len(qweight_stacked) >= n and len(scales_stacked) >= n and len(meta_stacked) >= n):
        raise ValueError("one qweight / scales / meta per output slice is required")
    K = x.shape[-1]
    x2 = x.view(-1, K)
    ind = indices.view(-1)
    out2 = output.view(-1, output.shape[-1])
    T = x2.shape[0]
    if sum(output_slices) > out2.shape[1]:
        raise ValueError("output_slices exceed the width of output")
    Ns = [int(v) for v in output_slices]
    offs = [sum(Ns[:j]) for j in range(n)]
    fits = (1 <= n <= 4 and T <= MAX_TOKENS_FUSED and out2.dtype == torch.float16 and out2.stride(1) == 1
            and out2.stride(0) % 4 == 0 and all(o % 4 == 0 for o in offs))
    if not fits:
        for j in range(n):
            add_delta_slice(out2, x2, qweight_stacked[j], None, scales_stacked[j], None, ind, 1.0, offs[j], Ns[j],
                            meta=meta_stacked[j])
        return out2.view_as(output)
    _need_cuda(x2, ind, out2, *qweight_stacked[:n], *scales_stacked[:n], *meta_stacked[:n])
    if x2.dtype != torch.float16 or not x2.is_contiguous():
        raise ValueError("x must be contiguous float16")
    if ind.dtype != torch.int64 or ind.numel() != T or not ind.is_contiguous():
        raise ValueError("indices must be a contiguous int64 tensor with one entry per token")
    if out2.shape[0] != T:
        raise ValueError("output must have one row per token")
    bits = _bits_from_shapes(qweight_stacked[0], K, Ns[0])
    S = qweight_stacked[0].shape[0]
    G = scales_stacked[0][0].numel() // Ns[0]
    group_size = -1 if G == 1 else K // G
    for j in range(n):
        cb, mb, sb = native_sizes(K, Ns[j], bits, group_size)
        q, m, sc = qweight_stacked[j], meta_stacked[j], scales_stacked[j]
        if (q.shape[0] != S or q[0].numel() * q.element_size() != cb or m[0].numel() * m.element_size() != mb
                or sc[0].numel() * sc.element_size() != sb or sc.dtype != torch.float16
                or not (q.is_contiguous() and m.is_contiguous() and sc.is_contiguous())):
            raise ValueError("stacked delta tensors do not match the native layout for these sizes")
    vp = C.c_void_p * n
    esz = out2.element_size()
    ws = _workspace(x2.device, T, K, sum(Ns))
    rc = _lib.lib().dz_multi_delta_linear_batch(
        n, vp(*[x2.data_ptr()] * n), vp(*[None] * n), vp(*[qweight_stacked[j].data_ptr() for j in range(n)]),
        vp(*[meta_stacked[j].data_ptr() for j in range(n)]), vp(*[scales_stacked[j].data_ptr() for j in range(n)]),
        ind.data_ptr(), vp(*[out2.data_ptr() + offs[j] * esz for j in range(n)]), (C.c_int * n)(*Ns),
        (C.c_int * n)(*[out2.stride(0)] * n), T, K, S, bits, group_size, 1, _order_ptr(order, T, ind.device),
        ws.data_ptr(), ws.numel(), _stream())
    _lib.check(rc, "dz_multi_delta_linear_batch")
    return out2.view_as(output)


def set_ksplit(nsplit: int) -> None:
    """Benchmark hook: force the number of K chunks of the fused kernel (0 = automatic)."""
    _lib.lib().dz_set_ksplit(int(nsplit))

