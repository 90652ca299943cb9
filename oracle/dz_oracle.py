"""CPU oracle for the multi-delta linear layer.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU and in numpy (+ torch CPU matmul), the algorithm that
eth-easl/deltazip runs for  y = x @ W_base.T + x @ dequant(delta[id(x)]).T .  It exists to
check the HIP kernels; only tests, the smoke check and the benchmark's CPU-baseline leg may
import it.  Nothing in the shipped package depends on it.

Every function names the reference lines it follows (paths relative to the reference root).

Pinning status (what independent evidence each function is checked against in tests/):
  quantize, find_params_sym     closed forms + known answers computed by hand          (pinned)
  find_params_sym(mse=True)     every candidate's error against plain-Python loops on exactly
                                representable rows, first-minimum rule, invariants      (pinned; the
                                reference's torch.sum order is undefined: near-ties may differ)
  prune_2of4_magnitude          brute force on tiny rows, group invariants             (pinned)
  pack_gptq / unpack_gptq       single-bit probes, hand-packed words, round trips      (pinned)
  dequant_gptq                  exhaustive fp16-scale sweep against exact rational math (pinned)
  forward_ref                   per-token python loop, F.linear special cases          (pinned)
  native layout functions       defined by this project; pinned by round trip through
                                dequant_gptq
  convert_mapping_ref           hand-computed index tensors for small batches          (pinned)
  embed_select_ref, linear_select_ref   plain row selection / torch CPU matmul per row, checked
                                against hand-built tables                              (pinned)
  hessian_add_batch_ref, hinv_upper_ref, obs_sweep_ref   float64 Gram matrix, identity-Hessian
                                reduction to the pinned quantizer, closed-form surgeon update,
                                first-order optimality of unvisited columns (pinned by mathematics;
                                the reference's matmul summation order and topk tie order are
                                undefined: "parity unpinned" against it on those two points)
The fused third-party kernel the reference calls on the serving path (triteia
`sbmm_4bit_2_4_native`, un-vendored and un-pinned: scripts/install.sh:2, call site
serving/vllm/delta/deltazip_marlin.py:18) cannot be inspected: its bit layout and rounding are
"parity unpinned".  Parity is anchored on the reference's in-tree CPU-runnable path instead.
"""
from __future__ import annotations

import numpy as np
import torch

# --------------------------------------------------------------------------------------
# a1/a2: quantizer  (deltazip/core/quant.py)
# --------------------------------------------------------------------------------------


def quantize(x: np.ndarray, scale: np.ndarray, zero: np.ndarray, maxq: int) -> np.ndarray:
    """deltazip/core/quant.py:9-18.  q = clamp(round(x/scale)+zero, 0, maxq); returns
    scale*(q-zero).  torch.round is round-half-to-even, as is np.rint.  fp32 throughout."""
    x = x.astype(np.float32)
    q = np.clip(np.rint(x / scale) + zero, 0, maxq).astype(np.float32)
    return (scale * (q - zero)).astype(np.float32)


def quantize_codes(x, scale, zero, maxq):
    """Integer codes of `quantize` (the q before it is mapped back), uint8."""
    x = x.astype(np.float32)
    return np.clip(np.rint(x / scale) + zero, 0, maxq).astype(np.uint8)


def find_params_sym(w: np.ndarray, bits: int, group_size: int = -1, mse: bool = False, norm: float = 2.4,
                    grid: int = 100, maxshrink: float = 0.8, return_errors: bool = False):
    """Symmetric per-output-row (optionally per (row, K-group)) scale and zero.

    deltazip/core/quant.py:48-130 with perchannel=True, sym=True, weight=True; mse=False is the
    configuration deltazip/modeling/_base.py:399-406 uses, mse=True adds the search over the
    clipping range (`_mse_search`).  `w` is [N, K] fp32.
    Returns (scale [N, G] fp32, zero [N, G] fp32) with G = 1 for group_size == -1.

    The reference computes the parameters on the un-pruned delta (core/sparsegpt.py:64-66).
    Grouping along K is a format-compatible extension (the reference's g_idx mechanism); each
    group is treated exactly like a full row is by the reference.
    """
    w = w.astype(np.float32)
    n, k = w.shape
    g = k if group_size in (-1, k) else group_size
    assert k % g == 0
    maxq = 2**bits - 1
    wg = w.reshape(n, k // g, g)
    xmin = np.minimum(wg.min(axis=2), 0.0).astype(np.float32)       # quant.py:69
    xmax = np.maximum(wg.max(axis=2), 0.0).astype(np.float32)       # quant.py:70
    xmax = np.maximum(np.abs(xmin), xmax)                           # quant.py:73
    neg = xmin < 0
    xmin = np.where(neg, -xmax, xmin)                               # quant.py:74-76
    both0 = (xmin == 0) & (xmax == 0)                               # quant.py:77-79
    xmin = np.where(both0, -1.0, xmin).astype(np.float32)
    xmax = np.where(both0, +1.0, xmax).astype(np.float32)
    scale = ((xmax - xmin) / np.float32(maxq)).astype(np.float32)   # quant.py:81
    zero = np.full_like(scale, (maxq + 1) / 2)                      # quant.py:83
    if mse:
        scale, errs = _mse_search(wg, xmin, xmax, scale, zero, maxq, norm, grid, maxshrink)
        if return_errors:
            return scale, zero, errs
    return scale, zero


def _mse_search(wg, xmin, xmax, scale, zero, maxq, norm, grid, maxshrink):
    """deltazip/core/quant.py:85-101 for sym=True: candidates p = 1 - i / grid, i = 0 ..
    int(maxshrink * grid) - 1; every candidate's range is (p * xmin, p * xmax), its scale
    (xmax1 - xmin1) / maxq, its zero the symmetric one; the error of a row (group) is the sum of
    |quantize(x) - x| ** norm, and a candidate replaces the best so far only when strictly better
    (`err < best`).  The elementwise arithmetic is fp32 as the reference's tensor ops; the
    reference's torch.sum has no defined order, here the sum is taken in float64.  Returns the
    chosen scale and the errors of all candidates [ncand, N, G] (for tests of near-ties)."""
    scale = scale.copy()
    best = np.full(scale.shape, np.inf)
    ncand = int(maxshrink * grid)
    errs = np.empty((ncand,) + scale.shape)
    for i in range(ncand):
        p = np.float32(1 - i / grid)                                 # a Python float times an fp32 tensor
        xmin1 = (p * xmin).astype(np.float32)
        xmax1 = (p * xmax).astype(np.float32)
        scale1 = ((xmax1 - xmin1) / np.float32(maxq)).astype(np.float32)
        q = quantize(wg, scale1[:, :, None], zero[:, :, None], maxq)   # quant.py:93
        d = np.abs((q - wg).astype(np.float32))
        e = np.power(d, np.float32(norm), dtype=np.float32)
        err = e.astype(np.float64).sum(axis=2)
        errs[i] = err
        better = err < best
        best = np.where(better, err, best)
        scale = np.where(better, scale1, scale).astype(np.float32)
    return scale, errs


# --------------------------------------------------------------------------------------
# a3: 2:4 mask rule (deltazip/core/sparsegpt.py:117-135 with H = I)
# --------------------------------------------------------------------------------------


def prune_2of4_magnitude(w: np.ndarray) -> np.ndarray:
    """Boolean keep-mask [N, K]: in every aligned group of 4 along K keep the 2 entries of
    largest |w|.  core/sparsegpt.py:123-125 prunes the `prunen`=2 entries with the smallest
    w^2/diag(Hinv)^2 in each group of `prunem`=4; with an identity Hessian that is the 2
    smallest |w|.  torch.topk leaves ties unspecified; here ties keep the lower column index.
    """
    n, k = w.shape
    assert k % 4 == 0
    a = np.abs(w.astype(np.float32)).reshape(n, k // 4, 4)
    # rank of each entry inside its group under (larger |w| first, lower index first on ties)
    rank = np.zeros(a.shape, dtype=np.int8)
    for i in range(4):
        for j in range(4):
            if i == j:
                continue
            ahead = (a[:, :, j] > a[:, :, i]) if j > i else (a[:, :, j] >= a[:, :, i])
            rank[:, :, i] += ahead
    return (rank < 2).reshape(n, k)


def compress_delta(delta32: np.ndarray, bits: int, group_size: int = -1):
    """delta [N, K] fp32 -> (codes [K, N] uint8, scales16 [G, N] fp16, zeros [G, N] int, keep).

    Order of operations follows core/sparsegpt.py:64-66 (parameters from the un-pruned
    delta), :123-135 (pruned entries are set to 0 and then quantized, so their code is the
    zero-point and they dequantize to exactly 0).
    """
    n, k = delta32.shape
    maxq = 2**bits - 1
    scale, zero = find_params_sym(delta32, bits, group_size)       # [N, G]
    g = k // scale.shape[1]
    keep = prune_2of4_magnitude(delta32)
    wp = np.where(keep, delta32.astype(np.float32), np.float32(0))
    scale_full = np.repeat(scale, g, axis=1)
    zero_full = np.repeat(zero, g, axis=1)
    codes = quantize_codes(wp, scale_full, zero_full, maxq)        # [N, K]
    return (np.ascontiguousarray(codes.T), np.ascontiguousarray(scale.T.astype(np.float16)),
            np.ascontiguousarray(zero.T.astype(np.int32)), keep)


# --------------------------------------------------------------------------------------
# a4: GPTQ-style packing (deltazip/nn_modules/qlinear_cuda.py:144-244)
# --------------------------------------------------------------------------------------


def pack_codes_gptq(codes: np.ndarray, zeros: np.ndarray, scales16: np.ndarray, bits: int):
    """codes [K, N] uint8, zeros [G, N] int (true zero-points), scales16 [G, N] fp16 ->
    (qweight [K/pf, N] int32, qzeros [G, N/pf] int32, scales [G, N] fp16, g_idx [K] int32).

    qlinear_cuda.py:177-182: qweight[r, n] |= code[r*pf + j, n] << (bits*j), j = 0..pf-1.
    qlinear_cuda.py:208-220: qzeros stores (zero - 1), packed along N the same way.
    qlinear_cuda.py:81-86 / sparsegpt.py:161-162: g_idx[k] = k // group_size.
    """
    assert bits in (2, 4, 8)
    k, n = codes.shape
    pf = 32 // bits
    assert k % pf == 0 and n % pf == 0
    c = codes.astype(np.uint32).reshape(k // pf, pf, n)
    qweight = np.zeros((k // pf, n), dtype=np.uint32)
    for j in range(pf):
        qweight |= c[:, j, :] << np.uint32(bits * j)
    g = zeros.shape[0]
    z = (zeros.astype(np.int64) - 1).astype(np.uint32).reshape(g, n // pf, pf)
    qzeros = np.zeros((g, n // pf), dtype=np.uint32)
    for j in range(pf):
        qzeros |= (z[:, :, j] & np.uint32(2**bits - 1)) << np.uint32(bits * j)
    group = k // g
    g_idx = (np.arange(k) // group).astype(np.int32)
    return qweight.view(np.int32), qzeros.view(np.int32), scales16.astype(np.float16), g_idx


def pack_from_weights(w_deq: np.ndarray, scale: np.ndarray, zero: np.ndarray, bits: int):
    """The reference's `QuantLinear.pack` starting, as it does, from the dequantized fp32
    weights: intweight[k, n] = round((W[n, k] + zero*scale) / half(scale))
    (qlinear_cuda.py:153-168; the division uses the fp16-rounded scale).  w_deq [N, K] fp32,
    scale/zero [N, G] fp32.  Returns the same tuple as pack_codes_gptq."""
    n, k = w_deq.shape
    g = scale.shape[1]
    group = k // g
    scales_t = np.ascontiguousarray(scale.T).astype(np.float32)       # [G, N]
    zeros_t = np.ascontiguousarray(zero.T).astype(np.float32)
    scale_zeros = zeros_t * scales_t
    scales16 = scales_t.astype(np.float16)
    gi = np.arange(k) // group
    num = w_deq.T.astype(np.float32) + scale_zeros[gi]                 # [K, N]
    codes = np.rint(num / scales16[gi].astype(np.float32)).astype(np.int64)
    codes = codes.astype(np.uint32).astype(np.uint8)
    return pack_codes_gptq(codes, zeros_t.astype(np.int32), scales16, bits)


def unpack_gptq(qweight: np.ndarray, qzeros: np.ndarray, bits: int):
    """qlinear_cuda.py:250-264 / quant_linear_naive.py:43-58: shift right by bits*j, mask with
    2^bits-1, zeros get +1.  Returns (codes [K, N] int8/int16, zeros [G, N] same dtype)."""
    assert bits in (2, 4, 8)
    pf = 32 // bits
    mask = 2**bits - 1
    dt = np.int16 if bits == 8 else np.int8
    wf = (np.arange(pf) * bits).astype(np.uint32)
    qw = qweight.view(np.uint32)
    codes = ((qw[:, None, :] >> wf[None, :, None]) & np.uint32(mask)).astype(dt)
    codes = codes.reshape(qw.shape[0] * pf, qw.shape[1])
    qz = qzeros.view(np.uint32)
    zeros = ((qz[:, :, None] >> wf[None, None, :]) & np.uint32(mask)).astype(dt) + dt(1)
    zeros = zeros.reshape(qz.shape[0], qz.shape[1] * pf)
    return codes, zeros


# --------------------------------------------------------------------------------------
# a5: dequantisation (qlinear_cuda.py:306-308, quant_linear_naive.py:65-67)
# --------------------------------------------------------------------------------------


def dequant_gptq(qweight, qzeros, scales16, g_idx, bits) -> np.ndarray:
    """delta^T [K, N] fp16 = scales[g_idx] * (codes - zeros[g_idx]).

    In the reference this is an fp16 tensor times an int8 tensor, which torch evaluates as
    one correctly rounded fp16 product.  The integer factor has at most 5 significant bits and
    the scale 11, so the fp32 product is exact and a single fp32->fp16 round-to-nearest-even
    reproduces it; that is what is computed here."""
    codes, zeros = unpack_gptq(qweight, qzeros, bits)
    gi = g_idx.astype(np.int64)
    m = (codes.astype(np.int32) - zeros[gi].astype(np.int32)).astype(np.float32)
    s = scales16.astype(np.float16)[gi].astype(np.float32)
    with np.errstate(over="ignore"):       # products beyond the fp16 range round to inf, as in torch
        return (s * m).astype(np.float16)


# --------------------------------------------------------------------------------------
# a6/a7/a8: forward
# --------------------------------------------------------------------------------------


def forward_ref(x16: np.ndarray, w_base16, delta_t_list, ids: np.ndarray) -> np.ndarray:
    """fp32 layer output [T, N].

    Semantics of apply_delta (serving/vllm/delta/deltazip_marlin.py:10-19; per-token rule
    spelled out at serving/vllm/delta/deltazip.py:24-30): token t uses W_base plus the delta
    in slot ids[t], ids[t] == -1 meaning base only.  The weight is formed as the reference's
    merge does, W = W_base + delta (deltazip/utils/generate.py:9-20), in fp32, and tokens are
    grouped by id with one dense product per id, the reference's own idiom for this
    (deltazip_marlin.py:44-53).  w_base16 may be None (delta-only, for the add_delta forms).
    delta_t_list[d] is delta^T [K, N] fp16 as dequant_gptq returns it."""
    x = torch.from_numpy(np.ascontiguousarray(x16).astype(np.float32))
    t = x.shape[0]
    n = (w_base16.shape[0] if w_base16 is not None else delta_t_list[0].shape[1])
    y = torch.zeros((t, n), dtype=torch.float32)
    wb = None if w_base16 is None else torch.from_numpy(np.ascontiguousarray(w_base16).astype(np.float32))
    ids = np.asarray(ids).astype(np.int64)
    for d in np.unique(ids):
        sel = torch.from_numpy(np.nonzero(ids == d)[0])
        if d >= 0:
            w = torch.from_numpy(np.ascontiguousarray(delta_t_list[int(d)]).astype(np.float32)).t()
            if wb is not None:
                w = wb + w
        else:
            if wb is None:
                continue
            w = wb
        y[sel] = x[sel] @ w.t()
    return y.numpy()


def forward_token_loop(x16, w_base16, delta_t_list, ids) -> np.ndarray:
    """Per-token loop in float64: the independent check for forward_ref, shaped like the
    reference's multi-adapter kernel test (serving/tests/lora/test_punica.py:18-42)."""
    t = x16.shape[0]
    n = w_base16.shape[0]
    y = np.zeros((t, n), dtype=np.float64)
    for i in range(t):
        xi = x16[i].astype(np.float64)
        y[i] = w_base16.astype(np.float64) @ xi
        if ids[i] >= 0:
            y[i] += xi @ delta_t_list[int(ids[i])].astype(np.float64)
    return y


def rel_err(y, y_ref) -> float:
    """max |y - y_ref| / max(|y_ref|, 1e-3 * max|y_ref|): the layer-output parity metric."""
    y = np.asarray(y, dtype=np.float64)
    y_ref = np.asarray(y_ref, dtype=np.float64)
    eps = 1e-3 * np.abs(y_ref).max()
    return float(np.max(np.abs(y - y_ref) / np.maximum(np.abs(y_ref), eps)))


# --------------------------------------------------------------------------------------
# native gfx950 layout (defined by this project)
# --------------------------------------------------------------------------------------
# Tiles: an "n-pair" is 32 output rows (two 16-row fragments), a "k-block" is 256 input
# columns (four 64-column steps).  One fragment = 16 rows x 64 columns; lane la = 16*ga + i of
# a 64-lane wavefront owns row i and the four aligned groups-of-4 starting at
#     k0(ga, p) = 16*(ga & 1) + 32*(ga >> 1) + 8*(p >> 1) + 4*(p & 1),   p = 0..3
# inside the step.  Each group contributes its two kept elements (ascending position): element
# e = 2p + w.  This is the operand order of the sparse matrix instruction
# v_smfmac_f32_16x16x64_f16 when the dense operand's 16 per-lane values are taken as columns
# 8*gb + (eb & 7) + 32*(eb >> 3).
#   meta  uint32 [N/32][K/256][64 lanes][4 steps]: bits [16*s + 2*e, +2) = position (0..3) of
#         element e of fragment (row-tile 2*np + s, step 4*kb + j).
#   codes 2-bit uint32 [N/32][K/256][64][4]: word j; for s in 0..1, m in 0..3, t = 4*s + m:
#         bits [2t, 2t+2) = code of element 2m, bits [16+2t, 16+2t+2) = code of element 2m+1.
#   codes 4-bit uint32 [N/32][K/256][2][64][4]: half hf covers steps 2*hf, 2*hf+1; word
#         w = 2*(j & 1) + s; bits [4m, 4m+4) = element 2m, bits [16+4m, 16+4m+4) = element 2m+1.
#   scales fp16 [G][N] unchanged.


def _frag_group_k0():
    ga = np.arange(4)[:, None]
    p = np.arange(4)[None, :]
    return 16 * (ga & 1) + 32 * (ga >> 1) + 8 * (p >> 1) + 4 * (p & 1)   # [ga, p]


def repack_native(qweight, qzeros, scales16, g_idx, bits):
    """GPTQ layout -> native (codes uint32, meta uint32, scales fp16).  Raises ValueError when
    the input is not 2:4 sparse, has a zero-point other than 2^(bits-1), or a g_idx other than
    k // group_size."""
    if bits not in (2, 4):
        raise ValueError("native layout supports 2 and 4 bits")
    codes, zeros = unpack_gptq(qweight, qzeros, bits)        # [K, N], [G, N]
    k, n = codes.shape
    if k % 256 or n % 32:
        raise ValueError("native layout needs K % 256 == 0 and N % 32 == 0")
    zp = 2 ** (bits - 1)
    if not np.all(zeros == zp):
        raise ValueError("only the symmetric zero-point 2^(bits-1) is supported")
    g = scales16.shape[0]
    if not np.array_equal(np.asarray(g_idx), np.arange(k) // (k // g)):
        raise ValueError("g_idx must be k // group_size")
    c = codes.T.astype(np.int32).reshape(n, k // 4, 4)        # [N, groups, 4]
    nz = c != zp
    if np.any(nz.sum(axis=2) > 2):
        raise ValueError("input is not 2:4 sparse")
    # kept positions: the non-zero-point entries, completed with the lowest free positions
    pos = np.arange(4)[None, None, :]
    key = np.where(nz, pos, pos + 4)                           # non-zero first, by position
    order = np.sort(key, axis=2)[:, :, :2] % 4                 # two kept positions
    order = np.sort(order, axis=2)                             # ascending position
    kept = np.take_along_axis(c, order, axis=2)                # [N, groups, 2]
    np_, nkb = n // 32, k // 256
    k0 = _frag_group_k0()                                      # [ga, p]
    # index arrays over (np, s, i, kb, j, ga, p)
    s_ = np.arange(2); i_ = np.arange(16); j_ = np.arange(4)
    meta = np.zeros((np_, nkb, 64, 4), dtype=np.uint32)
    if bits == 2:
        out = np.zeros((np_, nkb, 64, 4), dtype=np.uint32)
    else:
        out = np.zeros((np_, nkb, 2, 64, 4), dtype=np.uint32)
    rows = (np.arange(np_)[:, None, None] * 32 + s_[None, :, None] * 16 + i_[None, None, :])  # [np,s,i]
    for ga in range(4):
        for p in range(4):
            for j in range(4):
                grp = (np.arange(nkb) * 256 + 64 * j + k0[ga, p]) // 4          # [kb]
                pos2 = order[rows[:, :, :, None], grp[None, None, None, :]]     # [np,s,i,kb,2]
                val2 = kept[rows[:, :, :, None], grp[None, None, None, :]]
                for s in range(2):
                    la = 16 * ga + i_
                    for w in range(2):
                        e = 2 * p + w
                        pv = pos2[:, s, :, :, w].transpose(0, 2, 1).astype(np.uint32)  # [np,kb,i]
                        cv = val2[:, s, :, :, w].transpose(0, 2, 1).astype(np.uint32)
                        meta[:, :, la, j] |= pv << np.uint32(16 * s + 2 * e)
                        m = e // 2
                        if bits == 2:
                            t = 4 * s + m
                            out[:, :, la, j] |= cv << np.uint32(2 * t + 16 * (e & 1))
                        else:
                            out[:, :, j // 2, la, 2 * (j & 1) + s] |= cv << np.uint32(4 * m + 16 * (e & 1))
    return out, meta, scales16.astype(np.float16).copy()


def dequant_native(codes, meta, scales16, k, n, bits) -> np.ndarray:
    """native -> delta [N, K] fp16 (note: [N, K], the transpose of dequant_gptq's output)."""
    zp = 2 ** (bits - 1)
    np_, nkb = n // 32, k // 256
    g = scales16.shape[0]
    group = k // g
    out = np.zeros((n, k), dtype=np.float16)
    k0 = _frag_group_k0()
    i_ = np.arange(16)
    sc = scales16.astype(np.float32)                          # [G, N]
    for ga in range(4):
        la = 16 * ga + i_
        for p in range(4):
            for j in range(4):
                for s in range(2):
                    for w in range(2):
                        e = 2 * p + w
                        pos = (meta[:, :, la, j] >> np.uint32(16 * s + 2 * e)) & np.uint32(3)   # [np,kb,i]
                        m = e // 2
                        if bits == 2:
                            cv = (codes[:, :, la, j] >> np.uint32(2 * (4 * s + m) + 16 * (e & 1))) & np.uint32(3)
                        else:
                            cv = (codes[:, :, j // 2, la, 2 * (j & 1) + s] >> np.uint32(4 * m + 16 * (e & 1))) & np.uint32(15)
                        rows = (np.arange(np_)[:, None, None] * 32 + 16 * s + i_[None, None, :])
                        rows = np.broadcast_to(rows, pos.shape)
                        cols = (np.arange(nkb)[None, :, None] * 256 + 64 * j + k0[ga, p]) + pos.astype(np.int64)
                        val = (sc[cols // group, rows] * (cv.astype(np.float32) - zp)).astype(np.float16)
                        # a later kept element that dequantises to 0 must not erase an earlier value:
                        # positions are distinct within a group, so plain assignment is safe.
                        out[rows, cols] = val
    return out


# --------------------------------------------------------------------------------------
# a11: delta id -> slot index tensors (serving/vllm/delta/models.py:69-145)
# --------------------------------------------------------------------------------------


def convert_mapping_ref(index_mapping, prompt_mapping, delta_index_to_id, max_deltas, vocab_size,
                        extra_vocab_size):
    """Returns (base_indices [T], sampler_indices [P], sampler_indices_padded [P],
    embeddings_indices [2, T]) as int64 arrays.  `max_deltas` is what the caller passes there
    (the manager passes slots + 1, models.py:401).

    models.py:106-116: slot = delta_index_to_id.index(id) for id > 0 (raises ValueError when the
    id is in no slot), else -1; the embedding index uses 0 instead of -1 for the base model.
    models.py:122-126: embeddings_indices = [e * extra_vocab, e * (vocab + extra_vocab)], entries
    equal to -1 replaced by max_deltas - 1.  models.py:129-133: padded = arange(P) + s' * P with
    s' = s, or max_deltas - 1 where s == -1."""
    table = list(delta_index_to_id)
    slot = lambda x: table.index(x) if x > 0 else -1
    base = np.array([slot(x) for x in index_mapping], dtype=np.int64)
    emb = np.array([slot(x) if x > 0 else 0 for x in index_mapping], dtype=np.int64)
    sampler = np.array([slot(x) for x in prompt_mapping], dtype=np.int64)
    emb2 = np.stack([emb * extra_vocab_size, emb * (vocab_size + extra_vocab_size)]).astype(np.int64)
    emb2[emb2 == -1] = max_deltas - 1
    padded = sampler.copy()
    padded[padded == -1] = max_deltas - 1
    padded = np.arange(len(padded), dtype=np.int64) + padded * len(padded)
    return base, sampler, padded, emb2


# --------------------------------------------------------------------------------------
# uncompressed per-delta tables: embedding and output projection
# (serving/vllm/delta/deltazip_marlin.py:21-86)
# --------------------------------------------------------------------------------------


def embed_select_ref(tokens, delta_weights, ids, base_weight) -> np.ndarray:
    """deltazip_marlin.py:56-86: row tokens[t] of delta_weights[ids[t]], or of base_weight for
    ids[t] == -1 (the delta's table replaces the base table)."""
    out = np.zeros((len(tokens), base_weight.shape[1]), dtype=base_weight.dtype)
    for t, (tok, d) in enumerate(zip(tokens, ids)):
        out[t] = (base_weight if d == -1 else delta_weights[int(d)])[int(tok)]
    return out


def linear_select_ref(x16, delta_weights, ids, base_weight) -> np.ndarray:
    """deltazip_marlin.py:21-53: F.linear(x[t], W) with W = delta_weights[ids[t]] or base_weight
    for ids[t] == -1; fp32 result [T, N]."""
    x = torch.from_numpy(np.ascontiguousarray(x16).astype(np.float32))
    out = np.zeros((x.shape[0], base_weight.shape[0]), dtype=np.float32)
    for t, d in enumerate(ids):
        w = base_weight if d == -1 else delta_weights[int(d)]
        out[t] = (torch.from_numpy(np.ascontiguousarray(w).astype(np.float32)) @ x[t]).numpy()
    return out


# --------------------------------------------------------------------------------------
# seeded synthetic inputs for the benchmark configurations
# --------------------------------------------------------------------------------------


def _randn(shape, seed):
    g = torch.Generator(device="cpu").manual_seed(int(seed))
    return torch.randn(shape, generator=g, dtype=torch.float32).numpy()


def make_base(n, k, seed):
    return (_randn((n, k), seed) * np.float32(0.02)).astype(np.float16)


def make_delta(n, k, sigma, bits, group_size, seed):
    """Returns dict with GPTQ-format tensors of one synthetic 2:4 delta."""
    d = _randn((n, k), seed) * np.float32(sigma)
    codes, scales16, zeros, keep = compress_delta(d, bits, group_size)
    qweight, qzeros, scales, g_idx = pack_codes_gptq(codes, zeros, scales16, bits)
    return dict(qweight=qweight, qzeros=qzeros, scales=scales, g_idx=g_idx, bits=bits,
                delta32=d, keep=keep, codes=codes)


def make_x(t, k, seed):
    return _randn((t, k), seed).astype(np.float16)


def make_ids(kind, t, n_deltas, seed):
    g = torch.Generator(device="cpu").manual_seed(int(seed))
    if kind == "single":
        return np.zeros(t, dtype=np.int64)
    if kind == "uniform":
        return torch.randint(0, n_deltas, (t,), generator=g).numpy().astype(np.int64)
    if kind == "zipf":
        p = torch.arange(1, n_deltas + 1, dtype=torch.float64) ** -1.5
        return torch.multinomial(p / p.sum(), t, replacement=True, generator=g).numpy().astype(np.int64)
    if kind == "blocks":
        return np.repeat(np.arange(n_deltas), t // n_deltas).astype(np.int64)
    raise ValueError(kind)


# --------------------------------------------------------------------------------------
# f-4: the Hessian-aware sweep (deltazip/core/sparsegpt.py:25-146), n:m pruning with error
# compensation.  Pinned by what the mathematics fixes (tests/test_oracle_obs.py): an identity
# Hessian reduces it to prune_2of4_magnitude + quantize; without quantisation every kept weight to
# the right of the sweep satisfies the first-order optimality condition (W0 - W) H[:, todo] = 0;
# pruning one weight of a 1 x K row equals the closed-form optimal-brain-surgeon update.  The
# floating-point summation order of the reference's matmuls and torch.topk's tie order are not
# defined by the reference: here sums run in ascending index order with one rounding per operation
# and ties keep the lower column ("parity unpinned" against the reference for those two points).
# --------------------------------------------------------------------------------------


def hessian_add_batch_ref(H: np.ndarray, nsamples: int, inp: np.ndarray):
    """sparsegpt.py:27-40 for a linear layer: inp [B, L, K] (or [L, K] = one sample).
    H <- H * n/(n+B); inp <- sqrt(2/(n+B)) * inp; H <- H + inp^T inp.  Returns (H, n+B)."""
    x = np.asarray(inp, dtype=np.float32)
    b = 1 if x.ndim == 2 else x.shape[0]
    x = x.reshape(-1, x.shape[-1])
    H = (H.astype(np.float32) * np.float32(nsamples / (nsamples + b))).astype(np.float32)
    n = nsamples + b
    xs = (np.float32(np.sqrt(2.0 / n)) * x).astype(np.float32)
    acc = np.zeros_like(H)
    for t in range(xs.shape[0]):                       # ascending token order, one rounding per op
        acc = (acc + (xs[t][:, None] * xs[t][None, :]).astype(np.float32)).astype(np.float32)
    return (H + acc).astype(np.float32), n


def hinv_upper_ref(H: np.ndarray, W: np.ndarray, percdamp: float = 0.01):
    """sparsegpt.py:69-84: dead columns, dampening, H^-1 through Cholesky, its upper factor.
    Returns (Hinv_upper [K, K] fp32, W with dead columns zeroed).  torch CPU LAPACK in fp32."""
    H = torch.from_numpy(np.array(H, dtype=np.float32))
    W = np.array(W, dtype=np.float32)
    dead = torch.diag(H) == 0
    H[dead, dead] = 1
    W[:, dead.numpy()] = 0
    damp = percdamp * torch.mean(torch.diag(H))
    idx = torch.arange(H.shape[0])
    H[idx, idx] += damp
    H = torch.linalg.cholesky(H)
    H = torch.cholesky_inverse(H)
    H = torch.linalg.cholesky(H, upper=True)
    return np.ascontiguousarray(H.numpy()), W


def obs_sweep_ref(W: np.ndarray, hinv: np.ndarray, scale=None, bits: int = 4, prunen: int = 2,
                  prunem: int = 4, blocksize: int = 128, stop: int = None):
    """sparsegpt.py:92-146.  W [N, K] fp32, hinv = upper Cholesky factor of H^-1, scale [N] fp32
    (per-row symmetric scale, zero = 2^(bits-1)) or None for pruning without quantisation.
    Returns (W_out [N, K], losses [N]); columns >= `stop` (a multiple of blocksize) are left as
    the sweep has updated them so far (used by the optimality test)."""
    W = np.array(W, dtype=np.float32)
    n, k = W.shape
    hinv = np.asarray(hinv, dtype=np.float32)
    maxq = np.float32(2**bits - 1)
    zero = np.float32(2 ** (bits - 1))
    losses = np.zeros(n, dtype=np.float32)
    stop = k if stop is None else stop
    for i1 in range(0, stop, blocksize):
        i2 = min(i1 + blocksize, k)
        count = i2 - i1
        W1 = W[:, i1:i2].copy()
        Q1 = np.zeros_like(W1)
        Err1 = np.zeros_like(W1)
        H1 = hinv[i1:i2, i1:i2]
        dg = np.diag(H1).astype(np.float32)
        mask1 = np.zeros(W1.shape, dtype=bool)
        lsum = np.zeros(n, dtype=np.float32)
        for i in range(count):
            w = W1[:, i].copy()
            d = dg[i]
            if prunen != 0 and i % prunem == 0:
                tmp = (W1[:, i:i + prunem] ** 2).astype(np.float32) / (dg[i:i + prunem] ** 2).astype(np.float32)[None, :]
                # keep the (prunem - prunen) largest; ties keep the lower column
                m = tmp.shape[1]
                rank = np.zeros(tmp.shape, dtype=np.int8)
                for a in range(m):
                    for b in range(m):
                        if a != b:
                            rank[:, a] += (tmp[:, b] > tmp[:, a]) if b > a else (tmp[:, b] >= tmp[:, a])
                mask1[:, i:i + prunem] = rank >= (m - prunen)
            q = np.where(mask1[:, i], np.float32(0), w).astype(np.float32)
            if scale is not None:
                sc = scale.astype(np.float32)
                q = (sc * (np.clip(np.rint(q / sc) + zero, 0, maxq) - zero)).astype(np.float32)
            Q1[:, i] = q
            diff = (w - q).astype(np.float32)
            lsum = (lsum + ((diff * diff).astype(np.float32) / np.float32(d * d)).astype(np.float32)).astype(np.float32)
            err = (diff / d).astype(np.float32)
            W1[:, i:] = (W1[:, i:] - (err[:, None] * H1[i, i:][None, :]).astype(np.float32)).astype(np.float32)
            Err1[:, i] = err
        W[:, i1:i2] = Q1
        losses = (losses + lsum / np.float32(2)).astype(np.float32)
        if i2 < k:
            acc = np.zeros((n, k - i2), dtype=np.float32)
            for j in range(count):                      # ascending, one rounding per operation
                acc = (acc + (Err1[:, j][:, None] * hinv[i1 + j, i2:][None, :]).astype(np.float32)).astype(np.float32)
            W[:, i2:] = (W[:, i2:] - acc).astype(np.float32)
    return W, losses
