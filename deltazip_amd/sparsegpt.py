"""Hessian-aware compression of one linear layer's delta, with the reference's interface
(deltazip/core/sparsegpt.py: `SparseGPT`; deltazip/core/quant.py: `Quantizer`).

    gpt = SparseGPT(layer)                    # an nn.Linear on the GPU holding the fine-tuned weight
    gpt.quantizer = Quantizer(); gpt.quantizer.configure(4, perchannel=True, sym=True)
    for batch in calibration_inputs: gpt.add_batch(batch, None)
    scale, zero, g_idx, avg_loss, W = gpt.fasterprune(0.5, prunen=2, prunem=4, base_weight=base)
    qweight, meta, scales16 = gpt.pack()      # native layout of the compressed delta

The Hessian, the column sweep, the scales and the packing run in this library's HIP kernels; the
two Cholesky factorisations of the K x K Hessian are torch.linalg calls on the same device."""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from . import ops


class Quantizer:
    """Symmetric per-output-row weight quantizer (deltazip/core/quant.py:21-144; the settings
    deltazip/modeling/_base.py:399-406 uses are perchannel=True, sym=True, mse=False; mse=True, the
    search over the clipping range with `norm`, `grid` and `maxshrink`, is built too)."""

    def __init__(self):
        self.maxq = 0
        self.bits = 0
        self.scale: Optional[torch.Tensor] = None
        self.zero: Optional[torch.Tensor] = None

    def configure(self, bits, perchannel=True, sym=True, mse=False, norm=2.4, grid=100, maxshrink=0.8, grouprows=1):
        if bits not in (2, 4):
            raise NotImplementedError("Only 2 and 4 bits are supported.")
        if not (perchannel and sym) or grouprows != 1:
            raise NotImplementedError("only the per-channel symmetric quantizer is built")
        self.bits = bits
        self.maxq = 2 ** bits - 1
        self.mse, self.norm, self.grid, self.maxshrink = bool(mse), norm, grid, maxshrink

    def find_params(self, x: torch.Tensor, weight: bool = True):
        if not weight:
            raise NotImplementedError("activation quantisation is not part of this path")
        s32, _ = ops.quant_scales(x.float().contiguous(), self.bits, -1, mse=self.mse, norm=self.norm, grid=self.grid,
                                  maxshrink=self.maxshrink)
        self.scale = s32.reshape(-1, 1)                                  # [N, 1], as quant.py:118-121
        self.zero = torch.full_like(self.scale, (self.maxq + 1) / 2)

    def ready(self) -> bool:
        return self.scale is not None


def _inverse_hessian_factor(H: torch.Tensor, W: torch.Tensor, percdamp: float) -> torch.Tensor:
    """sparsegpt.py:69-84, in place on H and W: input columns that never fired get a unit diagonal and
    a zero weight column, the diagonal is raised by percdamp times its mean, and the upper Cholesky
    factor of the inverse comes back (the sweep reads its rows).  The factorisations are torch.linalg
    calls on the device the Hessian lives on."""
    d = torch.diagonal(H)                      # a view: writes go to H
    dead = d == 0
    d[dead] = 1
    W[:, dead] = 0
    d += percdamp * torch.mean(d)
    lower = torch.linalg.cholesky(H)
    hinv = torch.linalg.cholesky(torch.cholesky_inverse(lower), upper=True)
    if bool(torch.isnan(hinv).any()):
        raise ValueError("Hinv contains nan, aborting...")
    return hinv.contiguous()


class SparseGPT:
    def __init__(self, layer: nn.Linear):
        if not isinstance(layer, nn.Linear):
            raise NotImplementedError("only nn.Linear layers are on this path")
        self.layer = layer
        self.dev = layer.weight.device
        self.rows, self.columns = layer.weight.shape
        self.H = torch.zeros((self.columns, self.columns), dtype=torch.float32, device=self.dev)
        self.nsamples = 0
        self._packed_from = None

    def add_batch(self, inp: torch.Tensor, out=None):
        """sparsegpt.py:27-43: one more batch of layer inputs, [B, L, K] or [L, K] (= one sample)."""
        if inp.dim() == 2:
            inp = inp.unsqueeze(0)
        batch = inp.shape[0]
        x = inp.reshape(-1, inp.shape[-1])
        if x.dtype not in (torch.float16, torch.float32):
            x = x.float()
        self.nsamples = ops.hessian_add(self.H, x.contiguous(), self.nsamples, batch)
        if not bool(torch.any(self.H != 0)):
            raise ValueError("sparsity of H == 1, something is off, aborting")

    def fasterprune(self, sparsity, prunen=0, prunem=0, blocksize=128, percdamp=0.01, actorder=False,
                    base_weight: Optional[torch.Tensor] = None):
        """sparsegpt.py:46-197.  Returns (scale, zero, g_idx, avg_loss, W) like the reference and
        leaves `layer.weight` = compressed delta (+ base_weight).  n:m pruning (prunen, prunem) or no
        pruning (sparsity = 0); the reference's unstructured threshold mode and `actorder` are not
        built (the serving format is 2:4)."""
        if actorder:
            raise NotImplementedError("actorder is not built")
        if blocksize != 128:
            raise NotImplementedError("blocksize must be 128")
        if prunen == 0 and sparsity != 0:
            raise NotImplementedError("unstructured sparsity is not built; use prunen=2, prunem=4")
        W = self.layer.weight.data.clone().float()
        if base_weight is not None:
            if base_weight.shape != W.shape:
                raise ValueError("base_weight shape should be the same as W")
            W -= base_weight.float()
        quantizer = getattr(self, "quantizer", None)
        if quantizer is not None and not quantizer.ready():
            quantizer.find_params(W, weight=True)
        hinv = _inverse_hessian_factor(self.H, W, percdamp)
        self.H = None
        W = W.contiguous()
        scale = quantizer.scale.reshape(-1).contiguous() if quantizer is not None else None
        losses = ops.obs_sweep(W, hinv, scale, quantizer.bits if quantizer is not None else 4,
                               prunen, prunem)
        g_idx = torch.zeros(self.columns, dtype=torch.int32, device=self.dev)     # i // columns
        self._packed_from = W
        dtype = self.layer.weight.data.dtype
        Wq = W.to(dtype)
        self.layer.weight.data = (Wq + base_weight.to(dtype)).to(dtype) if base_weight is not None else Wq
        avg_loss = float(torch.sum(losses).item()) / max(self.nsamples, 1)
        if quantizer is not None:
            return quantizer.scale, quantizer.zero, g_idx, avg_loss, Wq
        return [], [], g_idx, avg_loss, Wq

    def pack(self):
        """(qweight, meta, scales16) of the compressed delta in the native serving layout (2:4 only)."""
        quantizer = getattr(self, "quantizer", None)
        if self._packed_from is None or quantizer is None:
            raise ValueError("fasterprune with a quantizer must run first")
        s32 = quantizer.scale.reshape(1, -1).contiguous()
        q, m = ops.pack_2of4(self._packed_from, s32, quantizer.bits, -1)
        return q, m, s32.half()

    def free(self):
        self.H = None
        self._packed_from = None
