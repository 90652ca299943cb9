"""QuantLinear: a single compressed delta as a linear layer.

Keeps the interface of the reference's QuantLinear
(serving/vllm/delta/quant_linears/quant_linear_naive.py:8-96 of eth-easl/deltazip):
`from_tensors(bitwidth, qweight, qzeros, scales, g_idx, bias, device_tensor)` takes the GPTQ-style
tensors that QuantLinear.pack writes (deltazip/nn_modules/qlinear_cuda.py:144-244) and
`forward(x)` returns x @ dequant(W) (+ bias) in fp16.  The tensors are converted once to the
native gfx950 layout; the product runs in the fused HIP kernel (delta-only form).
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from . import ops


class QuantLinear(nn.Module):
    def __init__(self, bits: int, infeatures: int, outfeatures: int, bias):
        super().__init__()
        if bits not in [2, 4]:
            # the reference accepts 2, 3, 4, 8 here and fails later for 3 (quant_linear_naive.py:60)
            raise NotImplementedError("Only 2 and 4 bits are supported.")
        self.infeatures = infeatures
        self.outfeatures = outfeatures
        self.bits = bits
        self.group_size = infeatures
        self.maxq = 2 ** self.bits - 1
        self.qweight = None
        self.qzeros = None
        self.scales = None
        self.g_idx = None
        self.bias = bias
        self._native = None      # (qweight, meta, scales) stacked with one slot, on the GPU
        self._zero_ids = None

    def _prepare(self, device: torch.device) -> None:
        q, m, s = ops.repack_gptq_to_native(self.qweight, self.qzeros, self.scales, self.g_idx, self.bits)
        self._native = (q.unsqueeze(0).to(device), m.unsqueeze(0).to(device), s.unsqueeze(0).to(device))
        self.group_size = self.infeatures // s.shape[0]

    def unpack(self) -> torch.Tensor:
        """fp16 [outfeatures, infeatures] weight, bit-exact with the reference's unpack
        (deltazip/nn_modules/qlinear_cuda.py:246-329)."""
        device = self.qweight.device if self.qweight.is_cuda else torch.device("cuda")
        if self._native is None:
            self._prepare(device)
        q, m, s = self._native
        return ops.dequant(q[0], m[0], s[0], self.infeatures, self.outfeatures, self.bits)

    @torch.inference_mode()
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        out_shape = x.shape[:-1] + (self.outfeatures,)
        x2 = x.reshape(-1, x.shape[-1]).half()
        if self._native is None:
            self._prepare(x2.device)
        q, m, s = self._native
        T = x2.shape[0]
        if self._zero_ids is None or self._zero_ids.numel() < T or self._zero_ids.device != x2.device:
            self._zero_ids = torch.zeros(max(T, 128), dtype=torch.int64, device=x2.device)
        out = ops.multi_delta_linear(x2, None, q, s, m, self._zero_ids[:T], bits=self.bits)
        out = out.reshape(out_shape)
        out = out + self.bias if self.bias is not None else out
        return out

    @classmethod
    def from_tensors(cls, bitwidth, qweight, qzeros, scales, g_idx, bias, device_tensor=None):
        infeatures = qweight.shape[0] * 32 // bitwidth
        outfeatures = qweight.shape[1]
        obj = cls(bitwidth, infeatures, outfeatures, bias)
        obj.qweight = qweight
        obj.qzeros = qzeros.to(qweight.device)
        obj.scales = scales.to(qweight.device)
        obj.g_idx = g_idx.to(qweight.device) if g_idx is not None else None
        return obj
