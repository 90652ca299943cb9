"""The reference's CPU-runnable forward, restated with torch CPU ops.  TEST INFRASTRUCTURE ONLY.

Used by the benchmark's CPU-baseline leg; tests/test_cpu_path.py holds it to the numpy oracle
(dequant_torch == dequant_gptq bit for bit, forward_cpu == forward_ref):
  * unpack + dequantise exactly as QuantLinear.forward does
    (serving/vllm/delta/quant_linears/quant_linear_naive.py:39-67): bitwise_right_shift by the
    per-position shifts, mask, zeros + 1, scales[g_idx] * (weight - zeros[g_idx]) in fp16;
  * W = W_base + delta in fp32 (deltazip/utils/generate.py:9-20, at fp32);
  * tokens grouped by id, one dense product per id (deltazip_marlin.py:44-53).
Nothing in the shipped package imports this module.
"""
from __future__ import annotations

import torch


def dequant_torch(qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor,
                  g_idx: torch.Tensor, bits: int) -> torch.Tensor:
    """delta^T [K, N] fp16; line-by-line restatement of quant_linear_naive.py:39-67."""
    wf = torch.tensor(list(range(0, 32, bits)), dtype=torch.int32).unsqueeze(0)
    zeros = torch.bitwise_right_shift(torch.unsqueeze(qzeros, 2).expand(-1, -1, 32 // bits),
                                      wf.unsqueeze(0)).to(torch.int8)
    torch.bitwise_and(zeros, (2 ** bits) - 1, out=zeros)
    zeros = zeros + 1
    zeros = zeros.reshape(scales.shape)
    weight = torch.bitwise_right_shift(torch.unsqueeze(qweight, 1).expand(-1, 32 // bits, -1),
                                       wf.unsqueeze(-1)).to(torch.int8)
    torch.bitwise_and(weight, (2 ** bits) - 1, out=weight)
    weight = weight.reshape(weight.shape[0] * weight.shape[1], weight.shape[2])
    return scales[g_idx.long()] * (weight - zeros[g_idx.long()])


def forward_cpu(x16: torch.Tensor, w_base16: torch.Tensor, deltas, ids: torch.Tensor, bits: int,
                predequantised=None) -> torch.Tensor:
    """fp32 [T, N].  `deltas[d]` = (qweight, qzeros, scales, g_idx).  With `predequantised`
    (list of delta^T fp16) the dequantisation is skipped: the matmul-only lower bound."""
    t = x16.shape[0]
    n = w_base16.shape[0]
    y = torch.zeros((t, n), dtype=torch.float32)
    xf = x16.float()
    wb = w_base16.float()
    for d in torch.unique(ids).tolist():
        sel = (ids == d).nonzero().flatten()
        if d >= 0:
            dt = predequantised[d] if predequantised is not None else dequant_torch(*deltas[d], bits)
            w = wb + dt.t().float()
        else:
            w = wb
        y[sel] = xf[sel] @ w.t()
    return y
