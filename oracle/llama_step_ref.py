"""CPU restatement of one decoder layer of the decode-step harness.  TEST INFRASTRUCTURE ONLY.

Follows the reference's serving model (serving/vllm/model_executor/models/llama.py:78-89 MLP,
:160-172 attention, :211-235 decoder layer; layernorm with fused residual add,
model_executor/layers/layernorm.py) with every projection computed by the layer oracle
(`dz_oracle.forward_ref`: W_base + delta of the token's id in fp32, one dense product per id) and
rounded to fp16 where the GPU layers hand over fp16 tensors.  Elementwise steps run as torch CPU
fp16 ops (computed in fp32, rounded once per op, like their GPU counterparts); reductions and the
attention run in fp32.  Checked by tests/test_llama_step.py against closed forms (a layer whose
projections are zero returns its residual; attention over a constant value cache returns that
value) before it is used as the checker.
"""
from __future__ import annotations

import numpy as np
import torch

from . import dz_oracle as o


def rms_norm(x16: torch.Tensor, weight16: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x16.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).half() * weight16


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def project(x16: torch.Tensor, w_base16: torch.Tensor, deltas_t, ids: np.ndarray) -> torch.Tensor:
    """fp16 [T, N]: the multi-delta layer's definition in fp32, rounded once."""
    y = o.forward_ref(x16.detach().numpy(), w_base16.detach().numpy(), deltas_t, ids)
    return torch.from_numpy(y).half()


def decoder_layer(hidden16, residual16, w, deltas, ids, k_cache16, v_cache16, context_len, num_heads, eps,
                  rope_theta=10000.0):
    """hidden16 [B, H] fp16, residual16 [B, H] fp16 or None.  w: dict with 'qkv', 'o', 'gate_up',
    'down' ([N, K] fp16 tensors), 'ln1', 'ln2' ([H] fp16).  deltas: dict with the same four
    projection names -> list over slots of delta^T [K, N] fp16 numpy arrays.  ids [B]: slot per row,
    -1 = base only.  k_cache16 / v_cache16 [B, heads, context_len + 1, head_dim] fp16; position
    context_len is filled in here (on copies).  Returns (hidden_out, residual_out) fp16."""
    B, H = hidden16.shape
    hd = H // num_heads
    if residual16 is None:
        residual16 = hidden16
        x = rms_norm(hidden16, w["ln1"], eps)
    else:
        residual16 = hidden16 + residual16
        x = rms_norm(residual16, w["ln1"], eps)
    qkv = project(x, w["qkv"], deltas["qkv"], ids)
    q, k, v = (t.reshape(B, num_heads, 1, hd) for t in qkv.chunk(3, dim=-1))
    inv = 1.0 / (rope_theta ** (torch.arange(0, hd, 2).float() / hd))
    ang = context_len * inv
    ang = torch.cat((ang, ang)).view(1, 1, 1, hd)
    cos, sin = ang.cos().half(), ang.sin().half()
    q = q * cos + rotate_half(q) * sin
    k = k * cos + rotate_half(k) * sin
    kc, vc = k_cache16.clone(), v_cache16.clone()
    kc[:, :, context_len] = k[:, :, 0]
    vc[:, :, context_len] = v[:, :, 0]
    scores = torch.matmul(q.float(), kc.float().transpose(-1, -2)) / np.sqrt(hd)     # [B, heads, 1, ctx + 1]
    attn = torch.matmul(torch.softmax(scores, dim=-1), vc.float()).half().reshape(B, H)
    out = project(attn, w["o"], deltas["o"], ids)
    residual16 = out + residual16
    x = rms_norm(residual16, w["ln2"], eps)
    gate_up = project(x, w["gate_up"], deltas["gate_up"], ids)
    gate, up = gate_up.chunk(2, dim=-1)
    act = torch.nn.functional.silu(gate.float()).half() * up
    return project(act, w["down"], deltas["down"], ids), residual16
