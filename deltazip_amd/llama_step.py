"""A Llama-style decoder for one decode step, every projection a multi-delta layer.

This is the harness around the hot path for the "full step" workload: the structure of the
reference's serving model (serving/vllm/model_executor/models/llama.py:58-89 LlamaMLP, :91-172
LlamaAttention, :175-235 LlamaDecoderLayer, :238-290 LlamaModel, :293-339 the delta module tables)
with the fused projections held as plain `torch.nn.Linear` modules, which
`create_delta_manager` (serving/vllm/delta/models.py:450-488, 606-626) replaces by delta layers.
RMSNorm, rotary embedding and attention over the KV context are plain PyTorch ops: they are not
part of the path this library accelerates and are here so that a step has its real shape.

Nothing in the package depends on this module.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F


@dataclass
class LlamaStepConfig:
    hidden_size: int = 4096
    intermediate_size: int = 11008
    num_attention_heads: int = 32
    num_hidden_layers: int = 32
    vocab_size: int = 32000
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    max_position_embeddings: int = 4096


class RMSNorm(nn.Module):
    """x * rsqrt(mean(x^2) + eps) * weight in fp32, with the fused residual add of the reference's
    layer (model_executor/layers/layernorm.py): forward(x, residual) returns (normed(x + residual),
    x + residual)."""

    def __init__(self, hidden_size: int, eps: float, device=None) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=torch.float16, device=device), requires_grad=False)
        self.eps = eps

    def forward(self, x: torch.Tensor, residual: Optional[torch.Tensor] = None):
        if residual is not None:
            x = x + residual
            residual = x
        xf = x.float()
        out = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps)).to(x.dtype) * self.weight
        return out if residual is None else (out, residual)


def _rotate_half(x: torch.Tensor) -> torch.Tensor:
    x1, x2 = x[..., : x.shape[-1] // 2], x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


class LlamaAttention(nn.Module):
    def __init__(self, cfg: LlamaStepConfig, device=None) -> None:
        super().__init__()
        h = cfg.hidden_size
        self.num_heads = cfg.num_attention_heads
        self.head_dim = h // self.num_heads
        self.qkv_proj = nn.Linear(h, 3 * h, bias=False, dtype=torch.float16, device=device)
        self.o_proj = nn.Linear(h, h, bias=False, dtype=torch.float16, device=device)

    def forward(self, hidden: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                kv_cache: Tuple[torch.Tensor, torch.Tensor], context_len: int) -> torch.Tensor:
        B = hidden.shape[0]
        qkv, _ = self.qkv_proj(hidden)
        q, k, v = (t.view(B, self.num_heads, 1, self.head_dim) for t in qkv.chunk(3, dim=-1))
        q = q * cos + _rotate_half(q) * sin
        k = k * cos + _rotate_half(k) * sin
        k_cache, v_cache = kv_cache              # [B, heads, context + 1, head_dim]
        k_cache[:, :, context_len] = k[:, :, 0]
        v_cache[:, :, context_len] = v[:, :, 0]
        out = F.scaled_dot_product_attention(q, k_cache[:, :, : context_len + 1], v_cache[:, :, : context_len + 1])
        out, _ = self.o_proj(out.reshape(B, -1))
        return out


class LlamaMLP(nn.Module):
    def __init__(self, cfg: LlamaStepConfig, device=None) -> None:
        super().__init__()
        self.gate_up_proj = nn.Linear(cfg.hidden_size, 2 * cfg.intermediate_size, bias=False, dtype=torch.float16,
                                      device=device)
        self.down_proj = nn.Linear(cfg.intermediate_size, cfg.hidden_size, bias=False, dtype=torch.float16,
                                   device=device)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        gate_up, _ = self.gate_up_proj(x)
        gate, up = gate_up.chunk(2, dim=-1)
        x, _ = self.down_proj(F.silu(gate) * up)
        return x


class LlamaDecoderLayer(nn.Module):
    def __init__(self, cfg: LlamaStepConfig, device=None) -> None:
        super().__init__()
        self.self_attn = LlamaAttention(cfg, device)
        self.mlp = LlamaMLP(cfg, device)
        self.input_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps, device)
        self.post_attention_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps, device)

    def forward(self, hidden, residual, cos, sin, kv_cache, context_len):
        if residual is None:
            residual = hidden
            hidden = self.input_layernorm(hidden)
        else:
            hidden, residual = self.input_layernorm(hidden, residual)
        hidden = self.self_attn(hidden, cos, sin, kv_cache, context_len)
        hidden, residual = self.post_attention_layernorm(hidden, residual)
        hidden = self.mlp(hidden)
        return hidden, residual


class _Layers(nn.Module):
    def __init__(self, cfg: LlamaStepConfig, device=None) -> None:
        super().__init__()
        self.embed_tokens = nn.Embedding(cfg.vocab_size, cfg.hidden_size, dtype=torch.float16, device=device)
        self.layers = nn.ModuleList([LlamaDecoderLayer(cfg, device) for _ in range(cfg.num_hidden_layers)])
        self.norm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps, device)


class _LogitsProcessor(nn.Module):
    """What the delta wrapper of the output projection needs of the serving engine's LogitsProcessor
    (model_executor/layers/logits_processor.py): the vocabulary size and `_get_logits`."""

    def __init__(self, vocab_size: int) -> None:
        super().__init__()
        self.vocab_size = vocab_size

    def _get_logits(self, hidden_states, embedding, embedding_bias=None):
        return hidden_states @ embedding.t()


class LlamaForDecodeStep(nn.Module):
    """The decoder with the module tables the delta manager looks for (llama.py:299-339).  The
    projections are created as `nn.Linear`; after `create_delta_manager(model, ...)` they are delta
    layers whose forward returns (output, bias) like the reference's parallel linears, which is what
    the blocks above expect -- the model runs only once the manager has wrapped them.  The output
    projection and the embedding stay on their base tables unless `vocab_deltas` is set (then
    they, too, are registered for per-delta tables)."""
    packed_modules_mapping = {"qkv_proj": ["q_proj", "k_proj", "v_proj"], "gate_up_proj": ["gate_proj", "up_proj"]}
    embedding_modules = {"embed_tokens": "input_embeddings", "lm_head": "output_embeddings"}

    def __init__(self, cfg: LlamaStepConfig, vocab_deltas: bool = False, device=None,
                 generator: Optional[torch.Generator] = None) -> None:
        super().__init__()
        self.config = cfg
        self.model = _Layers(cfg, device)
        self.lm_head = nn.Linear(cfg.hidden_size, cfg.vocab_size, bias=False, dtype=torch.float16, device=device)
        self.logits_processor = _LogitsProcessor(cfg.vocab_size)
        for p in self.parameters():
            p.requires_grad_(False)
        with torch.no_grad():   # random initialisation: weights N(0, 0.02), norm weights near 1
            for name, p in self.named_parameters():
                if p.dim() == 2:
                    p.normal_(0.0, 0.02, generator=generator)
                else:
                    p.copy_(1.0 + 0.1 * torch.randn(p.shape, device=p.device, generator=generator))
        self.supported_delta_modules = ["qkv_proj", "o_proj", "gate_up_proj", "down_proj"]
        if vocab_deltas:
            self.supported_delta_modules += ["embed_tokens", "lm_head"]
        hd = cfg.hidden_size // cfg.num_attention_heads
        inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, hd, 2, device=device).float() / hd))
        self.register_buffer("inv_freq", inv, persistent=False)

    def projections(self) -> List[Tuple[str, nn.Module]]:
        """(name, module) of every projection, in execution order."""
        out = []
        for i, layer in enumerate(self.model.layers):
            p = f"model.layers.{i}."
            out += [(p + "self_attn.qkv_proj", layer.self_attn.qkv_proj), (p + "self_attn.o_proj", layer.self_attn.o_proj),
                    (p + "mlp.gate_up_proj", layer.mlp.gate_up_proj), (p + "mlp.down_proj", layer.mlp.down_proj)]
        return out

    def make_kv_cache(self, batch: int, context_len: int, device, fill: float = 0.02):
        """Per layer (k, v) of [batch, heads, context_len + 1, head_dim]; the first context_len
        positions hold random history, the last one is written by the step."""
        cfg = self.config
        hd = cfg.hidden_size // cfg.num_attention_heads
        shape = (batch, cfg.num_attention_heads, context_len + 1, hd)
        return [(torch.randn(shape, device=device, dtype=torch.float16) * fill,
                 torch.randn(shape, device=device, dtype=torch.float16) * fill) for _ in range(cfg.num_hidden_layers)]

    @torch.no_grad()
    def decode_step(self, input_ids: torch.Tensor, kv_caches, context_len: int,
                    sample_rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """One decode step of `input_ids.numel()` sequences that all stand at position context_len:
        returns the logits [rows, vocab] of `sample_rows` (default: every sequence)."""
        cfg = self.config
        hd = cfg.hidden_size // cfg.num_attention_heads
        emb = self.model.embed_tokens(input_ids.view(-1))
        hidden = emb if not isinstance(emb, tuple) else emb[0]
        ang = context_len * self.inv_freq
        ang = torch.cat((ang, ang)).view(1, 1, 1, hd)
        cos, sin = ang.cos().to(hidden.dtype), ang.sin().to(hidden.dtype)
        residual = None
        for layer, kv in zip(self.model.layers, kv_caches):
            hidden, residual = layer(hidden, residual, cos, sin, kv, context_len)
        hidden, _ = self.model.norm(hidden, residual)
        if sample_rows is not None:
            hidden = hidden.index_select(0, sample_rows)
        return self.logits_processor._get_logits(hidden, self.lm_head.weight)
