"""Layer-by-layer compression of a fine-tuned model's delta with calibration data.

Mirrors `BaseDeltaZipModelForCausalLM.lossy_compress` (deltazip/modeling/_base.py:261-576): the
inputs of the first decoder layer are recorded by running the calibration examples through the
model with that layer replaced by a recorder that stops the forward pass; then, layer by layer
and -- with `true_sequential` -- group of projections by group, forward hooks collect each
projection's inputs into its Hessian (SparseGPT.add_batch), the projection's delta against the
base model goes through the Hessian-weighted 2:4 sweep (SparseGPT.fasterprune, which leaves the
projection holding base + compressed delta), and once a layer is done its outputs, computed with
the compressed projections, become the next layer's inputs.  So every Hessian sees the
activations the compressed model will produce, not those of the fine-tuned one.

The model is any torch module of the usual decoder shape: `layers` is its list of decoder layers,
each called as `layer(hidden_states, **kwargs)` and returning a tuple whose first entry is the new
hidden states; the projections are `nn.Linear` modules found by name inside a layer.  Hessian
accumulation, the sweep and the packing run in the HIP kernels behind `SparseGPT`.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn

from .checkpoint import PACK_MODULES, UNCOMPRESSED_MODULES, CompressionConfig, _emit_state_dict
from .sparsegpt import Quantizer, SparseGPT

# the groups of a llama-style layer, in execution order (deltazip/modeling/llama.py:9-14)
LLAMA_INSIDE_LAYER_MODULES: List[List[str]] = [
    ["self_attn.k_proj", "self_attn.v_proj", "self_attn.q_proj"],
    ["self_attn.o_proj"],
    ["mlp.up_proj", "mlp.gate_proj"],
    ["mlp.down_proj"],
]


class _StopForward(Exception):
    pass


class _LayerRecorder(nn.Module):
    """Stands in for the first decoder layer: keeps what it is called with and stops the pass
    (LayerHijacker, _base.py:290-331)."""

    def __init__(self, module: nn.Module, inputs: list, kwargs_list: list):
        super().__init__()
        self.module = module
        self._inputs, self._kwargs = inputs, kwargs_list

    def forward(self, inp=None, **kwargs):
        if inp is None:
            inp = kwargs.pop("hidden_states")
        else:
            kwargs.pop("hidden_states", None)
        self._inputs.append(inp)
        self._kwargs.append(kwargs)
        raise _StopForward


def _get(module: nn.Module, name: str) -> nn.Module:
    for part in name.split("."):
        module = getattr(module, part)
    return module


@torch.inference_mode()
def lossy_compress(model: nn.Module, examples: Sequence[Dict[str, torch.Tensor]], compress_config: CompressionConfig,
                   base_model: Optional[nn.Module] = None, layers_block_name: str = "model.layers",
                   inside_layer_modules: Optional[List[List[str]]] = None, layout: str = "native",
                   pack_modules: Optional[Dict[str, Tuple[str, int]]] = None) -> Dict[str, torch.Tensor]:
    """Compresses `model` (the fine-tuned model, on the GPU) against `base_model` in place -- on
    return every compressed projection holds base + compressed delta, as the reference leaves it
    (_base.py:536-571) -- and returns the state dict `compress_model` would: serving layout
    (layout="native") or the reference's checkpoint format (layout="gptq").  Without a base model
    the weights themselves are compressed.  `examples`: keyword arguments of `model(**example)`,
    one calibration batch each."""
    cfg = compress_config
    if cfg.bits not in (2, 4):
        raise NotImplementedError("Only 2 and 4 bits are supported.")
    if not (cfg.prunen == 2 and cfg.prunem == 4):
        raise NotImplementedError("only 2:4 pruning (prunen=2, prunem=4) is supported")
    if cfg.group_size != -1:
        raise NotImplementedError("the Hessian-weighted sweep uses per-channel scales (group_size -1)")
    if layout not in ("native", "gptq"):
        raise ValueError("layout must be 'native' or 'gptq'")
    groups = LLAMA_INSIDE_LAYER_MODULES if inside_layer_modules is None else inside_layer_modules
    if not cfg.true_sequential:
        groups = [sum(groups, [])]
    layers = _get(model, layers_block_name)
    base_sd = base_model.state_dict() if base_model is not None else None

    # inputs of the first layer
    layer_inputs: List[torch.Tensor] = []
    layer_kwargs: List[dict] = []
    first = layers[0]
    layers[0] = _LayerRecorder(first, layer_inputs, layer_kwargs)
    try:
        for example in examples:
            try:
                model(**example)
            except _StopForward:
                pass
    finally:
        layers[0] = first
    if not layer_inputs:
        raise ValueError("no calibration example reached the first decoder layer")

    native: Dict[str, Tuple[torch.Tensor, torch.Tensor, torch.Tensor, int]] = {}
    for i, layer in enumerate(layers):
        for names in groups:
            subset = {n: _get(layer, n) for n in names}
            gpts: Dict[str, SparseGPT] = {}
            handles = []
            for n, lin in subset.items():
                g = SparseGPT(lin)
                g.quantizer = Quantizer()
                g.quantizer.configure(cfg.bits, perchannel=True, sym=cfg.sym, mse=False)
                gpts[n] = g
                handles.append(lin.register_forward_hook(
                    lambda _m, inp, _out, g=g: g.add_batch(inp[0].data, None)))
            try:
                for x, kw in zip(layer_inputs, layer_kwargs):
                    layer(x, **kw)
            finally:
                for h in handles:
                    h.remove()
            for n, g in gpts.items():
                key = f"{layers_block_name}.{i}.{n}"
                base_w = base_sd[key + ".weight"].to(g.dev) if base_sd is not None else None
                g.fasterprune(cfg.sparsity, prunen=cfg.prunen, prunem=cfg.prunem, percdamp=cfg.damp_percent,
                              blocksize=cfg.block_size, actorder=cfg.desc_act, base_weight=base_w)
                q, m, s = g.pack()
                native[key] = (q.cpu(), m.cpu(), s.cpu(), g.columns)
                g.free()
        # the next layer sees what the compressed layer produces
        layer_inputs = [layer(x, **kw)[0] for x, kw in zip(layer_inputs, layer_kwargs)]

    out: Dict[str, torch.Tensor] = {}
    for key, w in model.state_dict().items():
        if key.endswith(".weight") and any(u in key for u in UNCOMPRESSED_MODULES):
            out[key if layout == "gptq" else key[: -len(".weight")] + ".0.weight"] = w.detach().cpu()
    return _emit_state_dict(native, out, layout, PACK_MODULES if pack_modules is None else pack_modules,
                            cfg.bits, cfg.group_size)
