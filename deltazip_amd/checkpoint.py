"""Reading compressed-delta checkpoints and converting them to the native layout.

Mirrors, for eth-easl/deltazip,
  deltazip/modeling/_base.py:596-645        what `save_compressed` writes: one file
                                            `deltazip-compressed.safetensors` whose keys are
                                            `{module}.qweight/.qzeros/.scales/.g_idx` (GPTQ-style,
                                            nn_modules/qlinear_cuda.py:144-244) plus the uncompressed
                                            parameters, and `compress_config.json`
  serving/vllm/delta/config.py:21-75        CompressionConfig (the JSON's fields)
  deltazip/utils/converter.py:13-101        convert_model: fuse q/k/v and gate/up along the output
                                            dimension, emit `{module}.{tp_rank}.qweight/.scales/.meta`
                                            and `{module}.{tp_rank}.weight`
  serving/vllm/delta/delta.py:6-35          DeltaLayerWeights
  serving/vllm/delta/models.py:155-264      DeltaModel, DeltaModel.from_checkpoint

The reference's converter dequantises every module and re-encodes it with a third-party packer.
Here the stored codes are kept as they are: the native layout orders words by blocks of 32 output
rows first, so fusing projections along the output dimension is a concatenation of their native
buffers, and the fused delta dequantises to exactly the values the separate ones did.

All of this is host work (CPU tensors in, CPU tensors out); the 2:4 / zero-point checks of the
repacker run on every module, so a checkpoint that is not 2:4 sparse and symmetric is refused.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, fields
from fractions import Fraction
from typing import Dict, Iterable, List, Optional, Tuple

import torch

from . import ops

CHECKPOINT_NAME = "deltazip-compressed.safetensors"
CONFIG_NAME = "compress_config.json"
# safetensors metadata entry that marks a serving-layout file as holding this library's bit layout
LAYOUT_KEY = "dz_layout"
NATIVE_LAYOUT = "native-gfx950-v1"

# sub-module -> (fused module, position inside it); llama-style naming, the same table the
# serving model declares as `packed_modules_mapping` (model_executor/models/llama.py:299-309)
PACK_MODULES: Dict[str, Tuple[str, int]] = {
    "self_attn.q_proj": ("self_attn.qkv_proj", 0),
    "self_attn.k_proj": ("self_attn.qkv_proj", 1),
    "self_attn.v_proj": ("self_attn.qkv_proj", 2),
    "mlp.gate_proj": ("mlp.gate_up_proj", 0),
    "mlp.up_proj": ("mlp.gate_up_proj", 1),
}
# parameters that stay uncompressed in a delta checkpoint (delta/models.py:207-213)
UNCOMPRESSED_MODULES = ("lm_head", "model.embed_tokens", "model.norm", "input_layernorm",
                        "post_attention_layernorm")


@dataclass
class CompressionConfig:
    """The fields of compress_config.json (serving/vllm/delta/config.py:21-75)."""
    bits: int = field(default=4, metadata={"choices": [2, 3, 4, 8, 16]})
    sparsity: float = 0.0
    prunen: int = 0
    prunem: int = 0
    group_size: int = -1
    group_rows: int = -1
    block_size: int = 128
    damp_percent: float = 0.01
    desc_act: bool = False
    sym: bool = True
    true_sequential: bool = True
    lossless: str = "none"
    dtype: str = "fp16"

    def __post_init__(self):
        if self.sparsity < 0 or self.sparsity > 1:
            raise ValueError("sparsity must be [0, 1]")
        if self.bits not in fields(self)[0].metadata["choices"]:
            raise ValueError(f"only support quantize to {fields(self)[0].metadata['choices']} bits.")
        if self.group_size != -1 and self.group_size <= 0:
            raise ValueError("unless equal to -1, group_size must greater then 0.")
        if not (0 < self.damp_percent < 1):
            raise ValueError("damp_percent must between 0 and 1.")
        self.pack_factor = Fraction(32, self.bits)

    def to_dict(self) -> dict:
        keys = ("bits", "group_size", "sparsity", "damp_percent", "desc_act", "sym", "true_sequential",
                "lossless", "prunen", "prunem", "block_size")
        return {k: getattr(self, k) for k in keys}

    def save_pretrained(self, save_dir: str, **kwargs) -> None:
        with open(os.path.join(save_dir, CONFIG_NAME), "w", encoding="utf-8") as f:
            json.dump(self.to_dict(), f, indent=2)

    @classmethod
    def from_pretrained(cls, save_dir: str) -> "CompressionConfig":
        with open(os.path.join(save_dir, CONFIG_NAME), "r", encoding="utf-8") as f:
            return cls(**json.load(f))


class DeltaLayerWeights:
    """Delta of one layer: either a native-layout compressed triple (qweight, scales, meta) or an
    uncompressed `weight` (serving/vllm/delta/delta.py:6-35)."""

    def __init__(self, module_name: str, qweight: Optional[torch.Tensor] = None,
                 qzeros: Optional[torch.Tensor] = None, scales: Optional[torch.Tensor] = None,
                 g_idx: Optional[torch.Tensor] = None, meta: Optional[torch.Tensor] = None,
                 compress_config: Optional[CompressionConfig] = None,
                 weight: Optional[torch.Tensor] = None) -> None:
        if weight is not None:
            self._compressed = False
            assert qweight is None, "qweight should be None if weight is provided"
        else:
            self._compressed = True
            assert qweight is not None, "qweight should not be None if weight is not provided"
        self.module_name = module_name
        self.config = compress_config
        self.qweight, self.qzeros, self.scales, self.g_idx, self.meta = qweight, qzeros, scales, g_idx, meta
        self.weight = weight

    def tensors(self) -> Iterable[torch.Tensor]:
        return [t for t in (self.qweight, self.qzeros, self.scales, self.g_idx, self.meta, self.weight)
                if t is not None]


def _fuse_native(parts: List[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]], K: int, bits: int,
                 group_size: int):
    """Concatenate native-layout deltas of the same K along the output dimension."""
    n_total = sum(s.shape[1] for _, _, s in parts)
    qs, ms, ss = ops.stacked_shapes(K, n_total, bits, group_size)
    q = torch.cat([p[0].reshape(-1) for p in parts]).view(qs)
    m = torch.cat([p[1].reshape(-1) for p in parts]).view(ms)
    s = torch.cat([p[2] for p in parts], dim=1).contiguous()
    assert tuple(s.shape) == tuple(ss)
    return q, m, s


@torch.no_grad()
def convert_model(tensors: Dict[str, torch.Tensor], bits: Optional[int] = None, verbose: bool = False,
                  pack_modules: Optional[Dict[str, Tuple[str, int]]] = None) -> Dict[str, torch.Tensor]:
    """GPTQ-style state dict of a compressed delta -> serving-layout state dict (tensor-parallel
    rank 0 of 1), the job of deltazip/utils/converter.py:13-101.

    Output keys: `{module}.0.qweight`, `{module}.0.scales`, `{module}.0.meta` for every compressed
    linear layer (q/k/v fused into `qkv_proj`, gate/up into `gate_up_proj`, in that order) and
    `{module}.0.weight` for every uncompressed parameter named in UNCOMPRESSED_MODULES.
    `bits` is needed when it cannot be read off the shapes (pass the checkpoint's config value)."""
    pack_modules = PACK_MODULES if pack_modules is None else pack_modules
    new_tensors: Dict[str, torch.Tensor] = {}
    remaining = list(tensors.keys())
    quantized = [k[: -len(".qweight")] for k in tensors if k.endswith(".qweight")]
    native: Dict[str, Tuple[torch.Tensor, torch.Tensor, torch.Tensor, int, int]] = {}
    for module in quantized:
        qweight, qzeros, scales = (tensors[module + s] for s in (".qweight", ".qzeros", ".scales"))
        g_idx = tensors.get(module + ".g_idx")
        b = bits if bits is not None else _bits_from_gptq(qweight, qzeros)
        q, m, s = ops.repack_gptq_to_native(qweight, qzeros, scales, g_idx, b)
        K = qweight.shape[0] * (32 // b)
        G = scales.shape[0]
        native[module] = (q, m, s, K, -1 if G == 1 else K // G)
        for suffix in (".qweight", ".qzeros", ".scales", ".g_idx"):
            if module + suffix in tensors:
                remaining.remove(module + suffix)
        if verbose:
            print(f"converted {module}: K={K} N={scales.shape[1]} bits={b}")
    plan: Dict[str, List[Tuple[int, str]]] = {}
    for module in quantized:
        hit = next((k for k in pack_modules if module.endswith("." + k) or module == k), None)
        if hit is None:
            q, m, s, _, _ = native[module]
            new_tensors[module + ".0.qweight"], new_tensors[module + ".0.meta"] = q, m
            new_tensors[module + ".0.scales"] = s
            continue
        target, pos = pack_modules[hit]
        plan.setdefault(module[: len(module) - len(hit)] + target, []).append((pos, module))
    for target, members in plan.items():
        members.sort()
        if [p for p, _ in members] != list(range(len(members))):
            raise ValueError(f"{target}: fused module has missing parts {[m for _, m in members]}")
        Ks = {native[m][3] for _, m in members}
        gss = {native[m][4] for _, m in members}
        if len(Ks) != 1 or len(gss) != 1:
            raise ValueError(f"{target}: parts disagree on in_features or group size")
        b = bits if bits is not None else _bits_from_gptq(tensors[members[0][1] + ".qweight"],
                                                          tensors[members[0][1] + ".qzeros"])
        q, m, s = _fuse_native([native[mod][:3] for _, mod in members], Ks.pop(), b, gss.pop())
        new_tensors[target + ".0.qweight"], new_tensors[target + ".0.meta"] = q, m
        new_tensors[target + ".0.scales"] = s
    for key in remaining:
        if key.endswith(".weight") and any(u in key for u in UNCOMPRESSED_MODULES):
            new_tensors[key[: -len(".weight")] + ".0.weight"] = tensors[key]
    return new_tensors


def _bits_from_gptq(qweight: torch.Tensor, qzeros: torch.Tensor) -> int:
    """qzeros is [G, N / pf] and qweight [K / pf, N]: N / (N / pf) gives the pack factor."""
    pf = qweight.shape[1] // qzeros.shape[1]
    if pf * qzeros.shape[1] != qweight.shape[1] or pf not in (8, 16):
        raise NotImplementedError("Only 2 and 4 bits are supported.")
    return 32 // pf


class DeltaModel:
    """A delta model compressed from a fine-tuned variant (serving/vllm/delta/models.py:155-264):
    module name -> DeltaLayerWeights, host tensors (pinned when a GPU is present, so the copies
    `set_delta` issues are asynchronous)."""

    def __init__(self, delta_model_id: int, bitwidth: int, deltas: Dict[str, DeltaLayerWeights]):
        self.id = delta_model_id
        self.deltas = deltas
        self.bitwidth = bitwidth

    def get_delta(self, module_name: str) -> Optional[DeltaLayerWeights]:
        return self.deltas.get(module_name, None)

    @classmethod
    def from_tensors(cls, tensors: Dict[str, torch.Tensor], id: int, compress_config: CompressionConfig,
                     pin_memory: Optional[bool] = None, layout: Optional[str] = None) -> "DeltaModel":
        """From a state dict in either layout: GPTQ-style keys (`*.qzeros` present) are converted
        first; serving-layout keys (`{module}.0.qweight/.scales/.meta`) are taken as they are, but only
        when `layout` says that their bits are this library's (`NATIVE_LAYOUT`).  The reference's own
        `save_compressed` writes its third-party kernel's (Marlin-style) bit layout under the same
        file name, key names and shapes (deltazip/modeling/_base.py:636-641,
        serving/vllm/delta/models.py:236-244): such tensors cannot be told apart by looking at them
        and would decode to wrong weights, so they are refused."""
        if compress_config.lossless != "none":
            raise NotImplementedError("losslessly packed checkpoints are not supported")
        if compress_config.bits not in (2, 4):
            raise NotImplementedError("Only 2 and 4 bits are supported.")
        if any(k.endswith(".qzeros") for k in tensors):
            tensors = convert_model(tensors, bits=compress_config.bits)
        elif any(k.endswith(".0.qweight") for k in tensors) and layout != NATIVE_LAYOUT:
            raise ValueError(
                "serving-layout tensors ({module}.0.qweight/.scales/.meta) without the layout mark "
                f"{LAYOUT_KEY}={NATIVE_LAYOUT}: a file written by the reference's save_compressed holds "
                "Marlin-layout bits under the same names and shapes, which this library cannot read. "
                "Load the GPTQ-style checkpoint ({module}.qweight/.qzeros/.scales/.g_idx) instead, or pass "
                f"layout='{NATIVE_LAYOUT}' for tensors that convert_model / compress_model of this library made.")
        pin = torch.cuda.is_available() if pin_memory is None else pin_memory

        def host(t: torch.Tensor) -> torch.Tensor:
            t = t.contiguous()
            return t.pin_memory() if pin else t

        modules: Dict[str, DeltaLayerWeights] = {}
        names = {k.rsplit(".", 2)[0] for k in tensors}
        for module in sorted(names):
            if f"{module}.0.qweight" in tensors:
                modules[module] = DeltaLayerWeights(
                    module_name=module, qweight=host(tensors[f"{module}.0.qweight"]),
                    scales=host(tensors[f"{module}.0.scales"]), meta=host(tensors[f"{module}.0.meta"]),
                    compress_config=compress_config)
            elif f"{module}.0.weight" in tensors:
                modules[module] = DeltaLayerWeights(module_name=module, weight=host(tensors[f"{module}.0.weight"]))
        return cls(id, compress_config.bits, modules)

    @classmethod
    def from_checkpoint(cls, path_or_name: str, id: int, device: Optional[int] = None,
                        pin_memory: Optional[bool] = None, layout: Optional[str] = None) -> "DeltaModel":
        """Read `deltazip-compressed.safetensors` + `compress_config.json` from a directory.  The
        layout of serving-layout tensors is taken from the file's metadata (`save_converted` marks
        its files) unless `layout` is given."""
        from safetensors import safe_open
        compress_config = CompressionConfig.from_pretrained(path_or_name)
        tensors: Dict[str, torch.Tensor] = {}
        with safe_open(os.path.join(path_or_name, CHECKPOINT_NAME), "pt") as f:
            if layout is None:
                layout = (f.metadata() or {}).get(LAYOUT_KEY)
            for key in f.keys():
                tensors[key] = f.get_tensor(key)
        return cls.from_tensors(tensors, id, compress_config, pin_memory, layout=layout)


def save_converted(tensors: Dict[str, torch.Tensor], compress_config: CompressionConfig, save_dir: str) -> None:
    """Write a serving-layout state dict the way the reference's `save_compressed` does after
    converting (deltazip/modeling/_base.py:636-645), with the metadata entry that tells
    `from_checkpoint` that the bits are in this library's layout."""
    from safetensors.torch import save_file
    os.makedirs(save_dir, exist_ok=True)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(save_dir, CHECKPOINT_NAME),
              metadata={LAYOUT_KEY: NATIVE_LAYOUT})
    compress_config.save_pretrained(save_dir)


def save_compressed(tensors: Dict[str, torch.Tensor], compress_config: CompressionConfig, save_dir: str) -> None:
    """Write a GPTQ-style state dict (`compress_model(..., layout="gptq")`) as the reference's
    `save_compressed` writes an unconverted delta (deltazip/modeling/_base.py:597-648): one
    `deltazip-compressed.safetensors` with `{module}.qweight/.qzeros/.scales/.g_idx` and the
    uncompressed parameters, plus `compress_config.json`.  The reference's loaders and this
    library's `from_checkpoint` both read it."""
    from safetensors.torch import save_file
    if any(k.endswith(".0.qweight") for k in tensors):
        raise ValueError("serving-layout tensors: use save_converted")
    os.makedirs(save_dir, exist_ok=True)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(save_dir, CHECKPOINT_NAME))
    compress_config.save_pretrained(save_dir)


@torch.no_grad()
def _compress_with_hessian(target: torch.Tensor, base: torch.Tensor, inputs: torch.Tensor,
                           cfg: CompressionConfig):
    """One module through SparseGPT with the reference's call sequence
    (deltazip/modeling/_base.py:399-470): Hessian from the layer inputs, per-channel symmetric
    quantizer, 2:4 sweep of target - base, native packing."""
    from .sparsegpt import Quantizer, SparseGPT
    layer = torch.nn.Linear(target.shape[1], target.shape[0], bias=False, dtype=target.dtype, device=target.device)
    layer.weight.data = target.clone()
    gpt = SparseGPT(layer)
    gpt.quantizer = Quantizer()
    gpt.quantizer.configure(cfg.bits, perchannel=True, sym=True, mse=False)
    gpt.add_batch(inputs, None)
    gpt.fasterprune(cfg.sparsity, prunen=cfg.prunen, prunem=cfg.prunem, percdamp=cfg.damp_percent, base_weight=base)
    out = gpt.pack()
    gpt.free()
    return out


def compress_model(base_state_dict: Dict[str, torch.Tensor], target_state_dict: Dict[str, torch.Tensor],
                   compress_config: CompressionConfig, device="cuda:0",
                   pack_modules: Optional[Dict[str, Tuple[str, int]]] = None,
                   calibration: Optional[Dict[str, torch.Tensor]] = None,
                   layout: str = "native") -> Dict[str, torch.Tensor]:
    """Fine-tuned model + base model -> serving-layout state dict of the compressed delta (what
    `convert_model` makes of a checkpoint the reference's compressor wrote), on the GPU.  With
    layout="gptq" the result is the unconverted checkpoint instead, in the reference's own format:
    `{module}.qweight/.qzeros/.scales/.g_idx` per compressed module (QuantLinear.pack,
    deltazip/nn_modules/qlinear_cuda.py:144-244; nothing fused) and the remaining parameters under
    their own names -- what `save_compressed` writes and the reference reads.

    Every 2-D `*.weight` outside UNCOMPRESSED_MODULES is compressed as the reference's per-layer
    step does it without calibration data: delta = target.float() - base.float()
    (deltazip/core/sparsegpt.py:55-62), scales from the un-pruned delta, 2:4 pruning by magnitude,
    round-to-nearest codes (`ops.compress_delta`).  A module whose weight key appears in
    `calibration` -- its layer inputs, [B, L, K] or [L, K], as the reference's compressor records them
    layer by layer (deltazip/modeling/_base.py:261-576) -- goes through the Hessian-weighted sweep
    with error feedback instead (`SparseGPT`, sparsegpt.py:27-146; per-channel scales only).  The
    remaining parameters are carried over from the fine-tuned model as they are, as the reference's
    command line tool saves them (cli/compress.py:134-152)."""
    if compress_config.bits not in (2, 4):
        raise NotImplementedError("Only 2 and 4 bits are supported.")
    if not (compress_config.prunen == 2 and compress_config.prunem == 4):
        raise NotImplementedError("only 2:4 pruning (prunen=2, prunem=4) is supported")
    if layout not in ("native", "gptq"):
        raise ValueError("layout must be 'native' or 'gptq'")
    pack_modules = PACK_MODULES if pack_modules is None else pack_modules
    bits, gs = compress_config.bits, compress_config.group_size
    out: Dict[str, torch.Tensor] = {}
    native: Dict[str, Tuple[torch.Tensor, torch.Tensor, torch.Tensor, int]] = {}
    for key, w in target_state_dict.items():
        if key.endswith(".weight") and w.dim() == 2 and not any(u in key for u in UNCOMPRESSED_MODULES):
            if calibration is not None and key in calibration:
                if gs not in (-1, w.shape[1]):
                    raise NotImplementedError("the Hessian-weighted sweep uses per-channel scales (group_size -1)")
                q, m, s = _compress_with_hessian(w.to(device), base_state_dict[key].to(device),
                                                 calibration[key].to(device), compress_config)
            else:
                delta = w.to(device).float() - base_state_dict[key].to(device).float()
                q, m, s = ops.compress_delta(delta.contiguous(), bits, gs)
            native[key[: -len(".weight")]] = (q.cpu(), m.cpu(), s.cpu(), w.shape[1])
        elif key.endswith(".weight") and any(u in key for u in UNCOMPRESSED_MODULES):
            out[key if layout == "gptq" else key[: -len(".weight")] + ".0.weight"] = w.detach().cpu()
    return _emit_state_dict(native, out, layout, pack_modules, bits, gs)


def _emit_state_dict(native: Dict[str, Tuple[torch.Tensor, torch.Tensor, torch.Tensor, int]],
                     out: Dict[str, torch.Tensor], layout: str, pack_modules: Dict[str, Tuple[str, int]],
                     bits: int, gs: int) -> Dict[str, torch.Tensor]:
    """Compressed modules {module: (qweight, meta, scales, K)} (native, unfused) + the uncompressed
    entries already in `out` -> the state dict of the requested layout."""
    if layout == "gptq":
        for module, (q, m, s, K) in native.items():
            qw, qz, sc, gi = ops.unrepack_native_to_gptq(q, m, s, K, s.shape[-1], bits)
            out[module + ".qweight"], out[module + ".qzeros"] = qw, qz
            out[module + ".scales"], out[module + ".g_idx"] = sc, gi
        return out
    plan: Dict[str, List[Tuple[int, str]]] = {}
    for module, (q, m, s, K) in native.items():
        hit = next((k for k in pack_modules if module.endswith("." + k) or module == k), None)
        if hit is None:
            out[module + ".0.qweight"], out[module + ".0.meta"], out[module + ".0.scales"] = q, m, s
        else:
            target, pos = pack_modules[hit]
            plan.setdefault(module[: len(module) - len(hit)] + target, []).append((pos, module))
    for target, members in plan.items():
        members.sort()
        if [p for p, _ in members] != list(range(len(members))):
            raise ValueError(f"{target}: fused module has missing parts {[m for _, m in members]}")
        q, m, s = _fuse_native([native[mod][:3] for _, mod in members], native[members[0][1]][3], bits, gs)
        out[target + ".0.qweight"], out[target + ".0.meta"], out[target + ".0.scales"] = q, m, s
    return out
