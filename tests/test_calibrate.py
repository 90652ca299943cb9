"""The layer-by-layer compression loop (deltazip/modeling/_base.py:261-576) on a toy decoder: every
projection's result is checked against the single-module route (`compress_model` with that
projection's recorded inputs), whose sweep is pinned against the oracle in test_checkpoint.py."""
import copy

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from deltazip_amd import checkpoint as ck
from deltazip_amd.calibrate import LLAMA_INSIDE_LAYER_MODULES, lossy_compress
from oracle import dz_oracle as o

H, I, HEADS, V = 256, 512, 4, 64


class _Norm(nn.Module):
    def __init__(self):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(H, dtype=torch.float16))

    def forward(self, x):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).half() * self.weight


class _Attn(nn.Module):
    def __init__(self):
        super().__init__()
        for n in ("q_proj", "k_proj", "v_proj", "o_proj"):
            setattr(self, n, nn.Linear(H, H, bias=False, dtype=torch.float16))

    def forward(self, x):
        B, L, _ = x.shape
        q, k, v = (p(x).view(B, L, HEADS, H // HEADS).transpose(1, 2) for p in (self.q_proj, self.k_proj, self.v_proj))
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        return self.o_proj(a.transpose(1, 2).reshape(B, L, H))


class _Mlp(nn.Module):
    def __init__(self):
        super().__init__()
        self.gate_proj = nn.Linear(H, I, bias=False, dtype=torch.float16)
        self.up_proj = nn.Linear(H, I, bias=False, dtype=torch.float16)
        self.down_proj = nn.Linear(I, H, bias=False, dtype=torch.float16)

    def forward(self, x):
        return self.down_proj(F.silu(self.gate_proj(x)) * self.up_proj(x))


class _Layer(nn.Module):
    def __init__(self):
        super().__init__()
        self.self_attn, self.mlp = _Attn(), _Mlp()
        self.input_layernorm, self.post_attention_layernorm = _Norm(), _Norm()

    def forward(self, hidden_states, attention_mask=None, position_ids=None):
        h = hidden_states + self.self_attn(self.input_layernorm(hidden_states))
        return (h + self.mlp(self.post_attention_layernorm(h)),)


class _Inner(nn.Module):
    def __init__(self, n_layers):
        super().__init__()
        self.embed_tokens = nn.Embedding(V, H, dtype=torch.float16)
        self.layers = nn.ModuleList([_Layer() for _ in range(n_layers)])
        self.norm = _Norm()


class _Toy(nn.Module):
    """The call shape of a Hugging Face causal LM: model(input_ids=..., attention_mask=...)."""

    def __init__(self, n_layers=2):
        super().__init__()
        self.model = _Inner(n_layers)
        self.lm_head = nn.Linear(H, V, bias=False, dtype=torch.float16)

    def forward(self, input_ids, attention_mask=None):
        h = self.model.embed_tokens(input_ids)
        for layer in self.model.layers:
            h = layer(h, attention_mask=attention_mask, position_ids=None)[0]
        return self.lm_head(self.model.norm(h))


def _models(dev, seed=3):
    torch.manual_seed(seed)
    base = _Toy()
    with torch.no_grad():
        for p in base.parameters():
            if p.dim() == 2:
                p.copy_((torch.randn(p.shape) * 0.05).half())
    ft = copy.deepcopy(base)
    with torch.no_grad():
        for name, p in ft.named_parameters():
            if p.dim() == 2 and "layers" in name:
                p.add_((torch.randn(p.shape) * 5e-3).half())
    return base.to(dev), ft.to(dev)


def test_unsupported_configurations_are_refused_before_any_work():
    toy = _Toy(1)
    with pytest.raises(NotImplementedError):
        lossy_compress(toy, [], ck.CompressionConfig(bits=8, sparsity=0.5, prunen=2, prunem=4))
    with pytest.raises(NotImplementedError):
        lossy_compress(toy, [], ck.CompressionConfig(bits=4, sparsity=0.5, prunen=0, prunem=0))
    with pytest.raises(NotImplementedError):
        lossy_compress(toy, [], ck.CompressionConfig(bits=4, sparsity=0.5, prunen=2, prunem=4, group_size=128))
    with pytest.raises(ValueError):
        lossy_compress(toy, [], ck.CompressionConfig(bits=4, sparsity=0.5, prunen=2, prunem=4), layout="marlin")


def _record(layer, names, x):
    """Inputs of the named projections when `layer` runs on x."""
    got, handles = {}, []
    for n in names:
        mod = layer
        for part in n.split("."):
            mod = getattr(mod, part)
        handles.append(mod.register_forward_hook(lambda _m, inp, _o, n=n: got.__setitem__(n, inp[0].detach().clone())))
    out = layer(x)[0]
    for h in handles:
        h.remove()
    return got, out


@pytest.mark.gpu
@pytest.mark.parametrize("true_sequential", [True, False])
def test_layer_by_layer_loop_matches_the_single_module_route(dev, true_sequential):
    """Replays the loop by hand with `compress_model(calibration=...)`: same groups, same order, the
    inputs of each group recorded from the layer as compressed so far, the next layer fed with the
    compressed layer's output.  One calibration batch, so both routes add the same single batch to
    each Hessian and the packed words agree bit for bit."""
    base, ft = _models(dev)
    cfg = ck.CompressionConfig(bits=4, sparsity=0.5, prunen=2, prunem=4, true_sequential=true_sequential)
    ids = torch.randint(0, V, (2, 96), generator=torch.Generator().manual_seed(5)).to(dev)
    ft_before = copy.deepcopy(ft)
    got = lossy_compress(ft, [dict(input_ids=ids, attention_mask=None)], cfg, base_model=base, layout="gptq")

    groups = LLAMA_INSIDE_LAYER_MODULES if true_sequential else [sum(LLAMA_INSIDE_LAYER_MODULES, [])]
    base_sd = base.state_dict()
    with torch.inference_mode():
        replay = copy.deepcopy(ft_before)
        x = replay.model.embed_tokens(ids)
        for i, layer in enumerate(replay.model.layers):
            for names in groups:
                inputs, _ = _record(layer, names, x)
                for n in names:
                    key = f"model.layers.{i}.{n}.weight"
                    mod = layer
                    for part in n.split("."):
                        mod = getattr(mod, part)
                    want = ck.compress_model({key: base_sd[key]}, {key: mod.weight.data}, cfg, device=dev,
                                             calibration={key: inputs[n]}, layout="gptq")
                    stem = key[: -len(".weight")]
                    for t in ("qweight", "qzeros", "scales", "g_idx"):
                        assert torch.equal(got[f"{stem}.{t}"], want[f"{stem}.{t}"]), (stem, t)
                    # what the loop leaves in the model: base + compressed delta
                    delta = o.dequant_gptq(*(want[f"{stem}.{t}"].numpy() for t in ("qweight", "qzeros", "scales", "g_idx")), 4).T
                    left = dict(ft.named_parameters())[key].detach().float().cpu().numpy()
                    np.testing.assert_allclose(left, base_sd[key].float().cpu().numpy() + delta.astype(np.float32),
                                               atol=2e-3 * float(np.abs(left).max()))
                    mod.weight.data = dict(ft.named_parameters())[key].data.clone()
            x = layer(x)[0]
    # uncompressed parameters are carried over under their own names
    assert torch.equal(got["lm_head.weight"], ft_before.lm_head.weight.cpu())
    assert torch.equal(got["model.layers.1.input_layernorm.weight"], ft_before.model.layers[1].input_layernorm.weight.cpu())


@pytest.mark.gpu
def test_later_layers_see_the_compressed_model(dev):
    """The Hessians of layer 1 come from what compressed layer 0 produces: compressing with the
    loop differs from compressing layer 1 on the fine-tuned model's own activations."""
    base, ft = _models(dev, seed=8)
    cfg = ck.CompressionConfig(bits=2, sparsity=0.5, prunen=2, prunem=4)
    ids = torch.randint(0, V, (2, 96), generator=torch.Generator().manual_seed(6)).to(dev)
    ft_before = copy.deepcopy(ft)
    got = lossy_compress(ft, [dict(input_ids=ids)], cfg, base_model=base, layout="gptq")
    key = "model.layers.1.self_attn.q_proj.weight"
    with torch.inference_mode():
        x0 = ft_before.model.embed_tokens(ids)
        x1 = ft_before.model.layers[0](x0)[0]                      # uncompressed layer 0
        inp = ft_before.model.layers[1].input_layernorm(x1)
    other = ck.compress_model({key: base.state_dict()[key]}, {key: ft_before.state_dict()[key]}, cfg, device=dev,
                              calibration={key: inp}, layout="gptq")
    stem = key[: -len(".weight")]
    assert not torch.equal(got[stem + ".qweight"], other[stem + ".qweight"])
    # and the native layout of the same run fuses q/k/v and gate/up
    nat = lossy_compress(copy.deepcopy(ft_before), [dict(input_ids=ids)], cfg, base_model=base)
    assert "model.layers.0.self_attn.qkv_proj.0.qweight" in nat and "model.layers.1.mlp.gate_up_proj.0.meta" in nat
    assert "model.layers.0.self_attn.o_proj.0.scales" in nat and "lm_head.0.weight" in nat
