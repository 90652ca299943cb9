"""Checkpoint reader and converter: a synthetic delta checkpoint in the reference's on-disk format
(deltazip/modeling/_base.py:596-645: GPTQ-style keys in deltazip-compressed.safetensors +
compress_config.json) is read, fused and converted to the native layout; every module must
dequantise, bit for bit, to what the reference's dequantisation gives for the separate modules."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import dz_oracle as o
from deltazip_amd import checkpoint as ck

H, I, V = 256, 512, 64        # hidden, intermediate, vocabulary of the toy model
SHAPES = {"self_attn.q_proj": (H, H), "self_attn.k_proj": (64, H), "self_attn.v_proj": (64, H),
          "self_attn.o_proj": (H, H), "mlp.gate_proj": (I, H), "mlp.up_proj": (I, H), "mlp.down_proj": (H, I)}


def make_state_dict(bits, gs, layers=2, seed=100):
    sd, ref = {}, {}
    for layer in range(layers):
        for j, (name, (n, k)) in enumerate(SHAPES.items()):
            d = o.make_delta(n, k, 1e-3, bits, gs, seed + 10 * layer + j)
            mod = f"model.layers.{layer}.{name}"
            for key in ("qweight", "qzeros", "scales", "g_idx"):
                sd[f"{mod}.{key}"] = torch.from_numpy(d[key].copy())
            ref[mod] = o.dequant_gptq(d["qweight"], d["qzeros"], d["scales"], d["g_idx"], bits).T  # [N, K]
        for name in ("input_layernorm", "post_attention_layernorm"):
            sd[f"model.layers.{layer}.{name}.weight"] = torch.full((H,), 0.5 + layer, dtype=torch.float16)
    sd["model.embed_tokens.weight"] = torch.arange(V * H, dtype=torch.float32).reshape(V, H).half()
    sd["lm_head.weight"] = torch.ones(V, H, dtype=torch.float16)
    sd["model.norm.weight"] = torch.ones(H, dtype=torch.float16)
    return sd, ref


def native_dequant(q, m, s, k, bits):
    n = s.shape[1]
    qn = q.numpy().view(np.uint32)
    codes = qn.reshape(n // 32, k // 256, 64, 4) if bits == 2 else qn.reshape(n // 32, k // 256, 2, 64, 4)
    meta = m.numpy().view(np.uint32).reshape(n // 32, k // 256, 64, 4)
    return o.dequant_native(codes, meta, s.numpy(), k, n, bits)


@pytest.mark.parametrize("bits,gs", [(4, -1), (2, -1), (4, 128)])
def test_convert_model_fuses_and_keeps_values(dzlib, bits, gs):
    sd, ref = make_state_dict(bits, gs)
    out = ck.convert_model(sd, bits=bits)
    for layer in range(2):
        p = f"model.layers.{layer}."
        fused = {"self_attn.qkv_proj": ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj"],
                 "mlp.gate_up_proj": ["mlp.gate_proj", "mlp.up_proj"],
                 "self_attn.o_proj": ["self_attn.o_proj"], "mlp.down_proj": ["mlp.down_proj"]}
        for target, parts in fused.items():
            want = np.concatenate([ref[p + x] for x in parts], axis=0)
            n, k = want.shape
            q, m, s = (out[f"{p}{target}.0.{x}"] for x in ("qweight", "meta", "scales"))
            pf = 32 // bits
            assert tuple(q.shape) == (k // (pf * 4), 2 * n) and tuple(m.shape) == (n, k // 16)
            assert tuple(s.shape) == (1 if gs == -1 else k // gs, n)
            got = native_dequant(q, m, s, k, bits)
            assert np.array_equal(got.view(np.uint16), np.ascontiguousarray(want).view(np.uint16)), target
        # the separate projections are gone, the layer norms are carried over
        assert f"{p}self_attn.q_proj.0.qweight" not in out
        assert torch.equal(out[f"{p}input_layernorm.0.weight"], sd[f"{p}input_layernorm.weight"])
    assert torch.equal(out["model.embed_tokens.0.weight"], sd["model.embed_tokens.weight"])
    assert torch.equal(out["lm_head.0.weight"], sd["lm_head.weight"])
    assert not any(k.endswith((".qzeros", ".g_idx")) for k in out)


def test_bits_are_read_off_the_shapes(dzlib):
    for bits in (2, 4):
        sd, _ = make_state_dict(bits, -1, layers=1)
        a = ck.convert_model(sd)             # no bits given
        b = ck.convert_model(sd, bits=bits)
        assert a.keys() == b.keys() and all(torch.equal(a[k], b[k]) for k in a)


def test_missing_part_of_a_fused_module_is_an_error(dzlib):
    sd, _ = make_state_dict(4, -1, layers=1)
    for key in ("qweight", "qzeros", "scales", "g_idx"):
        del sd[f"model.layers.0.self_attn.k_proj.{key}"]
    with pytest.raises(ValueError, match="missing parts"):
        ck.convert_model(sd, bits=4)


def test_compression_config_round_trip(tmp_path):
    cfg = ck.CompressionConfig(bits=2, sparsity=0.5, prunen=2, prunem=4, group_size=-1)
    cfg.save_pretrained(str(tmp_path))
    with open(tmp_path / "compress_config.json") as f:
        raw = json.load(f)
    assert raw["bits"] == 2 and raw["prunen"] == 2 and raw["prunem"] == 4 and raw["lossless"] == "none"
    back = ck.CompressionConfig.from_pretrained(str(tmp_path))
    assert back.to_dict() == cfg.to_dict() and back.pack_factor == 16
    with pytest.raises(ValueError):
        ck.CompressionConfig(bits=5)
    with pytest.raises(ValueError):
        ck.CompressionConfig(sparsity=1.5)
    with pytest.raises(ValueError):
        ck.CompressionConfig(group_size=0)


@pytest.mark.parametrize("converted_on_disk", [False, True])
def test_delta_model_from_checkpoint(dzlib, tmp_path, converted_on_disk):
    from safetensors.torch import save_file
    bits = 4
    sd, ref = make_state_dict(bits, -1)
    cfg = ck.CompressionConfig(bits=bits, sparsity=0.5, prunen=2, prunem=4)
    if converted_on_disk:
        ck.save_converted(ck.convert_model(sd, bits=bits), cfg, str(tmp_path))
    else:
        save_file(sd, os.path.join(tmp_path, ck.CHECKPOINT_NAME))
        cfg.save_pretrained(str(tmp_path))
    dm = ck.DeltaModel.from_checkpoint(str(tmp_path), id=7, pin_memory=False)
    assert dm.id == 7 and dm.bitwidth == bits
    names = set(dm.deltas)
    assert "model.layers.1.self_attn.qkv_proj" in names and "model.layers.0.mlp.gate_up_proj" in names
    assert "lm_head" in names and "model.embed_tokens" in names and "model.norm" in names
    assert not any(x.endswith(("q_proj", "k_proj", "v_proj", "gate_proj", "up_proj")) and "qkv" not in x
                   and "gate_up" not in x for x in names)
    d = dm.get_delta("model.layers.1.mlp.down_proj")
    assert d._compressed and d.meta is not None and d.qzeros is None
    got = native_dequant(d.qweight, d.meta, d.scales, I, bits)
    assert np.array_equal(got, ref["model.layers.1.mlp.down_proj"])
    e = dm.get_delta("model.embed_tokens")
    assert not e._compressed and torch.equal(e.weight, sd["model.embed_tokens.weight"])
    assert dm.get_delta("nope") is None


def test_serving_layout_tensors_without_the_layout_mark_are_refused(dzlib, tmp_path):
    """`{module}.0.qweight/.scales/.meta` written by the reference's own save_compressed hold another
    kernel's bit layout under the same names and shapes; without this library's mark they are not read."""
    from safetensors.torch import save_file
    bits = 4
    sd, _ = make_state_dict(bits, -1, layers=1)
    cfg = ck.CompressionConfig(bits=bits, sparsity=0.5, prunen=2, prunem=4)
    conv = ck.convert_model(sd, bits=bits)
    with pytest.raises(ValueError, match="Marlin"):
        ck.DeltaModel.from_tensors(conv, 1, cfg, pin_memory=False)
    assert ck.DeltaModel.from_tensors(conv, 1, cfg, pin_memory=False, layout=ck.NATIVE_LAYOUT).deltas
    save_file({k: v.contiguous() for k, v in conv.items()}, os.path.join(tmp_path, ck.CHECKPOINT_NAME))   # no mark
    cfg.save_pretrained(str(tmp_path))
    with pytest.raises(ValueError, match="Marlin"):
        ck.DeltaModel.from_checkpoint(str(tmp_path), id=1, pin_memory=False)
    assert ck.DeltaModel.from_checkpoint(str(tmp_path), id=1, pin_memory=False, layout=ck.NATIVE_LAYOUT).deltas
    ck.save_converted(conv, cfg, str(tmp_path))                                                          # marked
    assert ck.DeltaModel.from_checkpoint(str(tmp_path), id=1, pin_memory=False).deltas


def test_unsupported_checkpoints_are_refused(dzlib):
    sd, _ = make_state_dict(4, -1, layers=1)
    with pytest.raises(NotImplementedError):
        ck.DeltaModel.from_tensors(sd, 1, ck.CompressionConfig(bits=4, lossless="gdeflate"))
    with pytest.raises(NotImplementedError):
        ck.DeltaModel.from_tensors(sd, 1, ck.CompressionConfig(bits=8))
    # a dense (not 2:4) delta: the repacker's check fires
    k, n = 256, 32
    codes = np.full((k, n), 9, dtype=np.uint8)
    qw, qz, sc, gi = o.pack_codes_gptq(codes, np.full((1, n), 8), np.full((1, n), 0.5, np.float16), 4)
    bad = {"model.layers.0.self_attn.o_proj." + key: torch.from_numpy(v.copy())
           for key, v in (("qweight", qw), ("qzeros", qz), ("scales", sc), ("g_idx", gi))}
    with pytest.raises(ValueError):
        ck.convert_model(bad, bits=4)


@pytest.mark.gpu
@pytest.mark.parametrize("bits,gs", [(4, -1), (2, 128)])
def test_compress_model_on_gpu(dev, bits, gs):
    """Base + fine-tuned state dicts -> compressed serving-layout delta on the GPU; every fused
    module dequantises to what the reference's pipeline (restated by the oracle) gives for its
    parts, and the result loads like a checkpoint."""
    g = torch.Generator().manual_seed(11)
    base, target = {}, {}
    for name, (n, k) in SHAPES.items():
        key = f"model.layers.0.{name}.weight"
        base[key] = (torch.randn(n, k, generator=g) * 0.02).half()
        target[key] = (base[key].float() + torch.randn(n, k, generator=g) * 1e-3).half()
    for key, shape in (("model.embed_tokens.weight", (V, H)), ("lm_head.weight", (V, H)), ("model.norm.weight", (H,)),
                       ("model.layers.0.input_layernorm.weight", (H,))):
        base[key] = torch.randn(*shape, generator=g).half()
        target[key] = torch.randn(*shape, generator=g).half()
    cfg = ck.CompressionConfig(bits=bits, group_size=gs, sparsity=0.5, prunen=2, prunem=4)
    out = ck.compress_model(base, target, cfg, device=dev)
    want = {}
    for name, (n, k) in SHAPES.items():
        key = f"model.layers.0.{name}.weight"
        d32 = target[key].float().numpy() - base[key].float().numpy()
        codes, scales16, zeros, _ = o.compress_delta(d32, bits, gs)
        qw, qz, sc, gi = o.pack_codes_gptq(codes, zeros, scales16, bits)
        want[name] = o.dequant_gptq(qw, qz, sc, gi, bits).T
    fused = {"self_attn.qkv_proj": ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj"],
             "mlp.gate_up_proj": ["mlp.gate_proj", "mlp.up_proj"],
             "self_attn.o_proj": ["self_attn.o_proj"], "mlp.down_proj": ["mlp.down_proj"]}
    for tname, parts in fused.items():
        ref = np.concatenate([want[x] for x in parts], axis=0)
        q, m, s = (out[f"model.layers.0.{tname}.0.{x}"] for x in ("qweight", "meta", "scales"))
        got = native_dequant(q, m, s, ref.shape[1], bits)
        assert np.array_equal(got.view(np.uint16), np.ascontiguousarray(ref).view(np.uint16)), tname
    assert torch.equal(out["model.embed_tokens.0.weight"], target["model.embed_tokens.weight"])
    assert torch.equal(out["model.layers.0.input_layernorm.0.weight"], target["model.layers.0.input_layernorm.weight"])
    dm = ck.DeltaModel.from_tensors(out, 3, cfg, pin_memory=False, layout=ck.NATIVE_LAYOUT)
    assert dm.get_delta("model.layers.0.self_attn.qkv_proj")._compressed and not dm.get_delta("lm_head")._compressed
    with pytest.raises(NotImplementedError):
        ck.compress_model(base, target, ck.CompressionConfig(bits=4, prunen=0, prunem=0), device=dev)


@pytest.mark.gpu
@pytest.mark.parametrize("bits,gs", [(4, -1), (2, 128)])
def test_compress_model_writes_the_reference_format(dev, tmp_path, bits, gs):
    """compress_model(layout="gptq") + save_compressed: the file holds, per module, byte for byte the
    qweight/qzeros/scales/g_idx that the reference's pipeline (oracle: compress_delta +
    pack_codes_gptq) gives for that delta, and loads back to the same serving-layout tensors as
    the native path."""
    from safetensors import safe_open
    g = torch.Generator().manual_seed(13)
    base, target = {}, {}
    for name, (n, k) in SHAPES.items():
        key = f"model.layers.0.{name}.weight"
        base[key] = (torch.randn(n, k, generator=g) * 0.02).half()
        target[key] = (base[key].float() + torch.randn(n, k, generator=g) * 1e-3).half()
    for key, shape in (("model.embed_tokens.weight", (V, H)), ("lm_head.weight", (V, H)), ("model.norm.weight", (H,))):
        base[key] = torch.randn(*shape, generator=g).half()
        target[key] = torch.randn(*shape, generator=g).half()
    cfg = ck.CompressionConfig(bits=bits, group_size=gs, sparsity=0.5, prunen=2, prunem=4)
    out = ck.compress_model(base, target, cfg, device=dev, layout="gptq")
    ck.save_compressed(out, cfg, str(tmp_path))
    with safe_open(os.path.join(tmp_path, ck.CHECKPOINT_NAME), "pt") as f:
        disk = {k: f.get_tensor(k) for k in f.keys()}
    for name, (n, k) in SHAPES.items():
        key = f"model.layers.0.{name}"
        d32 = target[key + ".weight"].float().numpy() - base[key + ".weight"].float().numpy()
        codes, scales16, zeros, _ = o.compress_delta(d32, bits, gs)
        qw, qz, sc, gi = o.pack_codes_gptq(codes, zeros, scales16, bits)
        assert np.array_equal(disk[key + ".qweight"].numpy(), qw), name
        assert np.array_equal(disk[key + ".qzeros"].numpy(), qz), name
        assert np.array_equal(disk[key + ".scales"].numpy().view(np.uint16), sc.view(np.uint16)), name
        assert np.array_equal(disk[key + ".g_idx"].numpy(), gi.astype(np.int32)), name
    assert torch.equal(disk["lm_head.weight"], target["lm_head.weight"])
    dm = ck.DeltaModel.from_checkpoint(str(tmp_path), id=5, pin_memory=False)
    nat = ck.compress_model(base, target, cfg, device=dev)
    for mod in ("model.layers.0.self_attn.qkv_proj", "model.layers.0.mlp.gate_up_proj", "model.layers.0.mlp.down_proj"):
        d = dm.get_delta(mod)
        assert torch.equal(d.qweight, nat[mod + ".0.qweight"]) and torch.equal(d.meta, nat[mod + ".0.meta"])
        assert torch.equal(d.scales, nat[mod + ".0.scales"])


@pytest.mark.gpu
def test_compress_model_with_calibration_inputs(dev):
    """A module listed in `calibration` takes the Hessian-weighted path: its packed delta equals what
    the oracle's sweep gives for the same inputs, the others stay on the magnitude path."""
    g = torch.Generator().manual_seed(12)
    n, k = 64, 256
    keys = ["model.layers.0.self_attn.o_proj.weight", "model.layers.0.mlp.down_proj.weight"]
    base = {key: (torch.randn(n, k, generator=g) * 0.02).half() for key in keys}
    target = {key: (base[key].float() + torch.randn(n, k, generator=g) * 1e-2).half() for key in keys}
    x = torch.randn(4, 128, k, generator=g)
    x = (x + 0.5 * torch.roll(x, 1, dims=2)).half()
    cfg = ck.CompressionConfig(bits=4, sparsity=0.5, prunen=2, prunem=4)
    out = ck.compress_model(base, target, cfg, device=dev, calibration={keys[0]: x})
    # oracle for the calibrated module
    d32 = target[keys[0]].float().numpy() - base[keys[0]].float().numpy()
    H, _ = o.hessian_add_batch_ref(np.zeros((k, k), np.float32), 0, x.numpy())
    hinv, W0 = o.hinv_upper_ref(H, d32)
    scale, zero = o.find_params_sym(d32, 4)
    # the factor comes from the GPU's Cholesky in the product: compare through the compensated error
    want, _ = o.obs_sweep_ref(W0, hinv, scale[:, 0], 4)
    q, m, s = (out[f"model.layers.0.self_attn.o_proj.0.{t}"] for t in ("qweight", "meta", "scales"))
    got = native_dequant(q, m, s, k, 4).astype(np.float32)
    xf = x.float().numpy().reshape(-1, k)
    e_got = np.linalg.norm((d32 - got) @ xf.T)
    e_want = np.linalg.norm((d32 - want) @ xf.T)
    plain = o.quantize(np.where(o.prune_2of4_magnitude(d32), d32, np.float32(0)), scale, zero, 15)
    e_plain = np.linalg.norm((d32 - plain) @ xf.T)
    assert abs(e_got - e_want) <= 0.02 * e_want and e_got < 0.95 * e_plain
    # same integer codes, up to the few roundings that flip with the last bits of the GPU's factor
    s16 = s.numpy().astype(np.float32).reshape(-1, 1)
    assert (np.rint(got / s16) != np.rint(want / scale)).mean() < 0.02
    # the other module: magnitude path, bit for bit
    d2 = target[keys[1]].float().numpy() - base[keys[1]].float().numpy()
    codes, scales16, zeros, _ = o.compress_delta(d2, 4, -1)
    qw, qz, sc, gi = o.pack_codes_gptq(codes, zeros, scales16, 4)
    q2, m2, s2 = (out[f"model.layers.0.mlp.down_proj.0.{t}"] for t in ("qweight", "meta", "scales"))
    assert np.array_equal(native_dequant(q2, m2, s2, k, 4), o.dequant_gptq(qw, qz, sc, gi, 4).T)
