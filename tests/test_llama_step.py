"""The decode-step harness (deltazip_amd/llama_step.py): a small two-layer instance whose
projections were wrapped by create_delta_manager, compared layer by layer with the CPU oracle, and
the oracle's own pins."""
import numpy as np
import pytest
import torch

from oracle import dz_oracle as o
from oracle import llama_step_ref as ref

H, I, HEADS, LAYERS, V, CTX = 256, 512, 4, 2, 320, 24
BITS = 2


def test_oracle_layer_with_zero_projections_returns_the_residual_stream():
    """All weights zero: attention and MLP add nothing, so the layer's output is 0 and the residual
    stream is hidden + residual; pins the residual bookkeeping of the restatement."""
    B = 5
    g = torch.Generator().manual_seed(0)
    hid = torch.randn(B, H, generator=g).half()
    res = torch.randn(B, H, generator=g).half()
    z = lambda n, k: torch.zeros(n, k, dtype=torch.float16)
    w = {"qkv": z(3 * H, H), "o": z(H, H), "gate_up": z(2 * I, H), "down": z(H, I),
         "ln1": torch.ones(H, dtype=torch.float16), "ln2": torch.ones(H, dtype=torch.float16)}
    none = {k: [] for k in ("qkv", "o", "gate_up", "down")}
    kc = torch.zeros(B, HEADS, CTX + 1, H // HEADS, dtype=torch.float16)
    out, r = ref.decoder_layer(hid, res, w, none, np.full(B, -1), kc, kc.clone(), CTX, HEADS, 1e-5)
    assert (out == 0).all() and torch.equal(r, hid + res)
    out, r = ref.decoder_layer(hid, None, w, none, np.full(B, -1), kc, kc.clone(), CTX, HEADS, 1e-5)
    assert (out == 0).all() and torch.equal(r, hid)


def test_oracle_norm_rotary_and_attention_closed_forms():
    x = torch.tensor([[3.0, 4.0, 0.0, 0.0]]).half()
    # rms = sqrt(25 / 4) = 2.5
    assert torch.allclose(ref.rms_norm(x, torch.ones(4).half(), 0.0).float(), torch.tensor([[1.2, 1.6, 0, 0]]), atol=1e-3)
    assert ref.rotate_half(torch.tensor([1.0, 2.0, 3.0, 4.0])).tolist() == [-3.0, -4.0, 1.0, 2.0]
    # position 0: rotary is the identity; a value cache that is constant over positions comes back
    # whatever the scores are; with o = identity the attention output is that constant
    B, hd = 2, H // HEADS
    z = lambda n, k: torch.zeros(n, k, dtype=torch.float16)
    w = {"qkv": z(3 * H, H), "o": torch.eye(H, dtype=torch.float16), "gate_up": z(2 * I, H), "down": z(H, I),
         "ln1": torch.ones(H, dtype=torch.float16), "ln2": torch.ones(H, dtype=torch.float16)}
    none = {k: [] for k in ("qkv", "o", "gate_up", "down")}
    kc = torch.randn(B, HEADS, 1, hd).half()
    vc = torch.zeros(B, HEADS, 1, hd, dtype=torch.float16)          # context 0: only the new position, v = 0
    hid = torch.randn(B, H).half()
    out, r = ref.decoder_layer(hid, None, w, none, np.full(B, -1), kc, vc, 0, HEADS, 1e-5)
    assert torch.equal(r, hid) and (out == 0).all()
    vconst = torch.full((B, HEADS, 4, hd), 0.5, dtype=torch.float16)
    kc4 = torch.randn(B, HEADS, 4, hd).half()
    # v of the new position is 0 (zero qkv), the three old ones 0.5: equal scores (q = 0) -> mean 0.375
    out, r = ref.decoder_layer(hid, None, w, none, np.full(B, -1), kc4, vconst, 3, HEADS, 1e-5)
    assert torch.allclose((r - hid).float(), torch.full((B, H), 0.375), atol=2e-3)


def _close(got, want, tol=1e-2):
    """Largest deviation relative to the largest reference value, and the relative L2 deviation.
    A layer's output passes through some ten fp16 roundings (norm, rotary, attention, activation,
    four projections), each at most half a unit in the last place of values that reach the largest
    ones: element-wise relative error is meaningless for the entries near zero."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return (np.abs(got - want).max() <= tol * np.abs(want).max()
            and np.linalg.norm(got - want) <= 0.3 * tol * np.linalg.norm(want))


def _delta_state_dict(seed):
    shapes = {"self_attn.q_proj": (H, H), "self_attn.k_proj": (H, H), "self_attn.v_proj": (H, H),
              "self_attn.o_proj": (H, H), "mlp.gate_proj": (I, H), "mlp.up_proj": (I, H), "mlp.down_proj": (H, I)}
    sd, dq = {}, {}
    for layer in range(LAYERS):
        for j, (name, (n, k)) in enumerate(shapes.items()):
            d = o.make_delta(n, k, 2e-3, BITS, -1, seed + 20 * layer + j)
            for key in ("qweight", "qzeros", "scales", "g_idx"):
                sd[f"model.layers.{layer}.{name}.{key}"] = torch.from_numpy(d[key].copy())
            dq[(layer, name)] = o.dequant_gptq(d["qweight"], d["qzeros"], d["scales"], d["g_idx"], BITS)   # [K, N]
    fused = {}
    for layer in range(LAYERS):
        fused[(layer, "qkv")] = np.concatenate([dq[(layer, f"self_attn.{x}_proj")] for x in "qkv"], axis=1)
        fused[(layer, "o")] = dq[(layer, "self_attn.o_proj")]
        fused[(layer, "gate_up")] = np.concatenate([dq[(layer, "mlp.gate_proj")], dq[(layer, "mlp.up_proj")]], axis=1)
        fused[(layer, "down")] = dq[(layer, "mlp.down_proj")]
    return sd, fused


@pytest.mark.gpu
@pytest.mark.parametrize("B", [12, 40])
def test_decode_step_matches_the_oracle_layer_by_layer(dev, B):
    from deltazip_amd import CompressionConfig, DeltaConfig, DeltaMapping, DeltaModel, create_delta_manager
    from deltazip_amd.layers import LinearWithDelta
    from deltazip_amd.llama_step import LlamaForDecodeStep, LlamaStepConfig
    cfg = LlamaStepConfig(hidden_size=H, intermediate_size=I, num_attention_heads=HEADS, num_hidden_layers=LAYERS,
                          vocab_size=V)
    gen = torch.Generator(device=dev).manual_seed(3)
    model = LlamaForDecodeStep(cfg, device=dev, generator=gen)
    nd = 3
    mgr = create_delta_manager(model, max_num_seqs=64, max_num_batched_tokens=64, vocab_size=V,
                               delta_config=DeltaConfig(max_deltas=nd + 1, max_bitwidth=BITS))
    assert len(mgr.modules) == 4 * LAYERS and all(isinstance(m, LinearWithDelta) for m in mgr.modules.values())
    fused = {}
    for d in range(1, nd + 1):
        sd, fused[d] = _delta_state_dict(1000 * d)
        dm = DeltaModel.from_tensors(sd, d, CompressionConfig(bits=BITS, prunen=2, prunem=4, sparsity=0.5),
                                     pin_memory=False)
        mgr.add_delta(dm)
        mgr.activate_delta(d)
    rng = np.random.default_rng(B)
    delta_ids = rng.integers(0, nd + 1, B)          # 0 = base model
    delta_ids[:4] = (0, 1, 2, 3)
    mgr.set_delta_mapping(DeltaMapping(tuple(int(v) for v in delta_ids), tuple(int(v) for v in delta_ids)))
    slot_of = {d: mgr.delta_index_to_id.index(d) for d in range(1, nd + 1)}
    slots = np.array([slot_of[int(d)] if d > 0 else -1 for d in delta_ids])
    nslots = mgr.delta_slots
    tokens = torch.from_numpy(rng.integers(0, V, B)).to(dev)
    kv = model.make_kv_cache(B, CTX, dev, fill=0.5)
    kv_before = [(k.clone().cpu(), v.clone().cpu()) for k, v in kv]

    seen = []
    hooks = [layer.register_forward_hook(lambda mod, args, out: seen.append(
        (args[0].cpu(), None if args[1] is None else args[1].cpu(), out[0].cpu(), out[1].cpu())))
        for layer in model.model.layers]
    logits = model.decode_step(tokens, kv, CTX)
    torch.cuda.synchronize()
    for h in hooks:
        h.remove()
    assert len(seen) == LAYERS and tuple(logits.shape) == (B, V)

    for li, (hid, res, out_h, out_r) in enumerate(seen):
        layer = model.model.layers[li]
        w = {"qkv": layer.self_attn.qkv_proj.weight.detach().cpu(), "o": layer.self_attn.o_proj.weight.detach().cpu(),
             "gate_up": layer.mlp.gate_up_proj.weight.detach().cpu(), "down": layer.mlp.down_proj.weight.detach().cpu(),
             "ln1": layer.input_layernorm.weight.detach().cpu(), "ln2": layer.post_attention_layernorm.weight.detach().cpu()}
        deltas = {}
        for name in ("qkv", "o", "gate_up", "down"):
            per_slot = [None] * nslots
            for d, s in slot_of.items():
                per_slot[s] = fused[d][(li, name)]
            deltas[name] = per_slot
        want_h, want_r = ref.decoder_layer(hid, res, w, deltas, slots, kv_before[li][0], kv_before[li][1], CTX, HEADS,
                                           cfg.rms_norm_eps, cfg.rope_theta)
        assert _close(out_r.float().numpy(), want_r.float().numpy()), f"residual of layer {li}"
        assert _close(out_h.float().numpy(), want_h.float().numpy()), f"output of layer {li}"
        # the step wrote this position's keys and values into the cache
        assert not torch.equal(kv[li][0][:, :, CTX].cpu(), kv_before[li][0][:, :, CTX])
    # final norm + output projection on the last layer's output
    hid, res = seen[-1][2], seen[-1][3]
    x = ref.rms_norm(hid + res, model.model.norm.weight.detach().cpu(), cfg.rms_norm_eps)
    want = x.float() @ model.lm_head.weight.detach().cpu().float().t()
    assert _close(logits.float().cpu().numpy(), want.numpy())
    assert (slots >= 0).any() and (slots < 0).any()
    # the deltas matter at this tolerance: the oracle without them is far from the GPU result
    li, (hid, res, out_h, out_r) = 0, seen[0]
    layer = model.model.layers[0]
    w = {"qkv": layer.self_attn.qkv_proj.weight.detach().cpu(), "o": layer.self_attn.o_proj.weight.detach().cpu(),
         "gate_up": layer.mlp.gate_up_proj.weight.detach().cpu(), "down": layer.mlp.down_proj.weight.detach().cpu(),
         "ln1": layer.input_layernorm.weight.detach().cpu(), "ln2": layer.post_attention_layernorm.weight.detach().cpu()}
    none = {k: [] for k in ("qkv", "o", "gate_up", "down")}
    base_h, _ = ref.decoder_layer(hid, res, w, none, np.full(B, -1), kv_before[0][0], kv_before[0][1], CTX, HEADS,
                                  cfg.rms_norm_eps, cfg.rope_theta)
    assert not _close(out_h.float().numpy(), base_h.float().numpy())
