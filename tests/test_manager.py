"""Slot manager: bookkeeping on the CPU (no kernels), the oracle's convert_mapping restatement
against hand-computed answers, and on the GPU the device-side mapping and a checkpoint -> manager
-> layer forward pass checked against the oracle."""
import numpy as np
import pytest
import torch
import torch.nn as nn

from oracle import dz_oracle as o
from deltazip_amd import (DeltaConfig, DeltaMapping, DeltaModel, CompressionConfig, LRUCacheDeltaModelManager,
                          DeltaModelManager, create_delta_manager, convert_model)
from deltazip_amd.layers import (MergedQKVParallelLinearWithDelta, MergedColumnParallelLinearWithDelta,
                                 RowParallelLinearWithDelta, VocabParallelEmbeddingWithDelta,
                                 LogitsProcessorWithDelta)
from deltazip_amd.manager import LRUCache
from deltazip_amd import ops

H, I, V = 256, 512, 64


class Attn(nn.Module):
    def __init__(self, dev):
        super().__init__()
        self.qkv_proj = nn.Linear(H, H + 128, bias=False, dtype=torch.float16, device=dev)
        self.o_proj = nn.Linear(H, H, bias=False, dtype=torch.float16, device=dev)


class Mlp(nn.Module):
    def __init__(self, dev):
        super().__init__()
        self.gate_up_proj = nn.Linear(H, 2 * I, bias=False, dtype=torch.float16, device=dev)
        self.down_proj = nn.Linear(I, H, bias=False, dtype=torch.float16, device=dev)


class Block(nn.Module):
    def __init__(self, dev):
        super().__init__()
        self.self_attn, self.mlp = Attn(dev), Mlp(dev)


class Inner(nn.Module):
    def __init__(self, dev, layers):
        super().__init__()
        self.embed_tokens = nn.Embedding(V, H, dtype=torch.float16, device=dev)
        self.layers = nn.ModuleList([Block(dev) for _ in range(layers)])


class ToyLogitsProcessor(nn.Module):
    """The serving engine's LogitsProcessor reduced to what the delta wrapper uses: `vocab_size`
    and a forward that calls `_get_logits(hidden_states, embedding, embedding_bias)`."""

    def __init__(self, vocab_size):
        super().__init__()
        self.vocab_size = vocab_size
        self.scale = 1.0

    def _get_logits(self, hidden_states, embedding, embedding_bias=None):
        return hidden_states @ embedding.t()

    def forward(self, embedding, hidden_states):
        return self._get_logits(hidden_states, embedding, None) * self.scale


class ToyModel(nn.Module):
    """Module tree and class attributes shaped like the serving model
    (model_executor/models/llama.py:299-340)."""
    packed_modules_mapping = {"qkv_proj": ["q_proj", "k_proj", "v_proj"], "gate_up_proj": ["gate_proj", "up_proj"]}
    supported_delta_modules = ["qkv_proj", "o_proj", "gate_up_proj", "down_proj", "embed_tokens", "lm_head"]

    def __init__(self, dev="cpu", layers=1):
        super().__init__()
        self.model = Inner(dev, layers)
        self.lm_head = nn.Linear(H, V, bias=False, dtype=torch.float16, device=dev)
        self.logits_processor = ToyLogitsProcessor(V)
        with torch.no_grad():
            g = torch.Generator().manual_seed(5)
            for p in self.parameters():
                p.copy_((torch.randn(p.shape, generator=g) * 0.02).to(p.dtype))


SHAPES = {"self_attn.q_proj": (H, H), "self_attn.k_proj": (64, H), "self_attn.v_proj": (64, H),
          "self_attn.o_proj": (H, H), "mlp.gate_proj": (I, H), "mlp.up_proj": (I, H), "mlp.down_proj": (H, I)}


def make_delta_model(delta_id, bits, seed):
    """A DeltaModel built the way a checkpoint is read, plus the reference dequantisation [N, K] of
    every fused module."""
    sd, ref = {}, {}
    for j, (name, (n, k)) in enumerate(SHAPES.items()):
        d = o.make_delta(n, k, 1e-3, bits, -1, seed + j)
        for key in ("qweight", "qzeros", "scales", "g_idx"):
            sd[f"model.layers.0.{name}.{key}"] = torch.from_numpy(d[key].copy())
        ref[name] = o.dequant_gptq(d["qweight"], d["qzeros"], d["scales"], d["g_idx"], bits)   # [K, N]
    fused = {"self_attn.qkv_proj": np.concatenate([ref[f"self_attn.{x}_proj"] for x in "qkv"], axis=1),
             "self_attn.o_proj": ref["self_attn.o_proj"],
             "mlp.gate_up_proj": np.concatenate([ref["mlp.gate_proj"], ref["mlp.up_proj"]], axis=1),
             "mlp.down_proj": ref["mlp.down_proj"]}
    g = torch.Generator().manual_seed(seed + 77)
    sd["model.embed_tokens.weight"] = (torch.randn(V, H, generator=g) * 0.02).half()
    sd["lm_head.weight"] = (torch.randn(V, H, generator=g) * 0.02).half()
    sd["model.norm.weight"] = torch.ones(H, dtype=torch.float16)
    fused["model.embed_tokens"] = sd["model.embed_tokens.weight"].numpy()
    fused["lm_head"] = sd["lm_head.weight"].numpy()
    dm = DeltaModel.from_tensors(sd, delta_id, CompressionConfig(bits=bits, prunen=2, prunem=4, sparsity=0.5),
                                 pin_memory=False)
    return dm, fused


# ---------------------------------------------------------------------------------------------
# CPU
# ---------------------------------------------------------------------------------------------
def test_oracle_convert_mapping_known_answers():
    # slots: [id 7, free, id 3]; manager passes max_deltas = slots + 1 = 4
    base, samp, padded, emb = o.convert_mapping_ref((3, 3, 0, 7, 0), (3, 0, 7), [7, None, 3], 4, 100, 10)
    assert base.tolist() == [2, 2, -1, 0, -1]
    assert samp.tolist() == [2, -1, 0]
    assert padded.tolist() == [0 + 2 * 3, 1 + 3 * 3, 2 + 0 * 3]
    assert emb.tolist() == [[20, 20, 0, 0, 0], [220, 220, 0, 0, 0]]
    with pytest.raises(ValueError):
        o.convert_mapping_ref((5,), (), [7, None, 3], 4, 100, 0)


def test_oracle_table_selection_known_answers():
    base = np.arange(12, dtype=np.float16).reshape(4, 3)                 # row r = [3r, 3r+1, 3r+2]
    stack = np.stack([base + 100, base + 200]).astype(np.float16)
    got = o.embed_select_ref([3, 0, 2], stack, [-1, 1, 0], base)
    assert got.tolist() == [[9, 10, 11], [200, 201, 202], [106, 107, 108]]
    x = np.array([[1, 0, 0], [0, 1, 0], [1, 1, 1]], dtype=np.float16)
    y = o.linear_select_ref(x, stack, [0, -1, 1], base)
    assert y[0].tolist() == [100, 103, 106, 109]         # column 0 of table 0
    assert y[1].tolist() == [1, 4, 7, 10]                # column 1 of the base table
    assert y[2].tolist() == [603, 612, 621, 630]         # row sums of table 1


def test_lru_cache_order_and_callbacks():
    removed = []

    class C(LRUCache):
        def _on_remove(self, key, value):
            removed.append(key)

    c = C(2)
    c.put(1, "a"); c.put(2, "b"); c.get(1); c.put(3, "c")          # 2 is the oldest now
    assert removed == [2] and list(c.keys()) == [1, 3] and len(c) == 2
    c.touch(1); c.remove_oldest()
    assert removed == [2, 3] and 1 in c
    assert c.pop(1) == "a" and removed == [2, 3, 1] and c.pop(9, "x") == "x"


def test_manager_wraps_modules_and_tracks_slots(dzlib):
    model = ToyModel()
    cfg = DeltaConfig(max_deltas=2, max_bitwidth=4, max_cpu_deltas=3)
    mgr = create_delta_manager(model, 8, 64, V, cfg)
    assert isinstance(model.model.layers[0].self_attn.qkv_proj, MergedQKVParallelLinearWithDelta)
    assert isinstance(model.model.layers[0].mlp.gate_up_proj, MergedColumnParallelLinearWithDelta)
    assert isinstance(model.model.layers[0].mlp.down_proj, RowParallelLinearWithDelta)
    assert isinstance(model.model.embed_tokens, VocabParallelEmbeddingWithDelta)
    assert isinstance(model.logits_processor, LogitsProcessorWithDelta) and isinstance(model.lm_head, nn.Linear)
    assert mgr.modules["lm_head"] is model.logits_processor and model.logits_processor.scale == 1.0
    assert sorted(mgr.modules) == ["lm_head", "model.embed_tokens", "model.layers.0.mlp.down_proj",
                                   "model.layers.0.mlp.gate_up_proj", "model.layers.0.self_attn.o_proj",
                                   "model.layers.0.self_attn.qkv_proj"]
    assert mgr.packed_modules["model.layers.0.self_attn.qkv_proj"] == [
        "model.layers.0.self_attn.q_proj", "model.layers.0.self_attn.k_proj", "model.layers.0.self_attn.v_proj"]
    qkv = model.model.layers[0].self_attn.qkv_proj
    assert qkv.indices is mgr.base_indices and qkv.indices_len is mgr.indices_len
    assert model.delta_manager is mgr and mgr.capacity == 3 and mgr.delta_slots == 2

    dms = [make_delta_model(i, 4, 10 * i)[0] for i in (1, 2, 3)]
    assert [mgr.add_delta(d) for d in dms] == [True, True, True] and not mgr.add_delta(dms[0])
    with pytest.raises(RuntimeError, match="No free Delta slots"):
        mgr.add_delta(make_delta_model(4, 4, 40)[0])
    assert len(mgr) == 3 and set(mgr.list_deltas()) == {1, 2, 3} and mgr.get_delta(2) is dms[1]
    assert mgr.activate_delta(2) and not mgr.activate_delta(2) and mgr.activate_delta(1)
    assert mgr.delta_index_to_id == [2, 1]
    with pytest.raises(ValueError, match="No free delta slots"):
        mgr.activate_delta(3)
    # slot 0 of the fused qkv layer holds delta 2's tensors
    want = dms[1].get_delta("model.layers.0.self_attn.qkv_proj")
    assert torch.equal(qkv.qweight_stacked[0].reshape(-1), want.qweight.reshape(-1))
    assert torch.equal(qkv.scales_stacked[0].reshape(-1), want.scales.reshape(-1))
    assert torch.equal(model.model.embed_tokens.delta_weights[0], dms[1].get_delta("model.embed_tokens").weight)
    assert torch.equal(model.logits_processor.weight_stacked[1], dms[0].get_delta("lm_head").weight)
    assert mgr.deactivate_delta(2) and not mgr.deactivate_delta(2)
    assert mgr.delta_index_to_id == [None, 1]
    assert mgr.activate_delta(3) and mgr.delta_index_to_id == [3, 1]
    assert mgr.remove_delta(1) and mgr.delta_index_to_id == [3, None] and not mgr.remove_delta(1)
    mgr.remove_all_deltas()
    assert len(mgr) == 0 and mgr.delta_index_to_id == [None, None]
    # there is no CPU implementation of the mapping kernel
    with pytest.raises(ValueError, match="GPU"):
        mgr.set_delta_mapping(DeltaMapping((0, 0), (0,)))


def test_lru_manager_evicts_least_recently_used(dzlib):
    model = ToyModel()
    mgr = create_delta_manager(model, 8, 64, V, DeltaConfig(max_deltas=2, max_bitwidth=4, max_cpu_deltas=3),
                               delta_manager_cls=LRUCacheDeltaModelManager)
    for i in (1, 2, 3):
        assert mgr.add_delta(make_delta_model(i, 4, 10 * i)[0])
    assert not mgr.add_delta(mgr.get_delta(1))
    mgr.activate_delta(1); mgr.activate_delta(2)
    assert mgr.delta_index_to_id == [1, 2]
    mgr.activate_delta(1)                       # touch: 2 is now the least recently used
    mgr.activate_delta(3)
    assert mgr.delta_index_to_id == [1, 3]
    # host cache is full: the registered delta that was looked up longest ago (1: the second
    # activate_delta(1) returned before reading it) goes, and leaves its GPU slot as well
    mgr.add_delta(make_delta_model(4, 4, 40)[0])
    assert len(mgr) == 3 and set(mgr.list_deltas()) == {2, 3, 4} and mgr.delta_index_to_id == [None, 3]
    assert mgr.remove_oldest_delta() and len(mgr) == 2


def test_model_without_delta_support_is_refused():
    with pytest.raises(ValueError, match="not supported"):
        create_delta_manager(nn.Linear(4, 4), 1, 8, 10, DeltaConfig())


# ---------------------------------------------------------------------------------------------
# GPU
# ---------------------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("T,P,S", [(1, 1, 1), (5, 3, 3), (37, 37, 8), (300, 7, 64), (4096, 129, 700)])
def test_map_ids_matches_reference_loop(dev, T, P, S):
    from deltazip_amd import ops
    rng = np.random.default_rng(T + S)
    table = [None] * S
    resident = rng.choice(np.arange(1, 10 * S + 2), size=max(1, (2 * S) // 3), replace=False).tolist()
    for s_, d in zip(rng.permutation(S)[: len(resident)], resident):
        table[int(s_)] = int(d)
    pool = np.array(resident + [0, 0, -1])
    tok = rng.choice(pool, size=T).astype(np.int64)
    prm = rng.choice(pool, size=P).astype(np.int64)
    vocab, extra = 32000, 3
    tok_nonneg, prm_nonneg = np.maximum(tok, 0), np.maximum(prm, 0)
    want = o.convert_mapping_ref(tok_nonneg.tolist(), prm_nonneg.tolist(), table, S + 1, vocab, extra)
    n = T + 11
    base = torch.full((n,), -7, dtype=torch.long, device=dev)
    samp, padded = torch.full_like(base, -7), torch.full_like(base, -7)
    emb = torch.full((2, n), -7, dtype=torch.long, device=dev)
    missing = torch.zeros(1, dtype=torch.int32, device=dev)
    slots = torch.tensor([d if d is not None else 0 for d in table], dtype=torch.long, device=dev)
    ops.map_ids(torch.from_numpy(tok).to(dev), torch.from_numpy(prm).to(dev), slots, S + 1, vocab, extra,
                base, samp, padded, emb, missing)
    torch.cuda.synchronize()
    assert np.array_equal(base[:T].cpu().numpy(), want[0]) and np.array_equal(samp[:P].cpu().numpy(), want[1])
    assert np.array_equal(padded[:P].cpu().numpy(), want[2]) and np.array_equal(emb[:, :T].cpu().numpy(), want[3])
    # nothing written past the batch, nothing reported missing
    assert (base[T:] == -7).all() and (samp[P:] == -7).all() and (emb[:, T:] == -7).all()
    assert int(missing.item()) == 0
    # an id that is in no slot: -1 and counted
    tok2 = torch.tensor([10 * S + 5], dtype=torch.long, device=dev)
    ops.map_ids(tok2, None, slots, S + 1, vocab, extra, base, n_missing=missing)
    torch.cuda.synchronize()
    assert int(base[0].item()) == -1 and int(missing.item()) == 1


@pytest.mark.gpu
@pytest.mark.parametrize("T,S,V_,H_", [(1, 1, 64, 256), (37, 5, 1000, 264), (300, 9, 512, 4096)])
def test_embedding_select_is_exact(dev, T, S, V_, H_):
    from deltazip_amd import ops
    rng = np.random.default_rng(T)
    base = rng.standard_normal((V_, H_)).astype(np.float16)
    stack = rng.standard_normal((S, V_, H_)).astype(np.float16)
    tok = rng.integers(0, V_, size=T)
    ids = rng.integers(-1, S, size=T)
    got = ops.apply_delta_embed(torch.from_numpy(tok).to(dev), torch.from_numpy(stack).to(dev),
                                torch.from_numpy(ids).to(dev), torch.from_numpy(base).to(dev))
    torch.cuda.synchronize()
    want = o.embed_select_ref(tok, stack, ids, base)
    assert got.dtype == torch.float16 and np.array_equal(got.cpu().numpy().view(np.uint16), want.view(np.uint16))
    # a token id outside the vocabulary gives zeros, ids outside [0, S) read the base table
    got = ops.apply_delta_embed(torch.tensor([V_, 1], device=dev), torch.from_numpy(stack).to(dev),
                                torch.tensor([0, S + 3], device=dev), torch.from_numpy(base).to(dev))
    assert (got[0] == 0).all() and np.array_equal(got[1].cpu().numpy(), base[1])


@pytest.mark.gpu
@pytest.mark.parametrize("T,S,N,K", [(1, 1, 64, 256), (32, 8, 1000, 512), (128, 3, 32000, 256), (300, 4, 512, 320)])
def test_uncompressed_projection_matches_loop(dev, T, S, N, K):
    from deltazip_amd import ops
    rng = np.random.default_rng(T + N)
    base = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    stack = (rng.standard_normal((S, N, K)) * 0.05).astype(np.float16)
    x = rng.standard_normal((T, K)).astype(np.float16)
    ids = rng.integers(-1, S, size=T)
    if T > 2:
        ids[0], ids[1] = -1, S - 1
    got = ops.apply_delta_uncompressed(torch.from_numpy(x).to(dev), torch.from_numpy(stack).to(dev),
                                       torch.from_numpy(ids).to(dev), torch.from_numpy(base).to(dev))
    torch.cuda.synchronize()
    want = o.linear_select_ref(x, stack, ids, base)
    assert tuple(got.shape) == (T, N) and o.rel_err(got.float().cpu().numpy(), want) <= 1e-2
    # all rows on the base weight: the plain product
    got = ops.apply_delta_uncompressed(torch.from_numpy(x).to(dev), torch.from_numpy(stack).to(dev),
                                       torch.full((T,), -1, dtype=torch.long, device=dev),
                                       torch.from_numpy(base).to(dev))
    ref = x.astype(np.float32) @ base.astype(np.float32).T
    assert o.rel_err(got.float().cpu().numpy(), ref) <= 1e-2


@pytest.mark.gpu
def test_uncompressed_projection_never_reads_back_to_the_host(dev):
    """The per-delta output projection is captured into a HIP graph -- which any read-back of the
    group sizes to the host would refuse -- and every replay, with eager work and synchronisations
    in between and the ids rewritten in place, gives what the eager call gives."""
    from deltazip_amd import ops
    T, S, N, K = 48, 5, 1000, 512
    rng = np.random.default_rng(99)
    base_np = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    stack_np = (rng.standard_normal((S, N, K)) * 0.05).astype(np.float16)
    x_np = rng.standard_normal((T, K)).astype(np.float16)
    base, stack, x = (torch.from_numpy(a).to(dev) for a in (base_np, stack_np, x_np))
    ids = torch.from_numpy(rng.integers(-1, S, size=T)).to(dev)
    ops.apply_delta_uncompressed(x, stack, ids, base)          # first call outside the capture (one-time set-up)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            out = ops.apply_delta_uncompressed(x, stack, ids, base)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        new_ids = rng.integers(-1, S, size=T)
        if rep == 1:
            new_ids[:] = -1                                     # a batch without any delta
        ids.copy_(torch.from_numpy(new_ids).to(dev))
        eager = ops.apply_delta_uncompressed(x, stack, ids, base)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), rep
        assert o.rel_err(out.float().cpu().numpy(), o.linear_select_ref(x_np, stack_np, new_ids, base_np)) <= 1e-2


@pytest.mark.gpu
def test_checkpoint_to_manager_to_forward(dev):
    bits = 4
    model = ToyModel(dev)
    base = {n: m.weight.detach().cpu().numpy().copy() for n, m in model.named_modules()
            if isinstance(m, nn.Linear)}
    base_emb = model.model.embed_tokens.weight.detach().cpu().numpy().copy()
    mgr = create_delta_manager(model, 8, 64, V, DeltaConfig(max_deltas=3, max_bitwidth=bits, max_cpu_deltas=4),
                               delta_manager_cls=LRUCacheDeltaModelManager)
    fused = {}
    for did in (11, 12, 13, 14):
        dm, fused[did] = make_delta_model(did, bits, 100 * did)
        mgr.add_delta(dm)
    for did in (12, 11, 13):
        mgr.activate_delta(did)
    assert mgr.delta_index_to_id == [12, 11, 13]
    ids = (11, 11, 0, 13, 12, 12, 0, 13, 11)
    x = torch.from_numpy(o.make_x(len(ids), H, 3)).to(dev)

    def check(ids):
        mgr.set_delta_mapping(DeltaMapping(ids, ids[:2]))
        torch.cuda.synchronize()
        slots = [mgr.delta_index_to_id.index(i) if i > 0 else -1 for i in ids]
        assert mgr.base_indices[: len(ids)].tolist() == slots and list(mgr.indices_len) == [len(ids), 2, 2, len(ids)]
        for name in ("self_attn.qkv_proj", "self_attn.o_proj", "mlp.gate_up_proj"):
            layer = model.get_submodule("model.layers.0." + name)
            y, bias = layer(x)
            torch.cuda.synchronize()
            table = {i: fused[i][name] for i in fused}
            uniq = sorted({i for i in ids if i > 0})
            ref = o.forward_ref(x.cpu().numpy(), base["model.layers.0." + name], [table[i] for i in uniq],
                                np.array([uniq.index(i) if i > 0 else -1 for i in ids]))
            assert bias is None and o.rel_err(y.float().cpu().numpy(), ref) <= 1e-2, name
        # embedding and output projection: the delta's own tables
        slots_np = np.array(slots)
        tok = np.arange(len(ids)) % V
        by_slot = lambda name: np.stack([fused[d][name] if d is not None else np.zeros((V, H), np.float16)
                                         for d in mgr.delta_index_to_id])
        e = model.model.embed_tokens(torch.from_numpy(tok).to(dev))
        assert np.array_equal(e.cpu().numpy(), o.embed_select_ref(tok, by_slot("model.embed_tokens"), slots_np,
                                                                  base_emb))
        logits = model.logits_processor(model.lm_head.weight, x[:2])
        want = o.linear_select_ref(x[:2].cpu().numpy(), by_slot("lm_head"), slots_np[:2], base["lm_head"])
        assert o.rel_err(logits.float().cpu().numpy(), want) <= 1e-2

    check(ids)
    # delta 14 takes the least recently used slot (12's: 11 and 13 were activated after it)
    mgr.activate_delta(14)
    assert mgr.delta_index_to_id == [14, 11, 13]
    check((14, 11, 0, 13, 14, 14, 0, 13, 11))
    with pytest.raises(ValueError, match="not in list"):
        mgr.set_delta_mapping(DeltaMapping((12, 0), (12,)))
    # an unchanged mapping is not converted again
    m = DeltaMapping((11, 0), (11,))
    mgr.set_delta_mapping(m)
    before = mgr._staged
    mgr.set_delta_mapping(DeltaMapping((11, 0), (11,)))
    assert mgr._last_mapping == m and mgr._staged is before


@pytest.mark.gpu
def test_manager_makes_row_blocks_once_for_a_large_batch(dev):
    """A batch above the fused kernel's sizes: the manager orders the tokens by delta and cuts the row
    blocks once, with the mapping, and every layer call of the step uses them; a smaller batch
    afterwards drops them again."""
    bits = 4
    model = ToyModel(dev)
    base = {n: m.weight.detach().cpu().numpy().copy() for n, m in model.named_modules() if isinstance(m, nn.Linear)}
    mgr = create_delta_manager(model, 8, 1024, V, DeltaConfig(max_deltas=3, max_bitwidth=bits, max_cpu_deltas=4),
                               delta_manager_cls=LRUCacheDeltaModelManager)
    fused = {}
    for did in (11, 12):
        dm, fused[did] = make_delta_model(did, bits, 100 * did)
        mgr.add_delta(dm)
        mgr.activate_delta(did)
    rng = np.random.default_rng(5)
    ids = tuple(int(i) for i in rng.choice([0, 11, 12], size=600))
    assert not ops.takes_fused_chunks(len(ids), mgr.delta_slots)
    mgr.set_delta_mapping(DeltaMapping(ids, ids[:2]))
    blocks = mgr.row_blocks[0]
    assert isinstance(blocks, ops.RowBlocks) and blocks.T == 600
    x = torch.from_numpy(o.make_x(len(ids), H, 3)).to(dev)
    for name in ("self_attn.qkv_proj", "mlp.gate_up_proj"):
        layer = model.get_submodule("model.layers.0." + name)
        assert layer.row_blocks is mgr.row_blocks
        y, _ = layer(x)
        torch.cuda.synchronize()
        ref = o.forward_ref(x.cpu().numpy(), base["model.layers.0." + name], [fused[11][name], fused[12][name]],
                            np.array([{0: -1, 11: 0, 12: 1}[i] for i in ids]))
        assert o.rel_err(y.float().cpu().numpy(), ref) <= 1e-2, name
    assert mgr.row_blocks[0] is blocks          # made once, not per layer call
    mgr.set_delta_mapping(DeltaMapping(ids[:9], ids[:2]))
    assert mgr.row_blocks[0] is None


@pytest.mark.gpu
def test_manager_with_one_copy_of_the_base_weights(dev):
    """DeltaConfig.keep_row_major_base=False through the manager: every wrapped projection frees its
    row-major weight, and a decode-sized and a prefill-sized batch give, bit for bit, what a manager
    that keeps both copies gives on the same weights and deltas."""
    bits = 4
    torch.manual_seed(7)
    models = [ToyModel(dev), ToyModel(dev)]
    models[1].load_state_dict(models[0].state_dict())
    cfgs = [DeltaConfig(max_deltas=2, max_bitwidth=bits), DeltaConfig(max_deltas=2, max_bitwidth=bits,
                                                                       keep_row_major_base=False)]
    mgrs = [create_delta_manager(m, 8, 1024, V, c) for m, c in zip(models, cfgs)]
    for mgr in mgrs:
        for did in (11, 12):
            mgr.add_delta(make_delta_model(did, bits, 100 * did)[0])
            mgr.activate_delta(did)
    qkv = [m.get_submodule("model.layers.0.self_attn.qkv_proj") for m in models]
    assert qkv[0].base_layer.weight.numel() > 0 and qkv[1].base_layer.weight.numel() == 0
    assert qkv[1].base_shape == tuple(qkv[0].base_layer.weight.shape)
    rng = np.random.default_rng(11)
    for T in (9, 700):
        ids = tuple(int(i) for i in rng.choice([0, 11, 12], size=T))
        x = torch.from_numpy(o.make_x(T, H, 5)).to(dev)
        outs = []
        for mgr, model in zip(mgrs, models):
            mgr.set_delta_mapping(DeltaMapping(ids, ids[:2]))
            outs.append([model.get_submodule("model.layers.0." + name)(x)[0]
                         for name in ("self_attn.qkv_proj", "self_attn.o_proj", "mlp.gate_up_proj")])
        torch.cuda.synchronize()
        for a, b in zip(*outs):
            assert torch.equal(a, b), T
