"""GPU tests of the reference-shaped Python API: QuantLinear and the delta layers."""
import numpy as np
import pytest
import torch

from oracle import dz_oracle as o
from deltazip_amd import (DeltaConfig, MergedColumnParallelLinearWithDelta, QuantLinear,
                          RowParallelLinearWithDelta, convert_mapping, from_layer, ops)
from _util import TOL, make_problem

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits,gs", [(4, -1), (2, -1), (4, 128)])
def test_quant_linear_from_tensors_forward(dev, bits, gs):
    """QuantLinear.from_tensors(...).forward(x) == x @ dequant(W) (quant_linear_naive.py:35-96)."""
    dl = o.make_delta(64, 512, 2e-3, bits, gs, 42)
    t = lambda a: torch.from_numpy(a).to(dev)
    ql = QuantLinear.from_tensors(bits, t(dl["qweight"]), t(dl["qzeros"]), t(dl["scales"]), t(dl["g_idx"]), None, None)
    assert (ql.infeatures, ql.outfeatures) == (512, 64)
    x = torch.from_numpy(o.make_x(6, 512, 1)).to(dev).reshape(2, 3, 512)
    y = ql(x)
    assert y.shape == (2, 3, 64) and y.dtype == torch.float16
    dt = o.dequant_gptq(dl["qweight"], dl["qzeros"], dl["scales"], dl["g_idx"], bits)
    ref = x.reshape(6, 512).float().cpu().numpy() @ dt.astype(np.float32)
    assert o.rel_err(y.reshape(6, 64).cpu().numpy(), ref) <= TOL
    # the bias is added to the fp16 result, as the reference does (quant_linear_naive.py:82)
    bias = (torch.randn(64, device=dev) * 0.01).half()
    qb = QuantLinear.from_tensors(bits, t(dl["qweight"]), t(dl["qzeros"]), t(dl["scales"]), t(dl["g_idx"]), bias, None)
    assert torch.equal(qb(x), y + bias)
    w = ql.unpack().cpu().numpy()
    assert np.array_equal(w.view(np.uint16), np.ascontiguousarray(dt.T).view(np.uint16))


def test_layer_protocol(dev):
    """create_delta_weights -> set_delta -> set_mapping -> forward; reset_delta; buffer rewrite."""
    n, k, t, bits = 128, 512, 10, 4
    p = make_problem(n, k, bits, -1, 3, t, "uniform", 7, dev)
    base = torch.nn.Linear(k, n, bias=False, device=dev, dtype=torch.float16)
    with torch.no_grad():
        base.weight.copy_(p["wb"])
    cfg = DeltaConfig(max_deltas=4, max_bitwidth=bits)
    layer = from_layer(base, 4, cfg, ["gate_proj", "up_proj"])
    assert isinstance(layer, MergedColumnParallelLinearWithDelta)
    assert tuple(layer.qweight_stacked.shape) == (4, k // 32, 2 * n)
    assert tuple(layer.meta_stacked.shape) == (4, n, k // 16) and tuple(layer.scales_stacked.shape) == (4, 1, n)
    # slots 1..3 take the deltas: native tensors for two, GPTQ tensors (converted on the fly) for one
    layer.set_delta(1, bits, p["q"][0].cpu().pin_memory(), None, p["s"][0].cpu().pin_memory(), None, p["m"][0].cpu().pin_memory())
    layer.set_delta(2, bits, p["q"][1], None, p["s"][1], None, p["m"][1])
    g = p["gptq"][2]
    layer.set_delta(3, bits, torch.from_numpy(g["qweight"]), torch.from_numpy(g["qzeros"]),
                    torch.from_numpy(g["scales"]), torch.from_numpy(g["g_idx"]), None)
    assert layer.bitwidth == [0, bits, bits, bits]
    # manager side: delta ids 11, 12, 13 live in slots 1, 2, 3; id 0 = base
    index_buf = torch.full((16,), -1, dtype=torch.int64, device=dev)
    slot_ids = [None, 11, 12, 13]
    token_ids = [11, 0, 13, 12, 12, 0, 11, 13, 13, 11]
    idx = convert_mapping(token_ids, slot_ids, out=index_buf)
    layer.set_mapping(index_buf, None, None, None, [t])
    out, out_bias = layer(p["x"])
    assert out_bias is None
    oracle_ids = np.array([{0: -1, 11: 0, 12: 1, 13: 2}[i] for i in token_ids])
    ref = o.forward_ref(p["x_np"], p["wb_np"], p["dts"], oracle_ids)
    assert o.rel_err(out.cpu().numpy(), ref) <= TOL
    # the layer reads a tiled copy of its base weight (the default); without it: the same bits
    assert layer.base_tiled is not None and torch.equal(layer.base_tiled, ops.tile_base(base.weight))
    plain = from_layer(torch.nn.Linear(k, n, bias=False, device=dev, dtype=torch.float16), 4,
                       DeltaConfig(max_deltas=4, max_bitwidth=bits, tile_base_weights=False), ["gate_proj", "up_proj"])
    assert plain.base_tiled is None
    with torch.no_grad():
        plain.base_layer.weight.copy_(p["wb"])
    for slot in (1, 2, 3):
        plain.set_delta(slot, bits, layer.qweight_stacked[slot], None, layer.scales_stacked[slot], None, layer.meta_stacked[slot])
    plain.set_mapping(index_buf, None, None, None, [t])
    assert torch.equal(plain(p["x"])[0], out)
    # the base weight written in place after the layer was made: the tiles follow
    with torch.no_grad():
        base.weight.mul_(2.0)
    out_w2, _ = layer(p["x"])
    with torch.no_grad():
        base.weight.copy_(p["wb"])
    assert o.rel_err(out_w2.cpu().numpy(), o.forward_ref(p["x_np"], 2 * p["wb_np"], p["dts"], oracle_ids)) <= TOL
    assert torch.equal(layer(p["x"])[0], out)
    # the serving engine's way of loading a base weight: the parameter's weight_loader writes
    # param.data, which moves no version counter; a loader the parameter carried when the layer was
    # made is wrapped, so the tiles follow
    lin2 = torch.nn.Linear(k, n, bias=False, device=dev, dtype=torch.float16)
    lin2.weight.weight_loader = lambda param, loaded: param.data.copy_(loaded)
    wrapped = from_layer(lin2, 4, DeltaConfig(max_deltas=4, max_bitwidth=bits), ["gate_proj", "up_proj"])
    for slot in (1, 2, 3):
        wrapped.set_delta(slot, bits, layer.qweight_stacked[slot], None, layer.scales_stacked[slot], None, layer.meta_stacked[slot])
    wrapped.set_mapping(index_buf, None, None, None, [t])
    lin2.weight.weight_loader(lin2.weight, p["wb"])
    assert torch.equal(wrapped(p["x"])[0], out)
    # a write through .data from anywhere else cannot be seen by the layer (documented): the caller
    # refreshes the tiles
    lin2.weight.data.mul_(2.0)
    wrapped.refresh_base_tiles()
    assert torch.equal(wrapped(p["x"])[0], out_w2)
    # reset a slot: its tokens fall back to the base layer
    layer.reset_delta(2)
    out2, _ = layer(p["x"])
    ids2 = np.where(oracle_ids == 1, -1, oracle_ids)
    assert o.rel_err(out2.cpu().numpy(), o.forward_ref(p["x_np"], p["wb_np"], p["dts"], ids2)) <= TOL
    # the mapping buffer is rewritten in place for the next step
    convert_mapping([13] * t, slot_ids, out=index_buf)
    out3, _ = layer(p["x"])
    assert o.rel_err(out3.cpu().numpy(), o.forward_ref(p["x_np"], p["wb_np"], p["dts"], np.full(t, 2))) <= TOL
    with pytest.raises(ValueError):
        layer.set_delta(0, 2, p["q"][0], None, p["s"][0], None, p["m"][0])      # wrong bit width


@pytest.mark.parametrize("t", [8, 100, 300, 700])
def test_layer_with_only_the_tiled_base_weight(dev, t):
    """keep_row_major_base=False: after the tiles are made the row-major weight is freed; every batch
    size (fused kernel, its chunked form, the matrix-core kernel) reads the tiles and gives, bit for
    bit, what a layer with both copies gives.  The parameter's loader still works."""
    n, k, bits = 320, 1024, 2          # n is not a multiple of the matrix-core kernel's 256-feature tile
    p = make_problem(n, k, bits, -1, 3, t, "uniform", 31 + t, dev)
    def make(cfg):
        lin = torch.nn.Linear(k, n, bias=False, device=dev, dtype=torch.float16)
        with torch.no_grad():
            lin.weight.copy_(p["wb"])
        lin.weight.weight_loader = lambda param, loaded: param.data.copy_(loaded)
        layer = from_layer(lin, 3, cfg, [])
        for slot in range(3):
            layer.set_delta(slot, bits, p["q"][slot], None, p["s"][slot], None, p["m"][slot])
        layer.set_mapping(p["ids"], None, None, None, [t])
        return lin, layer
    lin_a, both = make(DeltaConfig(max_deltas=3, max_bitwidth=bits))
    free0 = torch.cuda.memory_allocated()
    lin_b, only = make(DeltaConfig(max_deltas=3, max_bitwidth=bits, keep_row_major_base=False))
    assert lin_b.weight.numel() == 0 and lin_a.weight.numel() == n * k
    assert torch.equal(only.base_tiled, both.base_tiled)
    assert torch.equal(ops.untile_base(only.base_tiled), p["wb"])
    ya, yb = both(p["x"])[0], only(p["x"])[0]
    torch.cuda.synchronize()
    assert torch.equal(ya, yb)
    ref = o.forward_ref(p["x_np"], p["wb_np"], p["dts"], p["ids_np"])
    assert o.rel_err(yb.cpu().numpy(), ref) <= TOL
    # loading another base weight through the parameter's loader: the row-major form comes back for
    # the load and is dropped again afterwards
    lin_b.weight.weight_loader(lin_b.weight, 2 * p["wb"])
    assert lin_b.weight.numel() == 0
    y2 = only(p["x"])[0]
    torch.cuda.synchronize()
    assert o.rel_err(y2.cpu().numpy(), o.forward_ref(p["x_np"], 2 * p["wb_np"], p["dts"], p["ids_np"])) <= TOL
    assert torch.equal(only.restore_row_major_base(), 2 * p["wb"]) and lin_b.weight.numel() == n * k
    with pytest.raises(ValueError):
        DeltaConfig(tile_base_weights=False, keep_row_major_base=False)


@pytest.mark.parametrize("bits,gs", [(2, -1), (4, 128)])
def test_matrix_core_kernel_reads_tiles_or_rows_alike(dev, bits, gs):
    """dz_multi_delta_gemm_tiled against dz_multi_delta_gemm on the same problem: equal bits, also
    with fewer features than a tile and with an output slice."""
    from deltazip_amd.prefill import multi_delta_linear_prefill
    for n, k, t in ((96, 768, 400), (544, 1024, 1000)):
        p = make_problem(n, k, bits, gs, 5, t, "uniform", 3 * n + bits, dev)
        wt = ops.tile_base(p["wb"])
        y0 = torch.zeros(t, n + 32, dtype=torch.float16, device=dev)
        y1 = torch.zeros_like(y0)
        multi_delta_linear_prefill(p["x"], p["wb"], p["q"], p["s"], p["m"], p["ids"], bits=bits, out=y0[:, 16:16 + n],
                                   accumulate=False)
        multi_delta_linear_prefill(p["x"], None, p["q"], p["s"], p["m"], p["ids"], bits=bits, out=y1[:, 16:16 + n],
                                   accumulate=False, base_tiled=wt)
        torch.cuda.synchronize()
        assert torch.equal(y0, y1)
        ref = o.forward_ref(p["x_np"], p["wb_np"], p["dts"], p["ids_np"])
        assert o.rel_err(y1[:, 16:16 + n].cpu().numpy(), ref) <= TOL


def test_row_parallel_rejects_bias_and_from_layer_passthrough(dev):
    lin = torch.nn.Linear(512, 64, bias=True, device=dev, dtype=torch.float16)
    cfg = DeltaConfig(max_deltas=1, max_bitwidth=4)
    layer = from_layer(lin, 1, cfg, [])
    assert isinstance(layer, RowParallelLinearWithDelta)
    layer.set_mapping(torch.full((4,), -1, dtype=torch.int64, device=dev), indices_len=[4])
    with pytest.raises(ValueError, match="bias"):
        layer(torch.zeros(4, 512, dtype=torch.float16, device=dev))
    act = torch.nn.ReLU()
    assert from_layer(act, 1, cfg, []) is act


def test_two_streams_use_separate_workspaces(dev):
    """The Python shim keeps one split-K workspace per (device, stream): calls issued on two streams
    at the same time must not share partial sums."""
    p1 = make_problem(256, 4096, 2, -1, 4, 32, "uniform", 11, dev)
    p2 = make_problem(256, 4096, 2, -1, 4, 32, "uniform", 12, dev)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    outs = {1: [], 2: []}
    for _ in range(8):
        with torch.cuda.stream(s1):
            outs[1].append(ops.apply_delta(p1["x"], p1["q"], p1["s"], p1["m"], p1["ids"], p1["wb"]))
        with torch.cuda.stream(s2):
            outs[2].append(ops.apply_delta(p2["x"], p2["q"], p2["s"], p2["m"], p2["ids"], p2["wb"]))
    torch.cuda.synchronize()
    for p, ys in ((p1, outs[1]), (p2, outs[2])):
        ref = o.forward_ref(p["x_np"], p["wb_np"], p["dts"], p["ids_np"])
        for y in ys:
            assert o.rel_err(y.cpu().numpy(), ref) <= TOL
            assert torch.equal(y, ys[0])
    assert len({k for k in ops._workspaces if k[0] == dev.index}) >= 2
