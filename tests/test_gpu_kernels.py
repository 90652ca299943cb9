"""GPU parity tests: every entry point is called through the C ABI (via the ctypes wrapper) and
compared with the CPU oracle on the same seeded inputs.  Dequantised deltas must match bit for
bit; layer outputs within TOL = 1e-2 max relative error (fp16 outputs vs the fp32 reference)."""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import dz_oracle as o
from deltazip_amd import ops
from _util import TOL, make_problem, run_layer

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits", [2, 4])
@pytest.mark.parametrize("gs", [-1, 64, 128, 256])
def test_dequant_bit_exact(dev, bits, gs):
    p = make_problem(96, 768, bits, gs, 2, 1, "single", 100 + bits + max(gs, 0), dev)
    for d in range(2):
        got = ops.dequant(p["q"][d], p["m"][d], p["s"][d], 768, 96, bits).cpu().numpy()
        assert np.array_equal(got.view(np.uint16), np.ascontiguousarray(p["dts"][d].T).view(np.uint16))


@pytest.mark.parametrize("bits", [2, 4])
def test_dequant_extreme_scales(dev, bits):
    """Subnormal, tiny and huge fp16 scales: one rounding of the exact product, no flush to zero."""
    k, n = 256, 32
    zp = 2 ** (bits - 1)
    rng = np.random.default_rng(5)
    codes = np.full((k, n), zp, dtype=np.uint8)
    pos = rng.integers(0, 4, size=(k // 4, n))
    for g in range(k // 4):                       # one non-zero code per group of 4
        codes[4 * g + pos[g], np.arange(n)] = rng.integers(0, 2 ** bits, size=n)
    scales = np.array([6e-8, 1.2e-7, 3e-6, 6.1e-5, 1e-3, 0.5, 1000.0, 8000.0] * 4, dtype=np.float16).reshape(1, n)
    qw, qz, sc, gi = o.pack_codes_gptq(codes, np.full((1, n), zp), scales, bits)
    ref = o.dequant_gptq(qw, qz, sc, gi, bits)
    q, m, s = ops.repack_gptq_to_native(torch.from_numpy(qw), torch.from_numpy(qz), torch.from_numpy(sc),
                                        torch.from_numpy(gi), bits)
    got = ops.dequant(q.to(dev), m.to(dev), s.to(dev), k, n, bits).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), np.ascontiguousarray(ref.T).view(np.uint16))
    assert np.any((ref != 0) & (np.abs(ref.astype(np.float32)) < 6.1e-5))   # subnormals were exercised


def test_merge_is_fp32_add_rounded_once(dev):
    p = make_problem(64, 512, 4, -1, 1, 1, "single", 31, dev)
    got = ops.merge(p["wb"], p["q"][0], p["m"][0], p["s"][0], 4).cpu().numpy()
    ref = (p["wb_np"].astype(np.float32) + p["dts"][0].T.astype(np.float32)).astype(np.float16)
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("t,s", [(1, 1), (9, 8), (128, 5), (1000, 3), (4099, 17)])
def test_segment(dev, t, s):
    rng = np.random.default_rng(t)
    ids = rng.integers(-1, s, size=t).astype(np.int64)
    ids[::7] = s + 3                               # out-of-range ids count as -1
    perm, off = ops.segment(torch.from_numpy(ids).to(dev), s)
    key = np.where((ids < 0) | (ids >= s), -1, ids)
    assert np.array_equal(perm.cpu().numpy(), np.argsort(key, kind="stable"))
    counts = [(key == v).sum() for v in range(-1, s)]
    assert off.cpu().numpy().tolist() == [0] + np.cumsum(counts).tolist()


CASES = [
    # n, k, bits, gs, deltas, tokens, ids
    (64, 512, 2, -1, 3, 5, "uniform"),
    (64, 512, 4, -1, 3, 16, "uniform"),
    (96, 768, 2, -1, 2, 1, "single"),
    (96, 768, 4, 64, 2, 17, "uniform"),
    (128, 1024, 2, 128, 4, 32, "uniform"),
    (128, 1024, 4, 128, 4, 32, "zipf"),
    (160, 1280, 2, -1, 8, 31, "uniform"),
    (256, 1024, 2, -1, 6, 48, "uniform"),
    (256, 1024, 4, -1, 6, 64, "zipf"),
    (256, 2048, 2, 256, 5, 100, "uniform"),
    (256, 1024, 4, 128, 12, 128, "zipf"),
    (32, 256, 2, -1, 1, 33, "single"),
]


@pytest.mark.parametrize("n,k,bits,gs,nd,t,kind", CASES)
def test_layer_parity(dev, n, k, bits, gs, nd, t, kind):
    p = make_problem(n, k, bits, gs, nd, t, kind, 1000 + n + k + t, dev)
    if t > 2:
        p["ids_np"][1] = -1
        p["ids"] = torch.from_numpy(p["ids_np"]).to(dev)
    y = run_layer(p).cpu().numpy()
    ref = o.forward_ref(p["x_np"], p["wb_np"], p["dts"], p["ids_np"])
    assert o.rel_err(y, ref) <= TOL
    assert ops.workspace_status() == 0


def test_edge_cases(dev):
    p = make_problem(64, 512, 4, -1, 2, 12, "uniform", 77, dev)
    base = o.forward_ref(p["x_np"], p["wb_np"], p["dts"], np.full(12, -1))
    # every token base-only == plain linear layer
    p["ids"] = torch.full((12,), -1, dtype=torch.int64, device=dev)
    assert o.rel_err(run_layer(p).cpu().numpy(), base) <= TOL
    # no slots at all (S = 0 is not allowed by the stacked tensors; one reset slot stands in)
    # a reset slot (zero scales) contributes exactly nothing
    p["s"].zero_()
    p["ids"] = torch.zeros(12, dtype=torch.int64, device=dev)
    y0 = run_layer(p)
    p["ids"] = torch.full((12,), -1, dtype=torch.int64, device=dev)
    assert torch.equal(y0, run_layer(p))


def test_out_of_range_ids_are_flagged_and_treated_as_base(dev):
    p = make_problem(64, 512, 2, -1, 2, 8, "uniform", 78, dev)
    ids = p["ids_np"].copy(); ids[3] = 2; ids[5] = -7
    p["ids"] = torch.from_numpy(ids).to(dev)
    y = run_layer(p).cpu().numpy()
    assert ops.workspace_status() & 1
    ids_eff = np.where((ids < 0) | (ids >= 2), -1, ids)
    assert o.rel_err(y, o.forward_ref(p["x_np"], p["wb_np"], p["dts"], ids_eff)) <= TOL
    ops._workspaces.clear()                        # fresh (zeroed) status word for later tests


GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_golden_fixtures(dev, path):
    g = np.load(path)
    bits = int(g["bits"])
    nd = sum(1 for k in g.files if k.endswith("_qweight"))
    qs, ms, ss = [], [], []
    for d in range(nd):
        q, m, s = ops.repack_gptq_to_native(*(torch.from_numpy(g[f"d{d}_{k}"]) for k in
                                              ("qweight", "qzeros", "scales", "g_idx")), bits)
        K, N = g[f"d{d}_dequant_t"].shape
        got = ops.dequant(q.to(dev), m.to(dev), s.to(dev), K, N, bits).cpu().numpy()
        assert np.array_equal(got.view(np.uint16), np.ascontiguousarray(g[f"d{d}_dequant_t"].T).view(np.uint16))
        qs.append(q); ms.append(m); ss.append(s)
    q, m, s = (torch.stack(v).to(dev) for v in (qs, ms, ss))
    x = torch.from_numpy(g["x"]).to(dev); ids = torch.from_numpy(g["ids"]).to(dev)
    y = ops.apply_delta(x, q, s, m, ids, torch.from_numpy(g["w_base"]).to(dev)).cpu().numpy()
    assert o.rel_err(y, g["y_ref"]) <= TOL
    yd = torch.zeros_like(torch.from_numpy(g["y_delta_only"])).half().to(dev)
    ops.add_delta(yd, x, q, None, s, None, ids, meta=m)
    assert o.rel_err(yd.cpu().numpy(), g["y_delta_only"]) <= TOL


def test_add_delta_slices_qkv_and_gate_up(dev):
    """In-place y[:, off:off+n] += x @ delta^T per output slice (deltazip.py:40-153)."""
    k, t = 512, 20
    slices = (128, 64, 64)                         # q, k, v
    probs = [make_problem(n, k, 4, -1, 3, t, "uniform", 300 + i, dev) for i, n in enumerate(slices)]
    ids_np = probs[0]["ids_np"]; ids = probs[0]["ids"]; x = probs[0]["x"]; x_np = probs[0]["x_np"]
    y0 = (torch.randn(t, sum(slices), device=dev) * 0.05).half()
    y = y0.clone()
    off = 0
    for p, n in zip(probs, slices):
        ops.add_delta_slice(y, x, p["q"], None, p["s"], None, ids, 1.0, off, n, meta=p["m"])
        off += n
    torch.cuda.synchronize()
    off = 0
    for p, n in zip(probs, slices):
        ref = y0[:, off:off + n].float().cpu().numpy() + o.forward_ref(x_np, None, p["dts"], ids_np)
        assert o.rel_err(y[:, off:off + n].cpu().numpy(), ref) <= TOL
        off += n
    # whole-width form
    p = probs[0]
    yy = torch.zeros(t, 128, dtype=torch.float16, device=dev)
    assert ops.add_delta(yy, x, p["q"], None, p["s"], None, ids, meta=p["m"]) is yy
    assert o.rel_err(yy.cpu().numpy(), o.forward_ref(x_np, None, p["dts"], ids_np)) <= TOL


@pytest.mark.parametrize("t,bits,gs", [(20, 4, -1), (100, 2, -1), (7, 4, 128), (300, 2, -1)])
def test_apply_delta_packed_nslice_and_in_place_apply_delta(dev, t, bits, gs):
    """The packed-sublayer op and the in-place apply_delta of the reference's non-fused module
    (deltazip.py:78-153), through its own names: every slice of `output` gains x @ delta_j^T of the
    token's delta, a base-only token (-1) gains nothing, columns outside the slices stay as they were."""
    from deltazip_amd import deltazip as dzmod
    k = 512
    slices = (128, 64, 96)
    nd = 4
    mixed = np.random.default_rng(t).integers(-1, nd, t).astype(np.int64)
    mixed[:2] = (-1, nd - 1)
    probs = [make_problem(n, k, bits, gs, nd, t, mixed, 700 + i, dev) for i, n in enumerate(slices)]
    ids_np = probs[0]["ids_np"]; ids = probs[0]["ids"]; x = probs[0]["x"]; x_np = probs[0]["x_np"]
    width = sum(slices) + 32                       # 32 columns that belong to no slice
    lead = (2, t // 2) if t % 2 == 0 else (t,)     # leading dimensions are flattened by the ops
    y0 = (torch.randn(*lead, width, device=dev) * 0.05).half()
    y = y0.clone()
    xin = x.view(*y.shape[:-1], k)
    got = dzmod.apply_delta_packed_nslice(xin, [p["q"] for p in probs], [None] * 3, [p["s"] for p in probs],
                                          [None] * 3, ids.view(*y.shape[:-1]), y, slices,
                                          meta_stacked=[p["m"] for p in probs])
    torch.cuda.synchronize()
    assert got.shape == y.shape and got.data_ptr() == y.data_ptr()
    y2, y02 = y.view(-1, width), y0.view(-1, width)
    off = 0
    for p, n in zip(probs, slices):
        ref = y02[:, off:off + n].float().cpu().numpy() + o.forward_ref(x_np, None, p["dts"], ids_np)
        assert o.rel_err(y2[:, off:off + n].cpu().numpy(), ref) <= TOL
        base_rows = torch.from_numpy(ids_np < 0).to(dev)
        assert torch.equal(y2[base_rows, off:off + n], y02[base_rows, off:off + n])
        off += n
    assert torch.equal(y2[:, off:], y02[:, off:])
    # the same slices one by one give the same bits (one launch or three)
    y3 = y0.clone().view(-1, width)
    off = 0
    for p, n in zip(probs, slices):
        ops.add_delta_slice(y3, x, p["q"], None, p["s"], None, ids, 1.0, off, n, meta=p["m"])
        off += n
    assert torch.equal(y3, y2)
    # in-place apply_delta over the first slice's delta
    p = probs[0]
    z0 = (torch.randn(*y.shape[:-1], slices[0], device=dev) * 0.05).half()
    z = z0.clone()
    out = dzmod.apply_delta(xin, p["q"], None, p["s"], None, ids.view(*y.shape[:-1]), z, meta_stacked=p["m"])
    torch.cuda.synchronize()
    assert out.shape == z.shape and out.data_ptr() == z.data_ptr()
    ref = z0.view(-1, slices[0]).float().cpu().numpy() + o.forward_ref(x_np, None, p["dts"], ids_np)
    assert o.rel_err(z.view(-1, slices[0]).cpu().numpy(), ref) <= TOL


def test_deterministic_and_order_independent(dev):
    p = make_problem(128, 1024, 2, -1, 5, 32, "uniform", 55, dev)
    y1 = run_layer(p); y2 = run_layer(p)
    assert torch.equal(y1, y2)                     # run-to-run bit identical (no float atomics)
    perm = torch.randperm(32, device=dev)
    q = dict(p); q["x"] = p["x"][perm].contiguous(); q["ids"] = p["ids"][perm].contiguous()
    assert torch.equal(run_layer(q), y1[perm])     # a token's result does not depend on its position
    srt = torch.argsort(p["ids"], stable=True)
    q["x"] = p["x"][srt].contiguous(); q["ids"] = p["ids"][srt].contiguous()
    assert torch.equal(run_layer(q), y1[srt])


@pytest.mark.parametrize("t", [32, 100])
def test_k_split_variants_agree(dev, t):
    p = make_problem(64, 2048, 4, 128, 3, t, "uniform", 66, dev)
    ref = o.forward_ref(p["x_np"], p["wb_np"], p["dts"], p["ids_np"])
    try:
        for ns in (1, 2, 3, 8):
            ops.set_ksplit(ns)
            assert o.rel_err(run_layer(p).cpu().numpy(), ref) <= TOL
            assert torch.equal(run_layer(p), run_layer(p))
    finally:
        ops.set_ksplit(0)


def test_indices_are_read_at_call_time(dev):
    """The manager rewrites the index buffer between steps (models.py:421-430); the layer must see it."""
    p = make_problem(64, 512, 4, -1, 3, 8, "uniform", 88, dev)
    buf = torch.zeros(16, dtype=torch.int64, device=dev)
    view = buf[:8]
    for ids in ([0, 1, 2, -1, 0, 1, 2, -1], [2, 2, 2, 2, -1, -1, 0, 0]):
        buf[:8].copy_(torch.tensor(ids))
        y = ops.apply_delta(p["x"], p["q"], p["s"], p["m"], view, p["wb"]).cpu().numpy()
        assert o.rel_err(y, o.forward_ref(p["x_np"], p["wb_np"], p["dts"], np.array(ids))) <= TOL


def test_gemm_f16(dev):
    from deltazip_amd.prefill import gemm_f16
    torch.manual_seed(0)
    x = torch.randn(300, 512, device=dev).half(); w = (torch.randn(256, 512, device=dev) * 0.05).half()
    y = gemm_f16(x, w)
    ref = x.float() @ w.float().t()
    assert o.rel_err(y.float().cpu().numpy(), ref.cpu().numpy()) <= 2e-3
    y2 = y.clone(); gemm_f16(x, w, y2, accumulate=True)
    assert o.rel_err(y2.float().cpu().numpy(), 2 * ref.cpu().numpy()) <= 3e-3


@pytest.mark.parametrize("kind", ["blocks", "uniform"])
def test_prefill_sized_call(dev, kind):
    """T > 128: per-segment merge + matrix-core GEMM; sorted (one delta per request) and unsorted."""
    p = make_problem(256, 1024, 2, -1, 4, 400, kind, 99, dev)
    y = run_layer(p).cpu().numpy()
    ref = o.forward_ref(p["x_np"], p["wb_np"], p["dts"], p["ids_np"])
    assert o.rel_err(y, ref) <= TOL


@pytest.mark.parametrize("bits,with_x", [(2, 0), (2, 1), (4, 1)])
def test_read_only_yardstick_runs_on_the_fused_launch_geometry(dev, bits, with_x):
    """dz_probe_read: the launch bench.py times beside the fused kernel reads the tiled base weight and
    the packed words of the first D slots with the fused kernel's grid and writes nothing (its sink
    stays as it was)."""
    import ctypes as C
    from deltazip_amd import _lib
    p1 = make_problem(256, 1024, bits, -1, 4, 32, "uniform", 3, dev)
    p2 = make_problem(96, 1024, bits, -1, 4, 32, "uniform", 4, dev)
    tiles = [ops.tile_base(p["wb"]) for p in (p1, p2)]
    sink = torch.full((64,), 7, dtype=torch.int32, device=dev)
    arr = lambda ts: (C.c_void_p * 2)(*[t.data_ptr() for t in ts])
    rc = _lib.lib().dz_probe_read(2, arr([p1["x"], p2["x"]]), arr(tiles), arr([p1["q"], p2["q"]]),
                                  arr([p1["m"], p2["m"]]), (C.c_int * 2)(256, 96), 32, 1024, bits, 4, with_x,
                                  sink.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == 0 and bool((sink == 7).all())


def test_row_blocks_made_once_per_batch(dev):
    """ops.row_blocks(indices, S) made once and passed as `order` to several calls gives, bit for
    bit, what each call gives when it orders the batch itself; blocks of another batch are refused."""
    p = make_problem(256, 1024, 2, -1, 4, 700, "uniform", 5, dev)
    blocks = ops.row_blocks(p["ids"], 4)
    assert blocks.T == 700 and blocks.S == 4 and blocks.perm.dtype == torch.int32
    y0 = run_layer(p)
    for _ in range(2):
        y1 = ops.multi_delta_linear(p["x"], p["wb"], p["q"], p["s"], p["m"], p["ids"], bits=2, order=blocks)
        torch.cuda.synchronize()
        assert torch.equal(y0, y1)
    with pytest.raises(ValueError):
        ops.multi_delta_linear(p["x"][:600], p["wb"], p["q"], p["s"], p["m"], p["ids"][:600].contiguous(), bits=2,
                               order=blocks)
    with pytest.raises(ValueError):
        ops.multi_delta_linear(p["x"][:64], p["wb"], p["q"], p["s"], p["m"], p["ids"][:64].contiguous(), bits=2,
                               order=blocks)


@pytest.mark.parametrize("t,nd", [(129, 3), (256, 40), (300, 4), (512, 17)])
def test_mid_size_batches_go_through_the_fused_kernel_in_chunks(dev, t, nd):
    """Between 129 tokens and a few hundred the matrix-core kernel would leave most of the GPU idle:
    the call is made of chunks of 128 tokens through the fused kernel.  Both routes match the oracle."""
    from deltazip_amd.prefill import multi_delta_linear_prefill
    assert ops.takes_fused_chunks(t, nd) and not ops.takes_fused_chunks(513, 64) and not ops.takes_fused_chunks(400, 4)
    p = make_problem(96, 512, 2, -1, nd, t, "uniform", 77 + t, dev)
    ref = o.forward_ref(p["x_np"], p["wb_np"], p["dts"], p["ids_np"])
    y = run_layer(p)
    assert o.rel_err(y.cpu().numpy(), ref) <= TOL
    y2 = torch.empty_like(y)
    multi_delta_linear_prefill(p["x"], p["wb"], p["q"], p["s"], p["m"], p["ids"], bits=2, out=y2, accumulate=False)
    torch.cuda.synchronize()
    assert o.rel_err(y2.cpu().numpy(), ref) <= TOL
    # in place, delta only, into a column slice: the chunks write their rows of the slice
    wide = torch.zeros(t, 96 + 64, device=dev, dtype=torch.float16)
    ops.add_delta_slice(wide, p["x"], p["q"], None, p["s"], None, p["ids"], 1.0, 32, 96, meta=p["m"])
    torch.cuda.synchronize()
    dref = ref - p["x_np"].astype(np.float32) @ p["wb_np"].astype(np.float32).T
    assert float(wide[:, :32].abs().max()) == 0 and float(wide[:, 128:].abs().max()) == 0
    assert np.abs(wide[:, 32:128].float().cpu().numpy() - dref).max() <= 2e-2 * np.abs(dref).max()


@pytest.mark.parametrize("n,k,bits,gs,nd,t", [(64, 512, 2, -1, 3, 1), (96, 768, 4, 128, 5, 16), (256, 4096, 2, -1, 8, 32),
                                              (160, 1024, 2, 64, 7, 33), (128, 2048, 4, -1, 12, 100), (512, 4096, 2, -1, 9, 128),
                                              (256, 1024, 2, -1, 6, 200)])   # 200 tokens: two chunks through the fused kernel
def test_tiled_base_weight_gives_the_same_bits(dev, n, k, bits, gs, nd, t):
    """The base weight converted to tiles (dz_tile_base) feeds the fused kernel the same operands in the
    same order: outputs equal the row-major call bit for bit, single and batched, and match the oracle.
    The conversion itself is a pure rearrangement (every value kept, at the position dz_layout.h gives)."""
    p = make_problem(n, k, bits, gs, nd, t, "uniform", 3000 + n + t, dev)
    tiled = ops.tile_base(p["wb"])
    w, tl = p["wb_np"], tiled.cpu().numpy().reshape(-1)
    for (np_, kb, s_, j, h, lane) in [(0, 0, 0, 0, 0, 0), (n // 32 - 1, k // 256 - 1, 1, 3, 1, 63), (0, k // 256 - 1, 1, 2, 0, 37)]:
        off = ((np_ * (k // 256) + kb) * 16384 + ((s_ * 4 + j) * 2 + h) * 1024 + lane * 16) // 2
        i, g = lane % 16, lane // 16
        row, col = 32 * np_ + 16 * s_ + i, 256 * kb + 64 * j + 16 * g + 8 * h
        assert np.array_equal(tl[off:off + 8], w[row, col:col + 8])
    assert np.array_equal(np.sort(tl.view(np.uint16)), np.sort(w.reshape(-1).view(np.uint16)))
    y0 = run_layer(p)
    y1 = ops.apply_delta(p["x"], p["q"], p["s"], p["m"], p["ids"], p["wb"], base_tiled=tiled)
    torch.cuda.synchronize()
    assert torch.equal(y0, y1)
    assert o.rel_err(y1.cpu().numpy(), o.forward_ref(p["x_np"], p["wb_np"], p["dts"], p["ids_np"])) <= TOL
    b0 = ops.apply_delta_batch(p["x"], [p["q"]] * 2, [p["s"]] * 2, [p["m"]] * 2, p["ids"], [p["wb"]] * 2)
    b1 = ops.apply_delta_batch(p["x"], [p["q"]] * 2, [p["s"]] * 2, [p["m"]] * 2, p["ids"], [p["wb"]] * 2,
                               base_tiled=[tiled] * 2)
    torch.cuda.synchronize()
    assert torch.equal(b0[0], b1[0]) and torch.equal(b0[1], b1[1])
    with pytest.raises(ValueError):
        ops.apply_delta(p["x"], p["q"], p["s"], p["m"], p["ids"], p["wb"], base_tiled=tiled[:, : k // 2])
    from deltazip_amd import _lib
    assert _lib.lib().dz_tile_base(p["wb"].data_ptr(), k, n, p["wb"].data_ptr(), None) != 0      # not in place
    assert _lib.lib().dz_tile_base(p["wb"].data_ptr(), k - 64, n, tiled.data_ptr(), None) != 0    # whole k-blocks only


def test_tiled_base_weight_wide_launch(dev):
    """12288 output rows (q, k and v of a 4096-wide model fused), split in K: the K split depends on
    the shapes only, so both forms of the base weight give the same bits here, too."""
    p = make_problem(12288, 2048, 2, -1, 4, 24, "uniform", 77, dev)
    ref = o.forward_ref(p["x_np"], p["wb_np"], p["dts"], p["ids_np"])
    y0 = run_layer(p)
    y1 = ops.apply_delta(p["x"], p["q"], p["s"], p["m"], p["ids"], p["wb"], base_tiled=ops.tile_base(p["wb"]))
    torch.cuda.synchronize()
    assert o.rel_err(y0.cpu().numpy(), ref) <= TOL
    assert torch.equal(y0, y1)


def test_fused_layer_calls_replay_from_a_graph(dev):
    """What a serving loop does with a decode step: the layer calls -- a single projection over the
    tiled base weight, two projections in one launch at 64 tokens (token order computed inside the
    call), a split-K launch -- are captured once into a HIP graph and replayed after the ids were
    rewritten in place, with eager work and synchronisations between the replays.  Every replay
    equals the eager call bit for bit: nothing in the path reads back to the host, allocates or
    depends on state a replay would find changed (the split-K workspace is left empty by every launch)."""
    a = make_problem(256, 4096, 2, -1, 6, 24, "uniform", 501, dev)      # split in K
    b = make_problem(160, 1024, 4, 128, 9, 64, "uniform", 502, dev)     # two chunks of tokens, grouped scales
    tiled = ops.tile_base(a["wb"])

    def step():
        y0 = ops.apply_delta(a["x"], a["q"], a["s"], a["m"], a["ids"], a["wb"], base_tiled=tiled)
        y1 = ops.apply_delta_batch(b["x"], [b["q"]] * 2, [b["s"]] * 2, [b["m"]] * 2, b["ids"], [b["wb"]] * 2)
        return y0, y1[0], y1[1]

    step()                                                               # one-time set-up outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            outs = step()
    torch.cuda.current_stream().wait_stream(side)
    rng = np.random.default_rng(5)
    for rep in range(4):
        ia, ib = rng.integers(-1, 6, size=24), rng.integers(-1, 9, size=64)
        if rep == 2:
            ia[:], ib[:] = -1, 3                                         # base only / one delta for every token
        a["ids"].copy_(torch.from_numpy(ia).to(dev))
        b["ids"].copy_(torch.from_numpy(ib).to(dev))
        eager = step()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(outs, eager):
            assert torch.equal(got, want), rep
        assert o.rel_err(outs[0].cpu().numpy(), o.forward_ref(a["x_np"], a["wb_np"], a["dts"], ia)) <= TOL
        assert o.rel_err(outs[2].cpu().numpy(), o.forward_ref(b["x_np"], b["wb_np"], b["dts"], ib)) <= TOL


def test_gemm_grouped(dev):
    """Grouped GEMM through the C ABI: ragged row blocks, a block without second weight, rows that no
    block covers (left untouched), an N that is not a multiple of the 256-wide tile, and the
    second-product-only form (w = NULL)."""
    from deltazip_amd import _lib
    L = _lib.lib()
    torch.manual_seed(1)
    T, K, N, G = 700, 512, 352, 3
    x = torch.randn(T, K, device=dev).half()
    w = (torch.randn(N, K, device=dev) * 0.05).half()
    w2 = (torch.randn(G, N, K, device=dev) * 0.05).half()
    blocks = [(0, 100, -1), (100, 356, 2), (356, 390, 2), (390, 391, 0), (400, 656, 1), (656, 700, 1)]
    tiles = torch.tensor([(lo, hi, g, 0) for lo, hi, g in blocks], dtype=torch.int32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    for with_base in (True, False):
        y = torch.full((T, N), 7.0, dtype=torch.float16, device=dev)
        rc = L.dz_gemm_f16_grouped(x.data_ptr(), w.data_ptr() if with_base else None, w2.data_ptr(), N * K,
                                   tiles.data_ptr(), len(blocks), y.data_ptr(), T, K, N, 0, N, st)
        assert rc == 0
        torch.cuda.synchronize()
        ref = torch.full((T, N), 7.0, dtype=torch.float32, device=dev)
        for lo, hi, g in blocks:
            r = x[lo:hi].float() @ w.float().t() if with_base else None
            if g >= 0:
                d = x[lo:hi].float() @ w2[g].float().t()
                r = d if r is None else r + d
            if r is not None:
                ref[lo:hi] = r
        assert o.rel_err(y.float().cpu().numpy(), ref.cpu().numpy()) <= 2e-3
        assert torch.equal(y[391:400], torch.full((9, N), 7.0, dtype=torch.float16, device=dev))
    # argument checks happen before the launch
    assert L.dz_gemm_f16_grouped(x.data_ptr(), w.data_ptr(), w2.data_ptr(), N * K, None, 1, y.data_ptr(),
                                 T, K, N, 0, N, st) != 0
    assert L.dz_gemm_f16_grouped(x.data_ptr(), w.data_ptr(), w2.data_ptr(), N * K, tiles.data_ptr(), 1,
                                 y.data_ptr(), T, K + 8, N, 0, N, st) != 0


def test_segment_limits(dev):
    ids = torch.zeros(10, dtype=torch.int64, device=dev)
    perm = torch.empty(10, dtype=torch.int32, device=dev)
    from deltazip_amd import _lib
    off = torch.empty(2000, dtype=torch.int32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    assert _lib.lib().dz_segment(ids.data_ptr(), 10, 768, perm.data_ptr(), off.data_ptr(), st) == 0
    assert _lib.lib().dz_segment(ids.data_ptr(), 10, 769, perm.data_ptr(), off.data_ptr(), st) != 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("t", [33, 64, 97, 128])
def test_unsorted_batches_above_32_tokens(dev, t):
    """33..128 tokens in arbitrary order with many deltas: the device-side ordering must bring every
    token back to its own output row."""
    p = make_problem(96, 768, 4, 128, 20, t, "uniform", 4242 + t, dev)
    p["ids_np"][::7] = -1
    p["ids"] = torch.from_numpy(p["ids_np"]).to(dev)
    y = run_layer(p).cpu().numpy()
    ref = o.forward_ref(p["x_np"], p["wb_np"], p["dts"], p["ids_np"])
    assert o.rel_err(y, ref) <= TOL
    assert ops.workspace_status() == 0


@pytest.mark.parametrize("t,kind", [(64, "zipf"), (128, "zipf"), (100, "single"), (77, "uniform")])
def test_dealt_chunks_skewed_mixes_and_many_slots(dev, t, kind):
    """33..128 tokens: the tokens are dealt to the 32-token chunks by delta (popular deltas split,
    rare ones spread); whatever the mix, every token must get its own delta's result in its own
    row -- also with far more slots than the sort used for long batches can take, most of them
    empty."""
    nd = 24
    p = make_problem(64, 512, 2, -1, nd, t, kind, 5150 + t, dev)
    S = 1000                                         # slots; deltas sit in scattered ones
    where = np.random.default_rng(t).choice(S, nd, replace=False)
    q = torch.zeros((S,) + tuple(p["q"].shape[1:]), dtype=p["q"].dtype, device=dev)
    m = torch.zeros((S,) + tuple(p["m"].shape[1:]), dtype=p["m"].dtype, device=dev)
    s = torch.zeros((S,) + tuple(p["s"].shape[1:]), dtype=p["s"].dtype, device=dev)
    idx = torch.from_numpy(where).to(dev)
    q[idx], m[idx], s[idx] = p["q"], p["m"], p["s"]
    ids_np = p["ids_np"].copy()
    slots_np = np.where(ids_np >= 0, where[np.maximum(ids_np, 0)], -1)
    slots_np[5] = -1
    ids_np[5] = -1
    perm = np.random.default_rng(t + 1).permutation(t)          # arbitrary arrival order
    y = ops.apply_delta(p["x"][torch.from_numpy(perm).to(dev)], q, s, m, torch.from_numpy(slots_np[perm]).to(dev),
                        p["wb"])
    torch.cuda.synchronize()
    ref = o.forward_ref(p["x_np"][perm], p["wb_np"], p["dts"], ids_np[perm])
    assert o.rel_err(y.cpu().numpy(), ref) <= TOL
    assert ops.workspace_status() == 0


PREFILL_CASES = [
    # n, k, bits, gs, deltas, tokens, ids
    (256, 1024, 2, -1, 4, 400, "uniform"),
    (352, 768, 4, -1, 3, 129, "uniform"),
    (352, 768, 2, 128, 5, 700, "zipf"),
    (512, 512, 4, 64, 2, 300, "blocks"),
    (96, 256, 2, -1, 9, 1000, "uniform"),
    (288, 1280, 4, 256, 6, 515, "uniform"),
]


@pytest.mark.parametrize("n,k,bits,gs,nd,t,kind", PREFILL_CASES)
def test_packed_delta_gemm_parity(dev, n, k, bits, gs, nd, t, kind):
    """T > 128 through dz_segment + dz_build_tiles + dz_multi_delta_gemm: unsorted ids, tokens
    without a delta, N that is not a multiple of the 256-wide tile, grouped scales, then the
    delta-only and accumulate forms."""
    p = make_problem(n, k, bits, gs, nd, t, kind, 4000 + n + k + t, dev)
    p["ids_np"][::7] = -1
    p["ids"] = torch.from_numpy(p["ids_np"]).to(dev)
    y = run_layer(p)
    ref = o.forward_ref(p["x_np"], p["wb_np"], p["dts"], p["ids_np"])
    assert o.rel_err(y.cpu().numpy(), ref) <= TOL
    # delta only, accumulated onto an existing output (the add_delta form)
    y0 = torch.from_numpy(o.make_x(t, n, 5)).to(dev)
    y1 = y0.clone()
    ops.multi_delta_linear(p["x"], None, p["q"], p["s"], p["m"], p["ids"], bits=bits, out=y1, accumulate=True)
    torch.cuda.synchronize()
    ref_d = o.forward_ref(p["x_np"], None, p["dts"], p["ids_np"]) + y0.float().cpu().numpy()
    assert o.rel_err(y1.cpu().numpy(), ref_d) <= TOL
    # delta only, not accumulated: rows without a delta are zero
    y2 = ops.multi_delta_linear(p["x"], None, p["q"], p["s"], p["m"], p["ids"], bits=bits)
    torch.cuda.synchronize()
    assert (y2[torch.from_numpy(p["ids_np"] < 0).to(dev)] == 0).all()
    assert o.rel_err(y2.cpu().numpy(), o.forward_ref(p["x_np"], None, p["dts"], p["ids_np"])) <= TOL


def test_build_tiles(dev):
    from deltazip_amd import _lib
    L = _lib.lib()
    off = [0, 10, 10, 600, 601, 1113, 1113]          # S = 4: segments of 10, 0, 590, 1, 512, 0 rows
    seg = torch.tensor(off, dtype=torch.int32, device=dev)
    tiles = torch.full((12, 4), 77, dtype=torch.int32, device=dev)
    assert L.dz_build_tiles(seg.data_ptr(), 5, tiles.data_ptr(), 12, torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    got = tiles.cpu().tolist()
    want = [[0, 10, -1, 0], [10, 266, 1, 0], [266, 522, 1, 0], [522, 600, 1, 0], [600, 601, 2, 0],
            [601, 857, 3, 0], [857, 1113, 3, 0]]
    assert got[:7] == want and all(r == [0, 0, -1, 0] for r in got[7:])
    assert L.dz_build_tiles(None, 5, tiles.data_ptr(), 12, None) == -1
    assert L.dz_build_tiles(seg.data_ptr(), 5000, tiles.data_ptr(), 12, None) == -2


@pytest.mark.parametrize("n,k,bits,gs", [(32, 256, 4, -1), (64, 512, 2, -1), (96, 768, 4, 128), (160, 1024, 2, 64),
                                         (256, 2048, 4, 256)])
def test_compressor_matches_reference_pipeline(dev, n, k, bits, gs):
    """dz_compress_2of4 against the oracle's restatement of the reference's pipeline (scales from the
    un-pruned delta, 2:4 by magnitude, quantise, GPTQ pack) followed by the repacker: same bytes.
    Rows that are all zero, rows without a negative value, magnitude ties and values that quantise to
    the zero-point are all present."""
    rng = np.random.default_rng(n + k + bits)
    d = (rng.standard_normal((n, k)) * 1e-3).astype(np.float32)
    d[3] = 0.0                                        # all-zero row: range (-1, 1)
    d[5] = np.abs(d[5])                               # no negative value: range (0, max)
    d[7, :64] = np.float32(2e-3) * rng.integers(-2, 3, 64)   # many exact ties and exact zeros
    d[9] *= 1e-4                                      # tiny values next to ...
    d[9, 17] = 1.0                                    # ... one large one: most codes are the zero-point
    codes, scales16, zeros, keep = o.compress_delta(d, bits, gs)
    qw, qz, sc, gi = o.pack_codes_gptq(codes, zeros, scales16, bits)
    want_c, want_m, want_s = o.repack_native(qw, qz, sc, gi, bits)
    q, m, s = ops.compress_delta(torch.from_numpy(d).to(dev), bits, gs)
    torch.cuda.synchronize()
    assert q.cpu().numpy().view(np.uint32).tobytes() == want_c.tobytes()
    assert m.cpu().numpy().view(np.uint32).tobytes() == want_m.tobytes()
    assert np.array_equal(s.cpu().numpy().view(np.uint16), want_s.view(np.uint16))
    # and it dequantises (on the GPU) to the reference dequantisation of those GPTQ tensors
    got = ops.dequant(q, m, s, k, n, bits).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), np.ascontiguousarray(o.dequant_gptq(qw, qz, sc, gi, bits).T).view(np.uint16))


def test_compressor_argument_checks(dev):
    with pytest.raises(ValueError):
        ops.compress_delta(torch.zeros(32, 256, device=dev, dtype=torch.float16), 4)
    with pytest.raises(NotImplementedError):
        ops.compress_delta(torch.zeros(32, 256, device=dev), 3)
    with pytest.raises(ValueError):
        ops.compress_delta(torch.zeros(32, 200, device=dev), 4)
    with pytest.raises(ValueError):
        ops.compress_delta(torch.zeros(32, 256), 4)


@pytest.mark.parametrize("bits,gs,t,ns,k", [(2, -1, 32, (128, 128, 128), 1024), (4, 128, 7, (64, 256), 1024),
                                            (2, -1, 64, (96, 32, 32, 160), 1024), (4, -1, 128, (64, 64), 1024),
                                            (2, -1, 32, (64, 96), 4096),
                                            # 2-bit deltas with scale groups of 64: the kernel variant under the
                                            # highest register pressure (it once spilled a register that an
                                            # in-flight load was still to fill)
                                            (2, 64, 32, (160, 160), 1024), (2, 64, 102, (96, 96), 768),
                                            (2, 64, 65, (32, 32), 4096), (2, 64, 7, (64, 32), 512)])
def test_batched_calls_equal_separate_calls(dev, bits, gs, t, ns, k):
    """Projections that share the tokens, in one launch: every output is bit for bit what the
    separate call gives when both split K the same way (1024 columns are never split; for 4096
    the split is pinned, since a batch chooses it by the n-pairs of all its calls and the fp32
    partial sums are then added in a different order), and matches the oracle."""
    nd = 5
    if k > 1024:
        ops.set_ksplit(2)
    try:
        _batched_equal_separate(dev, bits, gs, t, ns, k, nd)
    finally:
        ops.set_ksplit(0)
    if k > 1024:     # with the launch's own choice of split: equal within the parity bound
        ps = [make_problem(n, k, bits, gs, nd, t, "uniform", 700 + 10 * j + n, dev) for j, n in enumerate(ns)]
        ys = ops.apply_delta_batch(ps[0]["x"], [p["q"] for p in ps], [p["s"] for p in ps], [p["m"] for p in ps],
                                   ps[0]["ids"], [p["wb"] for p in ps])
        torch.cuda.synchronize()
        for p, y in zip(ps, ys):
            assert o.rel_err(y.cpu().numpy(), o.forward_ref(ps[0]["x_np"], p["wb_np"], p["dts"], ps[0]["ids_np"])) <= TOL


def _batched_equal_separate(dev, bits, gs, t, ns, k, nd):
    ps = [make_problem(n, k, bits, gs, nd, t, "uniform", 700 + 10 * j + n, dev) for j, n in enumerate(ns)]
    ids = ps[0]["ids"]
    ids_np = ps[0]["ids_np"]
    x = ps[0]["x"]
    ys = ops.apply_delta_batch(x, [p["q"] for p in ps], [p["s"] for p in ps], [p["m"] for p in ps], ids,
                               [p["wb"] for p in ps])
    torch.cuda.synchronize()
    for p, y in zip(ps, ys):
        sep = ops.apply_delta(x, p["q"], p["s"], p["m"], ids, p["wb"])
        torch.cuda.synchronize()
        assert torch.equal(y, sep)
        ref = o.forward_ref(ps[0]["x_np"], p["wb_np"], p["dts"], ids_np)
        assert o.rel_err(y.cpu().numpy(), ref) <= TOL
    # one x per projection
    ys2 = ops.apply_delta_batch([p["x"] for p in ps], [p["q"] for p in ps], [p["s"] for p in ps],
                                [p["m"] for p in ps], ids, [p["wb"] for p in ps])
    torch.cuda.synchronize()
    for p, y in zip(ps, ys2):
        assert torch.equal(y, ops.apply_delta(p["x"], p["q"], p["s"], p["m"], ids, p["wb"]))
    with pytest.raises(ValueError):
        ops.apply_delta_batch(x, [ps[0]["q"]] * 5, [ps[0]["s"]] * 5, [ps[0]["m"]] * 5, ids, [ps[0]["wb"]] * 5)


@pytest.mark.parametrize("t,kind", [(33, "uniform"), (64, "zipf"), (128, "uniform"), (20, "uniform")])
def test_token_order_is_a_permutation_and_reusable(dev, t, kind):
    """dz_token_order: a permutation of the tokens in which every delta's tokens are contiguous; passing
    it to the layer call gives bit for bit what the call computes with its own grouping."""
    p = make_problem(64, 512, 4, -1, 12, t, kind, 808 + t, dev)
    order = ops.token_order(p["ids"], 12)
    torch.cuda.synchronize()
    od = order.cpu().numpy()
    assert sorted(od.tolist()) == list(range(t))
    dealt = p["ids_np"][od]
    if t > 32:
        for c in range(0, t, 32):                      # inside a chunk every delta forms one run
            ch = dealt[c:c + 32]
            runs = 1 + int((ch[1:] != ch[:-1]).sum())
            assert runs == len(set(ch.tolist()))
    y0 = ops.apply_delta(p["x"], p["q"], p["s"], p["m"], p["ids"], p["wb"])
    y1 = ops.apply_delta(p["x"], p["q"], p["s"], p["m"], p["ids"], p["wb"], order=order)
    torch.cuda.synchronize()
    assert torch.equal(y0, y1)
    assert o.rel_err(y1.cpu().numpy(), o.forward_ref(p["x_np"], p["wb_np"], p["dts"], p["ids_np"])) <= TOL



def test_batched_calls_after_a_wide_single_call(dev):
    """The arrival counters of a batch must not sit where an earlier, wider call kept partial sums:
    a launch with three K chunks over 1024 rows (384 KiB of partial sums), then a batch whose
    second call follows 128 rows; every result must still match the oracle."""
    wide = make_problem(1024, 3072, 2, -1, 2, 31, "uniform", 41, dev)
    try:
        ops.set_ksplit(3)
        ref = o.forward_ref(wide["x_np"], wide["wb_np"], wide["dts"], wide["ids_np"])
        assert o.rel_err(run_layer(wide).cpu().numpy(), ref) <= TOL
        ops.set_ksplit(4)
        k, nd, t = 2048, 5, 32
        ns = (128, 96, 32, 160)
        ps = [make_problem(n, k, 2, -1, nd, t, "uniform", 900 + 10 * j + n, dev) for j, n in enumerate(ns)]
        ids, x = ps[0]["ids"], ps[0]["x"]
        ys = ops.apply_delta_batch(x, [p["q"] for p in ps], [p["s"] for p in ps], [p["m"] for p in ps], ids,
                                   [p["wb"] for p in ps])
        torch.cuda.synchronize()
        for p, y in zip(ps, ys):
            ref = o.forward_ref(ps[0]["x_np"], p["wb_np"], p["dts"], ps[0]["ids_np"])
            assert o.rel_err(y.cpu().numpy(), ref) <= TOL
    finally:
        ops.set_ksplit(0)
