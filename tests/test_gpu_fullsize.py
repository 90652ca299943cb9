"""Parity at the benchmark's full layer shapes (Llama-2-7B / 13B projections), on the deltas the
benchmark configurations describe: drawn from N(0, sigma), scales from the un-pruned values, pruned
2:4 by magnitude, quantised (compressed on the GPU by ops.compress_delta; sampled rows of the result
are held against the CPU restatement of that pipeline, bit for bit).

The CPU oracle cannot dequantise and multiply whole 4096 x 11008 layers in seconds, so each case is
checked three ways:
  * sampled blocks of 32 output rows: the GPU dequantisation is compared bit for bit with the
    oracle's, and the layer output at those columns with the oracle's fp32 forward;
  * the whole output against an fp32 reconstruction on the GPU that uses the (sample-verified)
    dequantised deltas: x.float() @ (W_base.float() + delta.float()).T per delta id;
  * size-independent properties: a batch of id -1 equals the base product; permuting the tokens
    permutes the output rows bit for bit.
"""
import numpy as np
import pytest
import torch

from oracle import dz_oracle as o
from deltazip_amd import ops
from deltazip_amd.synthetic import gaussian_native_stack

pytestmark = pytest.mark.gpu
TOL = 1e-2   # max relative error of fp16 outputs against the fp32 reference (floor 1e-3 * max|ref|)

# K, N, bits, group_size, slots, tokens, ids
CASES = [
    # configuration 1: one token, one 4-bit delta
    pytest.param(4096, 4096, 4, -1, 1, 1, "single", id="cfg1-7b-4096x4096-4bit-T1"),
    # configuration 2 (the headline): Llama-2-7B projections, 32 tokens, 8 deltas of 2 bits
    pytest.param(4096, 4096, 2, -1, 8, 32, "uniform", id="cfg2-7b-4096x4096-2bit-T32-D8"),
    pytest.param(4096, 11008, 2, -1, 8, 32, "uniform", id="cfg2-7b-4096x11008"),
    pytest.param(11008, 4096, 2, -1, 8, 32, "uniform", id="cfg2-7b-11008x4096"),
    pytest.param(4096, 12288, 2, -1, 8, 32, "uniform", id="cfg2-7b-fused-qkv"),
    # configuration 3: the same three shapes, 64 tokens, 32 deltas of 4 bits with group size 128, Zipf ids
    pytest.param(4096, 4096, 4, 128, 32, 64, "zipf", id="cfg3-7b-4096x4096-4bit-g128-T64-D32-zipf"),
    pytest.param(4096, 11008, 4, 128, 32, 64, "zipf", id="cfg3-7b-4096x11008-4bit-g128-T64-D32-zipf"),
    pytest.param(11008, 4096, 4, 128, 32, 64, "zipf", id="cfg3-7b-11008x4096-4bit-g128-T64-D32-zipf"),
    # configuration 4: Llama-2-13B prefill, 16 requests of 512 tokens, one 2-bit delta each
    pytest.param(5120, 5120, 2, -1, 16, 8192, "blocks", id="cfg4-13b-5120x5120-prefill-T8192-D16"),
    pytest.param(5120, 13824, 2, -1, 16, 8192, "blocks", id="cfg4-13b-5120x13824-prefill-T8192-D16"),
    pytest.param(13824, 5120, 2, -1, 16, 8192, "blocks", id="cfg4-13b-13824x5120-prefill-T8192-D16"),
    # configuration 5: Llama-2-7B projections at 128 tokens with 64 resident 2-bit deltas (the whole
    # decode step of that configuration is tests/test_llama_step.py)
    pytest.param(4096, 4096, 2, -1, 64, 128, "uniform", id="cfg5-7b-4096x4096-T128-D64"),
    pytest.param(4096, 11008, 2, -1, 64, 128, "uniform", id="cfg5-7b-4096x11008-T128-D64"),
    pytest.param(11008, 4096, 2, -1, 64, 128, "uniform", id="cfg5-7b-11008x4096-T128-D64"),
    # further shapes outside the configurations: 13B layers at decode sizes
    pytest.param(5120, 5120, 2, -1, 64, 128, "uniform", id="13b-5120x5120-T128-D64"),
    pytest.param(13824, 5120, 4, -1, 4, 16, "uniform", id="13b-down-4bit-T16"),
    # Llama-2-70B MLP layers (one tensor-parallel rank would hold a slice; the whole layer is the larger case)
    pytest.param(8192, 28672, 4, 128, 2, 100, "uniform", id="70b-8192x28672-4bit-g128-T100"),
    pytest.param(28672, 8192, 2, -1, 3, 32, "uniform", id="70b-28672x8192-2bit-T32"),
]


def _native_views(q, m, s, K, N, bits):
    """numpy views of one slot's tensors shaped as the oracle's native arrays."""
    qn = q.cpu().numpy().view(np.uint32)
    mn = m.cpu().numpy().view(np.uint32)
    codes = qn.reshape(N // 32, K // 256, 64, 4) if bits == 2 else qn.reshape(N // 32, K // 256, 2, 64, 4)
    meta = mn.reshape(N // 32, K // 256, 64, 4)
    return codes, meta, s.cpu().numpy()


def _ids(kind, t, nd, seed):
    if kind == "blocks":
        return np.repeat(np.arange(nd, dtype=np.int64), t // nd)
    ids = o.make_ids(kind, t, nd, seed)
    return np.sort(ids)


@pytest.mark.parametrize("K,N,bits,gs,nd,T,kind", CASES)
def test_full_size_layer(dev, K, N, bits, gs, nd, T, kind):
    gen = torch.Generator(device=dev).manual_seed(K + N + bits + T)
    ids_np = _ids(kind, T, nd, K + T)
    if T > 2:
        ids_np[0] = -1
    first = int(min(d for d in ids_np if d >= 0))
    sigma = 2e-3 if T == 1 else 1e-3          # configuration 1 draws its delta from N(0, 2e-3)
    q, m, s, fp32 = gaussian_native_stack(K, N, bits, gs, nd, dev, gen, sigma, keep_deltas=(first,))
    wb = (torch.randn((N, K), device=dev, generator=gen) * 0.02).half()
    x = torch.randn((T, K), device=dev, generator=gen).half()
    ids = torch.from_numpy(ids_np).to(dev)
    y = ops.apply_delta(x, q, s, m, ids, wb)
    torch.cuda.synchronize()
    assert ops.workspace_status() == 0

    present = [int(d) for d in np.unique(ids_np) if d >= 0]
    # ---- sampled 32-row blocks against the CPU oracle
    blocks = sorted({0, (N // 32) // 3, N // 32 - 1})
    rows = np.concatenate([np.arange(32 * b, 32 * b + 32) for b in blocks])
    check = present[:3] + present[-1:]
    dts = {}
    for d in sorted(set(check)):
        codes, meta, sc = _native_views(q[d], m[d], s[d], K, N, bits)
        ref = o.dequant_native(codes[blocks], meta[blocks], np.ascontiguousarray(sc[:, rows]), K, 32 * len(blocks), bits)
        got = ops.dequant(q[d], m[d], s[d], K, N, bits)[torch.from_numpy(rows).to(dev)].cpu().numpy()
        assert np.array_equal(got.view(np.uint16), ref.view(np.uint16)), f"dequant differs for slot {d}"
        dts[d] = ref
        if d in fp32:
            # the same rows through the CPU restatement of the reference's pipeline (scales from the
            # un-pruned delta, 2:4 by magnitude, round to nearest, pack, dequantise)
            rows_d = fp32[d][torch.from_numpy(rows).to(dev)].cpu().numpy()
            codes_o, sc_o, zeros_o, _ = o.compress_delta(rows_d, bits, gs)
            qw_o, qz_o, sc16_o, gidx_o = o.pack_codes_gptq(codes_o, zeros_o, sc_o, bits)
            want = o.dequant_gptq(qw_o, qz_o, sc16_o, gidx_o, bits)        # [K, rows]
            assert np.array_equal(got.view(np.uint16), np.ascontiguousarray(want.T).view(np.uint16)), \
                f"compressed delta of slot {d} differs from the CPU pipeline"
    del fp32
    tok = np.nonzero(np.isin(ids_np, list(dts.keys()) + [-1]))[0][:64]
    xs = x[torch.from_numpy(tok).to(dev)].cpu().numpy().astype(np.float32)
    wbs = wb[torch.from_numpy(rows).to(dev)].cpu().numpy().astype(np.float32)
    ref = np.empty((len(tok), len(rows)), np.float32)
    for r, t in enumerate(tok):
        w = wbs + dts[int(ids_np[t])].astype(np.float32) if ids_np[t] >= 0 else wbs
        ref[r] = w @ xs[r]
    got = y[torch.from_numpy(tok).to(dev)][:, torch.from_numpy(rows).to(dev)].cpu().numpy()
    assert o.rel_err(got, ref) <= TOL

    # ---- whole output against an fp32 reconstruction on the GPU
    yref = torch.empty((T, N), dtype=torch.float32, device=dev)
    xf = x.float()
    for d in [-1] + present:
        sel = (ids == d).nonzero().flatten()
        if sel.numel() == 0:
            continue
        w = wb.float()
        if d >= 0:
            w = w + ops.dequant(q[d], m[d], s[d], K, N, bits).float()
        yref[sel] = xf[sel] @ w.t()
        del w
    err = ((y.float() - yref).abs() / yref.abs().clamp_min(1e-3 * yref.abs().max())).max().item()
    assert err <= TOL

    if T > 128:
        return
    # ---- properties
    none = torch.full_like(ids, -1)
    yb = ops.apply_delta(x, q, s, m, none, wb)
    yb_ref = xf @ wb.float().t()
    errb = ((yb.float() - yb_ref).abs() / yb_ref.abs().clamp_min(1e-3 * yb_ref.abs().max())).max().item()
    assert errb <= TOL
    perm = torch.randperm(T, device=dev, generator=gen)
    yp = ops.apply_delta(x[perm].contiguous(), q, s, m, ids[perm].contiguous(), wb)
    assert torch.equal(yp, y[perm])
    # ---- the tiled copy of the base weight (what the delta layers read at these sizes): the same
    # products in the same order and the same K split, so the same bits
    yt = ops.apply_delta(x, q, s, m, ids, wb, base_tiled=ops.tile_base(wb))
    assert torch.equal(yt, y)
