"""Hessian-aware compression on the GPU (dz_hessian_add, dz_obs_sweep, dz_quant_scales,
dz_pack_2of4 through the C ABI) against the oracle's restatement of
deltazip/core/sparsegpt.py:25-146: bit for bit, since both sum in the same order."""
import numpy as np
import pytest
import torch

from oracle import dz_oracle as o
from deltazip_amd import ops
from deltazip_amd.sparsegpt import Quantizer, SparseGPT

pytestmark = pytest.mark.gpu


def _inputs(n, k, tokens, seed):
    rng = np.random.default_rng(seed)
    W = (rng.standard_normal((n, k)) * 0.01).astype(np.float32)
    X = rng.standard_normal((tokens, k)).astype(np.float32)
    X = (X + 0.5 * np.roll(X, 1, axis=1)).astype(np.float16)       # layer inputs are fp16
    return W, X


def test_hessian_add_bit_exact(dev):
    k = 256
    _, xa = _inputs(4, k, 3 * 40, 1)
    _, xb = _inputs(4, k, 77, 2)
    H = torch.zeros(k, k, dtype=torch.float32, device=dev)
    n = ops.hessian_add(H, torch.from_numpy(xa).to(dev), 0, 3)            # 3 samples of 40 tokens
    n = ops.hessian_add(H, torch.from_numpy(xb).float().to(dev), n, 1)    # one more, passed as fp32
    torch.cuda.synchronize()
    Href, nref = o.hessian_add_batch_ref(np.zeros((k, k), np.float32), 0, xa.reshape(3, 40, k))
    Href, nref = o.hessian_add_batch_ref(Href, nref, xb)
    assert n == nref == 4
    assert np.array_equal(H.cpu().numpy(), Href)


@pytest.mark.parametrize("n,k,bits,quant,prune", [(32, 256, 4, True, (2, 4)), (64, 384, 2, True, (2, 4)),
                                                  (32, 256, 4, False, (2, 4)), (40, 256, 4, True, (0, 0)),
                                                  (32, 256, 4, True, (4, 8)), (33, 128, 2, True, (1, 2)),
                                                  (256, 1024, 4, True, (2, 4))])
def test_obs_sweep_bit_exact(dev, n, k, bits, quant, prune):
    W, X = _inputs(n, k, 1024, 10 + n + k + bits)
    H, _ = o.hessian_add_batch_ref(np.zeros((k, k), np.float32), 0, X[:256] if k > 512 else X)
    if k > 512:
        H = H + np.eye(k, dtype=np.float32)                 # fewer samples than columns: keep it well conditioned
    hinv, W0 = o.hinv_upper_ref(H, W)
    scale, _ = o.find_params_sym(W, bits)
    sc = scale[:, 0].copy() if quant else None
    pn, pm = prune
    want, want_loss = o.obs_sweep_ref(W0, hinv, sc, bits, pn, pm)
    Wd = torch.from_numpy(W0.copy()).to(dev)
    loss = ops.obs_sweep(Wd, torch.from_numpy(hinv).to(dev), torch.from_numpy(sc).to(dev) if quant else None,
                         bits, pn, pm)
    torch.cuda.synchronize()
    assert np.array_equal(Wd.cpu().numpy(), want)
    assert np.array_equal(loss.cpu().numpy(), want_loss)


@pytest.mark.parametrize("n,k,bits,gs", [(64, 512, 4, -1), (96, 1024, 2, -1), (32, 512, 4, 128), (64, 256, 2, 64)])
def test_scales_with_the_search_over_the_clipping_range(dev, n, k, bits, gs):
    """dz_quant_scales_mse against the oracle's restatement of quant.py:85-101.  The candidates'
    errors are sums of |d| ** 2.4 whose last bits depend on the pow routine and the order of the
    sum, so where two candidates are within 1e-5 of each other either may win; everywhere else the
    chosen scale is the oracle's, bit for bit."""
    W, _ = _inputs(n, k, 8, 40 + n + bits)
    W[3, 5] = 25 * np.abs(W).max()                                # a row with an outlier
    W[7] = 0                                                      # an all-zero row
    W[9] = np.abs(W[9])                                           # a row without a negative value
    s32, s16 = ops.quant_scales(torch.from_numpy(W).to(dev), bits, gs, mse=True)
    scale, _, errs = o.find_params_sym(W, bits, gs, mse=True, return_errors=True)      # [N, G], [80, N, G]
    plain, _ = o.find_params_sym(W, bits, gs)
    got = s32.cpu().numpy().T                                                            # [N, G]
    assert got.shape == scale.shape
    differ = got != scale
    assert differ.mean() < 0.05
    for r, g in zip(*np.nonzero(differ)):
        cand = np.array([np.float32(np.float32(1 - i / 100) * plain[r, g]) for i in range(80)])
        i_got = int(np.argmin(np.abs(cand - got[r, g])))
        assert abs(cand[i_got] - got[r, g]) <= 1e-6 * got[r, g]                          # one of the candidates ...
        assert errs[i_got, r, g] <= errs[:, r, g].min() * (1 + 1e-5)                     # ... and as good as the best
    assert (got <= plain).all() and (got < plain).any()           # the search only ever shrinks the range
    assert np.array_equal(s16.cpu().numpy().view(np.uint16), s32.cpu().numpy().astype(np.float16).view(np.uint16))
    # the Quantizer front end with the reference's keywords
    from deltazip_amd.sparsegpt import Quantizer
    qz = Quantizer()
    qz.configure(bits, perchannel=True, sym=True, mse=True, norm=2.4, grid=100, maxshrink=0.8)
    qz.find_params(torch.from_numpy(W).to(dev), weight=True)
    if gs == -1:
        assert torch.equal(qz.scale[:, 0], s32[0]) and float(qz.zero[0, 0]) == 2 ** (bits - 1)


def test_scales_and_pack_match_the_reference_pipeline(dev):
    """Values on the grid with two zeros per group of four -> the same native bytes as compressing
    and packing the reference's way (oracle) and converting with the repacker."""
    n, k, bits = 64, 512, 4
    W, X = _inputs(n, k, 512, 3)
    s32, s16 = ops.quant_scales(torch.from_numpy(W).to(dev), bits)
    scale, zero = o.find_params_sym(W, bits)
    assert np.array_equal(s32.cpu().numpy()[0], scale[:, 0])
    assert np.array_equal(s16.cpu().numpy()[0].view(np.uint16), scale[:, 0].astype(np.float16).view(np.uint16))
    H, _ = o.hessian_add_batch_ref(np.zeros((k, k), np.float32), 0, X)
    hinv, W0 = o.hinv_upper_ref(H, W)
    out, _ = o.obs_sweep_ref(W0, hinv, scale[:, 0], bits)
    q, m = ops.pack_2of4(torch.from_numpy(out).to(dev), s32, bits)
    torch.cuda.synchronize()
    codes = o.quantize_codes(out, scale, zero, 2**bits - 1)                    # [N, K]
    qw, qz, sc16, gi = o.pack_codes_gptq(np.ascontiguousarray(codes.T), zero.T.astype(np.int32),
                                         scale.T.astype(np.float16), bits)
    rq, rm, rs = ops.repack_gptq_to_native(torch.from_numpy(qw), torch.from_numpy(qz), torch.from_numpy(sc16),
                                           torch.from_numpy(gi), bits)
    assert torch.equal(q.cpu(), rq) and torch.equal(m.cpu(), rm)
    # and the packed delta dequantises to the swept values rounded to fp16 the reference's way
    dq = ops.dequant(q, m, s16, k, n, bits).cpu().numpy()
    assert np.array_equal(dq, o.dequant_gptq(qw, qz, sc16, gi, bits).T)


def test_sparsegpt_interface_end_to_end(dev):
    """SparseGPT(layer).add_batch / fasterprune / pack with the reference's call sequence
    (deltazip/modeling/_base.py:399-470): the layer ends up holding base + compressed delta, the
    compensation lowers the layer's output error below plain magnitude pruning + rounding."""
    n, k, bits = 64, 256, 4
    rng = np.random.default_rng(7)
    base = (rng.standard_normal((n, k)) * 0.02).astype(np.float16)
    delta, X = _inputs(n, k, 2048, 8)
    target = (base.astype(np.float32) + delta).astype(np.float16)
    layer = torch.nn.Linear(k, n, bias=False, dtype=torch.float16, device=dev)
    layer.weight.data = torch.from_numpy(target).to(dev)
    gpt = SparseGPT(layer)
    gpt.quantizer = Quantizer()
    gpt.quantizer.configure(bits, perchannel=True, sym=True, mse=False)
    xs = torch.from_numpy(X).to(dev)
    for i in range(0, 2048, 512):
        gpt.add_batch(xs[i:i + 512].reshape(4, 128, k), None)
    assert gpt.nsamples == 16
    scale, zero, g_idx, avg_loss, Wc = gpt.fasterprune(0.5, prunen=2, prunem=4, base_weight=torch.from_numpy(base).to(dev))
    torch.cuda.synchronize()
    assert tuple(scale.shape) == (n, 1) and float(zero[0, 0]) == 8 and int(g_idx.abs().sum()) == 0 and avg_loss > 0
    d32 = target.astype(np.float32) - base.astype(np.float32)
    got = Wc.float().cpu().numpy()
    assert ((got.reshape(n, -1, 4) == 0).sum(axis=2) >= 2).all()
    sc, zr = o.find_params_sym(d32, bits)
    plain = o.quantize(np.where(o.prune_2of4_magnitude(d32), d32, np.float32(0)), sc, zr, 15)
    xf = X.astype(np.float32)
    assert np.linalg.norm((d32 - got) @ xf.T) < 0.95 * np.linalg.norm((d32 - plain) @ xf.T)
    assert torch.equal(layer.weight.data, (Wc + torch.from_numpy(base).to(dev)).half())
    q, m, s16 = gpt.pack()
    dq = ops.dequant(q, m, s16, k, n, bits).float().cpu().numpy()
    assert np.allclose(dq, got, rtol=2e-3, atol=1e-7)
    gpt.free()
    with pytest.raises(NotImplementedError):
        SparseGPT(layer).fasterprune(0.5)                       # unstructured sparsity
    with pytest.raises(NotImplementedError):
        SparseGPT(layer).fasterprune(0.0, actorder=True)
