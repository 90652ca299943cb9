"""Pins the oracle's dequantisation and forward (reference: qlinear_cuda.py:246-329,
quant_linear_naive.py:39-83, deltazip_marlin.py:10-53, utils/generate.py:9-20)."""
import numpy as np
import pytest
import torch

from oracle import dz_oracle as o


def _all_finite_fp16():
    bits = np.arange(0, 1 << 16, dtype=np.uint16)
    v = bits.view(np.float16)
    return v[np.isfinite(v)]


@pytest.mark.parametrize("bits", [2, 4])
def test_dequant_exhaustive_scales(bits):
    """fp16(scale) * (q - zero) for every finite fp16 scale and every code: the oracle must equal
    the exactly rounded product (computed in float64, where it is exact, then rounded once)."""
    scales = _all_finite_fp16()
    assert scales.size == 63488
    n = scales.size - scales.size % 32          # N must be a multiple of 32
    scales = scales[:n]
    maxq = 2 ** bits - 1
    zp = 2 ** (bits - 1)
    pf = 32 // bits
    # K = pf rows so that each code value appears (repeat to fill)
    k = 32
    codes = (np.arange(k)[:, None] % (maxq + 1)).astype(np.uint8).repeat(n, axis=1)
    qw, qz, sc, gi = o.pack_codes_gptq(codes, np.full((1, n), zp), scales.reshape(1, n), bits)
    got = o.dequant_gptq(qw, qz, sc, gi, bits)
    with np.errstate(over="ignore"):
        exact = (scales.astype(np.float64)[None, :] * (codes.astype(np.float64) - zp)).astype(np.float16)
    assert np.array_equal(got.view(np.uint16), exact.view(np.uint16))
    # and torch's own fp16 x int8 product (what the reference executes) agrees
    t = (torch.from_numpy(scales.copy()).reshape(1, n) * torch.from_numpy((codes.astype(np.int8) - zp))).numpy()
    assert np.array_equal(got.view(np.uint16), t.view(np.uint16))


def test_dequant_keeps_subnormals_and_zero():
    s = np.array([[6e-8, 5.96e-8, 1e-7, 6.1e-5] * 8], dtype=np.float16)    # subnormal scales
    codes = np.tile(np.array([[0], [1], [2], [3]] * 8, dtype=np.uint8), (1, 32))
    qw, qz, sc, gi = o.pack_codes_gptq(codes, np.full((1, 32), 2), s, 2)
    d = o.dequant_gptq(qw, qz, sc, gi, 2)
    assert np.all(d[2::4] == 0) and not np.any(np.signbit(d[2::4]))         # code == zero -> +0.0
    assert np.array_equal(d[3::4].view(np.uint16), np.tile(s, (8, 1)).view(np.uint16))
    assert np.array_equal(d[0::4], (-2 * np.tile(s, (8, 1)).astype(np.float32)).astype(np.float16))


def _small_problem(bits, gs, seed, n=32, k=256, nd=3, t=7):
    dts = []
    for d in range(nd):
        dl = o.make_delta(n, k, 1e-3, bits, gs, seed + 1 + d)
        dts.append(o.dequant_gptq(dl["qweight"], dl["qzeros"], dl["scales"], dl["g_idx"], bits))
    wb = o.make_base(n, k, seed)
    x = o.make_x(t, k, seed + 500)
    return x, wb, dts


@pytest.mark.parametrize("bits,gs", [(2, -1), (4, -1), (4, 128)])
def test_forward_ref_matches_token_loop(bits, gs):
    x, wb, dts = _small_problem(bits, gs, 11)
    ids = np.array([2, -1, 0, 2, 1, -1, 0], dtype=np.int64)
    y = o.forward_ref(x, wb, dts, ids)
    y64 = o.forward_token_loop(x, wb, dts, ids)
    assert np.max(np.abs(y - y64)) < 1e-5 * np.max(np.abs(y64))
    # order of tokens does not matter
    p = np.array([6, 5, 4, 3, 2, 1, 0])
    assert np.array_equal(o.forward_ref(x[p], wb, dts, ids[p]), y[p])


def test_forward_special_cases():
    x, wb, dts = _small_problem(4, -1, 12)
    t = x.shape[0]
    base = torch.nn.functional.linear(torch.from_numpy(x).float(), torch.from_numpy(wb).float()).numpy()
    assert np.allclose(o.forward_ref(x, wb, dts, np.full(t, -1)), base, rtol=0, atol=1e-6)
    # a delta whose codes all equal the zero-point is the base layer
    zero_delta = np.zeros_like(dts[0])
    assert np.allclose(o.forward_ref(x, wb, [zero_delta], np.zeros(t, np.int64)), base, rtol=0, atol=1e-6)
    # one delta for all tokens = one merged GEMM
    merged = wb.astype(np.float32) + dts[1].T.astype(np.float32)
    y = o.forward_ref(x, wb, dts, np.ones(t, np.int64))
    assert np.allclose(y, x.astype(np.float32) @ merged.T, rtol=1e-5, atol=1e-6)
    # delta only
    yd = o.forward_ref(x, None, dts, np.array([0, 1, 2, -1, 0, 1, 2]))
    assert np.all(yd[3] == 0)
    assert np.allclose(yd[0], x[0].astype(np.float32) @ dts[0].astype(np.float32), rtol=1e-5, atol=1e-7)
