"""Pins the oracle's GPTQ-style packing (reference: deltazip/nn_modules/qlinear_cuda.py:144-264)
against hand-packed words, single-bit probes and round trips."""
import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from oracle import dz_oracle as o


def _pack_one_column(codes, bits, zero):
    k = len(codes)
    n = 32 // bits  # qzeros needs N % pf == 0
    c = np.tile(np.asarray(codes, dtype=np.uint8).reshape(k, 1), (1, n))
    return o.pack_codes_gptq(c, np.full((1, n), zero), np.ones((1, n), np.float16), bits)


def test_known_words_4bit():
    # codes k = 0..7, lowest nibble = k = 0: 0x0F887988 computed by hand
    qw, qz, _, g_idx = _pack_one_column([8, 8, 9, 7, 8, 8, 15, 0], 4, 8)
    assert qw.view(np.uint32)[0, 0] == 0x0F887988
    assert qz.view(np.uint32)[0, 0] == 0x77777777      # stores zero - 1 = 7 in every nibble
    assert g_idx.tolist() == [0] * 8


def test_known_words_2bit():
    qw, qz, _, _ = _pack_one_column([2, 2, 3, 1, 2, 2, 0, 3, 2, 2, 2, 2, 1, 3, 2, 2], 2, 2)
    assert qw.view(np.uint32)[0, 0] == 0xADAACA7A
    assert qw[0, 0] == -1381315974                      # stored as int32
    assert qz.view(np.uint32)[0, 0] == 0x55555555


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_single_bit_probes(bits):
    """code[k, n] = 1 must set exactly bit bits*(k mod pf) of word [k // pf, n]."""
    pf = 32 // bits
    k, n = 2 * pf, pf
    for kk in range(k):
        for nn in (0, n - 1):
            codes = np.zeros((k, n), dtype=np.uint8)
            codes[kk, nn] = 1
            qw, _, _, _ = o.pack_codes_gptq(codes, np.ones((1, n), dtype=np.int32), np.ones((1, n), np.float16), bits)
            expect = np.zeros((k // pf, n), dtype=np.uint32)
            expect[kk // pf, nn] = np.uint32(1) << np.uint32(bits * (kk % pf))
            assert np.array_equal(qw.view(np.uint32), expect)


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_all_codes_round_trip(bits):
    pf = 32 // bits
    maxq = 2 ** bits - 1
    k, n = 4 * pf, 2 * pf
    rng = np.random.default_rng(0)
    codes = rng.integers(0, maxq + 1, size=(k, n)).astype(np.uint8)
    codes[: maxq + 1, 0] = np.arange(maxq + 1)[: k][: maxq + 1] if maxq + 1 <= k else codes[: maxq + 1, 0]
    zeros = rng.integers(1, maxq + 2, size=(2, n)).astype(np.int32)   # zero-1 must fit the field
    qw, qz, sc, g_idx = o.pack_codes_gptq(codes, zeros, np.ones((2, n), np.float16), bits)
    c2, z2 = o.unpack_gptq(qw, qz, bits)
    assert np.array_equal(c2.astype(np.int32), codes.astype(np.int32))
    assert np.array_equal(z2.astype(np.int32), zeros)
    assert g_idx.tolist() == [0] * (k // 2) + [1] * (k // 2)


@settings(max_examples=30, deadline=None)
@given(st.integers(1, 4), st.integers(1, 4), st.sampled_from([2, 4]), st.integers(0, 2 ** 31 - 1))
def test_random_round_trip(kf, nf, bits, seed):
    k, n = 32 * kf, 32 * nf
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 2 ** bits, size=(k, n)).astype(np.uint8)
    zeros = np.full((1, n), 2 ** (bits - 1), dtype=np.int32)
    qw, qz, _, _ = o.pack_codes_gptq(codes, zeros, np.ones((1, n), np.float16), bits)
    assert qw.shape == (k * bits // 32, n) and qz.shape == (1, n * bits // 32)
    c2, z2 = o.unpack_gptq(qw, qz, bits)
    assert np.array_equal(c2, codes.astype(c2.dtype)) and np.all(z2 == 2 ** (bits - 1))


@pytest.mark.parametrize("bits", [2, 4])
def test_pack_from_weights_recovers_codes(bits):
    """QuantLinear.pack starts from dequantised fp32 weights (qlinear_cuda.py:161-168); rounding
    (W + zero*scale) / half(scale) must give back the integer codes."""
    rng = np.random.default_rng(3)
    d = (rng.standard_normal((32, 64)) * 1e-3).astype(np.float32)
    scale, zero = o.find_params_sym(d, bits)
    codes, scales16, zeros, keep = o.compress_delta(d, bits)
    w_deq = o.quantize(np.where(keep, d, 0), scale, zero, 2 ** bits - 1)
    a = o.pack_from_weights(w_deq, scale, zero, bits)
    b = o.pack_codes_gptq(codes, zeros, scales16, bits)
    for x, y in zip(a, b):
        assert np.array_equal(x, y)
