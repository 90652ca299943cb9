"""Pins the oracle's quantizer and 2:4 mask (reference: deltazip/core/quant.py:9-18, 48-130;
deltazip/core/sparsegpt.py:117-135 with H = I) against closed forms and brute force."""
import itertools

import numpy as np
import pytest

from oracle import dz_oracle as o


def test_closed_form_4bit():
    row = np.array([[0.003, -0.001, 0.0005, -0.0029]], dtype=np.float32)
    scale, zero = o.find_params_sym(row, 4)
    assert zero[0, 0] == 8
    assert scale[0, 0] == np.float32(np.float32(0.006) / np.float32(15))      # 2*max|row|/15
    # 0.003/scale = 7.5 -> half-to-even 8 -> +8 = 16 -> clamp 15
    assert o.quantize_codes(row, scale, zero, 15).tolist() == [[15, 5, 9, 1]]


def test_closed_form_2bit():
    row = np.array([[0.003, -0.001, 0.0005, -0.0029]], dtype=np.float32)
    scale, zero = o.find_params_sym(row, 2)
    assert zero[0, 0] == 2 and scale[0, 0] == np.float32(np.float32(0.006) / np.float32(3))
    codes = o.quantize_codes(row, scale, zero, 3)
    assert codes.tolist() == [[3, 2, 2, 1]]
    deq = o.quantize(row, scale, zero, 3)
    assert np.allclose(deq, [[scale[0, 0], 0, 0, -scale[0, 0]]])


def test_all_zero_row_uses_unit_range():
    scale, zero = o.find_params_sym(np.zeros((1, 8), np.float32), 4)
    assert scale[0, 0] == np.float32(2.0 / 15) and zero[0, 0] == 8          # (xmin, xmax) = (-1, +1)


def test_all_non_negative_row_keeps_xmin_zero():
    # quant.py:74-76 mirrors the range only when the row has a negative entry
    row = np.array([[0.0, 0.25, 0.5, 1.0]], dtype=np.float32)
    scale, zero = o.find_params_sym(row, 4)
    assert scale[0, 0] == np.float32(1.0 / 15) and zero[0, 0] == 8
    # the top of the range clips: 1.0/scale = 15 -> +8 -> clamp 15 -> dequant 7*scale
    assert o.quantize_codes(row, scale, zero, 15)[0, 3] == 15


@pytest.mark.parametrize("bits", [2, 4])
def test_quantize_idempotent_and_bounded(bits):
    rng = np.random.default_rng(1)
    w = (rng.standard_normal((16, 64)) * 2e-3).astype(np.float32)
    scale, zero = o.find_params_sym(w, bits)
    maxq = 2 ** bits - 1
    q1 = o.quantize(w, scale, zero, maxq)
    q2 = o.quantize(q1, scale, zero, maxq)
    assert np.array_equal(q1, q2)
    lo, hi = -zero * scale, (maxq - zero) * scale
    inside = (w >= lo) & (w <= hi)
    assert np.all(np.abs(q1 - w)[inside] <= scale.repeat(64, 1)[inside] * 0.5000001)


def test_group_scales_equal_per_group_rows():
    rng = np.random.default_rng(2)
    w = (rng.standard_normal((4, 256)) * 1e-3).astype(np.float32)
    sg, zg = o.find_params_sym(w, 4, 128)
    for g in range(2):
        s1, _ = o.find_params_sym(w[:, 128 * g:128 * (g + 1)], 4)
        assert np.array_equal(sg[:, g], s1[:, 0])


def test_mask_brute_force_and_ties():
    # every ordering of 4 distinct magnitudes: keep the two largest
    for perm in itertools.permutations([1.0, 2.0, 3.0, 4.0]):
        for signs in itertools.product([1, -1], repeat=4):
            row = np.array([[p * s for p, s in zip(perm, signs)]], dtype=np.float32)
            keep = o.prune_2of4_magnitude(row)[0]
            assert sorted(np.abs(row[0])[keep].tolist()) == [3.0, 4.0]
    # ties keep the lower index
    assert o.prune_2of4_magnitude(np.array([[1, 1, 1, 1]], np.float32))[0].tolist() == [True, True, False, False]
    assert o.prune_2of4_magnitude(np.array([[0, 0, 0, 5]], np.float32))[0].tolist() == [True, False, False, True]
    assert o.prune_2of4_magnitude(np.array([[2, -3, 3, 2]], np.float32))[0].tolist() == [False, True, True, False]


@pytest.mark.parametrize("bits", [2, 4])
def test_compressed_delta_is_2of4(bits):
    rng = np.random.default_rng(4)
    d = (rng.standard_normal((32, 256)) * 1e-3).astype(np.float32)
    codes, scales16, zeros, keep = o.compress_delta(d, bits)
    zp = 2 ** (bits - 1)
    assert np.all(zeros == zp)
    c = codes.T.reshape(32, 64, 4)
    assert np.all((c == zp).sum(axis=2) >= 2)          # at least two zero-point codes per group
    assert np.all(keep.reshape(32, 64, 4).sum(axis=2) == 2)
    assert np.all(codes.T[~keep] == zp)                # pruned entries carry the zero-point


def test_compress_delta_known_answers():
    """The chain scales-from-unpruned -> 2:4 by magnitude -> quantise, on a row worked out by hand:
    b = 4: scale = 2 * 0.003 / 15 = 4e-4; 0.003 and -0.0029 stay; 0.003 / 4e-4 = 7.5 -> 8 (half to
    even) + 8 = 16 -> 15; -0.0029 / 4e-4 = -7.25 -> -7 + 8 = 1; the pruned pair carries the zero-point.
    b = 2: scale = 2e-3; 1.5 -> 2 + 2 = 4 -> 3; -1.45 -> -1 + 2 = 1."""
    row = np.array([[0.003, -0.001, 0.0005, -0.0029]], dtype=np.float32)
    codes, scales16, zeros, keep = o.compress_delta(row, 4)
    assert codes.T.tolist() == [[15, 8, 8, 1]] and keep.tolist() == [[True, False, False, True]]
    assert zeros.tolist() == [[8]] and scales16.view(np.uint16)[0, 0] == np.float16(4e-4).view(np.uint16)
    codes, scales16, zeros, keep = o.compress_delta(row, 2)
    assert codes.T.tolist() == [[3, 2, 2, 1]] and zeros.tolist() == [[2]]
    # the scale comes from the un-pruned row: a large value that is pruned away still sets it
    row = np.array([[0.004, 0.004, 0.004, -0.004, 0.0, 0.0, 0.001, 0.0]], dtype=np.float32)
    codes, scales16, _, keep = o.compress_delta(row, 4)
    assert keep.tolist() == [[True, True, False, False, True, False, True, False]]
    # scale = 0.008 / 15; 0.004 / scale = 7.5 -> 8 -> 16 -> 15; 0.001 / scale = 1.875 -> 2 -> 10
    assert codes.T.tolist() == [[15, 15, 8, 8, 8, 8, 10, 8]]


# ---- the search over the clipping range (quant.py:85-101, mse=True) --------------------------------
def _brute_force_mse(row, bits, norm, grid, maxshrink):
    """Plain Python floats and loops: every candidate's error, the first minimum wins."""
    import math
    maxq, zero = 2 ** bits - 1, 2 ** (bits - 1)
    xmin, xmax = min(min(row), 0.0), max(max(row), 0.0)
    xmax = max(abs(xmin), xmax)
    if xmin < 0:
        xmin = -xmax
    if xmin == 0 and xmax == 0:
        xmin, xmax = -1.0, 1.0
    out = []
    for i in range(int(maxshrink * grid)):
        p = 1 - i / grid
        s = (p * xmax - p * xmin) / maxq
        err = 0.0
        for v in row:
            # round half to even, as torch.round
            q = min(max(round(v / s) + zero, 0), maxq)
            err += abs(s * (q - zero) - v) ** norm
        out.append((err, s))
    return out


@pytest.mark.parametrize("bits", [2, 4])
def test_mse_search_against_brute_force(bits):
    rng = np.random.default_rng(7 + bits)
    for trial in range(40):
        # multiples of 1/64 in [-2, 2]: exact in fp32, so float64 loops and the fp32 oracle see the same values
        row = (rng.integers(-128, 129, size=12) / 64.0).astype(np.float32)
        if trial % 5 == 0:
            row[0] = 4.0                                              # an outlier: shrinking the range pays
        scale, zero, errs = o.find_params_sym(row[None, :], bits, mse=True, return_errors=True)
        cand = _brute_force_mse([float(v) for v in row], bits, 2.4, 100, 0.8)
        assert errs.shape[0] == len(cand) == 80
        np.testing.assert_allclose(errs[:, 0, 0], [c[0] for c in cand], rtol=2e-5, atol=1e-12)
        best = min(c[0] for c in cand)
        first = next(c for c in cand if c[0] == best)
        chosen = float(scale[0, 0])
        if abs(chosen - first[1]) > 1e-6 * first[1]:                  # only a near-tie may resolve differently
            e_chosen = next(c[0] for c in cand if abs(c[1] - chosen) <= 1e-6 * c[1])
            assert e_chosen <= best * (1 + 1e-5)
        assert zero[0, 0] == 2 ** (bits - 1)


def test_mse_search_with_only_the_full_range_as_candidate_changes_nothing():
    rng = np.random.default_rng(3)
    w = rng.standard_normal((5, 64)).astype(np.float32)
    plain, _ = o.find_params_sym(w, 4)
    one, _ = o.find_params_sym(w, 4, mse=True, grid=1, maxshrink=1.0)      # i = 0 only: p = 1
    none, _ = o.find_params_sym(w, 4, mse=True, grid=100, maxshrink=0.0)   # no candidate at all
    assert np.array_equal(plain, one) and np.array_equal(plain, none)


def test_mse_search_shrinks_for_an_outlier_and_scales_with_the_row():
    row = np.array([[1.0] + [0.3] * 20 + [-0.3] * 3], dtype=np.float32)
    plain, _ = o.find_params_sym(row, 2)
    searched, _, errs = o.find_params_sym(row, 2, mse=True, return_errors=True)
    assert searched[0, 0] < plain[0, 0]
    assert errs[:, 0, 0].min() < errs[0, 0, 0]                        # candidate 0 is the plain range
    # the grid is relative to the row's range: a row twice as large gets exactly twice the scale
    twice, _ = o.find_params_sym(2 * row, 2, mse=True)
    assert twice[0, 0] == 2 * searched[0, 0]
    # per group: each group is searched on its own
    two = np.concatenate([row, 4 * row], axis=1)
    two = np.pad(two, ((0, 0), (0, 128 - two.shape[1])))[:, :128]
    g, _ = o.find_params_sym(np.concatenate([np.pad(row, ((0, 0), (0, 40))), np.pad(4 * row, ((0, 0), (0, 40)))], axis=1), 2,
                             group_size=64, mse=True)
    assert g.shape == (1, 2) and g[0, 0] == searched[0, 0] and g[0, 1] == 4 * searched[0, 0]
