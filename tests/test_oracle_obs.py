"""The Hessian-aware sweep of the oracle (oracle.dz_oracle.obs_sweep_ref, after
deltazip/core/sparsegpt.py:25-146) against what the mathematics fixes: no reference code is run."""
import numpy as np
import pytest

from oracle import dz_oracle as o


def _problem(n, k, t, seed):
    rng = np.random.default_rng(seed)
    W = (rng.standard_normal((n, k)) * 0.01).astype(np.float32)
    X = rng.standard_normal((t, k)).astype(np.float32)
    # correlated inputs, so that the off-diagonal of H matters
    X = (X + 0.5 * np.roll(X, 1, axis=1)).astype(np.float32)
    H, ns = o.hessian_add_batch_ref(np.zeros((k, k), np.float32), 0, X)
    return W, X, H, ns


def test_hessian_is_two_over_n_times_gram_matrix():
    rng = np.random.default_rng(0)
    a = rng.standard_normal((3, 5, 8)).astype(np.float32)      # 3 samples of 5 tokens
    b = rng.standard_normal((7, 8)).astype(np.float32)         # one more sample
    H, n = o.hessian_add_batch_ref(np.zeros((8, 8), np.float32), 0, a)
    H, n = o.hessian_add_batch_ref(H, n, b)
    assert n == 4
    allx = np.concatenate([a.reshape(-1, 8), b]).astype(np.float64)
    assert np.allclose(H, 2.0 / 4 * allx.T @ allx, rtol=1e-5, atol=1e-5)


def test_identity_hessian_reduces_to_magnitude_pruning_and_rounding():
    rng = np.random.default_rng(1)
    W = (rng.standard_normal((16, 256)) * 0.01).astype(np.float32)
    hinv, W0 = o.hinv_upper_ref(np.eye(256, dtype=np.float32) * 3.0, W)
    assert np.allclose(hinv, np.diag(np.diag(hinv)))            # no coupling between columns
    for bits in (2, 4):
        scale, zero = o.find_params_sym(W, bits)
        out, _ = o.obs_sweep_ref(W0, hinv, scale[:, 0], bits)
        keep = o.prune_2of4_magnitude(W)
        want = o.quantize(np.where(keep, W, np.float32(0)), scale, zero, 2**bits - 1)
        assert np.array_equal(out, want)
    out, loss = o.obs_sweep_ref(W0, hinv, None)                  # pruning only
    assert np.array_equal(out, np.where(o.prune_2of4_magnitude(W), W, np.float32(0)))
    # loss = sum of pruned w^2 / d^2 / 2
    d = np.diag(hinv)[0]
    want_loss = (np.where(o.prune_2of4_magnitude(W), 0, W).astype(np.float64) ** 2).sum(axis=1) / d**2 / 2
    assert np.allclose(loss, want_loss, rtol=1e-4)


def test_single_pruned_weight_is_the_closed_form_surgeon_update():
    """Pruning weight p of a row changes the others by -w_p / [H^-1]_pp * H^-1[:, p] (Hassibi &
    Stork); the sweep freezes columns to the left, so take p = 0."""
    k = 8
    W, X, H, _ = _problem(1, k, 64, 2)
    Hd = H.astype(np.float64) + 0.01 * np.mean(np.diag(H)) * np.eye(k)
    Hinv = np.linalg.inv(Hd)
    hinv, _ = o.hinv_upper_ref(H, W)
    # force the mask: make column 0 tiny so that it is pruned, and stop pruning elsewhere by hand
    w = W.copy()
    w[0, 0] = 1e-6
    out, _ = o.obs_sweep_ref(w, hinv, None, prunen=1, prunem=8, blocksize=8)
    want = w[0].astype(np.float64) - w[0, 0] / Hinv[0, 0] * Hinv[:, 0]
    assert out[0, 0] == 0
    assert np.allclose(out[0, 1:], want[1:], rtol=2e-3, atol=1e-7)


@pytest.mark.parametrize("stop", [128, 256])
def test_untouched_columns_are_optimal_for_the_frozen_ones(stop):
    """After the sweep has passed `stop` columns (pruning only), the updated remaining columns
    minimise ||(W0 - W) X^T||: the gradient (W0 - W) H restricted to them vanishes."""
    n, k = 8, 384
    W, X, H, _ = _problem(n, k, 1024, 3)
    hinv, W0 = o.hinv_upper_ref(H, W)
    Hd = H.astype(np.float64) + 0.01 * np.mean(np.diag(H)) * np.eye(k)
    out, _ = o.obs_sweep_ref(W0, hinv, None, stop=stop)
    g = (W0.astype(np.float64) - out.astype(np.float64)) @ Hd
    scale = np.abs((W0.astype(np.float64) - out) @ Hd)[:, :stop].max()
    assert np.abs(g[:, stop:]).max() < 2e-3 * scale
    # and the frozen part is 2:4 sparse
    z = (out[:, :stop].reshape(n, -1, 4) == 0).sum(axis=2)
    assert (z >= 2).all()


def test_compensation_beats_plain_magnitude_pruning():
    n, k = 16, 256
    W, X, H, _ = _problem(n, k, 2048, 4)
    hinv, W0 = o.hinv_upper_ref(H, W)
    scale, zero = o.find_params_sym(W, 4)
    out, loss = o.obs_sweep_ref(W0, hinv, scale[:, 0], 4)
    plain = o.quantize(np.where(o.prune_2of4_magnitude(W), W, np.float32(0)), scale, zero, 15)
    e_obs = np.linalg.norm((W - out) @ X.T)
    e_plain = np.linalg.norm((W - plain) @ X.T)
    assert e_obs < 0.95 * e_plain
    # every value is on the row's grid and every group of 4 has two zeros
    q = out / scale
    assert np.allclose(q, np.rint(q), atol=1e-4) and np.abs(q).max() <= 8
    assert ((out.reshape(n, -1, 4) == 0).sum(axis=2) >= 2).all()
    assert (loss > 0).all()


def test_dead_columns_are_zeroed_and_get_unit_diagonal():
    W, X, H, _ = _problem(4, 128, 256, 5)
    X[:, 7] = 0
    H, _ = o.hessian_add_batch_ref(np.zeros((128, 128), np.float32), 0, X)
    hinv, W0 = o.hinv_upper_ref(H, W)
    assert (W0[:, 7] == 0).all() and np.isfinite(hinv).all()
