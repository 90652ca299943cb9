"""Seeded random sweeps of the layer call against the oracle: shapes, bit widths, scale groupings,
token counts on both sides of every internal threshold (16, 32, 128 tokens), id patterns with and
without base-only tokens, and the ways a call can be made (plain, delta-only accumulate, into a
column slice, batched; each with the base weight row-major and in tiles).  Some kernel variants -- 2-bit deltas with scale groups of 64 in a batched
launch is the one under the highest register pressure -- are reached only by such combinations."""
import numpy as np
import pytest
import torch

from _util import TOL, make_problem
from deltazip_amd import ops
from oracle import dz_oracle as o

pytestmark = pytest.mark.gpu


def _ids(rng, t, nd, kind):
    if kind == 0:
        ids = rng.integers(-1, nd, size=t)
    elif kind == 1:
        ids = np.sort(rng.integers(-1, nd, size=t))
    elif kind == 2:
        ids = np.minimum(rng.zipf(1.5, size=t) - 1, nd - 1)
    elif kind == 3:
        ids = np.full(t, -1)
    else:
        ids = np.full(t, int(rng.integers(0, nd)))
    return ids.astype(np.int64)


def _check(dev, rng, n, k, bits, gs, nd, t, mode):
    ids = _ids(rng, t, nd, int(rng.integers(0, 5)))
    seed = int(rng.integers(1, 10 ** 6))
    case = dict(n=n, k=k, bits=bits, gs=gs, nd=nd, t=t, mode=mode, seed=seed)
    p = make_problem(n, k, bits, gs, nd, t, ids, seed, dev)
    ref = o.forward_ref(p["x_np"], p["wb_np"], p["dts"], p["ids_np"])
    tol = TOL
    tiled = ops.tile_base(p["wb"])   # every call with a base weight is made in both forms: same bits
    if mode == 0:
        y = ops.apply_delta(p["x"], p["q"], p["s"], p["m"], p["ids"], p["wb"])
        assert torch.equal(y, ops.apply_delta(p["x"], p["q"], p["s"], p["m"], p["ids"], p["wb"], base_tiled=tiled)), case
    elif mode == 1:   # delta only, added to the base product (which is rounded to fp16 first)
        base16 = (p["x_np"].astype(np.float32) @ p["wb_np"].astype(np.float32).T).astype(np.float16)
        y = torch.from_numpy(base16).to(dev)
        ops.multi_delta_linear(p["x"], None, p["q"], p["s"], p["m"], p["ids"], bits=bits, out=y, accumulate=True)
        tol = 2 * TOL
    elif mode == 2:   # into a column slice of a wider tensor; the columns beside it stay untouched
        wide = torch.zeros(t, n + 64, device=dev, dtype=torch.float16)
        ops.multi_delta_linear(p["x"], p["wb"], p["q"], p["s"], p["m"], p["ids"], bits=bits, out=wide[:, 32:32 + n])
        assert float(wide[:, :32].abs().max()) == 0 and float(wide[:, 32 + n:].abs().max()) == 0, case
        y = wide[:, 32:32 + n]
        wide2 = torch.zeros_like(wide)
        ops.multi_delta_linear(p["x"], p["wb"], p["q"], p["s"], p["m"], p["ids"], bits=bits, out=wide2[:, 32:32 + n],
                               base_tiled=tiled)
        assert torch.equal(wide, wide2), case
    else:             # two calls in one launch
        y = ops.apply_delta_batch(p["x"], [p["q"]] * 2, [p["s"]] * 2, [p["m"]] * 2, p["ids"], [p["wb"]] * 2)[1]
        yt = ops.apply_delta_batch(p["x"], [p["q"]] * 2, [p["s"]] * 2, [p["m"]] * 2, p["ids"], [p["wb"]] * 2,
                                   base_tiled=[tiled] * 2)
        assert torch.equal(y, yt[1]) and torch.equal(yt[0], yt[1]), case
    torch.cuda.synchronize()
    err = o.rel_err(y.float().cpu().numpy(), ref)
    assert err <= tol, (case, err)


@pytest.mark.parametrize("seed", [11, 12])
def test_decode_sized_calls(dev, seed):
    rng = np.random.default_rng(seed)
    for _ in range(40):
        k = int(rng.choice([256, 512, 768, 1024, 2048, 4096]))
        gs = int(rng.choice([-1] + [g for g in (64, 128, 256) if k % g == 0 and g < k]))
        _check(dev, rng, int(rng.choice([32, 64, 96, 160, 256, 512])), k, int(rng.choice([2, 4])), gs,
               int(rng.choice([1, 2, 5, 9, 12, 24])), int(rng.choice([1, 2, 7, 16, 17, 31, 32, 33, 64, 65, 100, 128])),
               int(rng.integers(0, 4)))


def test_prefill_sized_calls(dev):
    rng = np.random.default_rng(21)
    for _ in range(30):
        k = int(rng.choice([256, 512, 1024, 2048]))
        gs = int(rng.choice([-1] + [g for g in (64, 128, 256) if k % g == 0 and g < k]))
        _check(dev, rng, int(rng.choice([32, 96, 256, 288, 544])), k, int(rng.choice([2, 4])), gs,
               int(rng.choice([1, 2, 5, 16])), int(rng.choice([129, 255, 256, 257, 400, 777])), int(rng.integers(0, 3)))
