"""The oracle reproduces the committed golden fixtures bit for bit (CPU only)."""
import glob
import os

import numpy as np
import pytest

from oracle import dz_oracle as o

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))


def test_fixtures_present():
    assert len(GOLDEN) == 4


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_oracle_matches_golden(path):
    g = np.load(path)
    bits = int(g["bits"])
    nd = sum(1 for k in g.files if k.endswith("_qweight"))
    dts = []
    for d in range(nd):
        dt = o.dequant_gptq(g[f"d{d}_qweight"], g[f"d{d}_qzeros"], g[f"d{d}_scales"], g[f"d{d}_g_idx"], bits)
        assert np.array_equal(dt.view(np.uint16), g[f"d{d}_dequant_t"].view(np.uint16))
        dts.append(dt)
        # the 2:4 structure the layer relies on
        k, n = dt.shape
        assert np.all((dt.T.reshape(n, k // 4, 4) != 0).sum(axis=2) <= 2)
    y = o.forward_ref(g["x"], g["w_base"], dts, g["ids"])
    assert np.array_equal(y, g["y_ref"])
    assert np.array_equal(o.forward_ref(g["x"], None, dts, g["ids"]), g["y_delta_only"])
