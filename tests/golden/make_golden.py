"""Writes the golden fixtures of tests/golden/ from the oracle's closed forms.

The reference repository holds no golden vectors, known-answer tests or fixtures for this path
(its README names tests/ that do not exist and serving/tests/ never touches vllm/delta/), so the
fixtures are generated here, from seeded inputs, by oracle/dz_oracle.py, whose functions are
pinned independently in tests/test_oracle_*.py.  They freeze those results: a later change to the
oracle or to the kernels that alters any bit shows up against these files.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import dz_oracle as o  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

CASES = [  # name, N, K, bits, group_size, deltas, tokens, ids
    ("b4_perchannel", 64, 256, 4, -1, 3, 9, [2, -1, 0, 2, 1, -1, 0, 1, 2]),
    ("b2_perchannel", 64, 256, 2, -1, 3, 9, [0, 0, 1, 1, 2, 2, -1, -1, 0]),
    ("b4_group128", 32, 512, 4, 128, 2, 5, [1, 0, -1, 1, 0]),
    ("b2_group64", 32, 256, 2, 64, 2, 17, [0, 1] * 8 + [-1]),
]


def main():
    for i, (name, n, k, bits, gs, nd, t, ids) in enumerate(CASES):
        seed = 9000 + 10 * i
        out = {"bits": np.int32(bits), "group_size": np.int32(gs), "ids": np.asarray(ids, np.int64)}
        dts = []
        for d in range(nd):
            dl = o.make_delta(n, k, 1e-3, bits, gs, seed + 1 + d)
            for key in ("qweight", "qzeros", "scales", "g_idx"):
                out[f"d{d}_{key}"] = dl[key]
            dt = o.dequant_gptq(dl["qweight"], dl["qzeros"], dl["scales"], dl["g_idx"], bits)
            out[f"d{d}_dequant_t"] = dt          # [K, N] fp16, the reference's unpack() orientation
            dts.append(dt)
        out["w_base"] = o.make_base(n, k, seed)
        out["x"] = o.make_x(t, k, seed + 500)
        out["y_ref"] = o.forward_ref(out["x"], out["w_base"], dts, out["ids"])
        out["y_delta_only"] = o.forward_ref(out["x"], None, dts, out["ids"])
        np.savez_compressed(os.path.join(HERE, f"{name}.npz"), **out)
        print(name, {k2: v.shape for k2, v in out.items() if hasattr(v, "shape") and v.shape})


if __name__ == "__main__":
    main()
