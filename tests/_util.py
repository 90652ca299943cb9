"""Helpers shared by the GPU tests: synthetic deltas from the oracle, moved to the device in the
native layout."""
import numpy as np
import torch

from oracle import dz_oracle as o
from deltazip_amd import ops


def make_problem(n, k, bits, gs, nd, t, ids_kind, seed, dev, sigma=1e-3):
    """Returns dict with device tensors (native stacks, base, x, ids) and oracle-side arrays."""
    qs, ms, ss, dts, gptq = [], [], [], [], []
    for d in range(nd):
        dl = o.make_delta(n, k, sigma, bits, gs, seed + 1 + d)
        q, m, s = ops.repack_gptq_to_native(torch.from_numpy(dl["qweight"]), torch.from_numpy(dl["qzeros"]),
                                            torch.from_numpy(dl["scales"]), torch.from_numpy(dl["g_idx"]), bits)
        qs.append(q); ms.append(m); ss.append(s)
        dts.append(o.dequant_gptq(dl["qweight"], dl["qzeros"], dl["scales"], dl["g_idx"], bits))
        gptq.append(dl)
    wb = o.make_base(n, k, seed)
    x = o.make_x(t, k, seed + 500)
    if isinstance(ids_kind, str):
        ids = o.make_ids(ids_kind, t, nd, seed + 900)
    else:
        ids = np.asarray(ids_kind, dtype=np.int64)
    return dict(q=torch.stack(qs).to(dev), m=torch.stack(ms).to(dev), s=torch.stack(ss).to(dev),
                wb=torch.from_numpy(wb).to(dev), x=torch.from_numpy(x).to(dev),
                ids=torch.from_numpy(ids).to(dev), wb_np=wb, x_np=x, ids_np=ids, dts=dts, gptq=gptq,
                bits=bits, n=n, k=k)


def run_layer(p, **kw):
    y = ops.apply_delta(p["x"], p["q"], p["s"], p["m"], p["ids"], p["wb"])
    torch.cuda.synchronize()
    return y


TOL = 1e-2   # max relative error of the fp16 layer output against the fp32 CPU reference
