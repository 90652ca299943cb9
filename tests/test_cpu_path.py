"""The torch-CPU restatement that the benchmark times as its CPU baseline (oracle/cpu_path.py) is
held to the numpy oracle: same dequantised bits, same layer output."""
import numpy as np
import pytest
import torch

from oracle import cpu_path
from oracle import dz_oracle as o

CASES = [(64, 512, 2, -1), (64, 512, 4, -1), (96, 1024, 4, 128), (32, 768, 2, 64)]   # (N, K, bits, group_size)


def _as_torch(dl):
    return tuple(torch.from_numpy(np.ascontiguousarray(dl[k])) for k in ("qweight", "qzeros", "scales", "g_idx"))


@pytest.mark.parametrize("n,k,bits,gs", CASES)
def test_dequant_torch_equals_oracle_bit_for_bit(n, k, bits, gs):
    dl = o.make_delta(n, k, 1e-3, bits, gs, 4100 + bits)
    want = o.dequant_gptq(dl["qweight"], dl["qzeros"], dl["scales"], dl["g_idx"], bits)   # [K, N] fp16
    got = cpu_path.dequant_torch(*_as_torch(dl), bits)
    assert got.dtype == torch.float16 and tuple(got.shape) == want.shape
    assert np.array_equal(got.numpy().view(np.uint16), want.view(np.uint16))
    assert np.count_nonzero(want) > 0


@pytest.mark.parametrize("n,k,bits,gs", CASES)
def test_forward_cpu_equals_forward_ref(n, k, bits, gs):
    nd, t = 3, 9
    dls = [o.make_delta(n, k, 1e-3, bits, gs, 4200 + d) for d in range(nd)]
    dts = [o.dequant_gptq(d["qweight"], d["qzeros"], d["scales"], d["g_idx"], bits) for d in dls]
    wb, x = o.make_base(n, k, 4300), o.make_x(t, k, 4400)
    ids = np.array([-1, 0, 2, 2, 1, -1, 0, 1, 2], dtype=np.int64)
    ref = o.forward_ref(x, wb, dts, ids)
    xt, wbt, idt = torch.from_numpy(x), torch.from_numpy(wb), torch.from_numpy(ids)
    got = cpu_path.forward_cpu(xt, wbt, [_as_torch(d) for d in dls], idt, bits).numpy()
    # both sum fp32 products of the same fp16 inputs; only the order of the additions differs
    assert o.rel_err(got, ref) <= 1e-5
    # the matmul-only form (deltas dequantised beforehand) is the same function
    pre = [torch.from_numpy(np.ascontiguousarray(d)) for d in dts]
    got2 = cpu_path.forward_cpu(xt, wbt, None, idt, bits, predequantised=pre).numpy()
    assert np.array_equal(got, got2)
    # a token without a delta is the plain linear layer
    base_rows = ids < 0
    assert o.rel_err(got[base_rows], x[base_rows].astype(np.float64) @ wb.astype(np.float64).T) <= 1e-4   # fp32 sums vs fp64
