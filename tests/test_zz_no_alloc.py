"""dz_multi_delta_linear_static, the entry point that allocates nothing: its workspace is a fixed
array inside the library.  Called through the C ABI twice in a row, the second call with a smaller
input, and compared with dz_multi_delta_linear (bit for bit: same kernels, same order of additions)
and with the CPU oracle (to the layer's tolerance).  That it allocates nothing is checked as well:
with the output tensor made beforehand, the device's free memory (hipMemGetInfo) and the bytes
torch's allocator holds are the same before and after the static calls."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import dz_oracle as o
from deltazip_amd import _lib, ops
from _util import make_problem, TOL


def _call(fn_name, p, ws=None, accumulate=0, out=None):
    L = _lib.lib()
    t, k, n = p["x"].shape[0], p["k"], p["n"]
    y = torch.full((t, n), 7.0, dtype=torch.float16, device=p["x"].device) if out is None else out
    if accumulate:
        y.copy_(p["y0"])
    gs = -1 if p["s"][0].numel() == n else k // (p["s"][0].numel() // n)
    args = [p["x"].data_ptr(), p["wb"].data_ptr(), p["q"].data_ptr(), p["m"].data_ptr(), p["s"].data_ptr(),
            p["ids"].data_ptr(), y.data_ptr(), t, k, n, p["q"].shape[0], p["bits"], gs, accumulate, n]
    if ws is not None:
        args += [ws.data_ptr(), ws.numel()]
    rc = getattr(L, fn_name)(*args, None)
    assert rc == 0, L.dz_strerror(rc)
    torch.cuda.synchronize()
    return y


def _workspace(p):
    t, k, n = p["x"].shape[0], p["k"], p["n"]
    return torch.zeros(_lib.lib().dz_workspace_bytes(t, k, n), dtype=torch.uint8, device=p["x"].device)


# (N, K, bits, group_size, deltas, tokens): the first of each pair is the larger call
PAIRS = [
    ((512, 4096, 2, -1, 8, 32), (128, 1024, 2, -1, 3, 7)),       # K split over workgroups, then not
    ((1024, 2048, 4, 128, 6, 100), (256, 2048, 4, 128, 6, 20)),  # grouped tokens (T > 32), 4-bit grouped scales
]


@pytest.mark.gpu
@pytest.mark.parametrize("big,small", PAIRS)
def test_static_entry_point_matches_workspace_entry_point(dev, big, small):
    for i, (n, k, bits, gs, nd, t) in enumerate((big, small)):
        p = make_problem(n, k, bits, gs, nd, t, "uniform", 300 + i, dev)
        want = _call("dz_multi_delta_linear", p, ws=_workspace(p))
        got = _call("dz_multi_delta_linear_static", p)     # first call on the device: looks up the array's address
        assert torch.equal(got, want)
        # nothing is allocated: neither from the device (hipMalloc would lower the free bytes) nor
        # from torch's allocator; the output tensor exists before the measurement starts
        out = torch.empty_like(got)
        torch.cuda.synchronize()
        free_before, reserved_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
        allocated_before = torch.cuda.memory_allocated()
        got2 = _call("dz_multi_delta_linear_static", p, out=out.fill_(7.0))
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.cuda.memory_reserved() == reserved_before
        assert torch.cuda.memory_allocated() <= allocated_before     # (a temporary of the test itself may have gone)
        assert torch.equal(got2, want)
        ref = o.forward_ref(p["x_np"], p["wb_np"], p["dts"], p["ids_np"])
        assert o.rel_err(got.cpu().numpy(), ref) <= TOL
        # y += result
        p["y0"] = torch.from_numpy(o.make_x(t, n, 900 + i)).to(dev)
        want = _call("dz_multi_delta_linear", p, ws=_workspace(p), accumulate=1)
        got = _call("dz_multi_delta_linear_static", p, accumulate=1)
        assert torch.equal(got, want)


def test_static_entry_point_rejects_sizes_beyond_its_array(dzlib):
    one = C.c_void_p(0x1000)   # never dereferenced: the size check comes first
    rc = dzlib.dz_multi_delta_linear_static(one, one, one, one, one, one, one, 4, 512, 16384 + 32, 2, 4, -1, 0,
                                            16384 + 32, None)
    assert rc == -11
    assert b"DZ_STATIC_MAX_N" in dzlib.dz_strerror(rc)
