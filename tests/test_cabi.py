"""The C ABI: the library loads, exports every function include/dz_amd.h declares, and rejects bad
arguments on the host before anything is launched (no GPU needed)."""
import ctypes as C
import os
import re

import pytest

from deltazip_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    # the layer's interface and, kept apart from it, the tuning hooks
    text = "".join(open(os.path.join(ROOT, "include", h)).read() for h in ("dz_amd.h", "dz_amd_tuning.h"))
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dz_[a-z0-9_]+)\s*\(", text)))


def test_header_functions_are_exported(dzlib):
    names = _declared_functions()
    assert len(names) >= 10
    for n in names:
        assert hasattr(dzlib, n), f"{n} declared in dz_amd.h but not exported"
    assert set(names) == set(_lib.SIGNATURES), "ctypes signatures out of step with the header"


def test_version_and_strerror(dzlib):
    assert dzlib.dz_version() >= 100
    assert dzlib.dz_strerror(0) == b"ok"
    for code in range(-11, 0):
        assert dzlib.dz_strerror(code) not in (b"", b"unknown error")


def test_argument_checks_happen_on_the_host(dzlib):
    one = C.c_void_p(0x1000)   # never dereferenced: every call below fails validation first
    f = dzlib.dz_multi_delta_linear
    ok = dict(T=4, K=512, N=64, S=2, bits=4, gs=-1, acc=0, ldy=64)

    def call(x=one, wb=one, q=one, m=one, s=one, idx=one, y=one, ws=one, wsb=1 << 30, **kw):
        if kw.get("S") == 0 and "wsb" not in kw and wb is not None:
            wsb = 16
        a = dict(ok); a.update(kw)
        return f(x, wb, q, m, s, idx, y, a["T"], a["K"], a["N"], a["S"], a["bits"], a["gs"], a["acc"], a["ldy"],
                 ws, wsb, None)

    assert call(x=None) == -1 and call(idx=None) == -1 and call(y=None) == -1 and call(q=None) == -1
    assert call(S=0, q=None, m=None, s=None) == -8          # no slots: dense product only; next check is the workspace size
    assert call(S=0, wb=None) == -1 and call(S=-1) == -1
    assert call(bits=3) == -3 and call(bits=8) == -3
    assert call(K=500) == -2 and call(N=48) == -2 and call(T=0) == -2 and call(T=129) == -2
    assert call(ldy=32) == -2 and call(ldy=66) == -2
    assert call(gs=100) == -4 and call(gs=96) == -4
    assert call(x=C.c_void_p(0x1004)) == -10 and call(y=C.c_void_p(0x1002)) == -10
    assert call(ws=None) == -8 and call(wsb=16) == -8
    assert dzlib.dz_workspace_bytes(32, 4096, 4096) > 4096 * 32 * 4
    assert dzlib.dz_dequant(None, one, one, 512, 64, 4, -1, one, None) == -1
    assert dzlib.dz_dequant(one, one, one, 512, 60, 4, -1, one, None) == -2
    assert dzlib.dz_merge(None, one, one, one, 512, 64, 4, -1, one, None) == -1
    assert dzlib.dz_segment(None, 4, 2, one, one, None) == -1
    assert dzlib.dz_segment(one, 0, 2, one, one, None) == -2
    mp = dzlib.dz_map_ids
    assert mp(None, 4, None, 0, one, 2, 3, 100, 0, one, None, None, None, 0, None, None) == -1
    assert mp(one, 4, None, 2, one, 2, 3, 100, 0, one, None, None, None, 0, None, None) == -1
    assert mp(one, 0, None, 0, one, 2, 3, 100, 0, one, None, None, None, 0, None, None) == -2
    assert mp(one, 4, None, 0, one, 5000, 3, 100, 0, one, None, None, None, 0, None, None) == -2
    assert mp(one, 4, None, 0, one, 2, 3, 100, 0, one, None, None, one, 3, None, None) == -2
    assert dzlib.dz_gemm_f16(one, one, one, 8, 100, 128, 0, 128, None) == -2
    assert dzlib.dz_gemm_f16(None, one, one, 8, 128, 128, 0, 128, None) == -1
    # the per-row table choice and the tiled form of the prefill entry point: missing tables / tiles
    sel = dzlib.dz_gemm_f16_select
    assert sel(one, one, one, 64 * 256, None, 4, one, one, 8, 256, 64, 0, 64, None) == -1      # no row blocks
    assert sel(one, None, one, 64 * 256, one, 4, one, one, 8, 256, 64, 0, 64, None) == -1     # no base table
    assert sel(one, one, None, 64 * 256, one, 4, one, one, 8, 256, 64, 0, 64, None) == -1     # no delta tables
    gt = dzlib.dz_multi_delta_gemm_tiled
    assert gt(one, None, one, one, one, 2, 4, -1, one, 4, None, one, 300, 512, 64, 0, 64, None) == -1
    assert gt(one, one, one, one, one, 2, 3, -1, one, 4, None, one, 300, 512, 64, 0, 64, None) == -3
    assert gt(one, one, one, one, one, 2, 4, -1, one, 4, None, one, 300, 500, 64, 0, 64, None) == -2
    # the read-only yardstick validates like the launch it stands beside
    arr = lambda v: (C.c_void_p * 1)(v)
    pr = dzlib.dz_probe_read
    n1 = (C.c_int * 1)(64)
    assert pr(0, arr(0x1000), arr(0x1000), arr(0x1000), arr(0x1000), n1, 8, 512, 2, 2, 0, one, None) == -1
    assert pr(1, arr(0x1000), arr(0x1000), arr(0x1000), arr(0x1000), n1, 8, 512, 2, 2, 0, None, None) == -1
    assert pr(1, arr(0x1000), arr(0x1000), arr(0x1000), arr(0x1000), n1, 33, 512, 2, 2, 0, one, None) == -2
    assert pr(1, arr(0x1000), arr(0x1000), arr(0x1000), arr(0x1000), n1, 8, 512, 2, 9, 0, one, None) == -2
    assert pr(1, arr(0x1000), arr(0x1000), arr(0x1000), arr(0x1000), n1, 8, 512, 3, 2, 0, one, None) == -3
    assert pr(1, arr(0x1000), arr(0x1000), arr(0x1000), arr(0x1000), n1, 8, 500, 2, 2, 0, one, None) == -2
    assert pr(1, arr(0x1000), arr(None), arr(0x1000), arr(0x1000), n1, 8, 512, 2, 2, 0, one, None) == -1


def test_compressor_entry_points_check_their_arguments(dzlib):
    one = C.c_void_p(0x1000)   # never dereferenced
    assert dzlib.dz_hessian_add(None, one, 1, 8, 256, 0.5, 0.5, None) == -1
    assert dzlib.dz_hessian_add(one, one, 1, 0, 256, 0.5, 0.5, None) == -2
    assert dzlib.dz_hessian_add(one, one, 1, 8, 100, 0.5, 0.5, None) == -2
    sweep = lambda **kw: dzlib.dz_obs_sweep(kw.get("W", one), one, kw.get("scale", one), kw.get("N", 32), kw.get("K", 256),
                                            kw.get("bits", 4), kw.get("pn", 2), kw.get("pm", 4), one, one, None)
    assert sweep(W=None) == -1
    assert sweep(K=192) == -2                    # whole blocks of 128 columns
    assert sweep(bits=5) == -3
    assert sweep(pn=2, pm=3) == -2               # group size must divide 64
    assert sweep(pn=4, pm=4) == -2
    assert sweep(pn=2, pm=16) == -2
    assert dzlib.dz_quant_scales(one, 256, 32, 3, -1, one, one, None) == -3
    assert dzlib.dz_quant_scales(one, 256, 32, 4, 100, one, one, None) == -4
    assert dzlib.dz_quant_scales_mse(one, 256, 32, 3, -1, 2.4, 100, 0.8, one, one, None) == -3
    assert dzlib.dz_quant_scales_mse(one, 256, 32, 4, -1, 2.4, 0, 0.8, one, one, None) == -1      # grid >= 1
    assert dzlib.dz_quant_scales_mse(one, 256, 32, 4, -1, 2.4, 100, 1.5, one, one, None) == -1    # maxshrink in [0, 1]
    assert dzlib.dz_pack_2of4(one, None, 256, 32, 4, -1, one, one, None) == -1
    assert dzlib.dz_pack_2of4(one, one, 250, 32, 4, -1, one, one, None) == -2


def test_python_wrappers_refuse_cpu_tensors(dzlib):
    import torch
    from deltazip_amd import ops, QuantLinear, DeltaConfig
    x = torch.zeros(2, 512, dtype=torch.float16)
    q = torch.zeros(1, 16, 128, dtype=torch.int32); m = torch.zeros(1, 64, 32, dtype=torch.int16)
    s = torch.zeros(1, 1, 64, dtype=torch.float16)
    with pytest.raises(ValueError, match="GPU"):
        ops.multi_delta_linear(x, None, q, s, m, torch.zeros(2, dtype=torch.int64), bits=4)
    with pytest.raises(NotImplementedError):
        QuantLinear(3, 512, 64, None)
    with pytest.raises(ValueError):
        DeltaConfig(max_bitwidth=8)
    with pytest.raises(ValueError):
        DeltaConfig(max_deltas=4, max_cpu_deltas=2)
    cfg = DeltaConfig(max_deltas=4, max_bitwidth=2)
    assert cfg.pack_factor == 16 and cfg.sparse_factor == 2 and cfg.max_cpu_deltas == 4
    assert ops.stacked_shapes(4096, 4096, 4) == ((128, 8192), (4096, 256), (1, 4096))
    assert ops.stacked_shapes(4096, 4096, 2, 128) == ((64, 8192), (4096, 256), (32, 4096))


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libdz_amd.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.lib()
