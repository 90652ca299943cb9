"""ctypes binding of libdz_amd.so (the C ABI declared in include/dz_amd.h).

There is no CPU fallback: if the library is missing, `lib()` raises.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdz_amd.so")

_lib = None

# name -> (restype, argtypes); mirrors include/dz_amd.h
_vp, _i, _sz = C.c_void_p, C.c_int, C.c_size_t
SIGNATURES = {
    "dz_version": (_i, []),
    "dz_strerror": (C.c_char_p, [_i]),
    "dz_native_sizes": (_i, [_i, _i, _i, _i, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz)]),
    "dz_repack_2of4": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp]),
    "dz_unrepack_2of4": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "dz_dequant": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp]),
    "dz_merge": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp]),
    "dz_segment": (_i, [_vp, _i, _i, _vp, _vp, _vp]),
    "dz_embedding_select": (_i, [_vp, _vp, _vp, _vp, C.c_longlong, _i, _vp, _i, _i, _i, _i, _vp]),
    "dz_build_tiles": (_i, [_vp, _i, _vp, _i, _vp]),
    "dz_multi_delta_gemm": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "dz_multi_delta_gemm_tiled": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "dz_compress_2of4": (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "dz_quant_scales": (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _vp]),
    "dz_quant_scales_mse": (_i, [_vp, _i, _i, _i, _i, C.c_float, _i, C.c_float, _vp, _vp, _vp]),
    "dz_pack_2of4": (_i, [_vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp]),
    "dz_hessian_add": (_i, [_vp, _vp, _i, _i, _i, C.c_float, C.c_float, _vp]),
    "dz_obs_sweep": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "dz_multi_delta_linear_batch": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp,
                                         _vp, C.c_size_t, _vp]),
    "dz_multi_delta_linear_batch_tiled": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i,
                                               _vp, _vp, C.c_size_t, _vp]),
    "dz_tile_base": (_i, [_vp, _i, _i, _vp, _vp]),
    "dz_token_order": (_i, [_vp, _i, _i, _vp, _vp]),
    "dz_map_ids": (_i, [_vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp]),
    "dz_workspace_bytes": (_sz, [_i, _i, _i]),
    "dz_multi_delta_linear": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i,
                                   _vp, _sz, _vp]),
    "dz_multi_delta_linear_static": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "dz_gemm_f16": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "dz_gemm_f16_pair": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "dz_gemm_f16_grouped": (_i, [_vp, _vp, _vp, C.c_longlong, _vp, _i, _vp, _i, _i, _i, _i, _i, _vp]),
    "dz_gemm_f16_select": (_i, [_vp, _vp, _vp, C.c_longlong, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "dz_set_ksplit": (None, [_i]),
    "dz_probe_read": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp]),
}


class DzError(RuntimeError):
    def __init__(self, code: int, what: str):
        self.code = code
        super().__init__(f"{what}: {lib().dz_strerror(code).decode()} (code {code})")


def lib():
    """The loaded library.  Raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m deltazip_amd.build` "
                "(there is no fallback implementation)")
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(code: int, what: str) -> None:
    """Turn a negative return code into the exception the reference API would raise:
    ValueError for argument problems, RuntimeError for launch failures."""
    if code == 0:
        return
    msg = f"{what}: {lib().dz_strerror(code).decode()} (code {code})"
    if code in (-9,):
        raise RuntimeError(msg)
    if code == -3:
        raise NotImplementedError(msg)
    raise ValueError(msg)
