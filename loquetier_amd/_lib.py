"""ctypes binding of libsmlm_hip.so (the C ABI declared in include/smlm.h).

There is no CPU fallback: if the library is missing or fails to load, every
operator raises.
"""
from __future__ import annotations

import ctypes as C
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "lib", "libsmlm_hip.so")

SMLM_DTYPE_F16, SMLM_DTYPE_BF16 = 0, 1
SMLM_KEY_NONE, SMLM_KEY_I32, SMLM_KEY_PTR, SMLM_KEY_PTR2 = 0, 1, 2, 3
SMLM_ERR_DTYPE = -2
SMLM_ERR_SCRATCH = -7
SMLM_STATIC_SCRATCH_BYTES = 8 << 20
SMLM_STAGE_SHRINK, SMLM_STAGE_EXPAND = 1, 2
SMLM_BWD_PRODUCTS, SMLM_BWD_DX, SMLM_BWD_WGRAD = 1, 2, 4

_vp, _i, _sz, _f = C.c_void_p, C.c_int, C.c_size_t, C.c_float
_psz = C.POINTER(C.c_size_t)
_pi = C.POINTER(C.c_int)
_pvp = C.POINTER(C.c_void_p)

class Dropout(C.Structure):
    """struct smlm_dropout of include/smlm.h."""
    _fields_ = [("seg_p", C.c_void_p), ("rows", C.c_int), ("seed", C.c_uint64), ("offset", C.c_uint64),
                ("mask_bits", C.c_void_p)]


class LoraOpts(C.Structure):
    """struct smlm_lora_opts of include/smlm.h."""
    _fields_ = [("dropout", C.POINTER(Dropout)), ("adapter_rank", C.c_void_p), ("packed_ranks", C.c_int),
                ("dx_rows", C.c_int), ("build_seg_indptr", C.c_void_p), ("build_seg_adapter", C.c_void_p), ("bwd_stages", C.c_int),
                ("w_row_major", C.c_int), ("build_seg_key_a", C.c_void_p), ("build_seg_key_b", C.c_void_p)]


_popts = C.POINTER(LoraOpts)

# name -> (restype, argtypes); must list every symbol include/smlm.h declares
SIGNATURES = {
    "smlm_abi_version": (_i, []),
    "smlm_strerror": (C.c_char_p, [_i]),
    "smlm_tmp_size": (_i, [_i, _psz]),
    "smlm_plan_size": (_i, [_i, _i, _psz]),
    "smlm_plan_build": (_i, [_vp, _sz, _vp, _vp, _i, _i, _i, _vp]),
    "smlm_plan_build2": (_i, [_vp, _sz, _vp, _vp, _vp, _i, _i, _vp]),
    "smlm_gemm_workspace_size": (_i, [_i, _i, _i, _i, _psz]),
    "smlm_gemm": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _i, _i, _i, _f, _vp, _vp]),
    "smlm_gemm_static": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _f, _vp, _vp]),
    "smlm_gemm_planned_workspace_size": (_i, [_i, _i, _i, _psz]),
    "smlm_gemm_planned": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _sz, _i, _i, _i, _i, _i, _i, _i, _f, _vp, _vp]),
    "smlm_lora_fwd_workspace_size": (_i, [_i, _i, _i, _i, _i, _psz]),
    "smlm_lora_fwd": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _sz, _i, _i, _i, _i, _i, _i, _f, _vp,
                           _vp]),
    "smlm_lora_fwd_multi_workspace_size": (_i, [_i, _i, _pi, _i, _psz]),
    "smlm_lora_fwd_multi": (_i, [_i, _pvp, _pvp, _pvp, _pvp, _pvp, _i, _pi, _pi, _vp, _vp, _sz, _i, _i, _i,
                                 _i, _f, _vp, _i, _vp]),
    "smlm_lora_fwd_multi_ex": (_i, [_i, _pvp, _pvp, _pvp, _pvp, _pvp, _i, _pi, _pi, _vp, _vp, _sz, _i, _i,
                                         _i, _i, _f, _vp, _i, _popts, _vp]),
    "smlm_lora_bwd_workspace_size": (_i, [_i, _i, _i, _i, _i, _i, _psz]),
    "smlm_lora_bwd": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _i, _i,
                           _i, _vp, _vp]),
    "smlm_lora_bwd_ex": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _i,
                                   _i, _i, _vp, _popts, _vp]),
    "smlm_lora_bwd_multi_workspace_size": (_i, [_i, _i, _i, _i, _pi, _pi, _i, _psz]),
    "smlm_lora_bwd_multi_ex": (_i, [_i, _pvp, _pvp, _pvp, _pvp, _pvp, _pvp, _pvp, _pvp, _vp, _vp, _sz, _i, _i,
                                    _i, _pi, _pi, _i, _i, _vp, _popts, _vp]),
    "smlm_rms_norm_fwd": (_i, [_vp, _vp, _vp, _vp, _i, _i, _f, _i, _vp]),
    "smlm_rms_norm_bwd_workspace_size": (_i, [_i, _i, _psz]),
    "smlm_rms_norm_bwd": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _vp]),
    "smlm_segments_build": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp]),
}

_lib = None


def load() -> C.CDLL:
    """Load the HIP library; raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m loquetier_amd.build` "
                "(hipcc, gfx950). There is no fallback path.")
        # torch ships its own copy of the HIP runtime (soname libamdhip64.so.7) and
        # hands out streams and device pointers that belong to that copy.  Importing
        # torch first makes the loader resolve this library's libamdhip64.so.7 to the
        # copy already in the process; the other order would put two runtimes in one
        # process and every launch on a torch stream would fail.
        import torch  # noqa: F401
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def strerror(code: int) -> str:
    return load().smlm_strerror(code).decode()


def check(code: int, what: str) -> None:
    if code != 0:
        raise RuntimeError(f"{what}: {strerror(code)} (code {code})")


_SIZES = {}  # the size queries are pure functions of their arguments: asked once each


def size_query(fn_name: str, *args: int) -> int:
    key = (fn_name,) + args
    n = _SIZES.get(key)
    if n is None:
        out = C.c_size_t(0)
        check(getattr(load(), fn_name)(*args, C.byref(out)), fn_name)
        n = _SIZES[key] = out.value
    return n
