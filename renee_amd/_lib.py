"""ctypes binding of the C-ABI library declared in include/xfc_mi355x.h.

There is no CPU or PyTorch fallback: if the library has not been built the
first call raises."""
from __future__ import annotations

import ctypes as C
import os

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libxfc_mi355x.so")  # written by renee_amd/build.py

_lib = None

# entry point -> argument types, in header order
_vp, _i64, _f32, _sz, _int = C.c_void_p, C.c_int64, C.c_float, C.c_size_t, C.c_int
_SIGNATURES = {
    "xfc_strerror": (C.c_char_p, [_int]),
    "xfc_abi_version": (_int, []),
    "xfc_init": (_int, []),
    "xfc_gemm_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "xfc_gemm": (_int, [_vp, _i64, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64,
                        _f32, _f32, _int, _vp, _sz, _vp]),
    "xfc_logits": (_int, [_vp, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _vp]),
    "xfc_fwd_grad_workspace_bytes": (_sz, [_i64, _i64]),
    "xfc_fwd_grad_csr": (_int, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _vp, _sz, _vp]),
    "xfc_fwd_grad_csr_static": (_int, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _vp]),
    "xfc_fwd_grad_coo": (_int, [_vp, _i64, _vp, _i64, _vp, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _sz, _vp]),
    "xfc_dx_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "xfc_dx": (_int, [_vp, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _f32, _vp, _sz, _vp]),
    "xfc_dw_update": (_int, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _f32, _f32, _f32,
                             _vp, _i64, _vp]),
    "xfc_dw_update_master": (_int, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _f32, _f32, _f32,
                                    _vp, _i64, _vp]),
    "xfc_sgd_momentum_master": (_int, [_vp, _vp, _vp, _vp, _i64, _f32, _f32, _f32, _vp]),
    "xfc_dw": (_int, [_vp, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _f32, _vp]),
    "xfc_sgd_momentum": (_int, [_vp, _vp, _vp, _i64, _f32, _f32, _f32, _vp]),
    "xfc_step_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64]),
    "xfc_step_csr": (_int, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _i64,
                            _f32, _f32, _f32, _f32, _vp, _sz, _vp]),
    "xfc_topk_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "xfc_layer_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64]),
    "xfc_topk": (_int, [_vp, _i64, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp, _vp, _vp, _sz, _vp]),
    "xfc_copy": (_int, [_vp, _vp, _i64, _vp]),
}

EXPORTS = tuple(_SIGNATURES)


class XfcError(RuntimeError):
    def __init__(self, code: int, where: str):
        self.code = code
        super().__init__(f"{where}: {lib().xfc_strerror(code).decode()} (code {code})")


def lib():
    """The loaded library; raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m renee_amd.build` "
                "(hipcc --offload-arch=gfx950); there is no fallback path")
        h = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(h, name)
            fn.restype, fn.argtypes = res, args
        _lib = h
    return _lib


def check(code: int, where: str) -> None:
    if code != 0:
        raise XfcError(code, where)
