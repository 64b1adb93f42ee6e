"""ctypes binding of libmatchattn_hip.so (declared in include/matchattn_hip.h).

The library is built in-tree by matchattention_amd/build.py; loading fails loudly
when it is missing -- there is no CPU or PyTorch fallback behind mat_impl='hip'.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmatchattn_hip.so")

F32, F16, BF16 = 0, 1, 2
ABI_VERSION = 4

# name -> (restype, argtypes); must list every symbol include/matchattn_hip.h declares
_vp, _i, _f, _sz, _cp, _ll = (ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t, ctypes.c_char_p,
                              ctypes.c_longlong)
SIGNATURES = {
    "matchattn_abi_version": (_i, []),
    "matchattn_last_error": (_cp, []),
    "matchattn_forward": (_i, [_vp] * 6 + [_i] * 7 + [_f, _i, _vp]),
    "matchattn_forward_workspace_bytes": (_sz, [_i] * 8),
    "matchattn_forward_ws": (_i, [_vp] * 7 + [_sz] + [_i] * 7 + [_f, _i, _vp]),
    "matchattn_static_scratch_bytes": (_sz, []),
    "matchattn_forward_static": (_i, [_vp] * 6 + [_i] * 7 + [_f, _i, _vp]),
    "matchattn_forward_fused_workspace_bytes": (_sz, [_i] * 8),
    "matchattn_forward_fused": (_i, [_vp, _i] + [_vp] * 5 + [_ll, _vp, _ll, _vp, _sz] + [_i] * 7 + [_f, _i, _vp]),
    "matchattn_backward_workspace_bytes": (_sz, [_i] * 8),
    "matchattn_backward": (_i, [_vp] * 11 + [_sz] + [_i] * 7 + [_f, _i, _vp]),
    "matchattn_set_option": (_i, [_cp, _i]),
    "matchattn_last_forward_kernel": (_cp, []),
    "matchattn_last_backward_kernel": (_cp, []),
    "matchattn_last_forward_kernel_ms": (ctypes.c_float, []),
    "matchattn_forward_deferred": (_i, [_vp, _sz] + [_i] * 8 + [_vp, ctypes.POINTER(ctypes.c_longlong)]),
}

_lib = None


class MatchAttnError(RuntimeError):
    pass


def load():
    """Load the shared library once; raise if it is absent or of another ABI."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MatchAttnError(
            f"{LIB_PATH} not found: build it with `python -m matchattention_amd.build` "
            "(mat_impl='hip' has no fallback path)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    if lib.matchattn_abi_version() != ABI_VERSION:
        raise MatchAttnError(f"{LIB_PATH}: ABI {lib.matchattn_abi_version()}, binding expects {ABI_VERSION}")
    _lib = lib
    return lib


def check(rc: int):
    if rc != 0:
        raise MatchAttnError(load().matchattn_last_error().decode() or f"matchattn error {rc}")


def set_option(name: str, value: int):
    check(load().matchattn_set_option(name.encode(), int(value)))


def last_forward_kernel() -> str:
    return load().matchattn_last_forward_kernel().decode()


def last_backward_kernel() -> str:
    return load().matchattn_last_backward_kernel().decode()
