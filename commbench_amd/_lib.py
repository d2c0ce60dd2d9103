"""ctypes binding of include/mi_ep.h.  There is no fallback: a missing library is an error."""
import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libmi_ep.so")

_c_int_p = ctypes.POINTER(ctypes.c_int)
_vp = ctypes.c_void_p
_int = ctypes.c_int
_size = ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/mi_ep.h declaration by declaration.
SIGNATURES = {
    "mi_ep_abi_version": (_int, []),
    "mi_ep_strerror": (ctypes.c_char_p, [_int]),
    "mi_ep_get_dispatch_layout": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp]),
    "mi_ep_workspace_bytes": (_size, [_int, _int, _int, _int]),
    "mi_ep_workspace_init": (_int, [_vp, _size, _vp]),
    "mi_ep_workspace_status": (_int, [_vp, _vp]),
    "mi_ep_workspace_set_wait_limit": (_int, [_vp, ctypes.c_uint, _vp]),
    "mi_ep_device_traits": (_int, [_c_int_p, _c_int_p, _c_int_p, _vp]),
    "mi_ep_dispatch_schedule_for": (_int, [_int, _int, _int, _int, _int, _int]),
    "mi_ep_dispatch_layout": (_int, [_vp, _int, _int, _int, _int, _int, _int,
                                     _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _vp, _vp, _vp, _vp,
                                     _vp, _size, _vp]),
    "mi_ep_dispatch_layout_static": (_int, [_vp, _int, _int, _int, _int, _int, _int,
                                            _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _vp, _vp, _vp, _vp,
                                            _vp, _vp]),
    "mi_ep_route_order_bytes": (_size, [_int, _int]),
    "mi_ep_dispatch": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _int, _int,
                              _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _vp]),
    "mi_ep_dispatch_strided_scales": (_int, [_vp, _vp, ctypes.c_longlong, ctypes.c_longlong, _vp, _vp, _vp, _vp, _vp,
                                             _vp, _int, _int, _int, _int, _int, _int, _vp, _vp,
                                             ctypes.c_longlong, ctypes.c_longlong, _vp, _vp, _vp, _vp, _int, _int,
                                             _vp]),
    "mi_ep_dispatch_ranks": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _vp, _vp, _int, _int, _int, _int, _int, _int,
                                    _int, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _vp]),
    "mi_ep_dispatch_ranks_strided_scales": (_int, [_vp, _vp, ctypes.c_longlong, ctypes.c_longlong, _vp, _vp, _vp,
                                                   _int, _vp, _vp, _int, _int, _int, _int, _int, _int, _int, _int,
                                                   _vp, _vp, ctypes.c_longlong, ctypes.c_longlong, _vp, _vp, _vp,
                                                   _vp, _vp, _vp, _int, _vp]),
    "mi_ep_combine_rank_weights": (_int, [_vp, _vp, _vp, _int, _int, _int, _vp, _vp, _vp]),
    "mi_ep_dispatch_cached": (_int, [_vp, _vp, _vp, _int, _int, _int, _int, _vp, _vp, _vp, _int, _vp]),
    "mi_ep_pull_indices": (_int, [_vp, _int, _int, _vp, _vp]),
    "mi_ep_combine": (_int, [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp, _vp, _vp, _int, _vp]),
    "mi_ep_host_get_dispatch_layout": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int]),
    "mi_ep_host_dispatch_layout": (_int, [_vp, _int, _int, _int, _int, _int, _int, _vp, _vp, _vp, _vp, _vp, _vp,
                                          _vp, _vp, _vp, _int, _vp, _vp, _vp, _vp]),
    "mi_ep_host_dispatch": (_int, [_vp, _vp, _vp, _vp, _int, _int, _int, _int, _int, _int, _int,
                                   _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int]),
    "mi_ep_host_dispatch_ranks": (_int, [_vp, _vp, _vp, _vp, _int, _int, _int, _int, _int, _int, _int, _int,
                                         _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int]),
    "mi_ep_host_dispatch_cached": (_int, [_vp, _vp, _vp, _int, _int, _int, _int, _vp, _vp]),
    "mi_ep_host_combine": (_int, [_vp, _int, _vp, _vp, _vp, _vp, _int, _int, _int, _vp]),
    "mi_ep_copy_yardstick": (_int, [_vp, _vp, _size, _vp]),
    "mi_ep_read_yardstick": (_int, [_vp, _size, _vp, _vp]),
    "mi_ep_write_yardstick": (_int, [_vp, _size, _vp]),
}

STATIC_SCRATCH = 256   # MI_EP_STATIC_SCRATCH: the library's own layout scratch, for the workspace calls

_lib = None


class MiEpError(RuntimeError):
    def __init__(self, code: int, where: str):
        self.code = code
        super().__init__(f"{where} failed: {code} ({strerror(code)})")


def bind(lib: ctypes.CDLL) -> ctypes.CDLL:
    """Gives every entry point of include/mi_ep.h its prototype on a loaded library."""
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m commbench_amd.build` "
                "(there is no CPU fallback for the HIP path)")
        _lib = bind(ctypes.CDLL(LIB_PATH))
    return _lib


def use(lib) -> None:
    """Makes `lib` (a library from commbench_amd.jit, already bound) the one every later call goes
    through; None goes back to the shipped library."""
    global _lib
    _lib = lib


def strerror(code: int) -> str:
    return load().mi_ep_strerror(code).decode()


def check(code: int, where: str) -> None:
    if code != 0:
        raise MiEpError(code, where)
