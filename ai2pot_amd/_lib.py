"""ctypes access to libai2pot_hip.so.  There is no fallback: if the library is missing or a
call fails, an exception is raised."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None

A2P_OK, A2P_ERR_INVALID, A2P_ERR_HIP, A2P_ERR_OVERFLOW, A2P_ERR_INPUT, A2P_ERR_SEGMENT, A2P_ERR_GRID = 0, 1, 2, 3, 4, 5, 6


class A2PError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("libai2pot_hip error %d: %s" % (code, message))
        self.code = code


def lib_path():
    env = os.environ.get("AI2POT_HIP_LIB")
    return env if env else os.path.join(_HERE, "libai2pot_hip.so")


def lib():
    global _lib
    if _lib is None:
        path = lib_path()
        if not os.path.exists(path):
            raise ImportError(
                "%s not found: build it with `python -m ai2pot_amd.build` (hipcc, gfx950). "
                "There is no CPU fallback." % path)
        _lib = ctypes.CDLL(path)
        _lib.a2p_last_error.restype = ctypes.c_char_p
    return _lib


def check(rc):
    if rc != A2P_OK:
        raise A2PError(rc, lib().a2p_last_error().decode("utf-8", "replace"))


def check_status(stream_ptr):
    """Raise if a kernel flagged an input violating the contract (synchronises the stream)."""
    check(lib().a2p_check_status(ctypes.c_void_p(stream_ptr)))
