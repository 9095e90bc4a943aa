"""ctypes binding of libyitu_host.so (CPU graph preparation: reorder, sampler)."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libyitu_host.so")
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libyitu_host.so is not built; run `python -m yitu_amd.build`")
        l = ctypes.CDLL(LIB_PATH)
        l.yitu_host_last_error.restype = ctypes.c_char_p
        l.yitu_sampler_last_error.restype = ctypes.c_char_p
        l.yitu_sampler_create.restype = ctypes.c_void_p
        l.yitu_sampler_create_modes.restype = ctypes.c_void_p
        l.yitu_sampler_num_blocks.restype = ctypes.c_int64
        _lib = l
    return _lib
