"""ctypes binding of libtandem_probe.so (include/tandem_probe.h): the stream-mix measurement
kernel. Not part of the plug-in: bench.py and the GPU tests load it, nothing in this package does."""

import ctypes
import os

PROBE_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libtandem_probe.so")
_probe = None


def lib():
    global _probe
    if _probe is None:
        if not os.path.exists(PROBE_PATH):
            raise RuntimeError(f"{PROBE_PATH} has not been built; run `python -m tandem_amd.build`")
        L = ctypes.CDLL(PROBE_PATH)
        L.tdm_probe_stream_mix.restype = ctypes.c_int
        L.tdm_probe_stream_mix.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_int, ctypes.POINTER(ctypes.c_void_p), ctypes.c_int,
                                           ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        L.tdm_probe_last_error.restype = ctypes.c_char_p
        L.tdm_probe_last_error.argtypes = []
        _probe = L
    return _probe


def check(status):
    if status == 0:
        return
    msg = lib().tdm_probe_last_error().decode(errors="replace")
    raise (ValueError if status == 1 else RuntimeError)(msg)
