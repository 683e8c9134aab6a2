"""ctypes binding of libfblt_probes.so: the measurement yardsticks bench.py's --probe-* modes run
(plain streaming copy and read, matrix / vector issue probe).  Not part of the attention backend."""
import ctypes as C
import os

LIB_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "lib", "libfblt_probes.so")

_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: run `python -m fblt_amd.build`" % LIB_PATH)
        import torch  # noqa: F401  (one HIP runtime per process: torch's comes first)
        lib = C.CDLL(LIB_PATH)
        lib.blt_probe_stream_copy.restype, lib.blt_probe_stream_copy.argtypes = None, [C.c_void_p, C.c_void_p, C.c_size_t]
        lib.blt_probe_stream_read.restype, lib.blt_probe_stream_read.argtypes = C.c_float, [C.c_void_p, C.c_size_t, C.c_int]
        lib.blt_probe_issue.restype, lib.blt_probe_issue.argtypes = C.c_float, [C.c_int, C.c_int]
        _lib = lib
    return _lib
