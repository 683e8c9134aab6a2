"""ctypes binding of libfblt_probes.so: the two yardsticks bench.py runs (a plain streaming copy of
known size for the hardware counters, an empty kernel for the launch floor).  Not part of the
attention backend."""
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
        fp = C.POINTER(C.c_float)
        lib.blt_probe_launch_floor.restype, lib.blt_probe_launch_floor.argtypes = None, [C.c_int, fp, fp, fp]
        _lib = lib
    return _lib


def launch_floor(launches=300):
    """{event_us_mean, event_us_median, back_to_back_wall_us} of an empty kernel."""
    mean, med, wall = C.c_float(), C.c_float(), C.c_float()
    load().blt_probe_launch_floor(launches, C.byref(mean), C.byref(med), C.byref(wall))
    return {"event_us_mean": mean.value, "event_us_median": med.value, "back_to_back_wall_us": wall.value}
