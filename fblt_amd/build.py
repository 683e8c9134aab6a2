"""Builds fblt_amd/lib/libfblt_hip.so: host C99 (gcc) + gfx950 HIP (hipcc); and the
bench-only counter yardstick fblt_amd/lib/libfblt_probes.so.

`python -m fblt_amd.build` or `fblt_amd.build.build()`.  Objects go to
fblt_amd/lib/obj; nothing is compiled at import time, and loading the library
never falls back to anything else.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(LIBDIR, "obj")
LIB = os.path.join(LIBDIR, "libfblt_hip.so")
# the counter yardstick of bench.py's --probe-copy-mib mode: its own small library, not in the backend's ABI
PROBES_SRC = os.path.join(HERE, "probes", "probes.hip")
PROBES_LIB = os.path.join(LIBDIR, "libfblt_probes.so")

HIP_SOURCES = ["memory.hip", "mask_builder.hip", "vecmath.hip", "attn_rows.hip", "attn_mfma.hip", "attn_wide.hip", "attn_fine.hip", "attn_once.hip", "matmul.hip", "rope.hip", "mha.hip", "layer_ops.hip", "encoder.hip", "stream.hip",
               "attn_decode.hip", "attn_decode_row.hip", "attn_verify.hip", "attn_verify_once.hip", "attn_api.hip", "profile.hip"]
C_SOURCES = ["host/blt_host.c"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
INCLUDES = ["-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
# -packed-fp32-ops off: hipcc must not form packed fp32 instructions on this pool
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"] + INCLUDES
C_FLAGS = ["-std=c99", "-O2", "-fPIC", "-Wall", "-Wextra", "-Werror=implicit-function-declaration", "-D_POSIX_C_SOURCE=200809L"] + INCLUDES


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError("build step failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(verbose=False, jobs=8):
    os.makedirs(OBJDIR, exist_ok=True)
    steps = []
    objs = []
    for src in HIP_SOURCES:
        obj = os.path.join(OBJDIR, os.path.basename(src) + ".o")
        objs.append(obj)
        steps.append([HIPCC] + HIP_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])
    for src in C_SOURCES:
        obj = os.path.join(OBJDIR, os.path.basename(src) + ".o")
        objs.append(obj)
        steps.append(["gcc"] + C_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])
    steps.append([HIPCC] + HIP_FLAGS + ["-shared", PROBES_SRC, "-o", PROBES_LIB])
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        for out in ex.map(_run, steps):
            if verbose and out.strip():
                print(out)
    out = _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
