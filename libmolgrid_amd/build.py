"""Compile the HIP kernels and the C ABI into ``libmolgrid_hip.so`` (gfx950 only).

Run as ``python libmolgrid_amd/build.py`` (by path: importing the package needs the library
this script creates).  hipcc cross-compiles without a GPU.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libmolgrid_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)

SOURCES = ["capi.hip", "transform.hip", "convert.hip", "forward_sorted.hip", "forward_vector.hip", "forward_vector_mfma.hip",
           "backward.hip", "second_order.hip", "interpolate.hip"]

# Packed FP32 instructions are kept out of the generated code.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wall", "-Wno-unused-function", "-Wno-pass-failed"]


def build(verbose=True):
    """Compile every source to an object in parallel, then link."""
    hipcc = os.environ.get("HIPCC", "hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    include = ["-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    procs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc] + HIP_FLAGS + include + ["-c", os.path.join(CSRC, src), "-o", obj]
        procs.append((src, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE,
                                                 stderr=subprocess.STDOUT, text=True)))
    objs = []
    for src, obj, p in procs:
        out, _ = p.communicate()
        # hipcc compiles every source twice, for gfx950 and for the host; the flag above names a
        # gfx950 feature, the device pass honours it (no v_pk_*_f32 in the ISA) and the HOST pass
        # (x86-64) says it does not know the feature -- that one line is dropped here
        out = "\n".join(l for l in out.splitlines()
                        if "packed-fp32-ops' is not a recognized feature" not in l)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        if verbose and out.strip():
            print(out)
        objs.append(obj)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB_PATH]
    subprocess.check_call(cmd)
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
