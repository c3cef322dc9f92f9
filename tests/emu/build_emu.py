"""TEST INFRASTRUCTURE: compiles the library's kernel sources and C ABI for the HOST against the
HIP emulation of hip_emu.h into tests/emu/libmolgrid_emu.so (same exported mg_* entry points, host
pointers in place of device pointers).  Nothing in the product loads it."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "libmolgrid_amd", "csrc")
LIB_PATH = os.path.join(HERE, "libmolgrid_emu.so")
SOURCES = ["capi.hip", "transform.hip", "convert.hip", "forward_sorted.hip", "forward_vector.hip",
           "forward_vector_mfma.hip", "backward.hip", "second_order.hip", "interpolate.hip"]


def _compiler():
    for c in (os.environ.get("EMU_CXX"), "/opt/rocm/llvm/bin/clang++", "/opt/rocm/lib/llvm/bin/clang++",
              "clang++"):
        if c and (os.path.sep not in c or os.path.exists(c)):
            return c
    raise RuntimeError("no clang++ found (the kernels use clang's vector extensions)")


def up_to_date():
    if not os.path.exists(LIB_PATH):
        return False
    t = os.path.getmtime(LIB_PATH)
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC)]
    deps += [os.path.join(HERE, f) for f in ("hip_emu.h", "hip_emu.cpp", "build_emu.py")]
    deps.append(os.path.join(ROOT, "include", "molgrid_hip.h"))
    return all(os.path.getmtime(d) <= t for d in deps)


def build(force=False, verbose=False):
    if not force and up_to_date():
        return LIB_PATH
    cxx = _compiler()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    flags = ["-std=c++17", "-O1", "-g", "-fPIC", "-ffp-contract=off", "-Wno-unknown-attributes",
             "-Wno-ignored-attributes", "-Wno-unused-value", "-Wno-pass-failed",
             "-I" + HERE, "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    procs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [cxx, "-x", "c++"] + flags + ["-c", os.path.join(CSRC, src), "-o", obj]
        procs.append((src, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE,
                                                 stderr=subprocess.STDOUT, text=True)))
    rt = os.path.join(objdir, "hip_emu.o")
    procs.append(("hip_emu.cpp", rt, subprocess.Popen(
        [cxx] + flags + ["-c", os.path.join(HERE, "hip_emu.cpp"), "-o", rt],
        stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    objs = []
    for src, obj, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError("host compile of %s failed:\n%s" % (src, out))
        if verbose and out.strip():
            print(out)
        objs.append(obj)
    subprocess.check_call([cxx, "-shared", "-fPIC"] + objs + ["-o", LIB_PATH])
    return LIB_PATH


if __name__ == "__main__":
    print(build(force=True, verbose="-v" in sys.argv))
