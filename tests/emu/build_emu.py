"""TEST INFRASTRUCTURE: compiles the library's kernel sources and C ABI for the HOST against the
HIP emulation of hip_emu.h into tests/emu/libmolgrid_emu.so (same exported mg_* entry points, host
pointers in place of device pointers).  Nothing in the product loads it."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "libmolgrid_amd", "csrc")
SOURCES = ["capi.hip", "transform.hip", "convert.hip", "forward_sorted.hip", "forward_vector.hip",
           "forward_vector_mfma.hip", "backward.hip", "second_order.hip", "interpolate.hip"]

# EMU_SANITIZE selects a second build of the same sources with clang's run-time checks, every report
# fatal: "1" the undefined-behaviour checks (array indices of fixed-size arrays -- the register and
# LDS arrays of the kernels --, shifts, signed overflow, float-to-int conversions out of range,
# misaligned accesses), "list" the same but reporting and going on (to see every place at once),
# "address" the address checks (every LDS array -- static storage here -- and every stack array gets
# poisoned neighbours, so an access through a pointer that leaves its array is caught as well).
# EMU_CONTRACT=1: a build that contracts a * b + c into one fused operation wherever the source
# allows it, as the device compiler does by default (the plain build contracts nothing): the paths
# that must match the reference bit for bit have to say so themselves (fp contract(off)).
CONTRACT = os.environ.get("EMU_CONTRACT", "") not in ("", "0")
SANITIZE = os.environ.get("EMU_SANITIZE", "")
if SANITIZE in ("0",):
    SANITIZE = ""
if SANITIZE == "address":
    SAN_FLAGS = ["-fsanitize=address", "-fno-omit-frame-pointer"]
    TAG = "asan"
else:
    SAN_FLAGS = ["-fsanitize=undefined,float-cast-overflow", "-fno-sanitize=vptr,function",
                 "-fsanitize-recover=all" if SANITIZE == "list" else "-fno-sanitize-recover=all"]
    TAG = "ubsan"
if CONTRACT and not SANITIZE:
    SANITIZE, TAG, SAN_FLAGS = "contract", "contract", []
LIB_PATH = os.path.join(HERE, "libmolgrid_emu_%s.so" % TAG if SANITIZE else "libmolgrid_emu.so")


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
    objdir = os.path.join(HERE, "build_" + TAG if SANITIZE else "build")
    os.makedirs(objdir, exist_ok=True)
    flags = ["-std=c++17", "-O1", "-g", "-fPIC", "-ffp-contract=off", "-Wno-unknown-attributes",
             "-Wno-ignored-attributes", "-Wno-unused-value", "-Wno-pass-failed",
             "-I" + HERE, "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    if SANITIZE:
        flags += SAN_FLAGS
    if CONTRACT:
        flags = [f for f in flags if f != "-ffp-contract=off"] + ["-ffp-contract=fast-honor-pragmas", "-mfma"]
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
    link = []
    if SANITIZE and SAN_FLAGS:      # the checks' runtime as a shared library, found beside the compiler
        rt = subprocess.check_output([cxx, "-print-resource-dir"], text=True).strip() + "/lib/linux"
        link = SAN_FLAGS + ["-shared-libsan", "-Wl,-rpath," + rt]
    subprocess.check_call([cxx, "-shared", "-fPIC"] + link + objs + ["-o", LIB_PATH])
    return LIB_PATH


def build_cpp_api_test():
    """tests/cpp/test_api.cpp (the C++ classes of include/libmolgrid) compiled against the emulation
    and linked with the emulated library: the C++ host layer on the CPU."""
    lib = build()
    out = os.path.join(HERE, "test_api_emu")
    src = os.path.join(ROOT, "tests", "cpp", "test_api.cpp")
    deps = [src, lib] + [os.path.join(ROOT, "include", "libmolgrid", f)
                         for f in os.listdir(os.path.join(ROOT, "include", "libmolgrid"))]
    if os.path.exists(out) and all(os.path.getmtime(d) <= os.path.getmtime(out) for d in deps):
        return out
    subprocess.check_call([_compiler(), "-std=c++17", "-O1", "-g", "-Wno-unknown-attributes",
                           "-Wno-ignored-attributes", "-I" + HERE, "-I" + os.path.join(ROOT, "include"),
                           src, "-o", out, "-L" + HERE, "-l" + os.path.basename(lib)[3:-3],
                           "-Wl,-rpath,$ORIGIN"])
    return out


if __name__ == "__main__":
    print(build(force=True, verbose="-v" in sys.argv))
