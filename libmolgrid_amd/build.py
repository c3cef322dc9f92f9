"""Compile the HIP kernels and the C ABI into ``libmolgrid_hip.so`` (gfx950 only).

Run as ``python libmolgrid_amd/build.py`` (by path: importing the package needs the library
this script creates).  hipcc cross-compiles without a GPU.
"""
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libmolgrid_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)

SOURCES = ["capi.hip", "transform.hip", "forward_index.hip", "forward_channel.hip", "forward_vector.hip", "forward_vector_mfma.hip",
           "backward.hip", "second_order.hip", "interpolate.hip"]

# Packed FP32 instructions are kept out of the generated code.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wall", "-Wno-unused-function", "-Wno-pass-failed"]


# Sources whose kernels keep data in vector registers that the compiler does not manage (from
# v<MG_ACC_BASE> upwards, touched only inside asm statements).
RESERVED_REGISTER_SOURCES = ["forward_index.hip"]


def check_reserved_registers(asm_path, base):
    """Fail if compiler-generated code (anything outside an inline-asm block) of any kernel in the
    device assembly ``asm_path`` names a vector register >= ``base``, or if a kernel uses scratch
    memory.  Returns {kernel: highest compiler-used register}."""
    used, kernel, in_asm = {}, None, False
    for line in open(asm_path):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            kernel = m.group(1)
            used[kernel] = -1
            continue
        if "#ASMSTART" in line:
            in_asm = True
            continue
        if "#ASMEND" in line:
            in_asm = False
            continue
        m = re.match(r"^; ScratchSize: (\d+)", line)
        if m and int(m.group(1)) != 0:
            raise RuntimeError("%s: a kernel spills to scratch memory" % asm_path)
        stripped = line.strip()
        if in_asm or kernel is None or stripped.startswith((".", ";")):
            continue
        code = line.split(";")[0]
        regs = [int(b) for _, b in re.findall(r"\bv\[(\d+):(\d+)\]", code)]
        regs += [int(a) for a in re.findall(r"\bv(\d+)\b", code)]
        for r in regs:
            used[kernel] = max(used[kernel], r)
            if r >= base:
                raise RuntimeError("%s: compiler-allocated v%d reaches the reserved registers "
                                   "(v%d and up) in %s:\n  %s" % (asm_path, r, base, kernel, stripped))
    return used


def build(verbose=True):
    """Compile every source to an object in parallel, then link."""
    hipcc = os.environ.get("HIPCC", "hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    include = ["-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    procs = []
    checks = []
    for src in RESERVED_REGISTER_SOURCES:
        text = open(os.path.join(CSRC, src)).read()
        base = int(re.search(r"#define\s+MG_ACC_BASE\s+(\d+)", text).group(1))
        asm = os.path.join(objdir, src.replace(".hip", ".s"))
        cmd = [hipcc] + HIP_FLAGS + include + ["-S", "--cuda-device-only", os.path.join(CSRC, src),
                                               "-o", asm]
        checks.append((src, asm, base, subprocess.Popen(cmd, stdout=subprocess.PIPE,
                                                        stderr=subprocess.STDOUT, text=True)))
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc] + HIP_FLAGS + include + ["-c", os.path.join(CSRC, src), "-o", obj]
        procs.append((src, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE,
                                                 stderr=subprocess.STDOUT, text=True)))
    objs = []
    for src, obj, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines()
                        if "packed-fp32-ops' is not a recognized feature" not in l)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        if verbose and out.strip():
            print(out)
        objs.append(obj)
    for src, asm, base, p in checks:
        out, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError("hipcc -S failed on %s:\n%s" % (src, out))
        used = check_reserved_registers(asm, base)
        if verbose:
            print("%s: compiler uses at most v%d, v%d and up are reserved"
                  % (src, max(used.values()), base))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB_PATH]
    subprocess.check_call(cmd)
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
