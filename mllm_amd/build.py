"""Compiles the HIP sources under mllm_amd/csrc for gfx950 into mllm_amd/lib/libmllm_hip_qlinear.so.

hipcc cross-compiles without a GPU.  The library is built in-tree so that it travels with the source tree.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libmllm_hip_qlinear.so")
HOST_LIB = os.path.join(LIBDIR, "libmllm_hip_backend.so")  # C++ op-factory layer on top of the C ABI
HOST = os.path.join(CSRC, "host")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# no fast-math: the activation quantization needs correctly rounded fp32 division and plain multiplies;
# packed fp32 instructions are switched off (hipcc may otherwise form them from scalar code).
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-fno-fast-math",
         "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, "-Wall", "-Wno-unused-function"]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src, keep_asm=False):
    obj = os.path.join(LIBDIR, "obj", src[:-4] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    if keep_asm:
        cmd += ["--save-temps=obj"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(keep_asm=False, jobs=8):
    os.makedirs(os.path.join(LIBDIR, "obj"), exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, keep_asm), sources()))
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs,
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    build_host()
    return LIB


def build_host():
    """The C++ host layer (mllm-compatible Backend / ops) as its own library, linked against the kernel library."""
    srcs = sorted(os.path.join(HOST, f) for f in os.listdir(HOST) if f.endswith(".cpp"))
    cmd = [HIPCC, "-x", "hip", "--offload-arch=gfx950", "-O2", "-std=c++20", "-fPIC", "-shared", "-fvisibility=hidden",
           "-I" + os.path.join(ROOT, "include"), "-I" + HOST, "-Wall", "-o", HOST_LIB] + srcs + [
           "-L" + LIBDIR, "-lmllm_hip_qlinear", "-Wl,-rpath,$ORIGIN", "-ldl"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("host layer build failed:\n" + err)
    if err.strip():
        sys.stderr.write(err + "\n")
    return HOST_LIB


if __name__ == "__main__":
    print(build(keep_asm="--asm" in sys.argv))
