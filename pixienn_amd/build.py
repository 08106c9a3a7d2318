"""Builds libpixienn_hip.so (the gfx950 kernels + C ABI) in-tree with hipcc."""
import concurrent.futures
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
OBJ = os.path.join(PKG, "build")
LIB = os.path.join(PKG, "libpixienn_hip.so")

SOURCES = ["runtime.hip", "epilogue.hip", "elementwise.hip", "pool.hip", "yolo.hip", "nms.hip"]

# -ffp-contract=off: the bit-exact kernels must not fuse a*b+c; packed fp32 VALU forms are
# switched off for every kernel.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-std=c++20", "-O3", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wextra", "-Wno-unused-parameter", "-Wno-unknown-attributes",
]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(src):
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc()] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    return src, obj, proc


def build_library(verbose=True):
    """Compiles every HIP source for gfx950 and links the shared library.  Always recompiles."""
    os.makedirs(OBJ, exist_ok=True)
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        for src, obj, proc in pool.map(_compile, SOURCES):
            noise = "\n".join(l for l in proc.stderr.splitlines()
                              if "packed-fp32-ops" not in l and l.strip())
            if proc.returncode != 0:
                raise RuntimeError("hipcc failed on %s:\n%s" % (src, proc.stderr))
            if verbose and noise:
                print(noise, file=sys.stderr)
            objs.append(obj)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    subprocess.check_call(cmd)
    return LIB


def build_host(verbose=True):
    """Compiles the C++ layer interface (host/pixienn/*.h, header-only) as a translation unit of
    its own: the check that it builds against the C ABI alone."""
    host = os.path.join(PKG, "host")
    probe = os.path.join(OBJ, "host_headers.cpp")
    os.makedirs(OBJ, exist_ok=True)
    with open(probe, "w") as f:
        f.write('#include "pixienn/Layers.h"\n#include "pixienn/OptimizerState.h"\n#include "pixienn/CapturedSequence.h"\n#include "pixienn/ParameterSet.h"\n#include "pixienn/WeightsFile.h"\n#include "pixienn/DeviceTraits.h"\nstatic_assert(std::is_same_v<px::hip::DeviceTraits<px::hip::Device::HIP>::ValueType, float>);\nstatic_assert(px::hip::IsHipDevice<px::hip::Device::HIP>::value && !px::hip::IsHipDevice<px::hip::Device::CPU>::value);\nint pixienn_host_headers_compile() { return PXH_OK; }\n')
    obj = os.path.join(OBJ, "host_headers.o")
    cmd = [hipcc(), "-std=c++20", "-O1", "-Wall", "-Wextra", "-Wno-unused-parameter", "-I" + os.path.join(ROOT, "include"),
           "-I" + host, "-c", probe, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("host headers do not compile:\n" + proc.stderr)
    if verbose and proc.stderr.strip():
        print(proc.stderr, file=sys.stderr)
    return obj


if __name__ == "__main__":
    print(build_library())
    print(build_host())
