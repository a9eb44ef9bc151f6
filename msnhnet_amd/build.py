"""Builds the shared libraries of the package in-tree:

  msnhnet_amd/lib/libmsnh_hip.so   HIP kernels + C ABI (include/msnh_hip.h), hipcc --offload-arch=gfx950
  msnhnet_amd/lib/libMsnhnet.so    C++ host side (NetBuilder, Parser, layers) + C facade (include/msnhnet_c.h)
  msnhnet_amd/lib/libmsnh_diag.so  timing diagnostics (include/msnh_hip_diag.h; measurement only, nothing in the product loads it)

Run as `python -m msnhnet_amd.build` or through `__graft_entry__.build()`.
"""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "msnhnet_amd")
LIB = os.path.join(PKG, "lib")
OBJ = os.path.join(PKG, "build")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument", "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(PKG, "csrc")]
HOST_FLAGS = ["-O3", "-march=x86-64-v3", "-ffp-contract=off", "-std=c++17", "-fPIC", "-fopenmp-simd", "-Wall", "-Wextra", "-I" + os.path.join(ROOT, "include"),
              "-I" + os.path.join(PKG, "host", "include")]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    return out


# `python -m msnhnet_amd.build --changed` (a developer convenience; build_all() itself always compiles everything) skips a
# source whose object is newer than the source and every header of the tree.
ONLY_CHANGED = False


def _newest_header():
    hs = glob.glob(os.path.join(PKG, "csrc", "*.hpp")) + glob.glob(os.path.join(ROOT, "include", "*.h")) + \
        glob.glob(os.path.join(PKG, "host", "include", "**", "*.h"), recursive=True)
    return max(os.path.getmtime(h) for h in hs)


def _compile(src, obj, flags, compiler):
    os.makedirs(os.path.dirname(obj), exist_ok=True)
    if ONLY_CHANGED and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), _newest_header()):
        return ""
    return _run([compiler, *flags, "-c", src, "-o", obj])


def build_hip(verbose=True):
    srcs = sorted(glob.glob(os.path.join(PKG, "csrc", "*.hip")))
    objs = [os.path.join(OBJ, "hip", os.path.basename(s) + ".o") for s in srcs]
    diag_srcs = sorted(glob.glob(os.path.join(PKG, "csrc", "diag", "*.hip")))
    diag_objs = [os.path.join(OBJ, "hip", "diag_" + os.path.basename(s) + ".o") for s in diag_srcs]
    with ThreadPoolExecutor(max_workers=8) as ex:
        for out in ex.map(lambda so: _compile(so[0], so[1], HIP_FLAGS, HIPCC), zip(srcs + diag_srcs, objs + diag_objs)):
            if verbose and out.strip():
                print(out)
    os.makedirs(LIB, exist_ok=True)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", os.path.join(LIB, "libmsnh_hip.so"), *objs])
    if diag_objs:
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", os.path.join(LIB, "libmsnh_diag.so"), *diag_objs,
              "-L" + LIB, "-lmsnh_hip", "-Wl,-rpath,$ORIGIN"])
    return os.path.join(LIB, "libmsnh_hip.so")


def build_host(verbose=True):
    srcs = sorted(glob.glob(os.path.join(PKG, "host", "src", "*.cpp")))
    if not srcs:
        return None
    objs = [os.path.join(OBJ, "host", os.path.basename(s) + ".o") for s in srcs]
    with ThreadPoolExecutor(max_workers=8) as ex:
        for out in ex.map(lambda so: _compile(so[0], so[1], HOST_FLAGS, "g++"), zip(srcs, objs)):
            if verbose and out.strip():
                print(out)
    os.makedirs(LIB, exist_ok=True)
    _run(["g++", "-shared", "-fPIC", "-o", os.path.join(LIB, "libMsnhnet.so"), *objs,
          "-L" + LIB, "-lmsnh_hip", "-Wl,-rpath,$ORIGIN", "-lpthread"])
    return os.path.join(LIB, "libMsnhnet.so")


def build_all(verbose=True):
    a = build_hip(verbose)
    b = build_host(verbose)
    return a, b


if __name__ == "__main__":
    import sys
    ONLY_CHANGED = "--changed" in sys.argv[1:]
    print(build_all())
