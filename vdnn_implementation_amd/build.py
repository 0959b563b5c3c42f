"""Builds the native parts of the package for gfx950, in-tree.

  libvdnn_amd.so : device back end (HIP kernels behind include/vdnn_backend.h) + the C++ host classes
                   (Layer, Network) + their C API (include/vdnn_capi.h)
  bin/vdnn       : the command-line front end, `vdnn MODEL POLICY ALGO`

Usage: python -m vdnn_implementation_amd.build [--force]
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
OBJ = os.path.join(PKG, "build")
LIB = os.path.join(PKG, "libvdnn_amd.so")
BIN = os.path.join(PKG, "bin", "vdnn")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops is switched off: some packed fp32 forms have given wrong results on this hardware
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
COMMON = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-command-line-argument", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]

DEVICE_SOURCES = ["backend.hip", "eltwise.hip", "conv.hip", "fc.hip", "zvc.hip"]
HOST_SOURCES = ["pool.cpp", "layer.cpp", "network.cpp", "capi.cpp"]
CLI_SOURCE = "vdnn_main.cpp"


def _deps_newer(target, sources):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    hdrs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hdrs += [os.path.join(ROOT, "include", f) for f in os.listdir(os.path.join(ROOT, "include"))]
    return any(os.path.getmtime(s) > t for s in list(sources) + hdrs)


def _compile(src, force):
    path = os.path.join(CSRC, src)
    obj = os.path.join(OBJ, src + ".o")
    if not force and not _deps_newer(obj, [path]):
        return obj
    if src.endswith(".hip"):
        cmd = [HIPCC] + COMMON + DEVICE_FLAGS + ["-c", path, "-o", obj]
    else:
        # host code: no contraction, so the seeded generator rounds the same way everywhere
        cmd = [HIPCC] + COMMON + ["-ffp-contract=off", "-c", path, "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("compile failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        sys.stderr.write(out + "\n")
    return obj


def build(force=False, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(os.path.dirname(BIN), exist_ok=True)
    sources = [s for s in DEVICE_SOURCES + HOST_SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with ThreadPoolExecutor(max_workers=min(8, len(sources))) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), sources))
    if force or _deps_newer(LIB, objs):
        cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
        subprocess.check_call(cmd)
    cli = os.path.join(CSRC, CLI_SOURCE)
    if os.path.exists(cli) and (force or _deps_newer(BIN, [cli, LIB])):
        cmd = [HIPCC] + COMMON + ["-ffp-contract=off", cli, "-o", BIN, "-L" + PKG, "-lvdnn_amd", "-Wl,-rpath,$ORIGIN/.."]
        subprocess.check_call(cmd)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
