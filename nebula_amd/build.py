"""Builds the product libraries in-tree with hipcc (gfx950 only).

    python -m nebula_amd.build          # libnebula_hip.so (+ libnebula_layers.so when its sources exist)

The flags switch off packed-fp32 code generation for the device pass, as this pool of machines requires.
"""
import glob
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(PKG, "host")
LIBDIR = os.path.join(PKG, "lib")
HIP_SO = os.path.join(LIBDIR, "libnebula_hip.so")
LAYERS_SO = os.path.join(LIBDIR, "libnebula_layers.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option"]


def _run(cmd):
    print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_hip(verbose=True):
    os.makedirs(LIBDIR, exist_ok=True)
    objs = []
    procs = []
    for src in sorted(glob.glob(os.path.join(CSRC, "*.hip"))):
        obj = os.path.join(LIBDIR, os.path.basename(src)[:-4] + ".o")
        cmd = [HIPCC] + DEVICE_FLAGS + ["-I", os.path.join(ROOT, "include"), "-I", CSRC, "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd)))
        objs.append(obj)
    for src, p in procs:
        if p.wait() != 0:
            raise RuntimeError("hipcc failed on " + src)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", HIP_SO] + objs)
    return HIP_SO


def build_layers(verbose=True):
    srcs = sorted(glob.glob(os.path.join(HOST, "*.cc")))
    if not srcs:
        return None
    _run(["g++", "-O2", "-std=c++11", "-fPIC", "-shared", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I", "/opt/rocm/include",
          "-I", os.path.join(ROOT, "include"), "-I", HOST,
          "-o", LAYERS_SO] + srcs + ["-L", LIBDIR, "-lnebula_hip", "-L", "/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib"])
    return LAYERS_SO


def build_all():
    build_hip()
    build_layers()


if __name__ == "__main__":
    build_all()
    print("built:", HIP_SO, file=sys.stderr)
