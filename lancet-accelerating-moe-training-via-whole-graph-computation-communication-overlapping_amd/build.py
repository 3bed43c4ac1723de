"""Builds the in-tree native libraries with hipcc for gfx950.

liblancet_hip.so      HIP kernels + the C ABI declared in include/lancet_hip.h
liblancet_raf_ops.so  C++ op layer (RAF OpEnv / dialect vocabulary) on top of the C ABI

Run `python build.py` (or __graft_entry__.build()).  hipcc cross-compiles without a GPU.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")

HIP_SOURCES = ["capi.hip", "moe_route.hip", "moe_bpr.hip", "moe_rows.hip", "moe_gate_grad.hip", "sparse_copy.hip", "lans.hip", "static_scratch.hip"]
HIP_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC",
    # Packed fp32 arithmetic stays off for every kernel of this library.  The option reaches both passes of
    # hipcc: the device pass (gfx950) takes it, the host pass (x86-64) prints "'-packed-fp32-ops' is not a
    # recognized feature for this target (ignoring feature)" once per file, which is harmless; the driver has
    # no form of it that reaches the device pass alone (-Xarch_device does not forward -Xclang).
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _hipcc():
    return shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.stdout.strip():
        print(proc.stdout, flush=True)   # everything the compiler says
    if proc.returncode != 0:
        raise RuntimeError("command failed (%d): %s" % (proc.returncode, " ".join(cmd)))


def build_hip(verbose=True):
    os.makedirs(LIBDIR, exist_ok=True)
    objs = []
    for src in HIP_SOURCES:
        obj = os.path.join(LIBDIR, src.replace(".hip", ".o"))
        _run([_hipcc()] + HIP_FLAGS + os.environ.get("LANCET_EXTRA_HIPFLAGS", "").split() + ["-c", os.path.join(CSRC, src), "-o", obj])
        objs.append(obj)
    out = os.path.join(LIBDIR, "liblancet_hip.so")
    _run([_hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", out] + objs)
    return out


def build_ops():
    src_dir = os.path.join(HERE, "raf_hip")
    srcs = sorted(os.path.join(src_dir, f) for f in os.listdir(src_dir) if f.endswith(".cc"))
    if not srcs:
        return None
    out = os.path.join(LIBDIR, "liblancet_raf_ops.so")
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-I", os.path.join(ROOT, "include"),
          "-I", src_dir, "-o", out] + srcs +
         ["-L", LIBDIR, "-llancet_hip", "-Wl,-rpath,$ORIGIN"])
    return out


def build_all():
    a = build_hip()
    b = build_ops()
    return [p for p in (a, b) if p]


if __name__ == "__main__":
    for p in build_all():
        print("built", p)
    sys.exit(0)
