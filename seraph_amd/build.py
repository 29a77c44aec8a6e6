"""Builds the native libraries in-tree.

  seraph_amd/lib/libseraph_hip.so          HIP kernels + C ABI (hipcc, gfx950 only)
  seraph_amd/lib/libseraph_hip_backend.so  host C: vulkan_* compatible backend, the packed
                                           training-step drivers and the file formats (gcc, no HIP headers)
  seraph_amd/bin/seraph-train-hip          the batched training front end (gcc)

Run as `python -m seraph_amd.build` (add --force to rebuild everything).
"""
import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
SRC = os.path.join(HERE, "src")
LIB = os.path.join(HERE, "lib")
OBJ = os.path.join(LIB, "obj")
INCLUDE = os.path.join(ROOT, "include")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-I", INCLUDE, "-I", CSRC,
             # keep the compiler from forming packed-FP32 VALU ops
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option"]
CC = os.environ.get("CC", "gcc")
C_FLAGS = ["-O2", "-std=gnu11", "-fPIC", "-Wall", "-Wextra", "-I", INCLUDE, "-I", SRC]

CLI = os.path.join(HERE, "cli")
BIN = os.path.join(HERE, "bin")
KERNEL_LIB = os.path.join(LIB, "libseraph_hip.so")
TRAIN_BIN = os.path.join(BIN, "seraph-train-hip")
BACKEND_LIB = os.path.join(LIB, "libseraph_hip_backend.so")


def _newer(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + p.stdout + "\n")
        raise RuntimeError("build step failed: " + os.path.basename(cmd[-1]))
    warn = [l for l in p.stdout.splitlines() if "warning" in l and "packed-fp32-ops" not in l and "target feature" not in l]
    if warn:
        sys.stderr.write("\n".join(warn[:20]) + "\n")


def build_kernels(force=False, jobs=8):
    os.makedirs(OBJ, exist_ok=True)
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")] + \
              [os.path.join(INCLUDE, "seraph_hip.h")]
    srcs = sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))
    objs, todo = [], []
    for f in srcs:
        o = os.path.join(OBJ, f[:-4] + ".o")
        objs.append(o)
        if force or _newer(o, [os.path.join(CSRC, f)] + headers):
            todo.append([HIPCC] + HIP_FLAGS + ["-c", os.path.join(CSRC, f), "-o", o])
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(_run, todo))
    if todo or force or not os.path.exists(KERNEL_LIB):
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", KERNEL_LIB] + objs)
    return KERNEL_LIB


def build_backend(force=False):
    if not os.path.isdir(SRC):
        return None
    srcs = sorted(os.path.join(SRC, f) for f in os.listdir(SRC) if f.endswith(".c"))
    if not srcs:
        return None
    deps = srcs + [os.path.join(INCLUDE, f) for f in os.listdir(INCLUDE)] + \
        [os.path.join(SRC, f) for f in os.listdir(SRC) if f.endswith(".h")]
    if force or _newer(BACKEND_LIB, deps + [KERNEL_LIB]):
        _run([CC] + C_FLAGS + ["-shared", "-o", BACKEND_LIB] + srcs +
             ["-L", LIB, "-lseraph_hip", "-Wl,-rpath,$ORIGIN", "-lm"])
    return BACKEND_LIB


def build_cli(force=False):
    src = os.path.join(CLI, "seraph_train_hip.c")
    if not os.path.exists(src):
        return None
    os.makedirs(BIN, exist_ok=True)
    deps = [src, BACKEND_LIB] + [os.path.join(INCLUDE, f) for f in os.listdir(INCLUDE)]
    if force or _newer(TRAIN_BIN, deps):
        _run([CC] + [f for f in C_FLAGS if f != "-fPIC"] + ["-o", TRAIN_BIN, src, "-L", LIB, "-lseraph_hip_backend",
             "-lseraph_hip", "-Wl,-rpath,$ORIGIN/../lib", "-lm"])
    return TRAIN_BIN


def build_all(force=False):
    k = build_kernels(force)
    b = build_backend(force)
    c = build_cli(force)
    return k, b, c


if __name__ == "__main__":
    print(build_all(force="--force" in sys.argv))
