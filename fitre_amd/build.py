"""Builds the two shared libraries of the package, in-tree.

  libfitre_hip.so  HIP kernels + the C-ABI device layer (include/fitre_hip.h), hipcc, gfx950
  libfitre_cnn.so  C host code: model layout, cnnForward / cnnBackward / computeCNNGradient and
                   the reference-named device shim (include/fitre_cnn.h, include/fitre_shim.h), gcc

Run as ``python -m fitre_amd.build``.  hipcc cross-compiles for gfx950 without a GPU.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "fitre_amd")
HIP_DIR = os.path.join(PKG, "csrc", "hip")
HOST_DIR = os.path.join(PKG, "csrc", "host")
INC = os.path.join(ROOT, "include")
OBJ = os.path.join(PKG, "csrc", "build")

HIP_LIB = os.path.join(PKG, "libfitre_hip.so")
CNN_LIB = os.path.join(PKG, "libfitre_cnn.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-I" + INC, "-I" + HIP_DIR,
    # keep the compiler from forming packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]
HIPCC_FLAGS += os.environ.get("FITRE_HIPCC_EXTRA", "").split()  # e.g. -D switches while tuning a kernel
GCC_FLAGS = ["-O2", "-std=c11", "-fPIC", "-Wall", "-Wextra", "-I" + INC]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def _sources(directory, ext):
    return sorted(os.path.join(directory, f) for f in os.listdir(directory) if f.endswith(ext))


def build_hip(verbose=True, jobs=8):
    os.makedirs(OBJ, exist_ok=True)
    srcs = _sources(HIP_DIR, ".hip")
    objs = [os.path.join(OBJ, os.path.basename(s)[:-4] + ".o") for s in srcs]

    def compile_one(pair):
        src, obj = pair
        out = _run(["hipcc"] + HIPCC_FLAGS + ["-c", src, "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, zip(srcs, objs)))
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", HIP_LIB] + objs)
    return HIP_LIB


def build_host(verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    srcs = _sources(HOST_DIR, ".c")
    objs = []
    for src in srcs:
        obj = os.path.join(OBJ, "host_" + os.path.basename(src)[:-2] + ".o")
        out = _run(["gcc"] + GCC_FLAGS + ["-c", src, "-o", obj])
        if verbose and out.strip():
            print(out)
        objs.append(obj)
    _run(["gcc", "-shared", "-fPIC", "-o", CNN_LIB] + objs +
         ["-L" + PKG, "-lfitre_hip", "-Wl,-rpath,$ORIGIN", "-lm"])
    return CNN_LIB


def stamp_tree():
    """Notes the commit the libraries are built from (fitre_amd/BUILD_TREE, a '+' behind it when the tree has changes
    that are not committed): what bench.py reports where the tree travels without its history."""
    try:
        rev = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], stdout=subprocess.PIPE, stderr=subprocess.DEVNULL,
                             text=True, timeout=10).stdout.strip()
        dirty = subprocess.run(["git", "-C", ROOT, "status", "--porcelain", "--untracked-files=no"], stdout=subprocess.PIPE,
                               stderr=subprocess.DEVNULL, text=True, timeout=10).stdout.strip()
    except (OSError, subprocess.SubprocessError):
        return
    if rev:
        with open(os.path.join(PKG, "BUILD_TREE"), "w") as f:
            f.write(rev + ("+" if dirty else "") + "\n")


def build_all(verbose=True):
    build_hip(verbose)
    build_host(verbose)
    stamp_tree()
    return HIP_LIB, CNN_LIB


if __name__ == "__main__":
    libs = build_all()
    print("built:", *libs, file=sys.stderr)
