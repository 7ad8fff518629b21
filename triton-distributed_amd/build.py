"""Builds libtdist_hip.so (gfx950) from csrc/*.hip with hipcc, in-tree.

    python triton-distributed_amd/build.py            # build if sources are newer than the library
    python triton-distributed_amd/build.py --force    # always rebuild

The library lands in triton_dist/_lib/ next to the Python package that loads it with ctypes.
hipcc cross-compiles for gfx950 without a GPU present.
"""
import argparse
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")
OUT_DIR = os.path.join(HERE, "triton_dist", "_lib")
OBJ_DIR = os.path.join(HERE, "build")
LIB_NAME = "libtdist_hip.so"
SOURCES = ["lib.hip", "reduce.hip", "moe.hip", "decode.hip", "gemm.hip"]

# -packed-fp32-ops is removed from the device target on purpose: no v_pk_*_f32 in any kernel.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I", INCLUDE,
    "-I", CSRC,
]


def lib_path():
    return os.path.join(OUT_DIR, LIB_NAME)


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")
    return exe


def _inputs():
    files = [os.path.join(CSRC, s) for s in SOURCES]
    files += [os.path.join(CSRC, "common.h"), os.path.join(INCLUDE, "tdist.h")]
    return files


def is_stale():
    lib = lib_path()
    if not os.path.exists(lib):
        return True
    t = os.path.getmtime(lib)
    return any(os.path.getmtime(f) > t for f in _inputs())


def _compile_one(hipcc, src):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the device-only target feature; that line is noise
    log = "\n".join(l for l in res.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, log))
    return obj, log


def build(force=False, verbose=True):
    """Compiles every source and links the shared library. Returns its path."""
    if not force and not is_stale():
        return lib_path()
    hipcc = _hipcc()
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(OUT_DIR, exist_ok=True)
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(len(SOURCES), 8)) as pool:
        for obj, log in pool.map(lambda s: _compile_one(hipcc, s), SOURCES):
            objs.append(obj)
            if verbose and log.strip():
                print(log, file=sys.stderr)
    tmp = lib_path() + ".tmp"
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", tmp] + objs
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stdout)
    os.replace(tmp, lib_path())
    if verbose:
        print("built", lib_path(), file=sys.stderr)
    return lib_path()


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    args = ap.parse_args()
    print(build(force=args.force))
