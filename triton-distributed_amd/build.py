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


# The four-wave GEMM instances (one wave per SIMD, 256 accumulators in AGPRs) are only fast while the compiler keeps
# their loops free of spills, and they must leave registers for a copy kernel's wave beside them on the SIMD (the
# register file holds 512 per lane). Small edits far from the K loop have tipped the allocation over, so every build
# checks the compiler's own resource report.
GEMM_REGISTER_BUDGET = 480   # architectural + accumulation registers per lane
_RESOURCE_FLAG = "-Rpass-analysis=kernel-resource-usage"


def _check_gemm_resources(report):
    import re
    name, vgprs, agprs, offenders = None, 0, 0, []
    for line in report.splitlines():
        m = re.search(r"remark: (?:Function Name: (\S+)|\s+(VGPRs|AGPRs|ScratchSize \[bytes/lane\]): (\d+))", line)
        if not m:
            continue
        if m.group(1):
            name, vgprs, agprs = m.group(1), 0, 0
        elif m.group(2) == "VGPRs":
            vgprs = int(m.group(3))
        elif m.group(2) == "AGPRs":
            agprs = int(m.group(3))
        elif name and "gemm_kernel" in name and re.search(r"ELi2ELi2ELi\d+ELb", name):   # WM = WN = 2
            total = (vgprs + 7) // 8 * 8 + agprs
            if int(m.group(3)) != 0 or total > GEMM_REGISTER_BUDGET:
                offenders.append("%s: %d + %d registers, %s bytes of scratch" % (name, vgprs, agprs, m.group(3)))
    if offenders:
        raise RuntimeError("gemm.hip: four-wave instances over the register budget (%d, no scratch):\n  %s"
                           % (GEMM_REGISTER_BUDGET, "\n  ".join(offenders)))


def _compile_one(hipcc, src):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    if src == "gemm.hip":
        cmd += [_RESOURCE_FLAG, "-fno-caret-diagnostics"]   # (no source excerpt under each of the report's lines)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if src == "gemm.hip" and res.returncode == 0:
        _check_gemm_resources(res.stdout)
    # the host pass does not know the device-only target feature; that line is noise, and so is the resource report
    log = "\n".join(l for l in res.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l and "-Rpass-analysis" not in l)
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
