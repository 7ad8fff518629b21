"""Builds libtdist_hip.so (gfx950) from csrc/*.hip with hipcc, in-tree.

    python triton-distributed_amd/build.py            # build if sources are newer than the library
    python triton-distributed_amd/build.py --force    # always rebuild

The libraries land in triton_dist/_lib/ next to the Python package that loads them with ctypes.
hipcc cross-compiles for gfx950 without a GPU present.
"""
import argparse
import concurrent.futures
import os
import re
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
SOURCES = ["gemm.hip", "decode.hip", "moe.hip", "lib.hip", "reduce.hip"]
BENCH_SOURCES = ["bench_probes.hip"]   # libtdist_bench.so: measurement helpers, not part of the product library
BENCH_LIB_NAME = "libtdist_bench.so"

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


def bench_lib_path():
    return os.path.join(OUT_DIR, BENCH_LIB_NAME)


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")
    return exe


def _inputs():
    files = [os.path.join(CSRC, s) for s in SOURCES + BENCH_SOURCES]
    files += [os.path.join(CSRC, "common.h"), os.path.join(INCLUDE, "tdist.h"), os.path.join(INCLUDE, "tdist_bench.h")]
    return files


def is_stale():
    lib = lib_path()
    if not os.path.exists(lib) or not os.path.exists(bench_lib_path()):
        return True
    t = os.path.getmtime(lib)
    return any(os.path.getmtime(f) > t for f in _inputs())


# The GEMM instances on the 16-row MFMA blocks keep their accumulators in fixed accumulation registers that only
# their inline assembly names: the compiler must not place anything of its own there, the kernels must not spill, and
# the large ones must leave 24 registers for the producer kernel's wave beside them on the SIMD (the register file
# holds 512 per lane). Every build checks the compiler's resource report and the generated assembly for that.
GEMM_REGISTER_BUDGET = 488   # architectural (rounded up to the allocation unit of 8) + accumulation registers
PRODUCER_REGISTER_BUDGET = 24
_RESOURCE_FLAG = "-Rpass-analysis=kernel-resource-usage"
_FIXED_ACC = re.compile(r"gemm_kernelINS_\d+Elem(?:BF16|F16|FP8)NE")


def _resource_report(report):
    """[(kernel name, VGPRs, AGPRs, scratch bytes)] from the compiler's remarks."""
    out, name, vgprs, agprs = [], None, 0, 0
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
        elif name:
            out.append((name, vgprs, agprs, int(m.group(3))))
    return out


def _check_gemm_resources(report):
    offenders = []
    for name, vgprs, agprs, scratch in _resource_report(report):
        if "gemm_kernel" not in name:
            continue
        total = (vgprs + 7) // 8 * 8 + agprs
        if scratch != 0 or total > GEMM_REGISTER_BUDGET:
            offenders.append("%s: %d + %d registers, %d bytes of scratch" % (name, vgprs, agprs, scratch))
    if offenders:
        raise RuntimeError("gemm.hip: instances over the register budget (%d, no scratch):\n  %s"
                           % (GEMM_REGISTER_BUDGET, "\n  ".join(offenders)))


def _check_producer_resources(report):
    for name, vgprs, _, scratch in _resource_report(report):
        if "producer_push_kernel" in name and ((vgprs + 7) // 8 * 8 > PRODUCER_REGISTER_BUDGET or scratch != 0):
            raise RuntimeError("lib.hip: producer_push_kernel needs %d registers (budget %d: its waves must fit beside "
                               "a GEMM wave on the SIMD)" % (vgprs, PRODUCER_REGISTER_BUDGET))


def _check_fixed_accumulators(asm_text):
    """In the kernels with fixed accumulators no instruction the compiler wrote may touch an accumulation register:
    only the inline assembly (between the compiler's ASMSTART / ASMEND marks) does."""
    name, in_asm, offenders = None, False, {}
    for line in asm_text.splitlines():
        m = re.match(r"^(_ZN5tdist11gemm_kernel\S+):", line)
        if m:
            name, in_asm = (m.group(1) if _FIXED_ACC.search(m.group(1)) else None), False
            continue
        if name is None:
            continue
        t = line.strip()
        if t.startswith("s_endpgm"):
            name = None
        elif t.startswith(";;#ASMSTART"):
            in_asm = True
        elif t.startswith(";;#ASMEND"):
            in_asm = False
        elif not in_asm and t and t[0] not in ";.":
            code = t.split(";")[0]
            if re.search(r"(?<![A-Za-z0-9_.])a(\d+|\[)", code):
                offenders.setdefault(name, []).append(code.strip())
    if offenders:
        raise RuntimeError("gemm.hip: the compiler placed values in accumulation registers of kernels whose accumulators "
                           "are fixed:\n  " + "\n  ".join("%s: %s" % (k, v[0]) for k, v in offenders.items()))


def _compile_one(hipcc, src, flags=None):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc] + (flags or HIPCC_FLAGS) + ["-c", os.path.join(CSRC, src), "-o", obj]
    if src in ("gemm.hip", "lib.hip"):
        cmd += [_RESOURCE_FLAG, "-fno-caret-diagnostics"]   # (no source excerpt under each of the report's lines)
    if src == "gemm.hip":
        cmd += ["-save-temps=obj"]                          # keeps the device assembly next to the object
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode == 0 and src == "gemm.hip":
        _check_gemm_resources(res.stdout)
        with open(os.path.join(OBJ_DIR, "gemm-hip-amdgcn-amd-amdhsa-gfx950.s")) as f:
            _check_fixed_accumulators(f.read())
    if res.returncode == 0 and src == "lib.hip":
        _check_producer_resources(res.stdout)
    # the host pass does not know the device-only target feature; that line is noise, and so is the resource report
    log = "\n".join(l for l in res.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l and "-Rpass-analysis" not in l
                    and "argument unused during compilation" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, log))
    return obj, log


def _link(hipcc, objs, out):
    tmp = out + ".tmp"
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", tmp] + objs
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stdout)
    os.replace(tmp, out)


def build(force=False, verbose=True):
    """Compiles every source and links the two shared libraries: libtdist_hip.so (the product) and
    libtdist_bench.so (measurement helpers for bench.py). Returns the product library's path."""
    if not force and not is_stale():
        return lib_path()
    hipcc = _hipcc()
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(OUT_DIR, exist_ok=True)
    objs = {}
    with concurrent.futures.ThreadPoolExecutor(max_workers=8) as pool:
        for src, (obj, log) in zip(SOURCES + BENCH_SOURCES, pool.map(lambda s: _compile_one(hipcc, s), SOURCES + BENCH_SOURCES)):
            objs[src] = obj
            if verbose and log.strip():
                print(log, file=sys.stderr)
    _link(hipcc, [objs[s] for s in BENCH_SOURCES], bench_lib_path())
    _link(hipcc, [objs[s] for s in SOURCES], lib_path())
    if verbose:
        print("built", lib_path(), file=sys.stderr)
    return lib_path()


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    args = ap.parse_args()
    print(build(force=args.force))
