"""The build refuses a GEMM whose instances spill, leave no registers for the producer kernel's wave beside them, or
in which the compiler used a register that the kernels with fixed accumulators reserve for their assembly (host logic
only: the checks read the compiler's resource report and its assembly output)."""
import importlib.util
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load_build():
    spec = importlib.util.spec_from_file_location("tdist_build", os.path.join(ROOT, "triton-distributed_amd", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def report(name, vgprs, agprs, scratch):
    tag = " [-Rpass-analysis=kernel-resource-usage]"
    return "\n".join(["gemm.hip:1:1: remark: Function Name: %s%s" % (name, tag), "gemm.hip:1:1: remark:     SGPRs: 100" + tag,
                      "gemm.hip:1:1: remark:     VGPRs: %d%s" % (vgprs, tag), "gemm.hip:1:1: remark:     AGPRs: %d%s" % (agprs, tag),
                      "gemm.hip:1:1: remark:     ScratchSize [bytes/lane]: %d%s" % (scratch, tag)]) + "\n"


LARGE_TILE = "_ZN5tdist11gemm_kernelINS_9ElemBF16NELi256ELi256ELi128ELi2ELi2ELi5ELb0ELb0EEEvNS_10GemmParamsE"
SMALL_TILE = "_ZN5tdist11gemm_kernelINS_8ElemBF16ELi128ELi128ELi64ELi2ELi2ELi4ELb0ELb0EEEvNS_10GemmParamsE"
PRODUCER = "_ZN5tdist20producer_push_kernelENS_10PushParamsE"


def test_register_budget_guard():
    build = load_build()
    build._check_gemm_resources(report(LARGE_TILE, 171, 256, 0))
    build._check_gemm_resources(report(LARGE_TILE, 225, 256, 0))          # 232 + 256 = 488: the producer's 24 still fit
    build._check_gemm_resources(report(SMALL_TILE, 121, 64, 0))
    build._check_gemm_resources(report("_ZN5tdist20decode_split_kernelE", 300, 256, 64))   # other kernels are not its business
    with pytest.raises(RuntimeError, match="register budget"):
        build._check_gemm_resources(report(LARGE_TILE, 233, 256, 0))       # no room for another wave on the SIMD
    with pytest.raises(RuntimeError, match="register budget"):
        build._check_gemm_resources(report(LARGE_TILE, 140, 256, 40))      # spills
    with pytest.raises(RuntimeError, match="register budget"):
        build._check_gemm_resources(report(SMALL_TILE, 120, 64, 8))
    with pytest.raises(RuntimeError, match="register budget"):
        build._check_gemm_resources(report(LARGE_TILE, 140, 256, 0) + report(LARGE_TILE.replace("BF16N", "F16N"), 256, 256, 0))


def test_producer_budget_guard():
    build = load_build()
    build._check_producer_resources(report(PRODUCER, 22, 0, 0))
    build._check_producer_resources(report("_ZN5tdist16flag_fill_kernelEPiii", 99, 0, 0))
    with pytest.raises(RuntimeError, match="producer_push_kernel"):
        build._check_producer_resources(report(PRODUCER, 26, 0, 0))


def asm_kernel(name, body):
    return "%s:\n%s\n\ts_endpgm\n" % (name, "\n".join("\t" + l for l in body))


def test_fixed_accumulator_guard():
    build = load_build()
    ok = ["v_add_u32_e32 v1, v2, v3", ";;#ASMSTART", "v_mfma_f32_16x16x32_bf16 a[0:3], v[2:5], v[6:9], a[0:3]", ";;#ASMEND",
          "global_load_dwordx4 v[10:13], v1, s[2:3] ; a comment that names a5", "s_load_dwordx2 s[4:5], s[0:1], 0x0"]
    build._check_fixed_accumulators(asm_kernel(LARGE_TILE, ok))
    # the compiler's own use of accumulation registers is fine where it allocates the accumulators itself
    build._check_fixed_accumulators(asm_kernel(SMALL_TILE, ["v_accvgpr_write_b32 a15, 0", "v_mfma_f32_32x32x16_bf16 a[0:15], v[0:3], v[4:7], a[0:15]"]))
    for line in ("v_accvgpr_write_b32 a7, v3", "global_load_dwordx4 a[8:11], v1, s[2:3]", "v_accvgpr_read_b32 v0, a200"):
        with pytest.raises(RuntimeError, match="accumulation registers"):
            build._check_fixed_accumulators(asm_kernel(LARGE_TILE, ok + [line]))
