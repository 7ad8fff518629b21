"""The build refuses a GEMM whose four-wave instances spill or leave no registers for a copy kernel's wave beside them
(host logic only: the check reads the compiler's resource report)."""
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


FOUR_WAVE = "_ZN5tdist11gemm_kernelINS_8ElemBF16ELi256ELi256ELi128ELi2ELi2ELi5ELb0ELb0EEEvNS_10GemmParamsE"
EIGHT_WAVE = "_ZN5tdist11gemm_kernelINS_7ElemFP8ELi256ELi256ELi128ELi2ELi4ELi5ELb1ELb0EEEvNS_10GemmParamsE"


def test_register_budget_guard():
    build = load_build()
    build._check_gemm_resources(report(FOUR_WAVE, 140, 256, 0))
    build._check_gemm_resources(report(EIGHT_WAVE, 256, 0, 96))           # the measurement variants are not held to it
    build._check_gemm_resources(report("_ZN5tdist20decode_split_kernelE", 300, 256, 64))
    with pytest.raises(RuntimeError, match="register budget"):
        build._check_gemm_resources(report(FOUR_WAVE, 250, 256, 0))        # no room for another wave on the SIMD
    with pytest.raises(RuntimeError, match="register budget"):
        build._check_gemm_resources(report(FOUR_WAVE, 140, 256, 40))       # spills
    with pytest.raises(RuntimeError, match="register budget"):
        build._check_gemm_resources(report(FOUR_WAVE, 140, 256, 0) + report(FOUR_WAVE.replace("BF16", "F16x"), 256, 256, 0))
