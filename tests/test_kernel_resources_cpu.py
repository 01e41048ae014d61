"""What the compiler reported for every kernel of the built library (written next to the
library by tracea_amd/build.py from -Rpass-analysis=kernel-resource-usage).

No kernel of this library is meant to touch scratch memory.  Twice a kernel did after an
innocent-looking change (a run-time index into the accumulators; the argument block read
through nested lambdas): the results stayed right and the kernel ran at half speed.  No
exceptions: the register-staged 256x256 tiles that used to spill are no longer built."""
import json
import os
import re

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
PATH = os.path.join(HERE, "..", "tracea_amd", "lib", "kernel_resources.json")

CONTRACTION = re.compile(r"contraction_kernelILi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)E")


def _resources():
    if not os.path.exists(PATH):
        pytest.skip("library not built by tracea_amd/build.py in this tree")
    return json.load(open(PATH))


def test_every_kernel_family_is_listed():
    names = " ".join(_resources())
    for family in ("contraction_kernel", "conv_patch_kernel", "gemm_f32_dma_kernel", "gemm_f32_kernel", "fa2_fwd",
                   "splitk_reduce_kernel", "phase_filter_kernel", "softmax", "global_avg_pool_kernel"):
        assert family in names, family


def test_no_kernel_uses_scratch_memory():
    bad = []
    for name, r in _resources().items():
        scratch = r.get("scratch_bytes", 0)
        if scratch > 0:
            bad.append((scratch, name))
        assert r.get("vgpr_spills", 0) == 0, name
    assert not bad, "kernels with a private segment: %s" % sorted(bad, reverse=True)[:8]


def test_two_workgroups_of_the_headline_kernels_fit_a_cu():
    # 512 registers per SIMD lane: the 8-wave 256x256 GEMM tile and the fp32 128x128 tile rely on
    # two resident workgroups (two and one wave per SIMD each), the 8-wave patch convolution on two
    res = _resources()
    for name, r in res.items():
        regs = r.get("vgprs", 0) + r.get("agprs", 0)
        m = CONTRACTION.search(name)
        if m and m.group(2, 3, 5, 6, 8) == ("256", "256", "2", "4", "2"):
            assert regs <= 256, (name, regs)
        if "gemm_f32_dma_kernelILi2ELi2ELi1E" in name:
            assert regs <= 256, (name, regs)
        if "conv_patch_kernel" in name and "ELi256ELi64ELi8ELi1E" in name:
            assert regs <= 128, (name, regs)
