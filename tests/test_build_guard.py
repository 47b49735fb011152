"""The build refuses to ship tile kernels that spill: the two-buffer direct-to-LDS loops read their MFMA operands
through inline assembly with hand-counted waits, which is only correct while no fragment register is spilled or
copied between the read and its wait.  Checked here: the parser of the compiler's resource report, the guard's
rules on synthetic reports, and the report of the library that is actually built in-tree."""
import json
import os

import pytest

import importlib

B = importlib.import_module("fgrpo.build")     # the package re-exports the function `build` under the same name

ASM_KERNEL = "_ZN5fgrpo17lmhead_fwd_kernelINS_7TileCfgILi256ELi256ELi64ELi2ELi4ELi2ELi2ELb1EEEEEvNS_9FwdParamsE"
REG_KERNEL = "_ZN5fgrpo17gemm_store_kernelINS_7TileCfgILi256ELi256ELi64ELi2ELi2ELi1ELi2ELb0EEELb0ELb0EEEvNS_11StoreParamsE"


def remarks(name, vgprs=200, agprs=0, scratch=0, vspill=0, sspill=0):
    tag = "[-Rpass-analysis=kernel-resource-usage]"
    return "\n".join([
        f"x.hip:52:1: remark: Function Name: {name} {tag}",
        "   52 | template <class C>",
        "      | ^",
        f"x.hip:52:1: remark:     TotalSGPRs: 96 {tag}",
        f"x.hip:52:1: remark:     VGPRs: {vgprs} {tag}",
        f"x.hip:52:1: remark:     AGPRs: {agprs} {tag}",
        f"x.hip:52:1: remark:     ScratchSize [bytes/lane]: {scratch} {tag}",
        f"x.hip:52:1: remark:     Dynamic Stack: False {tag}",
        f"x.hip:52:1: remark:     Occupancy [waves/SIMD]: 2 {tag}",
        f"x.hip:52:1: remark:     SGPRs Spill: {sspill} {tag}",
        f"x.hip:52:1: remark:     VGPRs Spill: {vspill} {tag}",
        f"x.hip:52:1: remark:     LDS Size [bytes/block]: 0 {tag}",
    ])


def full_report(**over):
    """A report that names every guarded family once (so that only the kernel under test can trip the guard)."""
    text = remarks(ASM_KERNEL, **over)
    for other in ("lmhead_ds_kernelI_plain", "gemm_store_kernelI_plain", "varlen_attn_fwd_kernelILi128ELi1EE",
                  "varlen_attn_dq_kernelILi128ELi1EE", "varlen_attn_dkv_kernelILi128EE", "varlen_attn_fwd2_kernelILi128ELi1EE",
                  "varlen_attn_dq2_kernelILi128ELi1EE", "varlen_attn_dkv2_kernelILi128EE"):
        text += "\n" + remarks("_ZN5fgrpo" + other)
    return B.parse_resource_usage(text)


def test_parser_reads_every_field():
    u = B.parse_resource_usage(remarks(ASM_KERNEL, vgprs=226, agprs=0, scratch=24, vspill=5, sspill=102))
    assert u == {ASM_KERNEL: dict(sgprs=96, vgprs=226, agprs=0, scratch=24, occupancy=2, sgpr_spill=102,
                                  vgpr_spill=5, lds=0)}


def test_guard_accepts_a_clean_report_and_sgpr_spills():
    assert B.check_resource_usage(full_report()) == []
    assert B.check_resource_usage(full_report(sspill=120)) == []      # scalar spills live in vector lanes: harmless


@pytest.mark.parametrize("over", [dict(vspill=5, scratch=24), dict(scratch=8), dict(vgprs=260), dict(agprs=16)])
def test_guard_rejects_spills_and_lost_occupancy(over):
    problems = B.check_resource_usage(full_report(**over))
    assert problems and ASM_KERNEL in problems[0]


def test_guard_ignores_spills_of_loops_the_compiler_schedules():
    """Register-staged loops (LDS reads the compiler sees and waits for) may spill: slow, but correct."""
    u = full_report()
    u.update(B.parse_resource_usage(remarks(REG_KERNEL, vgprs=256, agprs=256, scratch=440, vspill=113)))
    assert B.check_resource_usage(u) == []


def test_guard_notices_a_family_that_vanished():
    u = full_report()
    u = {k: v for k, v in u.items() if "varlen_attn_dkv" not in k}
    assert any("varlen_attn_dkv_kernel" in p for p in B.check_resource_usage(u))


def test_built_library_passed_the_guard():
    if not (os.path.exists(B.LIB_PATH) and os.path.exists(B.USAGE_PATH)):
        B.build(verbose=False)
    rep = json.load(open(B.USAGE_PATH))
    assert rep["problems"] == []
    assert B.check_resource_usage(rep["kernels"]) == []
    names = list(rep["kernels"])
    for family in B.MUST_EXIST:
        assert any(family in n for n in names)
    assert os.path.getmtime(B.USAGE_PATH) >= os.path.getmtime(B.LIB_PATH) - 5


def test_guard_covers_the_hand_scheduled_attention_kernels():
    """Their LDS reads are inline assembly too: a spill fails the build."""
    base = full_report()
    name = "_ZN5fgrpovarlen_attn_dkv2_kernelILi128EE"
    assert name in base
    spilled = dict(base)
    spilled[name] = dict(base[name], vgpr_spill=3, scratch=12)
    problems = B.check_resource_usage(spilled)
    assert problems and any("varlen_attn_dkv2_kernel" in x for x in problems)
    gone = {k: v for k, v in base.items() if "varlen_attn_dq2_kernel" not in k}
    assert any("varlen_attn_dq2_kernel" in x for x in B.check_resource_usage(gone))
