"""The build script's own guard: kernels whose K loop is hand-placed register text may not use scratch memory."""
import importlib.util
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _build_module():
    spec = importlib.util.spec_from_file_location("_dfa_build_checks", os.path.join(ROOT, "deeplink.framework_amd", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_scratch_guard_reads_the_resource_usage_remarks():
    b = _build_module()
    remark = "gemm.hip:806:1: remark: {} [-Rpass-analysis=kernel-resource-usage]"
    clean = "\n".join(remark.format(t) for t in ["Function Name: _ZN3amd19gemmMfma4WaveKernelIDF16bLi0EEEvNS_8MfmaArgsE", "    VGPRs: 250",
                                                  "    ScratchSize [bytes/lane]: 0", "    SGPRs Spill: 0", "    VGPRs Spill: 0"])
    assert b.scratch_users(clean, ("gemmMfma4WaveKernel",)) == []
    spilled = clean.replace("ScratchSize [bytes/lane]: 0", "ScratchSize [bytes/lane]: 52").replace("VGPRs Spill: 0", "VGPRs Spill: 13")
    bad = b.scratch_users(spilled, ("gemmMfma4WaveKernel",))
    assert len(bad) == 2 and "ScratchSize" in bad[0] and "VGPRs Spill: 13" in bad[1]
    # scalar registers parked in lanes of a vector register are not scratch
    lanes = clean.replace("SGPRs Spill: 0", "SGPRs Spill: 2")
    assert b.scratch_users(lanes, ("gemmMfma4WaveKernel",)) == []
    # another kernel's scratch is not this guard's business
    other = spilled.replace("gemmMfma4WaveKernel", "gemmFmaKernel")
    assert b.scratch_users(other, ("gemmMfma4WaveKernel",)) == []
    assert "gemm.hip" in b.NO_SCRATCH_KERNELS
