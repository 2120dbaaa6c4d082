"""The build refuses kernels that keep loads in flight and spill registers (qwen-llm_amd/build.py): the check on
hipcc's resource-usage remarks, fed with remark text of the shape the compiler prints.  Host logic, no GPU."""
import importlib.util
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _build_module():
    spec = importlib.util.spec_from_file_location("_dflash_build_for_test", os.path.join(ROOT, "qwen-llm_amd", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def remarks(name, vgpr_spill, scratch=0):
    tag = "[-Rpass-analysis=kernel-resource-usage]"
    lines = [f"x.hip:10:1: remark: Function Name: {name} {tag}", "   10 | __global__ void k() {", "      | ^"]
    for key, val in (("TotalSGPRs", 100), ("VGPRs", 120), ("ScratchSize [bytes/lane]", scratch), ("VGPRs Spill", vgpr_spill)):
        lines += [f"x.hip:10:1: remark:     {key}: {val} {tag}", "   10 | __global__ void k() {", "      | ^"]
    return "\n".join(lines) + "\n"


def test_a_guarded_kernel_that_spills_is_refused():
    b = _build_module()
    bad = b.check_no_scratch(remarks("_ZN12_GLOBAL__N_123gemm_q4k_experts_kernelIffLb0EEEvPKh", 13, 52), expect=())
    assert len(bad) == 2 and all("gemm_q4k_experts_kernel" in m for m in bad) and "52" in bad[0] and "13" in bad[1]
    # a scratch frame without a spill count is refused as well
    bad = b.check_no_scratch(remarks("_ZN12_GLOBAL__N_123gemm_q4k_experts_kernelIffLb0EEEvPKh", 0, 16), expect=())
    assert len(bad) == 1 and "scratch" in bad[0]


def test_guarded_kernels_without_spills_and_other_kernels_pass():
    b = _build_module()
    text = remarks("_ZN12_GLOBAL__N_121gemm_q4k_tiled_kernelIfEEvPKh", 0) + remarks("_Z15rms_norm_kernelPKf", 7, 28)
    assert b.check_no_scratch(text, expect=()) == []


def test_a_guarded_kernel_missing_from_the_remarks_fails_the_guard():
    """A changed remark format or a dropped flag must not make the guard pass vacuously."""
    b = _build_module()
    text = remarks("_ZN12_GLOBAL__N_121gemm_q4k_tiled_kernelIfEEvPKh", 0)
    bad = b.check_no_scratch(text)  # every other guarded kernel is unreported
    assert len(bad) == len(b.NO_SCRATCH_KERNELS) - 1 and all("no resource-usage remark" in m for m in bad)
    assert b.check_no_scratch("nothing of the kind\n", expect=("gemm_q4k_tiled_kernel",)) != []


def test_inspected_exceptions_hold_only_at_their_recorded_counts():
    b = _build_module()
    b.INSPECTED_SPILLS = {"gemm_q6k_stream_kernelILi16EfE": 13}
    name = "_ZN12_GLOBAL__N_122gemm_q6k_stream_kernelILi16EfEEvPKhPKT0_PfS6_iiii"
    assert b.check_no_scratch(remarks(name, 13), expect=()) == []
    assert len(b.check_no_scratch(remarks(name, 14), expect=())) == 1
    assert len(b.check_no_scratch(remarks(name, 0), expect=())) == 1  # the code changed: read the generated code again


def test_remarks_are_stripped_from_what_the_build_prints():
    b = _build_module()
    text = remarks("_Z1kv", 0) + "y.hip:3:5: warning: unused variable 'q' [-Wunused-variable]\n    3 |     int q;\n"
    out = b.strip_remarks(text)
    assert "remark" not in out and "unused variable 'q'" in out
