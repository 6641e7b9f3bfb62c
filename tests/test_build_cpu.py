"""The build script's register report: a kernel of the GEMM files that needs scratch memory fails the build."""
import importlib.util
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

REMARKS = """In file included from gemm.hip:6:
./gemm_skinny.h:90:1: remark: Function Name: kernel_a [-Rpass-analysis=kernel-resource-usage]
   90 | __global__ void kernel_a(Args g) {
      | ^
./gemm_skinny.h:90:1: remark:     TotalSGPRs: 106 [-Rpass-analysis=kernel-resource-usage]
./gemm_skinny.h:90:1: remark:     VGPRs: 196 [-Rpass-analysis=kernel-resource-usage]
./gemm_skinny.h:90:1: remark:     AGPRs: 0 [-Rpass-analysis=kernel-resource-usage]
./gemm_skinny.h:90:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
./gemm_skinny.h:90:1: remark:     Occupancy [waves/SIMD]: 2 [-Rpass-analysis=kernel-resource-usage]
./gemm_skinny.h:90:1: remark:     SGPRs Spill: 38 [-Rpass-analysis=kernel-resource-usage]
./gemm_skinny.h:90:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
./gemm_big.h:57:1: remark: Function Name: kernel_b [-Rpass-analysis=kernel-resource-usage]
./gemm_big.h:57:1: remark:     TotalSGPRs: 90 [-Rpass-analysis=kernel-resource-usage]
./gemm_big.h:57:1: remark:     VGPRs: 256 [-Rpass-analysis=kernel-resource-usage]
./gemm_big.h:57:1: remark:     AGPRs: 12 [-Rpass-analysis=kernel-resource-usage]
./gemm_big.h:57:1: remark:     ScratchSize [bytes/lane]: 596 [-Rpass-analysis=kernel-resource-usage]
./gemm_big.h:57:1: remark:     Occupancy [waves/SIMD]: 2 [-Rpass-analysis=kernel-resource-usage]
./gemm_big.h:57:1: remark:     VGPRs Spill: 318 [-Rpass-analysis=kernel-resource-usage]
./gemm_big.h:57:1: remark: Function Name: kernel_b [-Rpass-analysis=kernel-resource-usage]
./gemm_big.h:57:1: remark:     VGPRs: 1 [-Rpass-analysis=kernel-resource-usage]
"""


def _build_module():
    spec = importlib.util.spec_from_file_location("sglamd_build", os.path.join(ROOT, "sglang_amd", "csrc", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_resource_table_reads_each_kernel_once():
    rows = _build_module()._resource_table(REMARKS)
    assert rows == [("kernel_a", 196, 0, 106, 0, 2), ("kernel_b", 256, 12, 90, 596, 2)]


def test_scratch_guard_refuses_an_empty_or_unreadable_report():
    import pytest

    mod = _build_module()
    with pytest.raises(RuntimeError, match="no kernel-resource-usage remarks"):
        mod._require_complete_report("gemm.hip", mod._resource_table("warning: something else entirely\n"))
    broken = REMARKS.replace("ScratchSize [bytes/lane]: 0", "ScratchBytes: 0")
    with pytest.raises(RuntimeError, match="kernel_a"):
        mod._require_complete_report("gemm.hip", mod._resource_table(broken))
    mod._require_complete_report("gemm.hip", mod._resource_table(REMARKS))


def test_gemm_sources_are_guarded_and_requested_from_the_compiler():
    mod = _build_module()
    assert {"gemm_mode_block_fp8.hip", "gemm_mode_row_fp8.hip", "gemm_mode_row_int8.hip", "gemm_mode_block_int8.hip",
            "moe.hip"} <= mod.NO_SCRATCH
    assert mod.NO_SCRATCH <= set(mod.SOURCES)
    assert "-Rpass-analysis=kernel-resource-usage" in mod.HIPCC_FLAGS


def test_last_build_left_no_gemm_kernel_in_scratch():
    """When the library has been built in this tree, its report must show every GEMM kernel in registers."""
    import pytest

    for src in ("gemm_mode_block_fp8", "gemm_mode_row_fp8", "gemm_mode_row_int8", "gemm_mode_block_int8", "moe"):
        path = os.path.join(ROOT, "sglang_amd", "csrc", "build", src + ".resources.txt")
        if not os.path.exists(path):
            pytest.skip("no build report in this tree")
        lines = open(path).read().strip().splitlines()[1:]
        assert lines, path
        for line in lines:
            name, vgprs, agprs, sgprs, scratch, waves = line.split()
            assert int(scratch) == 0, f"{name} uses {scratch} bytes of scratch per lane"
