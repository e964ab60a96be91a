"""The build's own checks: kernels that count their outstanding vector-memory operations may
not use scratch memory, and the build refuses a compile in which one does."""
import pytest

from sparse_amd import build

REMARKS = """\
a.hip:91:1: remark: Function Name: _ZN6sparse23prefill_tile_map_kernelENS_9PfMapArgsE [-Rpass-analysis=kernel-resource-usage]
   91 | __global__ void prefill_tile_map_kernel(const PfMapArgs a) {
      | ^
a.hip:91:1: remark:     VGPRs: 20 [-Rpass-analysis=kernel-resource-usage]
a.hip:91:1: remark:     ScratchSize [bytes/lane]: 16 [-Rpass-analysis=kernel-resource-usage]
a.hip:137:1: remark: Function Name: _ZN6sparse18prefill_ffn_kernelILb1ELb0EEEvNS_11PrefillArgsE [-Rpass-analysis=kernel-resource-usage]
a.hip:137:1: remark:     VGPRs: 237 [-Rpass-analysis=kernel-resource-usage]
a.hip:137:1: remark:     ScratchSize [bytes/lane]: %d [-Rpass-analysis=kernel-resource-usage]
a.hip:137:1: remark:     Occupancy [waves/SIMD]: 2 [-Rpass-analysis=kernel-resource-usage]
"""


def test_scratch_is_read_per_kernel():
    table = build.scratch_by_kernel(REMARKS % 0)
    assert table == {"_ZN6sparse23prefill_tile_map_kernelENS_9PfMapArgsE": 16,
                     "_ZN6sparse18prefill_ffn_kernelILb1ELb0EEEvNS_11PrefillArgsE": 0}


def test_build_refuses_scratch_in_a_kernel_with_counted_waits():
    build.check_no_scratch("swiglu_prefill.hip", REMARKS % 0)       # the map kernel's scratch is no concern
    with pytest.raises(RuntimeError, match="uses scratch memory"):
        build.check_no_scratch("swiglu_prefill.hip", REMARKS % 264)
    with pytest.raises(RuntimeError, match="no resource remarks"):
        build.check_no_scratch("swiglu_prefill.hip", "")
    build.check_no_scratch("router.hip", "")                          # not a guarded source


def test_every_guarded_source_is_built():
    assert set(build.NO_SCRATCH) <= set(build.SOURCES)
