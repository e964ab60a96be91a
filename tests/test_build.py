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


def _hot_loops(asm: str, kernel_prefix: str):
    """Basic blocks with at least 16 MFMAs of every function whose name starts with ``kernel_prefix``,
    as lists of instruction mnemonics + operands."""
    import re
    loops, name, block = [], None, None
    for line in asm.splitlines():
        text = line.strip()
        m = re.match(r"^(_Z\w+):", line)
        if m:
            name, block = m.group(1), None
            continue
        if line.startswith(".Lfunc_end"):
            name, block = None, None
            continue
        if name is None or not name.startswith(kernel_prefix):
            continue
        if re.match(r"^\.LBB\d+_\d+:", line):
            block = []
            loops.append((name, block))
            continue
        if block is not None and text and not text.startswith((";", ".")):
            block.append(text)
    return [(n, b) for n, b in loops if sum(i.startswith("v_mfma") for i in b) >= 16]


@pytest.mark.parametrize("source,prefix", [("swiglu_prefill.hip", "_ZN6sparse18prefill_ffn_kernel"),
                                           ("swiglu_prefill_merged.hip", "_ZN6sparse21prefill_merged_kernel")])
def test_prefill_k_loop_issues_its_vector_memory_operations_as_the_counted_wait_assumes(tmp_path, source, prefix):
    """The prefill kernel waits for "all but the 20 newest" vector memory operations before the barrier that
    closes a k slab.  That is exact only if every slab issues, in this order, the 4 LDS copies of the slab
    after next and then 8 fragment loads, and nothing else that the counter counts (no scratch traffic, no
    other global access).  Checked on the compiler's output for the counted-wait kernels
    (the one-tile-per-workgroup form and the merged routed + shared form)."""
    import re
    import subprocess
    hipcc = build._hipcc()
    out = tmp_path / "prefill.s"
    cmd = [hipcc, *[f for f in build.HIP_FLAGS if f not in ("-fPIC",)], f"-I{build.INCLUDE}", f"-I{build.CSRC}", "-S",
           "--cuda-device-only", str(build.CSRC / source), "-o", str(out)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    loops = _hot_loops(out.read_text(), prefix)
    # counted-wait variants only: the last template argument (kDrainWaits) is false
    loops = [(n, b) for n, b in loops if re.search(r"ELb[01]ELb0EEEv", n)]
    assert len(loops) >= 8          # bf16 and fp16, gate/up and down, several tile heights each
    slabs = 0
    for name, block in loops:
        segment = []
        for ins in block:
            if ins.startswith("s_barrier"):
                vm = [i for i in segment if i.startswith(("global_", "scratch_", "buffer_", "flat_"))]
                kinds = ["copy" if i.startswith("global_load_lds") else "frag" if i.startswith("global_load_dwordx4")
                         else "other" for i in vm]
                if kinds:           # (a block may begin in the middle of a slab: only whole slabs are judged)
                    if len(kinds) == 12:
                        assert kinds == ["copy"] * 4 + ["frag"] * 8, (name, kinds)
                        waits = [i for i in segment if i.startswith("s_waitcnt") and "vmcnt" in i]
                        assert waits and "vmcnt(20)" in waits[-1], (name, waits[-3:])
                        slabs += 1
                    else:
                        assert "other" not in kinds, (name, kinds)
                segment = []
            else:
                segment.append(ins)
    assert slabs >= 8
