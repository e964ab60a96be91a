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


def _function_instructions(asm: str, kernel_prefix: str):
    """``{function name: [instruction text, ...]}`` in the order the compiler laid them out."""
    import re
    out, name = {}, None
    for line in asm.splitlines():
        m = re.match(r"^(_Z\w+):", line)
        if m:
            name = m.group(1) if m.group(1).startswith(kernel_prefix) else None
            if name:
                out[name] = []
            continue
        if line.startswith(".Lfunc_end"):
            name = None
            continue
        text = line.strip()
        if name and text and not text.startswith((";", ".")):
            out[name].append(text.split(";")[0].strip())
    return out


def test_decode_combine_hand_off_as_the_compiler_emits_it(tmp_path):
    """The decode down kernel hands rows and partial sums from every workgroup of a 32-column tile to the
    one that arrives last, without a release / acquire fence.  That is sound only if, in the machine code:
    the rows and partial sums leave as device-scope (sc1) stores, which gfx950 writes through to memory;
    the wavefront waits for all its vector memory operations (s_waitcnt vmcnt(0): stores are acknowledged
    from memory) and for the workgroup's barrier before one thread adds to the tile's counter, with no data
    store in between; every read behind the counter is a device-scope (sc1) load, which does not hit a
    stale line of the reader's L2; and no cache-wide write-back or invalidate is there to hide a mistake
    in the above.  Checked for every instantiation of the down kernel."""
    import re
    import subprocess
    hipcc = build._hipcc()
    out = tmp_path / "decode.s"
    cmd = [hipcc, *[f for f in build.HIP_FLAGS if f not in ("-fPIC",)], f"-I{build.INCLUDE}", f"-I{build.CSRC}", "-S",
           "--cuda-device-only", str(build.CSRC / "swiglu_decode.hip"), "-o", str(out)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    funcs = _function_instructions(out.read_text(), "_ZN6sparse17decode_ffn_kernel")
    down = {n: ins for n, ins in funcs.items() if re.search(r"ELb0ELi\dELi\dEEEv", n)}
    gateup = {n: ins for n, ins in funcs.items() if re.search(r"ELb1ELi\dELi\dEEEv", n)}
    assert len(down) == 6 and len(gateup) == 6          # bf16 and fp16, three tile shapes each
    is_vmem = lambda i: i.startswith(("global_", "buffer_", "flat_", "scratch_"))
    for name, ins in down.items():
        adds = [k for k, i in enumerate(ins) if i.startswith("global_atomic_add")]
        assert len(adds) == 1, (name, "one counter increment expected", len(adds))
        add = adds[0]
        assert re.search(r"\bsc0\b", ins[add]), (name, ins[add])                 # returns the count before it
        # the barrier in front of the increment, and the full wait in front of that barrier
        barrier = max(k for k in range(add) if ins[k].startswith("s_barrier"))
        wait = max(k for k in range(barrier) if ins[k].startswith("s_waitcnt") and "vmcnt(0)" in ins[k])
        assert not any(is_vmem(i) for i in ins[wait + 1:barrier]), (name, ins[wait:barrier + 1])
        assert not any(i.startswith(("global_store", "flat_store", "buffer_store")) for i in ins[barrier:add]), name
        # data stores of the handed-off kind: before the wait, 8 bytes each, device scope
        handed = [i for i in ins[:wait] if i.startswith("global_store") and re.search(r"\bsc1\b", i)]
        assert len(handed) >= 3 and all(i.startswith("global_store_dwordx2") for i in handed), (name, handed)
        # behind the increment: the counter's reset (device scope) and the final rows (plain, nobody in this
        # launch reads them); every 8-byte read is device scope
        after = ins[add + 1:]
        loads = [i for i in after if i.startswith("global_load_dwordx2")]
        assert len(loads) >= 3 and all(re.search(r"\bsc1\b", i) for i in loads), (name, [i for i in loads
                                                                                         if "sc1" not in i][:3])
        assert any(i.startswith("global_store_dword ") and re.search(r"\bsc1\b", i) for i in after), name
        assert not any(i.startswith(("buffer_wbl2", "buffer_inv", "buffer_gl")) for i in ins), name
    # the gate/up kernel hands nothing over inside a launch: no device-scope data stores, no counter add
    for name, ins in gateup.items():
        assert not any(i.startswith("global_atomic") for i in ins), name
