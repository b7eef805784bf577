"""Static check of the compiled stage-1 MFMA kernels (device assembly, no GPU needed).

The kernel loads its Q rows with inline-assembly global loads that the compiler's wait
insertion does not see, and waits for them by hand. Between such a load and the wait the
destination registers hold stale values and receive the data at an unknown moment: if the
compiler copied, spilled or reused them there, the late data would land in whatever lives
in them by then (an address, say). This test reads the assembly hipcc emits for every
instantiation and asserts that nothing touches those registers inside the window."""
import os
import re
import subprocess
import tempfile

import pytest

from flash_tree_attn_amd import build as fta_build

SRC = os.path.join(fta_build.CSRC, "stage1_mfma.hip")
REG = re.compile(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]")


def regs_of(text):
    out = set()
    for m in REG.finditer(text):
        if m.group(1) is not None:
            out.add(int(m.group(1)))
        else:
            out.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return out


@pytest.fixture(scope="module")
def kernels():
    if not os.path.exists(fta_build.HIPCC):
        pytest.skip("hipcc not available")
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "stage1_mfma.s")
        cmd = [fta_build.HIPCC, *fta_build.FLAGS, "--cuda-device-only", "-S", "-x", "hip", SRC, "-o", out]
        subprocess.run(cmd, check=True, capture_output=True)
        text = open(out).read()
    bodies = {}
    for m in re.finditer(r"^(_ZN3fta\S*stage1_mfma_kernel[^:\s]*):[^\n]*\n(.*?)^\.Lfunc_end", text, flags=re.S | re.M):
        lines = [l.split(";")[0].strip() if not l.strip().startswith(";;#ASM") else l.strip() for l in m.group(2).split("\n")]
        bodies[m.group(1)] = [l for l in lines if l and not l.startswith(".") and not l.endswith(":")]
    assert len(bodies) >= 12, "expected every dtype x head_dim x variant x paged instantiation"
    return bodies


def test_untracked_q_loads_are_not_touched_before_their_wait(kernels):
    for name, ins in kernels.items():
        # inline-assembly register loads without a cache-scope modifier = the Q rows
        in_asm, q_loads = False, []
        for i, l in enumerate(ins):
            if l.startswith(";;#ASMSTART"):
                in_asm = True
            elif l.startswith(";;#ASMEND"):
                in_asm = False
            elif in_asm and l.startswith("global_load_dwordx4") and "sc1" not in l:
                q_loads.append(i)
        # the Q loads are the first group of such loads; the merge code (sc1) is excluded above, and
        # nothing else in the kernel uses an untracked register load
        first = q_loads[0]
        group = [i for i in q_loads if i - first < 200]
        assert len(group) in (4, 8, 16) and group == q_loads, (name, q_loads)
        dests = set()
        for i in group:
            dests |= regs_of(ins[i].split(",")[0])
        assert len(dests) == 4 * len(group), name
        # no instruction between the loads other than address arithmetic that stays off the destinations
        for i in range(group[0], group[-1] + 1):
            if i in group or ins[i].startswith(";;#ASM"):
                continue
            assert not (regs_of(ins[i]) & dests), (name, ins[i])
        # after the last load: a manual wait must come before the first instruction that names a destination
        seen_wait = False
        for i in range(group[-1] + 1, len(ins)):
            l = ins[i]
            if l.startswith("s_waitcnt") and "vmcnt" in l:
                seen_wait = True
            if not l.startswith(";;#ASM") and regs_of(l) & dests:
                assert seen_wait, (name, "destination of an in-flight Q load is used before any vmcnt wait", l)
                break
        else:
            pytest.fail(f"{name}: the Q registers are never used")


def test_no_scratch_or_stack_use_in_the_pipelined_loop(kernels):
    """The 256-row kernels must keep their fused loop free of spill traffic: a scratch access there
    is a vector-memory instruction the manual vmcnt accounting does not expect."""
    for name, ins in kernels.items():
        if "Li8ELi3ELb1" not in name:   # <.., 8 waves, K ring 3, pipelined, ..>
            continue
        mfma_blocks, cur = [], []
        for l in ins:
            if l.startswith("s_cbranch") or l.startswith("s_branch"):
                mfma_blocks.append(cur)
                cur = []
            else:
                cur.append(l)
        hot = [b for b in mfma_blocks if sum(1 for l in b if l.startswith("v_mfma")) >= 16 and any("v_exp_f32" in l for l in b)]
        assert hot, name
        for b in hot:
            assert not any(l.startswith("scratch_") or l.startswith("buffer_") for l in b), name
