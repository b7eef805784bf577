"""Static checks of the stage-1 MFMA kernels: the device assembly hipcc emits for them and the
hand-scheduled loop's generator (no GPU needed).

The kernels wait for their HBM -> LDS loads by hand (`s_waitcnt vmcnt(n)` with n counted from
the loads the code itself issued). That is only sound for loads whose destination is LDS: a
hand-issued load into REGISTERS is invisible to the compiler's wait insertion, and until the
hand-written wait the compiler may copy, spill or reuse the destination. The kernels therefore
contain no such load, and the first test keeps it that way.

The 64-row-wave loop is one inline-assembly statement over fixed physical registers. The
compiler keeps its own values in every register the statement does not declare, so the
statement's operand and clobber lists must name every register its text touches: the
generator checks that when it renders, and the tests here check the checker."""
import importlib.util
import os
import re
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

import pytest

from flash_tree_attn_amd import build as fta_build

UNITS = ["stage1_mfma.hip", "stage1_mfma_wide.hip", "stage1_mfma_splitkeys.hip"]


def _generator():
    spec = importlib.util.spec_from_file_location("gen_wide_loop", os.path.join(fta_build.CSRC, "gen_wide_loop.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="module")
def kernels():
    """name -> (instruction lines, metadata dict) of every stage1_mfma_kernel instantiation."""
    if not os.path.exists(fta_build.HIPCC):
        pytest.skip("hipcc not available")
    with tempfile.TemporaryDirectory() as tmp:
        def compile_unit(src):
            out = os.path.join(tmp, src + ".s")
            cmd = [fta_build.HIPCC, *fta_build.FLAGS, "--cuda-device-only", "-S", "-x", "hip", os.path.join(fta_build.CSRC, src), "-o", out]
            subprocess.run(cmd, check=True, capture_output=True)
            return open(out).read()
        with ThreadPoolExecutor(max_workers=3) as pool:
            texts = list(pool.map(compile_unit, UNITS))
    found = {}
    for text in texts:
        meta = {}
        for entry in text.split("\n  - .agpr_count:")[1:]:
            field = lambda key: re.search(rf"^\s+\.{key}:\s+(\S+)", entry, flags=re.M).group(1)
            meta[field("name")] = {"agpr": int(entry.split()[0]), "scratch": int(field("private_segment_fixed_size")), "vgpr": int(field("vgpr_count"))}
        for m in re.finditer(r"^(_ZN3fta\S*stage1_mfma_kernel[^:\s]*):[^\n]*\n(.*?)^\.Lfunc_end", text, flags=re.S | re.M):
            lines = [l.strip() if l.strip().startswith(";;#ASM") else l.split(";")[0].strip() for l in m.group(2).split("\n")]
            found[m.group(1)] = ([l for l in lines if l and not l.startswith(".") and not l.endswith(":")], meta[m.group(1)])
    # 2 dtypes x paged/contiguous x (pipelined D 128, 64 + plain D 128, 64, 256 + key halves D 128, 64) + 2 dtypes x wide D 128, 64
    assert len(found) == 2 * 2 * 7 + 2 * 2, sorted(found)
    return found


def asm_regions(ins):
    """Yields the instruction lists of the inline-assembly statements of one kernel."""
    cur = None
    for l in ins:
        if l.startswith(";;#ASMSTART"):
            cur = []
        elif l.startswith(";;#ASMEND"):
            yield cur
            cur = None
        elif cur is not None:
            cur.append(l)


def test_no_hand_issued_load_into_registers(kernels):
    for name, (ins, _) in kernels.items():
        for region in asm_regions(ins):
            for l in region:
                op = l.split()[0]
                if op.startswith(("global_load", "buffer_load", "flat_load", "scratch_load")) and "_lds_" not in op:
                    # the merge code's reads of other workgroups' partial results (device-scope, `sc1`) sit in one
                    # statement with their own vmcnt(0), outputs bound by constraints: the compiler sees them complete
                    assert "sc1" in l, (name, l)


REG = re.compile(r"\b([va])(\d+)\b|\b([va])\[(\d+):(\d+)\]")


def vector_regs(text):
    out = set()
    for m in REG.finditer(text):
        if m.group(1):
            out.add((m.group(1), int(m.group(2))))
        else:
            out.update((m.group(3), i) for i in range(int(m.group(4)), int(m.group(5)) + 1))
    return out


def touches_of_in_flight_lds_reads(ins):
    """Operand fragments are read with hand-written `ds_read` instructions and awaited by separate hand-written
    `s_waitcnt lgkmcnt(n)`: between the two the compiler believes the destination holds its value. Walks one
    kernel in layout order, keeps the destinations of the hand-issued reads that no wait has covered yet (LDS
    reads return in order, a wait for n leaves the newest n in flight) and reports every instruction that
    names such a register. Returns (problems, reads seen)."""
    in_asm, pending, problems, reads = False, [], [], 0
    for idx, l in enumerate(ins):
        if l.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if l.startswith(";;#ASMEND"):
            in_asm = False
            continue
        op = l.split()[0]
        if op == "s_waitcnt":
            m = re.search(r"lgkmcnt\((\d+)\)", l)
            if m:
                pending = pending[len(pending) - int(m.group(1)):] if int(m.group(1)) else []
            continue
        live = set().union(*pending) if pending else set()
        if in_asm and op.startswith("ds_read"):
            reads += 1
            dest = vector_regs(l.split(",")[0])
            if dest & live:
                problems.append((idx, l))
            pending.append(dest)
        elif vector_regs(l) & live:
            problems.append((idx, l))
    return problems, reads


def test_registers_of_in_flight_lds_reads_are_left_alone(kernels):
    for name, (ins, _) in kernels.items():
        problems, reads = touches_of_in_flight_lds_reads(ins)
        assert reads >= (20 if "Li3ELb" in name else 32), (name, reads)   # every variant reads its K and V fragments this way (key halves: half as many)
        assert not problems, (name, problems[:3])
    # the check sees what it is meant to see: a copy of a destination right behind its read is reported
    name, (ins, _) = next(iter(kernels.items()))
    at = next(i for i, l in enumerate(ins) if l.startswith("ds_read") and ins[i - 1].startswith(";;#ASMSTART"))
    first = sorted(vector_regs(ins[at].split(",")[0]))[0]
    spoiled = ins[:at + 2] + [f"v_mov_b32 v255, {first[0]}{first[1]}"] + ins[at + 2:]
    assert touches_of_in_flight_lds_reads(spoiled)[0]


def test_the_whole_tile_pipelined_loop_has_no_spill_traffic(kernels):
    """Scratch accesses are vector-memory instructions too: inside the fused loop of the 8-wave
    kernels they would sit between the tile requests and the hand-counted waits and make every
    wait longer than intended (never shorter: the counter retires in order)."""
    checked = 0
    for name, (ins, _) in kernels.items():
        if "Li1ELi8ELi3ELi1ELb" not in name:   # <.., 32-row waves, 8 waves, K requested 3 ahead, pipelined, ..>
            continue
        blocks, cur = [], []
        for l in ins:
            if l.startswith("s_cbranch") or l.startswith("s_branch"):
                blocks.append(cur)
                cur = []
            else:
                cur.append(l)
        hot = [b for b in blocks if sum(1 for l in b if l.startswith("v_mfma")) >= 16 and any("v_exp_f32" in l for l in b)]
        assert hot, name
        for b in hot:
            assert not any(l.startswith("scratch_") or l.startswith("buffer_") for l in b), name
        checked += 1
    assert checked == 8


def test_wide_kernels_hold_the_generated_loop_and_fit_the_register_file(kernels):
    gen = _generator()
    wide = {n: v for n, v in kernels.items() if "Li2ELi4ELi4ELi2ELb0" in n}   # <.., 64-row waves, 4 waves, K ring 4, wide, contiguous>
    assert len(wide) == 4
    for name, (ins, meta) in wide.items():
        D = 128 if "Li128E" in name else 64
        dtype = "bf16" if "IDF16b" in name else "f16"
        want = [l.split(";")[0].strip() for l in gen.gen(D, dtype)]
        want = [l for l in want if l and not l.endswith(":")]
        regions = [r for r in asm_regions(ins) if len(r) > 1000]
        assert len(regions) == 1, (name, [len(r) for r in asm_regions(ins)])
        # `%=` in a label is the statement's number in the compiled code
        got = [re.sub(r"(\.L\w+_)\d+$", r"\1%=", l) for l in regions[0] if not l.endswith(":")]
        assert got == want, name   # the compiled loop IS the generator's text, register for register
        # one wave per SIMD: accumulation and vector registers share a file of 512
        assert meta["vgpr"] <= 512 and meta["agpr"] >= gen.A_Q + 8 * (D // 16), (name, meta)


def test_committed_loop_text_is_what_the_generator_renders():
    gen = _generator()
    with open(os.path.join(fta_build.CSRC, "wide_loop_asm.inc")) as f:
        assert f.read() == gen.render()


def test_generator_rejects_undeclared_registers():
    gen = _generator()
    body, ops = gen.gen(128, "bf16"), gen.operands(128)
    gen.verify(body, ops, "as rendered")
    # a temporary the statement writes but does not list as clobbered
    tmp = f'"s{gen.S_TMP + 7}"'
    assert tmp in ops
    with pytest.raises(AssertionError, match="writes undeclared"):
        gen.verify(body, ops.replace(tmp + ", ", ""), "clobber dropped")
    # a vector temporary
    vt = f'"v{gen.V_T}"'
    assert vt in ops
    with pytest.raises(AssertionError, match="undeclared"):
        gen.verify(body, ops.replace(vt + ", ", ""), "clobber dropped")
    # an input the statement reads but the operand list does not bind
    inp = f'"{{v{gen.V_KOFF}}}"(w_koff), '
    assert inp in ops
    with pytest.raises(AssertionError, match="reads undeclared"):
        gen.verify(body, ops.replace(inp, ""), "input dropped")
    # a write to an input-only operand
    with pytest.raises(AssertionError, match="writes undeclared"):
        gen.verify(body + [f"v_mov_b32 v{gen.V_KOFF}, 0"], ops, "input written")
    # register tuples of vector registers start on an even register
    with pytest.raises(AssertionError, match="misaligned"):
        gen.verify(body + [f"v_mov_b64 v[{gen.V_T + 0 | 1}:{(gen.V_T + 0 | 1) + 1}], 0"], ops, "odd tuple")
    # the named registers are held to the same rule: M0 (the LDS destination of the tile requests; the compiler's
    # own requests around the statement use it as well), VCC (vector compares), SCC (scalar compares and arithmetic)
    for named, what in (("m0", "s_mov_b32 m0"), ("vcc", "v_cmp"), ("scc", "s_")):
        assert f'"{named}"' in ops and any(l.startswith(what) for l in body)
        with pytest.raises(AssertionError, match=rf"writes undeclared \['{named}'\]"):
            gen.verify(body, ops.replace(f'"{named}", ', ""), "named clobber dropped")
    with pytest.raises(AssertionError, match=r"writes undeclared \['exec'\]"):
        gen.verify(body + ["s_and_saveexec_b64 s[86:87], vcc"], ops, "exec written")
    # the masked-half statements go through the same check
    for H in (0, 1):
        gen.verify(gen.gen_masked(64, "f16", H), gen.operands_masked(64), "masked")
        with pytest.raises(AssertionError, match="undeclared"):
            gen.verify(gen.gen_masked(64, "f16", H), gen.operands_masked(64).replace(f'"v{gen.V_R}", ', ""), "masked, clobber dropped")


def test_generator_rejects_issue_hazards():
    """The rules the hardware does not enforce (wait states behind v_dot2c, transcendentals, M0 writes and MFMA
    results; SCC between a compare and its consumer; the fence at the end of a statement): the rendered text
    passes, and each rule fires on a text that breaks it."""
    gen = _generator()
    body = gen.gen(128, "bf16")
    for D in (64, 128):
        for dtype in ("bf16", "f16"):
            gen.hazards(gen.gen(D, dtype), "loop")
            for H in (0, 1):
                gen.hazards(gen.gen_masked(D, dtype, H), "masked")

    def first(pred):
        return next(i for i, l in enumerate(body) if pred(l))

    broken = list(body)
    broken.pop(first(lambda l: l.startswith("s_nop 3")))                      # the gap behind a group of v_dot2c
    with pytest.raises(AssertionError, match="v_dot2c.*needs 3"):
        gen.hazards(broken, "dot")
    at = first(lambda l: l.startswith("v_exp_f32"))
    dest = body[at].split()[1].rstrip(",")
    with pytest.raises(AssertionError, match="v_exp_f32.*needs 1"):
        gen.hazards(body[:at + 1] + [f"v_add_f32 v{gen.V_T}, {dest}, {dest}"] + body[at + 1:], "trans")
    at = first(lambda l: l.startswith("s_cselect"))
    with pytest.raises(AssertionError, match="overwrites SCC"):
        gen.hazards(body[:at] + [f"s_add_u32 s{gen.S_TMP}, s{gen.S_TMP}, 1"] + body[at:], "scc")
    at = first(lambda l: l.startswith("v_mfma") and l.split()[1].startswith("v["))
    with pytest.raises(AssertionError, match="needs 11"):
        gen.hazards(body[:at + 1] + [f"v_add_f32 v{gen.V_T}, v{gen.V_S}, v{gen.V_S}"] + body[at + 1:], "mfma result")
    at = first(lambda l: l.startswith("s_mov_b32 m0"))
    assert body[at + 1].startswith("s_nop")
    with pytest.raises(AssertionError, match="m0.*needs 1"):
        gen.hazards(body[:at + 1] + body[at + 2:], "m0")
    end = max(i for i, l in enumerate(body) if l.startswith("s_nop 15"))
    with pytest.raises(AssertionError, match="statement ends"):
        gen.hazards(body[:end] + ["s_nop 3"] + body[end + 1:], "fence")


def test_instruction_mix_of_the_generated_loop_per_tile():
    """What one wave issues per 64-key tile in the steady state of the 64-row-wave loop (the text between the loop
    label and the backward branch; the exact redo sits outside of it). These are the figures the design argues with:
    every K or V fragment read feeds two matrix products, 3.4 vector instructions per product, one barrier and one
    round of tile requests per tile. A change of the generator that moves them has to move this test."""
    import collections
    gen = _generator()
    for D, want in ((128, dict(mfma=64, lds=48, dma=8)), (64, dict(mfma=32, lds=24, dma=4))):
        for dtype in ("bf16", "f16"):
            body = gen.gen(D, dtype)
            first = next(i for i, l in enumerate(body) if l.startswith(".Lloop_"))
            last = next(i for i, l in enumerate(body) if l.startswith("s_cbranch_scc1 .Lloop_"))
            mix = collections.Counter()
            for line in body[first + 1:last + 1]:
                line = line.split(";")[0].strip()
                if not line or line.endswith(":"):
                    continue
                op = line.split()[0]
                kind = ("mfma" if op.startswith("v_mfma") else "lds" if op.startswith("ds_") else "dma" if op.startswith("global_load_lds") else
                        "exp" if op.startswith("v_exp") else "valu" if op.startswith("v_") else "barrier" if op == "s_barrier" else "other")
                mix[kind] += 1
            assert {k: mix[k] for k in want} == want, (D, dtype, mix)
            assert mix["lds"] * 4 == mix["mfma"] * 3                       # 2 K + 1 V^T pair of reads per four products
            assert mix["exp"] == 64 and mix["barrier"] == 1               # 64 rows x 64 keys over 64 lanes; one synchronisation point
            assert mix["valu"] + mix["exp"] <= 216, (D, dtype, mix)        # 3.4 per matrix product at head_dim 128
