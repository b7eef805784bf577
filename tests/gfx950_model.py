"""A small functional model of the gfx950 instructions that the generated stage-1 loop uses
(flash_tree_attn_amd/csrc/gen_wide_loop.py), so that the generated TEXT can be executed on the CPU:
one workgroup of four 64-lane waves, their registers, one LDS array, a flat global memory, barriers.

Test infrastructure only. It models results, not time: every load delivers its data at once. What it
does keep is the BOOKKEEPING of the wait counters, so that a missing wait is an error even though the
data would have been there:
  * LDS reads retire in order; a register that a read has not delivered yet (no `s_waitcnt lgkmcnt(n)`
    has covered it) may not be named by any other instruction;
  * tile requests (global_load_lds) retire in order per wave; the LDS bytes of a request are readable by
    the requesting wave once its `s_waitcnt vmcnt(n)` has covered the request, and by the other waves
    after the next barrier behind that wait; a read of bytes that are still in flight, or a request into
    bytes that any wave reads between the same two barriers, is an error (the ring's stages are reused).
Issue hazards (wait states between dependent instructions) are the generator's `hazards()` check.

Lane layouts of the matrix instruction v_mfma_f32_32x32x16_{bf16,f16} (D = A.B + C, A 32x16, B 16x32):
lane l holds, of A, row l % 32 and the 8 values k = 8 * (l // 32) .. + 7 (four registers, two values
each, low half first); of B, column l % 32 and the same k; of C / D, column l % 32 and the 16 rows
8 * (r // 4) + 4 * (l // 32) + r % 4, r = 0 .. 15 (one register each).
ds_read_b64_tr_b16: the 16 lanes of a group each fetch 8 bytes (four 16-bit values); the 16 x 4 values
of the group, read as four rows of sixteen (row e = the values of lanes 4e .. 4e + 3 in order), are
returned transposed: lane s gets element s of each of the four rows."""
import re

import numpy as np

LANES = 64


def bf16_to_f32(u16):
    return (u16.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(x):
    """Round to nearest even, as v_cvt_pk_bf16_f32 does; NaN stays NaN."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = np.isnan(np.asarray(x, dtype=np.float32))
    return np.where(nan, np.uint16(0x7FC0), rounded)


def halves_to_f32(words, dtype):
    """uint32[...] -> float32[..., 2] (low half, high half)."""
    lo, hi = (words & 0xFFFF).astype(np.uint16), (words >> 16).astype(np.uint16)
    if dtype == "bf16":
        return np.stack([bf16_to_f32(lo), bf16_to_f32(hi)], axis=-1)
    return np.stack([lo.view(np.float16).astype(np.float32), hi.view(np.float16).astype(np.float32)], axis=-1)


class Memory:
    """Flat byte-addressed global memory at a 64-bit base address."""

    def __init__(self, base, size):
        self.base, self.data = base, np.zeros(size, dtype=np.uint8)

    def place(self, offset, array):
        raw = np.ascontiguousarray(array).view(np.uint8).reshape(-1)
        self.data[offset:offset + raw.size] = raw
        return self.base + offset

    def read16(self, addr):
        off = int(addr) - self.base
        if off < 0 or off + 16 > self.data.size:
            raise IndexError(f"global read at {addr:#x} outside the modelled memory")
        return self.data[off:off + 16]


REG_RE = re.compile(r"^(-?)([vas])(?:(\d+)|\[(\d+):(\d+)\])$")


class Wave:
    def __init__(self, lds, mem, dtype):
        self.v = np.zeros((256, LANES), dtype=np.uint32)
        self.a = np.zeros((256, LANES), dtype=np.uint32)
        self.s = np.zeros(128, dtype=np.uint64)     # 32-bit values, kept wide so that carries are explicit
        self.vcc = np.zeros(LANES, dtype=bool)
        self.scc = 0
        self.m0 = 0
        self.lds, self.mem, self.dtype = lds, mem, dtype
        self.executed = 0
        self.taken = []          # labels branched to (in order), for tests that want to see a path taken
        self.lds_pending = []    # destination registers of LDS reads no lgkmcnt wait has covered yet, oldest first
        self.vm_pending = []     # (lo, hi) LDS byte ranges of tile requests no vmcnt wait has covered yet, oldest first
        self.vm_own = []         # ranges whose wait this wave has passed, not yet published to the others by a barrier
        self.epoch_reads = []    # (lo, hi) LDS ranges read since the last barrier
        self.epoch_requests = [] # (lo, hi) LDS ranges requested into since the last barrier, with the reads that preceded them
        self.shared = None       # the workgroup's bookkeeping (set by run_workgroup)

    # ---- operands
    def _reg(self, tok):
        m = REG_RE.match(tok)
        if not m:
            return None
        neg, kind = m.group(1) == "-", m.group(2)
        lo = int(m.group(3)) if m.group(3) is not None else int(m.group(4))
        n = 1 if m.group(3) is not None else int(m.group(5)) - lo + 1
        return neg, kind, lo, n

    def src32(self, tok):
        """The 32-bit value of a source operand in every lane (uint32[64]); a leading '-' flips the float sign."""
        r = self._reg(tok)
        if r is not None:
            neg, kind, lo, n = r
            assert n == 1, tok
            val = (self.v[lo] if kind == "v" else self.a[lo] if kind == "a" else np.full(LANES, self.s[lo] & 0xFFFFFFFF, dtype=np.uint32)).copy()
            return val ^ np.uint32(0x80000000) if neg else val
        if tok == "m0":
            return np.full(LANES, self.m0, dtype=np.uint32)
        if tok.startswith("0x"):
            return np.full(LANES, int(tok, 16), dtype=np.uint32)
        if re.fullmatch(r"-?\d+", tok):
            return np.full(LANES, int(tok) & 0xFFFFFFFF, dtype=np.uint32)
        return np.full(LANES, np.float32(float(tok)).view(np.uint32), dtype=np.uint32)   # 1.0, 0.5 ... inline float constants

    def f(self, tok):
        return self.src32(tok).view(np.float32)

    def scalar(self, tok):
        if tok == "m0":
            return self.m0
        r = self._reg(tok)
        if r is not None:
            assert r[1] == "s" and r[3] == 1, tok
            return int(self.s[r[2]]) & 0xFFFFFFFF
        return int(tok, 0) & 0xFFFFFFFF

    def set_scalar(self, tok, value):
        if tok == "m0":
            self.m0 = value & 0xFFFFFFFF
        else:
            r = self._reg(tok)
            assert r[1] == "s" and r[3] == 1, tok
            self.s[r[2]] = value & 0xFFFFFFFF

    def put(self, tok, values):
        r = self._reg(tok)
        assert r is not None and r[3] == 1 and not r[0], tok
        (self.v if r[1] == "v" else self.a)[r[2]] = np.asarray(values).view(np.uint32) if np.asarray(values).dtype != np.uint32 else values

    def tuple_regs(self, tok):
        r = self._reg(tok)
        assert r is not None and not r[0], tok
        return (self.v if r[1] == "v" else self.a), r[2], r[3]

    # ---- the matrix instruction
    def mfma(self, d, a, b, c):
        fa, la, na = self.tuple_regs(a)
        fb, lb, nb = self.tuple_regs(b)
        assert na == 4 and nb == 4
        lane = np.arange(LANES)
        A = np.zeros((32, 16), dtype=np.float32)
        B = np.zeros((16, 32), dtype=np.float32)
        av = halves_to_f32(fa[la:la + 4], self.dtype)      # [4 regs, 64 lanes, 2]
        bv = halves_to_f32(fb[lb:lb + 4], self.dtype)
        for reg in range(4):
            for half in range(2):
                k = 8 * (lane // 32) + 2 * reg + half
                A[lane % 32, k] = av[reg, :, half]
                B[k, lane % 32] = bv[reg, :, half]
        fd, ld, nd = self.tuple_regs(d)
        assert nd == 16
        rows = np.array([[8 * (r // 4) + 4 * (l // 32) + r % 4 for l in range(LANES)] for r in range(16)])
        cols = np.tile(lane % 32, (16, 1))
        if c == "0":
            C = np.zeros((32, 32), dtype=np.float32)
        else:
            fc, lc, nc = self.tuple_regs(c)
            C = np.zeros((32, 32), dtype=np.float32)
            C[rows, cols] = fc[lc:lc + 16].view(np.float32)
        with np.errstate(all="ignore"):
            D = (A.astype(np.float64) @ B.astype(np.float64) + C.astype(np.float64)).astype(np.float32)
        fd[ld:ld + 16] = D[rows, cols].view(np.uint32)

    # ---- bookkeeping of the wait counters (see the module text)
    def note_lds_read(self, addr, nbytes, text):
        lo, hi = int(addr.min()), int(addr.max()) + nbytes
        for other in (self.shared or [self]):
            busy = other.vm_pending + ([] if other is self else other.vm_own)
            for r_lo, r_hi in busy:
                if lo < r_hi and hi > r_lo and bool(((addr < r_hi) & (addr + nbytes > r_lo)).any()):
                    who = "this wave has not waited for" if other is self else "another wave has not published"
                    raise RuntimeError(f"`{text}` reads LDS bytes {r_lo}..{r_hi} of a tile request that {who}")
        self.epoch_reads.append((lo, hi))

    def note_request(self, lo, hi, text):
        for other in (self.shared or []):
            if other is self:
                continue
            for r_lo, r_hi in other.epoch_reads:
                if lo < r_hi and hi > r_lo:
                    raise RuntimeError(f"`{text}` requests a tile into LDS bytes {lo}..{hi} that another wave reads before the next barrier")
        self.vm_pending.append((lo, hi))

    # ---- LDS
    def lds_read(self, addr, nbytes):
        out = np.zeros((LANES, nbytes), dtype=np.uint8)
        for l in range(LANES):
            a = int(addr[l])
            if a < 0 or a + nbytes > self.lds.size:
                raise IndexError(f"LDS read at {a} outside the array")
            out[l] = self.lds[a:a + nbytes]
        return out


_VREG_RE = re.compile(r"\b([va])(\d+)\b|\b([va])\[(\d+):(\d+)\]")


def _vector_regs(text):
    out = set()
    for m in _VREG_RE.finditer(text.split(";")[0]):
        if m.group(1):
            out.add((m.group(1), int(m.group(2))))
        else:
            out.update((m.group(3), i) for i in range(int(m.group(4)), int(m.group(5)) + 1))
    return frozenset(out)


def _strip(op):
    return re.sub(r"_(e32|e64)$", "", op)


def run_wave(w: Wave, body):
    """Generator: executes `body` (the generator's lines) on wave `w`, yielding at every s_barrier."""
    ins, labels = [], {}
    for line in body:
        line = line.split(";")[0].strip()
        if not line:
            continue
        if line.endswith(":"):
            labels[line[:-1]] = len(ins)
            continue
        parts = line.split(None, 1)
        ins.append((_strip(parts[0]), [x.strip() for x in parts[1].split(",")] if len(parts) > 1 else [], line))
    pc = 0
    fmax = lambda x, y: np.fmax(x, y)
    named = [_vector_regs(text) if op[0] in "vdg" else frozenset() for op, _, text in ins]   # vector registers each instruction names
    with np.errstate(all="ignore"):
        while pc < len(ins):
            op, a, text = ins[pc]
            touched = named[pc]
            pc += 1
            w.executed += 1
            if op == "s_nop":
                continue
            if op == "s_waitcnt":
                m = re.search(r"lgkmcnt\((\d+)\)", text)
                if m:
                    w.lds_pending = w.lds_pending[len(w.lds_pending) - int(m.group(1)):] if int(m.group(1)) else []
                m = re.search(r"vmcnt\((\d+)\)", text)
                if m:
                    keep = int(m.group(1))
                    done = len(w.vm_pending) - keep
                    if done > 0:
                        w.vm_own += w.vm_pending[:done]
                        w.vm_pending = w.vm_pending[done:]
                continue
            if w.lds_pending and touched:
                for dest in w.lds_pending:
                    if dest & touched:
                        raise RuntimeError(f"`{text}` names a register of an LDS read that no lgkmcnt wait has covered")
            if op == "s_barrier":
                yield "barrier"
            elif op == "s_branch":
                w.taken.append(a[0]); pc = labels[a[0]]
            elif op == "s_cbranch_scc1":
                if w.scc:
                    w.taken.append(a[0]); pc = labels[a[0]]
            elif op == "s_cbranch_vccnz":
                if w.vcc.any():
                    w.taken.append(a[0]); pc = labels[a[0]]
            elif op == "s_cbranch_vccz":
                if not w.vcc.any():
                    w.taken.append(a[0]); pc = labels[a[0]]
            elif op == "s_mov_b32":
                w.set_scalar(a[0], w.scalar(a[1]))
            elif op == "s_mov_b64":
                if a[1] == "vcc":
                    lo = w._reg(a[0])[2]
                    bits = sum(1 << i for i in range(LANES) if w.vcc[i])
                    w.s[lo], w.s[lo + 1] = bits & 0xFFFFFFFF, bits >> 32
                else:
                    d, s_ = w._reg(a[0])[2], w._reg(a[1])[2]
                    w.s[d], w.s[d + 1] = w.s[s_], w.s[s_ + 1]
            elif op in ("s_or_b64", "s_and_b64"):
                def mask64(tok):
                    if tok == "vcc":
                        return sum(1 << i for i in range(LANES) if w.vcc[i])
                    lo = w._reg(tok)[2]
                    return int(w.s[lo]) | (int(w.s[lo + 1]) << 32)
                bits = mask64(a[1]) | mask64(a[2]) if op == "s_or_b64" else mask64(a[1]) & mask64(a[2])
                if a[0] == "vcc":
                    w.vcc = np.array([(bits >> i) & 1 == 1 for i in range(LANES)])
                else:
                    lo = w._reg(a[0])[2]
                    w.s[lo], w.s[lo + 1] = bits & 0xFFFFFFFF, bits >> 32
                w.scc = int(bits != 0)
            elif op == "s_add_u32":
                r = w.scalar(a[1]) + w.scalar(a[2])
                w.scc = int(r > 0xFFFFFFFF)
                w.set_scalar(a[0], r)
            elif op == "s_addc_u32":
                r = w.scalar(a[1]) + w.scalar(a[2]) + w.scc
                w.scc = int(r > 0xFFFFFFFF)
                w.set_scalar(a[0], r)
            elif op == "s_sub_u32":
                x, y = w.scalar(a[1]), w.scalar(a[2])
                w.scc = int(y > x)
                w.set_scalar(a[0], x - y)
            elif op == "s_cmp_eq_u32":
                w.scc = int(w.scalar(a[0]) == w.scalar(a[1]))
            elif op == "s_cmp_lg_u32":
                w.scc = int(w.scalar(a[0]) != w.scalar(a[1]))
            elif op == "s_cmp_gt_u32":
                w.scc = int(w.scalar(a[0]) > w.scalar(a[1]))
            elif op == "s_cselect_b32":
                w.set_scalar(a[0], w.scalar(a[1]) if w.scc else w.scalar(a[2]))
            elif op in ("v_mov_b32", "v_accvgpr_read_b32", "v_accvgpr_write_b32"):
                w.put(a[0], w.src32(a[1]))
            elif op == "v_add_u32":
                w.put(a[0], (w.src32(a[1]).astype(np.uint64) + w.src32(a[2])).astype(np.uint32))
            elif op == "v_lshlrev_b32":
                w.put(a[0], (w.src32(a[2]).astype(np.uint64) << (w.src32(a[1]) & 31)).astype(np.uint32))
            elif op == "v_and_b32":
                w.put(a[0], w.src32(a[1]) & w.src32(a[2]))
            elif op == "v_add_f32":
                w.put(a[0], (w.f(a[1]) + w.f(a[2])).astype(np.float32))
            elif op == "v_sub_f32":
                w.put(a[0], (w.f(a[1]) - w.f(a[2])).astype(np.float32))
            elif op == "v_mul_f32":
                w.put(a[0], (w.f(a[1]) * w.f(a[2])).astype(np.float32))
            elif op == "v_fma_f32":
                x, y, z = w.f(a[1]).astype(np.float64), w.f(a[2]).astype(np.float64), w.f(a[3]).astype(np.float64)
                w.put(a[0], (x * y + z).astype(np.float32))
            elif op == "v_max_f32":
                w.put(a[0], fmax(w.f(a[1]), w.f(a[2])))
            elif op == "v_max3_f32":
                w.put(a[0], fmax(fmax(w.f(a[1]), w.f(a[2])), w.f(a[3])))
            elif op == "v_exp_f32":
                w.put(a[0], np.exp2(w.f(a[1]).astype(np.float64)).astype(np.float32))
            elif op == "v_cmp_neq_f32":
                assert a[0] == "vcc"
                w.vcc = ~(w.f(a[1]) == w.f(a[2]))
            elif op == "v_cmp_nge_f32":
                assert a[0] == "vcc"
                w.vcc = ~(w.f(a[1]) >= w.f(a[2]))
            elif op == "v_cndmask_b32":
                assert a[3] == "vcc"
                w.put(a[0], np.where(w.vcc, w.src32(a[2]), w.src32(a[1])))
            elif op in ("v_cvt_pk_bf16_f32", "v_cvt_pk_f16_f32"):
                x, y = w.f(a[1]), w.f(a[2])
                if op == "v_cvt_pk_bf16_f32":
                    lo, hi = f32_to_bf16(x), f32_to_bf16(y)
                else:
                    lo, hi = x.astype(np.float16).view(np.uint16), y.astype(np.float16).view(np.uint16)
                w.put(a[0], lo.astype(np.uint32) | (hi.astype(np.uint32) << 16))
            elif op in ("v_dot2c_f32_bf16", "v_dot2c_f32_f16"):
                kind = "bf16" if op.endswith("bf16") else "f16"
                x, y = halves_to_f32(w.src32(a[1]), kind), halves_to_f32(w.src32(a[2]), kind)
                acc = w.f(a[0]).astype(np.float64) + (x.astype(np.float64) * y).sum(axis=-1)
                w.put(a[0], acc.astype(np.float32))
            elif op == "v_cvt_f32_f16":
                w.put(a[0], (w.src32(a[1]) & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float32))
            elif op == "v_cvt_f32_f16_sdwa":
                src, mods = a[1].split(None, 1)
                assert "src0_sel:WORD_1" in mods and "dst_sel:DWORD" in mods, text
                w.put(a[0], (w.src32(src) >> 16).astype(np.uint16).view(np.float16).astype(np.float32))
            elif op == "v_permlane32_swap_b32":
                f0, r0, _ = w.tuple_regs(a[0])
                f1, r1, _ = w.tuple_regs(a[1])
                upper0, lower1 = f0[r0, 32:].copy(), f1[r1, :32].copy()
                f0[r0, 32:], f1[r1, :32] = lower1, upper0
            elif op in ("v_mfma_f32_32x32x16_bf16", "v_mfma_f32_32x32x16_f16"):
                assert op.endswith(w.dtype)
                w.mfma(a[0], a[1], a[2], a[3])
            elif op in ("ds_read_b128", "ds_read_b64_tr_b16"):
                addr_tok, off = a[1].split() if " " in a[1] else (a[1], "offset:0")
                addr = w.src32(addr_tok).astype(np.int64) + int(off.split(":")[1], 0)
                fd, ld, nd = w.tuple_regs(a[0])
                w.note_lds_read(addr, 16 if op == "ds_read_b128" else 8, text)
                w.lds_pending.append(frozenset(("v" if fd is w.v else "a", ld + i) for i in range(nd)))
                if op == "ds_read_b128":
                    assert nd == 4
                    fd[ld:ld + 4] = w.lds_read(addr, 16).view(np.uint32).reshape(LANES, 4).T
                else:
                    assert nd == 2
                    got = w.lds_read(addr, 8).view(np.uint16).reshape(LANES, 4)      # [lane, 4 values]
                    out = np.zeros((LANES, 4), dtype=np.uint16)
                    for g in range(LANES // 16):
                        block = got[16 * g:16 * g + 16].reshape(4, 16)                 # row e = lanes 4e .. 4e + 3 in order
                        out[16 * g:16 * g + 16] = block.T                             # lane s: element s of each row
                    fd[ld:ld + 2] = out.view(np.uint32).reshape(LANES, 2).T
            elif op == "global_load_lds_dwordx4":
                lo = w._reg(a[1])[2]
                base = int(w.s[lo]) | (int(w.s[lo + 1]) << 32)
                off = w.src32(a[0])
                w.note_request(w.m0, w.m0 + 16 * LANES, text)
                for l in range(LANES):
                    dst = w.m0 + 16 * l
                    if dst + 16 > w.lds.size:
                        raise IndexError(f"LDS write at {dst} outside the array")
                    w.lds[dst:dst + 16] = w.mem.read16(base + int(off[l]))
            else:
                raise NotImplementedError(text)


def run_workgroup(waves, bodies):
    """Runs the waves of one workgroup to completion; all live waves meet at every barrier. `bodies[i]` is
    the instruction text of wave i (waves may run different statements with the same barrier count)."""
    gens = [run_wave(w, b) for w, b in zip(waves, bodies)]
    for w in waves:
        w.shared = waves
        w.epoch_reads = []
    live = list(range(len(gens)))
    barriers = 0
    while live:
        arrived, done = [], []
        for i in live:
            try:
                next(gens[i])
                arrived.append(i)
            except StopIteration:
                done.append(i)
        if arrived and done:
            raise RuntimeError(f"waves {done} finished while waves {arrived} wait at a barrier")
        barriers += bool(arrived)
        live = arrived
        for w in waves:       # behind the barrier: what each wave had waited for is everybody's, and a new span of reads begins
            w.vm_own = []
            w.epoch_reads = []
    return barriers
