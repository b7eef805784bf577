"""The generated 64-row-wave loop (csrc/gen_wide_loop.py), executed instruction by instruction on a
functional model of the instructions it uses (tests/gfx950_model.py), against attention computed with
numpy in float64. One workgroup: four waves of 64 query rows, the K / V rings in a modelled LDS, the
tile requests served from a modelled global memory.

The operands are set up the way the kernel sets them up before the statement
(stage1_mfma_kernel.h, the 64-row-wave branch: ring offsets, per-lane read addresses, the Q fragments in
the accumulation registers, the address of the next tile to request), so the test also pins that
contract. What the model cannot see (waits, issue hazards, registers the compiler owns) is checked on
the text by the generator itself and on the GPU by the parity tests."""
import importlib.util
import math
import os

import numpy as np
import pytest

from flash_tree_attn_amd import build as fta_build
from gfx950_model import LANES, Memory, Wave, bf16_to_f32, f32_to_bf16, run_workgroup

NW, NSK, NSV, KEY_TILE = 4, 4, 5, 64
SMEM_BASE = 3072            # the kernel's static LDS arrays come first
LDS_BYTES = 160 * 1024


def _generator():
    spec = importlib.util.spec_from_file_location("gen_wide_loop", os.path.join(fta_build.CSRC, "gen_wide_loop.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


GEN = _generator()


def to_storage(x, dtype):
    """float array -> (uint16 storage, the values that storage holds as float64)."""
    if dtype == "bf16":
        u = f32_to_bf16(x.astype(np.float32))
        return u, bf16_to_f32(u).astype(np.float64)
    h = x.astype(np.float16)
    return h.view(np.uint16), h.astype(np.float64)


class Workgroup:
    """LDS, memory and four waves with the operands of the loop statement in place."""

    def __init__(self, D, dtype, q, k, v, first_stage_tile=0, row_pad=0, seed_state=None):
        self.D, self.dtype = D, dtype
        self.lay = GEN.layout(D)
        lay = self.lay
        self.KS, self.DB, self.RPB = D // 16, D // 32, lay["rpb"]
        self.kvring = NSK * lay["tile"]
        assert SMEM_BASE + (NSK + NSV) * lay["tile"] <= LDS_BYTES
        self.lds = np.full(LDS_BYTES, 0xFF, dtype=np.uint8)       # NaN patterns wherever nothing was loaded
        rows, _ = k.shape
        self.row_bytes = 2 * (D + row_pad)
        self.k_store, self.k_val = to_storage(k, dtype)
        self.v_store, self.v_val = to_storage(v, dtype)
        self.q_store, self.q_val = to_storage(q, dtype)
        # a base whose low word is about to overflow: the 64-bit address arithmetic of the tile requests must carry
        self.mem = Memory(0x7F00FFFF0000, 2 * rows * self.row_bytes + 4096)
        padded = lambda st: np.concatenate([st, np.full((rows, row_pad), 0x7FC0, dtype=np.uint16)], axis=1) if row_pad else st
        self.k_addr = self.mem.place(1024, padded(self.k_store))
        self.v_addr = self.mem.place(2048 + rows * self.row_bytes, padded(self.v_store))
        self.c0 = first_stage_tile      # ring position of the first cache tile (tree tiles came before it)
        self.waves = [Wave(self.lds, self.mem, dtype) for _ in range(NW)]
        self.seed_state = seed_state

    def at(self, r, c):
        lay = self.lay
        return (r // self.RPB) * lay["pitch"] + c * lay["chunk"] + (r % self.RPB) * 16

    def fill_stage(self, ring_base, stage, store, tile):
        """What the tile requests of one full tile leave in a ring stage."""
        for r in range(KEY_TILE):
            row = store[tile * KEY_TILE + r]
            for c in range(self.D // 8):
                a = SMEM_BASE + ring_base + stage * self.lay["tile"] + self.at(r, c)
                self.lds[a:a + 16] = row[8 * c:8 * c + 8].view(np.uint8)

    def setup_waves(self, sm_scale):
        """Per-wave values that every statement of the kernel shares: Q fragments, the state (m, l, O), the
        per-lane read addresses, the scale."""
        g, D, KS, DB, RPB = GEN, self.D, self.KS, self.DB, self.RPB
        c = sm_scale * math.log2(math.e)
        lane = np.arange(LANES)
        li, lh = lane & 31, lane >> 5
        for wi, w in enumerate(self.waves):
            for qb in range(2):
                rows = wi * 64 + qb * 32 + li
                for ks in range(KS):
                    cols = (16 * ks + 8 * lh)[:, None] + np.arange(8)[None, :]
                    frag = self.q_store[rows[:, None], cols]                                   # [64 lanes, 8]
                    words = frag[:, 0::2].astype(np.uint32) | (frag[:, 1::2].astype(np.uint32) << 16)
                    for e in range(4):
                        w.a[g.A_Q + 4 * (qb * KS + ks) + e] = words[:, e]
                if self.seed_state is None:
                    w.v[g.V_M + qb] = np.full(LANES, -np.inf, dtype=np.float32).view(np.uint32)
                    w.v[g.V_L + qb] = 0
                else:
                    m, l, o = self.seed_state      # m [256], l [256, 2 halves], o [256, D]: an earlier part of the same softmax
                    w.v[g.V_M + qb] = m[rows].astype(np.float32).view(np.uint32)
                    w.v[g.V_L + qb] = l[rows, lh].astype(np.float32).view(np.uint32)
                    for db in range(DB):
                        for r in range(16):
                            col = db * 32 + 8 * (r // 4) + 4 * lh + r % 4
                            w.a[g.A_O + 16 * (db * 2 + qb) + r] = o[rows, col].astype(np.float32).view(np.uint32)
            w.v[g.V_KRD] = SMEM_BASE + np.array([self.at(int(i), int(h)) for i, h in zip(li, lh)], dtype=np.uint32)
            w.v[g.V_VRD] = SMEM_BASE + self.kvring + np.array(
                [self.at(4 * int(h) + (int(l) & 15) // 4, 2 * ((int(l) >> 4) & 1) + ((int(l) >> 1) & 1)) + (int(l) & 1) * 8 for l, h in zip(lane, lh)],
                dtype=np.uint32)
            w.v[g.V_KOFF] = ((lane % RPB) * self.row_bytes + (lane // RPB) * 16).astype(np.uint32)
            w.v[g.V_VOFF] = w.v[g.V_KOFF]
            w.s[g.S_C] = int(np.float32(c).view(np.uint32))
        return c

    def setup_loop(self, full_tiles, first_cache_tile=0):
        """The operands of the loop statement for `full_tiles` full tiles starting at cache tile
        `first_cache_tile`, and the ring as the kernel's synchronisation point before the loop leaves it."""
        g, lay, RPB = GEN, self.lay, self.RPB
        c0 = self.c0
        issued = min(full_tiles, NSK)
        for i in range(issued):
            self.fill_stage(0, (c0 + i) % NSK, self.k_store, first_cache_tile + i)
            self.fill_stage(self.kvring, (c0 + i) % NSV, self.v_store, first_cache_tile + i)
        nreal = max(0, full_tiles - NSK)
        ktile = KEY_TILE * self.row_bytes
        for wi, w in enumerate(self.waves):
            s = w.s
            first_row = (first_cache_tile + issued) * KEY_TILE + wi * RPB
            krun = self.k_addr + first_row * self.row_bytes - (0 if nreal else ktile)
            vrun = self.v_addr + first_row * self.row_bytes - (0 if nreal else ktile)
            s[g.S_KRUN], s[g.S_KRUN + 1] = krun & 0xFFFFFFFF, krun >> 32
            s[g.S_VRUN], s[g.S_VRUN + 1] = vrun & 0xFFFFFFFF, vrun >> 32
            step = NW * RPB * self.row_bytes
            s[g.S_KSTEP], s[g.S_KSTEP + 1], s[g.S_VSTEP], s[g.S_VSTEP + 1] = step, 0, step, 0
            s[g.S_KTILE], s[g.S_KTILE + 1], s[g.S_VTILE], s[g.S_VTILE + 1] = ktile, 0, ktile, 0
            s[g.S_KCUR], s[g.S_KNEXT] = (c0 % NSK) * lay["tile"], ((c0 + 1) % NSK) * lay["tile"]
            s[g.S_VCUR], s[g.S_VPREV] = (c0 % NSV) * lay["tile"], ((c0 + NSV - 1) % NSV) * lay["tile"]
            s[g.S_PVOFF] = int(s[g.S_VCUR]) + 2 * lay["v16"]
            s[g.S_KDST], s[g.S_VDST] = SMEM_BASE + wi * lay["pitch"], SMEM_BASE + self.kvring + wi * lay["pitch"]
            s[g.S_NT], s[g.S_NREAL] = full_tiles, nreal

    def setup(self, full_tiles, sm_scale):
        c = self.setup_waves(sm_scale)
        self.setup_loop(full_tiles)
        return c

    def fill_edge_stage(self, ring_base, stage, store, key0, key_lim):
        """A ragged or tree tile: rows past the limit repeat the last valid row (stage1_mfma_kernel.h, issue_edge_tile)."""
        for r in range(KEY_TILE):
            row = store[min(key0 + r, key_lim - 1)]
            for c in range(self.D // 8):
                a = SMEM_BASE + ring_base + stage * self.lay["tile"] + self.at(r, c)
                self.lds[a:a + 16] = row[8 * c:8 * c + 8].view(np.uint8)

    def run_masked_half(self, H, ring_tile, key0, key_lim, add_of_row_and_key):
        """One masked half step on every wave (stage1_mfma_kernel.h, masked_half): scores of keys key0 .. key0 + 31
        of the tile in ring position `ring_tile`, plus add_of_row_and_key[row, key] * log2(e), -inf from key_lim on."""
        g, lay = GEN, self.lay
        lane = np.arange(LANES)
        li, lh = lane & 31, lane >> 5
        for wi, w in enumerate(self.waves):
            for qb in range(2):
                rows = wi * 64 + qb * 32 + li
                for r in range(16):
                    j = key0 + (r >> 2) * 8 + 4 * lh + (r & 3)
                    add = np.zeros(LANES) if add_of_row_and_key is None else add_of_row_and_key[rows, np.minimum(j, key_lim - 1)] * math.log2(math.e)
                    w.v[g.V_MADD + 16 * qb + r] = np.where(j < key_lim, add, -np.inf).astype(np.float32).view(np.uint32)
            w.s[g.S_KCUR] = (ring_tile % NSK) * lay["tile"] + H * lay["kb_off"]
            w.s[g.S_VCUR] = (ring_tile % NSV) * lay["tile"] + H * 2 * lay["v16"]
        body = GEN.gen_masked(self.D, self.dtype, H)
        assert run_workgroup(self.waves, [body] * NW) == 0       # no barrier inside a masked half

    def results(self):
        """(m [256], l_total [256], O [256, D]) in the kernel's conventions after the statement."""
        g, DB = GEN, self.DB
        lane = np.arange(LANES)
        li, lh = lane & 31, lane >> 5
        m, l, o = np.zeros(256), np.zeros(256), np.zeros((256, self.D))
        for wi, w in enumerate(self.waves):
            for qb in range(2):
                rows = wi * 64 + qb * 32 + li
                mm = w.v[g.V_M + qb].view(np.float32)
                assert np.array_equal(mm[:32], mm[32:])                  # both half-waves hold the same reference for a row
                m[rows[:32]] = mm[:32]
                ll = w.v[g.V_L + qb].view(np.float32).astype(np.float64)
                l[rows[:32]] = ll[:32] + ll[32:]                          # the epilogue's cross-half sum
                for db in range(DB):
                    for r in range(16):
                        col = db * 32 + 8 * (r // 4) + 4 * lh + r % 4
                        o[rows, col] = w.a[g.A_O + 16 * (db * 2 + qb) + r].view(np.float32)
        return m, l, o


def reference(q_val, k_val, v_val, keys, sm_scale):
    s = (q_val @ k_val[:keys].T) * sm_scale
    p = np.exp(s - s.max(axis=1, keepdims=True))
    return (p / p.sum(axis=1, keepdims=True)) @ v_val[:keys], s.max(axis=1) + np.log(p.sum(axis=1))


def make_case(seed, D, tiles, spread=1.0):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((256, D))
    k = rng.standard_normal((tiles * KEY_TILE, D)) * spread
    v = rng.standard_normal((tiles * KEY_TILE, D))
    return q, k, v


@pytest.mark.parametrize("D,dtype,tiles,c0,pad", [
    (128, "bf16", 1, 0, 0), (128, "bf16", 3, 0, 0), (128, "bf16", 6, 1, 0), (128, "f16", 5, 2, 8),
    (64, "bf16", 6, 0, 0), (64, "f16", 9, 3, 0), (128, "bf16", 10, 2, 64),
])
def test_loop_against_numpy_attention(D, dtype, tiles, c0, pad):
    q, k, v = make_case(11 * tiles + D, D, tiles)
    wg = Workgroup(D, dtype, q, k, v, first_stage_tile=c0, row_pad=pad)
    sm_scale = 1.0 / math.sqrt(D)
    wg.setup(tiles, sm_scale)
    body = GEN.gen(D, dtype)
    barriers = run_workgroup(wg.waves, [body] * NW)
    assert barriers == tiles                                             # one synchronisation point per tile
    m, l, o = wg.results()
    ref_o, ref_lse = reference(wg.q_val, wg.k_val, wg.v_val, tiles * KEY_TILE, sm_scale)
    out = o / l[:, None]
    lse = (m + np.log2(l)) * math.log(2.0)
    np.testing.assert_allclose(lse, ref_lse, atol=2e-3, rtol=0)
    np.testing.assert_allclose(out, ref_o, atol=2e-3, rtol=1e-2)
    # the first step starts from m = -inf, so every wave took the exact step once at least; the pipeline
    # re-entered the loop after it
    for w in wg.waves:
        assert any(t.startswith(".Lfix0") for t in w.taken)
    # ring bookkeeping: requests went out for tiles 4 .. tiles - 1 (and stand-ins after them): every K / V
    # value the products used came from the right tile, which the comparison above could not pass otherwise


def test_loop_continues_a_softmax_that_other_keys_started():
    """The statement takes over (m, l, O) from the tree phase: results must be those of one softmax over both parts."""
    D, dtype, tiles = 128, "bf16", 4
    q, k, v = make_case(5, D, tiles + 1)
    sm_scale = 1.0 / math.sqrt(D)
    c = sm_scale * math.log2(math.e)
    probe = Workgroup(D, dtype, q, k[KEY_TILE:], v[KEY_TILE:])
    # exact state after the first 64 keys, in the kernel's form: m in scaled log2 units, l split over the two half-waves, O unnormalised
    s0 = (probe.q_val @ to_storage(k[:KEY_TILE], dtype)[1].T) * c
    m0 = s0.max(axis=1)
    p0 = np.exp2(s0 - m0[:, None])
    l0 = np.stack([p0[:, :32].sum(axis=1), p0[:, 32:].sum(axis=1)], axis=1)
    o0 = p0 @ to_storage(v[:KEY_TILE], dtype)[1]
    wg = Workgroup(D, dtype, q, k[KEY_TILE:], v[KEY_TILE:], first_stage_tile=1, seed_state=(m0, l0, o0))
    wg.setup(tiles, sm_scale)
    run_workgroup(wg.waves, [GEN.gen(D, dtype)] * NW)
    m, l, o = wg.results()
    k_all = np.concatenate([to_storage(k[:KEY_TILE], dtype)[1], wg.k_val])
    v_all = np.concatenate([to_storage(v[:KEY_TILE], dtype)[1], wg.v_val])
    ref_o, ref_lse = reference(wg.q_val, k_all, v_all, (tiles + 1) * KEY_TILE, sm_scale)
    np.testing.assert_allclose((m + np.log2(l)) * math.log(2.0), ref_lse, atol=2e-3, rtol=0)
    np.testing.assert_allclose(o / l[:, None], ref_o, atol=2e-3, rtol=1e-2)


def test_a_late_key_that_raises_the_maximum_takes_the_exact_step():
    """Lazy softmax: the reference is only raised when a half tile's sums run away. A key far above all
    earlier ones, late in the stream, must send its step through the exact redo, and the result must not
    change."""
    D, dtype, tiles = 128, "f16", 6
    q, k, v = make_case(9, D, tiles)
    k[5 * KEY_TILE + 40] = q[:4].mean(axis=0) * 6.0          # tile 5, second half: step 0 of the loop's last pass
    k[2 * KEY_TILE + 3] = q[200] * 4.0                        # tile 2, first half: step 1
    wg = Workgroup(D, dtype, q, k, v)
    sm_scale = 1.0 / math.sqrt(D)
    wg.setup(tiles, sm_scale)
    run_workgroup(wg.waves, [GEN.gen(D, dtype)] * NW)
    m, l, o = wg.results()
    ref_o, ref_lse = reference(wg.q_val, wg.k_val, wg.v_val, tiles * KEY_TILE, sm_scale)
    np.testing.assert_allclose((m + np.log2(l)) * math.log(2.0), ref_lse, atol=2e-3, rtol=0)
    np.testing.assert_allclose(o / l[:, None], ref_o, atol=4e-3, rtol=1e-2)
    fixes = [sum(1 for t in w.taken if t.startswith(".Lfix")) for w in wg.waves]
    assert fixes[3] >= 2 and fixes[0] >= 2, fixes           # the first step and the late key (rows 200 and 0..3)
    assert all(np.isfinite(o).ravel())


def tree_mask(rng, L):
    """Additive mask of a random tree: row i attends to itself and to its ancestors."""
    parents = [-1] + [int(rng.integers(0, i)) for i in range(1, L)]
    allowed = np.zeros((L, L), dtype=bool)
    for i in range(L):
        j = i
        while j >= 0:
            allowed[i, j] = True
            j = parents[j]
    return np.where(allowed, 0.0, -np.inf)


@pytest.mark.parametrize("D,dtype,L,heads,full_tiles,tail", [
    (128, "bf16", 64, 4, 5, 37),        # a whole tree tile, five full cache tiles, a ragged tile of 37 keys
    (64, "f16", 40, 6, 2, 0),           # 240 of 256 rows hold queries; the tree tile ends at key 40; no ragged tile
    (128, "f16", 64, 4, 0, 50),         # no full tile at all: tree + ragged tile only
    (128, "bf16", 32, 8, 7, 33),        # a tree of exactly one half tile; the ragged tile needs both halves
])
def test_a_whole_split_tree_tiles_loop_and_ragged_tail(D, dtype, L, heads, full_tiles, tail):
    """The statements in the order the kernel runs them for the split that owns the end of a sequence
    (stage1_mfma_kernel.h, phases A, B, C of the 64-row-wave branch): masked halves over the tree tile, the
    loop over the full cache tiles, masked halves over the ragged last tile; state stays in the registers.
    Expected: one softmax per query row over [cache keys ; tree keys under the mask]."""
    rng = np.random.default_rng(1000 * L + full_tiles)
    T = full_tiles * KEY_TILE + tail
    rows = heads * L
    assert rows <= 256
    q = np.zeros((256, D))
    q[:rows] = rng.standard_normal((rows, D))               # rows past the unit hold zeros, as the kernel loads them
    cache_rows = max(T, 1)
    k, v = rng.standard_normal((cache_rows, D)), rng.standard_normal((cache_rows, D))
    tk, tv = rng.standard_normal((L, D)), rng.standard_normal((L, D))
    mask = tree_mask(rng, L)
    add = np.zeros((256, L))
    add[:rows] = mask[np.arange(rows) % L]                  # row r of the unit is tree token r % L of head r // L
    sm_scale = 1.0 / math.sqrt(D)
    tree_tiles = 1
    wg = Workgroup(D, dtype, q, k, v, first_stage_tile=tree_tiles)
    tk_store, tk_val = to_storage(tk, dtype)
    tv_store, tv_val = to_storage(tv, dtype)
    wg.setup_waves(sm_scale)
    # phase A: the tree tile sits in ring position 0
    wg.fill_edge_stage(0, 0, tk_store, 0, L)
    wg.fill_edge_stage(wg.kvring, 0, tv_store, 0, L)
    wg.run_masked_half(0, 0, 0, L, add)
    assert all(w.taken == [".Lnoscale_%="] for w in wg.waves)         # nothing accumulated yet: O is not rescaled
    if 32 < L:
        wg.run_masked_half(1, 0, 32, L, add)
        assert any(len(w.taken) == 1 for w in wg.waves)               # some row's reference moved: this time it is
    # phase B
    if full_tiles:
        wg.setup_loop(full_tiles)
        assert run_workgroup(wg.waves, [GEN.gen(D, dtype)] * NW) == full_tiles
    # phase C: the ragged tile takes the next ring position
    if tail:
        t = tree_tiles + full_tiles
        wg.fill_edge_stage(0, t % NSK, wg.k_store, full_tiles * KEY_TILE, T)
        wg.fill_edge_stage(wg.kvring, t % NSV, wg.v_store, full_tiles * KEY_TILE, T)
        wg.run_masked_half(0, t, full_tiles * KEY_TILE, T, None)
        if full_tiles * KEY_TILE + 32 < T:
            wg.run_masked_half(1, t, full_tiles * KEY_TILE + 32, T, None)
    m, l, o = wg.results()
    s_cache = (wg.q_val[:rows] @ wg.k_val[:T].T) * sm_scale
    s_tree = (wg.q_val[:rows] @ tk_val.T) * sm_scale + add[:rows]
    s = np.concatenate([s_cache, s_tree], axis=1)
    p = np.exp(s - s.max(axis=1, keepdims=True))
    ref = (p / p.sum(axis=1, keepdims=True)) @ np.concatenate([wg.v_val[:T], tv_val])
    ref_lse = s.max(axis=1) + np.log(p.sum(axis=1))
    np.testing.assert_allclose(((m + np.log2(l)) * math.log(2.0))[:rows], ref_lse, atol=2e-3, rtol=0)
    np.testing.assert_allclose((o / l[:, None])[:rows], ref, atol=2e-3, rtol=1e-2)
    assert np.isfinite(o).all() and np.isfinite(l).all()    # rows past the unit (zero queries) stay finite too


def _run_mutated(mutate, D=64, dtype="bf16", tiles=8):
    q, k, v = make_case(1, D, tiles)
    wg = Workgroup(D, dtype, q, k, v)
    wg.setup(tiles, 1.0 / math.sqrt(D))
    body = mutate(list(GEN.gen(D, dtype)))
    run_workgroup(wg.waves, [body] * NW)


def test_the_model_holds_the_loop_to_its_waits():
    """The model delivers every load at once, but keeps the books of the wait counters: a text whose waits are
    weaker than its reads need, or whose requests overtake the barrier, must fail although the data is there."""
    import re
    _run_mutated(lambda b: b)                                            # as rendered: clean
    base = GEN.gen(64, "bf16")
    stop = next(i for i, l in enumerate(base) if l.startswith(".Lfix0"))
    waits = [i for i, l in enumerate(base) if l.startswith("s_waitcnt lgkmcnt") and i < stop]
    assert len(waits) >= 20
    for i in waits[::3]:                                                 # every wait is exactly as strong as it must be
        def weaker(b, i=i):
            n = int(re.search(r"\((\d+)\)", b[i]).group(1))
            b[i] = f"s_waitcnt lgkmcnt({n + 1})"
            return b
        with pytest.raises(RuntimeError, match="no lgkmcnt wait has covered"):
            _run_mutated(weaker, tiles=2)

    def weaker_tile_wait(b):
        i = next(i for i, l in enumerate(b) if l.startswith("s_waitcnt vmcnt"))
        n = int(re.search(r"\((\d+)\)", b[i]).group(1))
        b[i] = f"s_waitcnt vmcnt({n * 3 // 2})"                          # leaves three tiles in flight instead of two
        return b
    with pytest.raises(RuntimeError, match="this wave has not waited for"):
        _run_mutated(weaker_tile_wait)

    def no_barrier(b):
        b[b.index("s_barrier")] = "s_nop 0"
        return b
    with pytest.raises(RuntimeError, match="another wave has not published"):
        _run_mutated(no_barrier)

    def request_ahead_of_the_barrier(b):
        bar = b.index("s_barrier")
        load = next(i for i, l in enumerate(b) if l.startswith("global_load_lds"))
        group = b[load - 3:load + 1]                                     # address, M0, gap, request
        del b[load - 3:load + 1]
        where = next(i for i, l in enumerate(b) if l.startswith(f"s_add_u32 s{GEN.S_TMP + 6}"))
        landing = b.pop(where)                                           # the LDS address the request lands at
        b[bar:bar] = [landing] + group
        return b
    with pytest.raises(RuntimeError):
        _run_mutated(request_ahead_of_the_barrier)


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_error_margin_of_the_loop_at_the_headline_chunk(dtype):
    """One workgroup of the headline plan (33 full tiles = 2112 keys, head_dim 128) with the instruction-exact
    roundings of the model (probabilities and row sums in 16 bits, fp32 accumulation): the largest error as a
    share of the tolerance, printed, and held to half of it."""
    D, tiles = 128, 33
    q, k, v = make_case(77, D, tiles)
    wg = Workgroup(D, dtype, q, k, v)
    sm_scale = 1.0 / math.sqrt(D)
    wg.setup(tiles, sm_scale)
    run_workgroup(wg.waves, [GEN.gen(D, dtype)] * NW)
    m, l, o = wg.results()
    ref, _ = reference(wg.q_val, wg.k_val, wg.v_val, tiles * KEY_TILE, sm_scale)
    err = np.abs(o / l[:, None] - ref)
    share = (err / (2e-3 + 1e-2 * np.abs(ref))).max()
    print(f"\n64-row-wave loop, {dtype}, 2112 keys: max abs err {err.max():.3e}, largest share of the tolerance {share:.3f}")
    assert share <= 0.5
