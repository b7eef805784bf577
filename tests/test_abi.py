"""CPU-only checks of the C-ABI library: it loads, exports every symbol include/fta.h
declares, validates arguments like the reference's asserts (flash_tree_attn.py:263-291)
and plans splits sensibly. No kernel is launched here."""
import ctypes as C
import os
import re
import subprocess

import pytest

from flash_tree_attn_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def base_args(**kw):
    a = _lib.FtaArgs()
    ptr = 0x1000  # never dereferenced by validate/plan
    for f in ("q", "k_cache", "v_cache", "cur_k", "cur_v", "mask", "kv_seq_len", "out"):
        setattr(a, f, ptr)
    cfg = dict(bsz=8, num_q_heads=32, num_kv_heads=8, cur_heads=8, q_len=64, head_dim=128, cache_len=8192,
               v_cache_len=8192, block_size=64, max_seq_len_hint=0, mid_splits=0, dtype=_lib.FTA_BF16,
               len_dtype=_lib.FTA_I64, force_splits=0, force_kernel=-1, sm_scale=128 ** -0.5)
    cfg.update(kw)
    for k, v in cfg.items():
        setattr(a, k, v)
    D, L, T = a.head_dim, a.q_len, a.cache_len
    a.q_stride[:] = [a.num_q_heads * L * D, L * D, D]
    a.k_stride[:] = [a.num_kv_heads * T * D, T * D, D]
    a.v_stride[:] = a.k_stride[:]
    a.ck_stride[:] = [a.cur_heads * L * D, L * D, D]
    a.cv_stride[:] = a.ck_stride[:]
    a.mask_stride[:] = [0, 0, L]
    a.out_stride[:] = a.q_stride[:]
    return a


def plan(fta_lib, a, cus=256):
    pl = _lib.FtaPlanOut()
    st = fta_lib.fta_plan(C.byref(a), cus, C.byref(pl))
    return st, pl


def test_header_symbols_exported(fta_lib):
    header = open(os.path.join(ROOT, "include", "fta.h")).read()
    declared = set(re.findall(r"^\s*(?:int|const char\*)\s+(fta_\w+)\s*\(", header, flags=re.M))
    assert declared == set(_lib.EXPORTED_SYMBOLS)
    for name in declared:
        assert hasattr(fta_lib, name), name
    assert fta_lib.fta_abi_version() == _lib.ABI_VERSION
    assert int(re.search(r"#define FTA_ABI_VERSION (\d+)", header).group(1)) == _lib.ABI_VERSION


def test_struct_layout_matches_header(fta_lib, tmp_path):
    # 12 pointers, 18 int32 + 1 float (padded to 8), 9 stride arrays (8 of 3 + 1 of 4 int64), 1 int64
    assert C.sizeof(_lib.FtaArgs) == 12 * 8 + 20 * 4 + (8 * 3 + 4) * 8 + 8
    assert C.sizeof(_lib.FtaPlanOut) == 10 * 4 + 2 * 8 + 2 * _lib.LEN_BUCKETS * 4
    # ... and field by field against what a C compiler makes of include/fta.h
    fields = [n for n, _ in _lib.FtaArgs._fields_]
    plan_fields = [n for n, _ in _lib.FtaPlanOut._fields_]
    append_fields = [n for n, _ in _lib.FtaAppendArgs._fields_]
    src = tmp_path / "layout.c"
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "fta.h"', 'int main(void) {',
             '  printf("%zu %zu %zu\\n", sizeof(fta_args), sizeof(fta_plan_out), sizeof(fta_append_args));']
    lines += [f'  printf("%zu\\n", offsetof(fta_args, {n}));' for n in fields]
    lines += [f'  printf("%zu\\n", offsetof(fta_plan_out, {n}));' for n in plan_fields]
    lines += [f'  printf("%zu\\n", offsetof(fta_append_args, {n}));' for n in append_fields]
    lines += ['  return 0;', '}']
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    assert [int(v) for v in out[:3]] == [C.sizeof(_lib.FtaArgs), C.sizeof(_lib.FtaPlanOut), C.sizeof(_lib.FtaAppendArgs)]
    offs = [int(v) for v in out[3:]]
    n1, n2 = len(fields), len(fields) + len(plan_fields)
    assert offs[:n1] == [getattr(_lib.FtaArgs, n).offset for n in fields]
    assert offs[n1:n2] == [getattr(_lib.FtaPlanOut, n).offset for n in plan_fields]
    assert offs[n2:] == [getattr(_lib.FtaAppendArgs, n).offset for n in append_fields]


def test_strerror(fta_lib):
    assert fta_lib.fta_strerror(0) == b"ok"
    seen = set()
    for st in range(-11, 0):
        s = fta_lib.fta_strerror(st)
        assert s and s != b"unknown fta status"
        seen.add(s)
    assert len(seen) == 11
    assert fta_lib.fta_strerror(-99) == b"unknown fta status"


@pytest.mark.parametrize("kw, status", [
    (dict(head_dim=96), -2), (dict(head_dim=512), -2),          # flash_tree_attn.py:263
    (dict(block_size=48), -3), (dict(block_size=256), -3),      # flash_tree_attn.py:268
    (dict(v_cache_len=4096), -4),                               # flash_tree_attn.py:264
    (dict(dtype=7), -6), (dict(len_dtype=3), -6),
    (dict(bsz=0), -7), (dict(num_q_heads=30), -7), (dict(cur_heads=16), -7), (dict(q_len=0), -7),
    (dict(force_kernel=5), -9),
])
def test_validate_rejects(fta_lib, kw, status):
    a = base_args(**kw)
    assert fta_lib.fta_validate(C.byref(a)) == status
    assert plan(fta_lib, a)[0] == status


def test_validate_pointer_and_stride_rules(fta_lib):
    a = base_args()
    assert fta_lib.fta_validate(C.byref(a)) == 0
    assert fta_lib.fta_validate(None) == -1
    a.mask = None
    assert fta_lib.fta_validate(C.byref(a)) == -1
    a = base_args()
    a.k_stride[2] = 130  # rows no longer 16-byte aligned
    assert fta_lib.fta_validate(C.byref(a)) == -8
    a = base_args()
    a.q = 0x1004
    assert fta_lib.fta_validate(C.byref(a)) == -8
    a = base_args()
    a.v_stride[0] = -1
    assert fta_lib.fta_validate(C.byref(a)) == -8


def test_decode_without_scratch_or_device_fails_cleanly(fta_lib):
    """fta_decode validates before touching HIP; on a GPU-less host it must return an
    error status instead of crashing."""
    a = base_args(head_dim=96)
    assert fta_lib.fta_decode(C.byref(a), None) == -2
    import torch
    if not torch.cuda.is_available():
        a = base_args()
        assert fta_lib.fta_decode(C.byref(a), None) == -11


CASES = [
    dict(),                                                                                     # cfg3_gqa_8b_bf16
    dict(bsz=4, num_q_heads=32, num_kv_heads=32, cur_heads=32, q_len=26, cache_len=4096, v_cache_len=4096, dtype=_lib.FTA_F16),
    dict(bsz=1, cache_len=131072, v_cache_len=131072),                                          # config 4
    dict(bsz=64, num_q_heads=64, q_len=16, cache_len=32768, v_cache_len=32768),                 # config 5
    dict(bsz=1, num_q_heads=8, num_kv_heads=8, cur_heads=8, q_len=4, head_dim=64, cache_len=256, v_cache_len=256, dtype=_lib.FTA_F32),
    dict(bsz=2, cache_len=0, v_cache_len=0),
    dict(bsz=3, cache_len=100, v_cache_len=100, block_size=16),
    dict(bsz=2, cache_len=100000, v_cache_len=100000, block_size=128, max_seq_len_hint=777),
    dict(head_dim=256),                                                                         # 256 rows per unit at head_dim 256: two row blocks of 128
    dict(head_dim=256, num_q_heads=8, num_kv_heads=8, cur_heads=8, q_len=1),                    # plain decode at head_dim 256
    dict(num_q_heads=32, num_kv_heads=32, cur_heads=32, q_len=1),                               # plain decode: one row per unit, MFMA kernel
    dict(sm_scale=-0.1),                                                                        # the MFMA kernel needs a positive scale
]


@pytest.mark.parametrize("kw", CASES)
@pytest.mark.parametrize("cus", [256, 64, 1])
def test_plan_properties(fta_lib, kw, cus):
    a = base_args(**kw)
    st, pl = plan(fta_lib, a, cus)
    assert st == 0
    t_cap = min(a.max_seq_len_hint, a.cache_len) if a.max_seq_len_hint else a.cache_len
    gran = max(a.block_size, 64)
    assert pl.num_splits >= 1
    assert pl.chunk % a.block_size == 0 and pl.chunk % 64 == 0 and pl.chunk >= gran
    # the splits cover every key exactly once ...
    assert pl.num_splits * pl.chunk >= t_cap
    assert (pl.num_splits - 1) * pl.chunk < max(t_cap, 1)
    # ... and never outnumber the reference's block count, so its scratch shapes fit
    assert pl.num_splits <= max(1, -(-t_cap // a.block_size))
    hpu = a.num_q_heads // a.num_kv_heads if a.cur_heads == a.num_kv_heads else 1
    assert pl.rows_per_group == hpu * a.q_len
    assert pl.row_blocks == -(-pl.rows_per_group // pl.rows_per_wg)
    if a.head_dim == 256:
        assert pl.rows_per_wg in (16, 128)   # no 256-row variant: its rings would not fit the LDS
    assert pl.num_workgroups == a.bsz * (a.num_q_heads // hpu) * pl.row_blocks * pl.num_splits
    if pl.num_splits > 1:
        assert pl.mid_lse_elems == a.bsz * a.num_q_heads * pl.num_splits * a.q_len
        assert pl.mid_o_elems == pl.mid_lse_elems * a.head_dim
    else:
        assert pl.mid_o_elems == 0 and pl.mid_lse_elems == 0
    mfma_ok = a.dtype in (_lib.FTA_F16, _lib.FTA_BF16) and a.head_dim in (64, 128, 256) and a.sm_scale > 0
    assert pl.kernel == (_lib.KERNEL_MFMA if mfma_ok else _lib.KERNEL_SHUFFLE)
    # one counter per (sequence, unit, row block) where the merge can run inside stage 1
    fusable = pl.num_splits > 1 and pl.kernel == _lib.KERNEL_MFMA
    assert pl.counter_elems == (pl.num_workgroups // pl.num_splits if fusable else 0)
    slots = cus * (2 if pl.rows_per_wg == 128 and a.head_dim <= 128 else 1)   # the 128-row variant shares a CU with a second workgroup (MFMA plans only reach here)
    assert pl.single_launch == int(fusable and pl.num_splits <= 2 and pl.num_workgroups <= slots)


def test_plan_headline_shape_fills_the_gpu(fta_lib):
    """bsz 8 x 8 kv heads x 256 rows: 64 independent streams must be split so that at
    least one workgroup lands on each of the 256 CUs."""
    st, pl = plan(fta_lib, base_args())
    assert st == 0 and pl.kernel == _lib.KERNEL_MFMA
    assert pl.rows_per_group == 256 and pl.num_workgroups >= 256
    st, pl4 = plan(fta_lib, base_args(bsz=1, cache_len=131072, v_cache_len=131072))
    assert pl4.num_workgroups >= 256


@pytest.mark.parametrize("kw,splits,chunk", [
    (dict(bsz=4, num_q_heads=32, num_kv_heads=32, cur_heads=32, q_len=26, cache_len=4096, v_cache_len=4096, dtype=_lib.FTA_F16), 4, 1088),
    (dict(), 4, 2112),                                                                            # config 3
    (dict(bsz=1, cache_len=131072, v_cache_len=131072), 32, 4160),                                # config 4
    (dict(bsz=64, num_q_heads=64, q_len=16, cache_len=32768, v_cache_len=32768), 3, 11008),      # config 5
    (dict(bsz=32, num_q_heads=32, num_kv_heads=32, cur_heads=32, q_len=128, cache_len=4096, v_cache_len=4096,
          dtype=_lib.FTA_F16, block_size=128), 1, 4096),                                          # the reference test's shape: one pass
])
def test_plan_of_the_measured_workloads(fta_lib, kw, splits, chunk):
    """The split counts the published measurements were taken with (each the measured optimum
    or within 2 % of it on a 256-CU part): a change of the cost model that moves them needs new measurements."""
    st, pl = plan(fta_lib, base_args(**kw))
    assert st == 0 and (pl.num_splits, pl.chunk) == (splits, chunk)


def test_plan_overrides(fta_lib):
    st, pl = plan(fta_lib, base_args(force_splits=3))
    assert st == 0 and pl.num_splits == 3
    st, pl = plan(fta_lib, base_args(force_kernel=_lib.KERNEL_SHUFFLE))
    assert st == 0 and pl.kernel == _lib.KERNEL_SHUFFLE and pl.rows_per_wg == 16
    st, _ = plan(fta_lib, base_args(force_kernel=_lib.KERNEL_MFMA, dtype=_lib.FTA_F32))
    assert st == -9


def _live_workgroups(pl, lengths, units_x_row_blocks):
    """Stage-1 workgroups that have keys to process, the way the kernels count them."""
    chunk = pl.chunk_for(max(lengths))
    return sum(min(pl.num_splits, max(1, -(-t // chunk))) for t in lengths) * units_x_row_blocks


@pytest.mark.parametrize("kw", [
    dict(), dict(bsz=1), dict(bsz=3, q_len=16), dict(head_dim=64, dtype=_lib.FTA_F16), dict(q_len=1, num_q_heads=8, num_kv_heads=8, cur_heads=8),
    dict(dtype=_lib.FTA_F32), dict(block_size=128), dict(force_splits=7), dict(cache_len=100, v_cache_len=100), dict(cache_len=0, v_cache_len=0),
    dict(max_seq_len_hint=3000), dict(head_dim=256, q_len=8),
])
@pytest.mark.parametrize("capacity", [None, 131072])
def test_chunk_table_invariants(fta_lib, kw, capacity):
    kw = dict(kw)
    if capacity and "cache_len" not in kw:
        kw.update(cache_len=capacity, v_cache_len=capacity)
    a = base_args(**kw)
    st, pl = plan(fta_lib, a)
    assert st == 0
    cap = max(1, min(a.cache_len, a.max_seq_len_hint) if a.max_seq_len_hint else a.cache_len)
    bounds, chunks = list(pl.len_bound), list(pl.chunk_by_len)
    gran = max(a.block_size, 64)
    assert bounds == sorted(bounds) and bounds[-1] == cap and chunks[-1] == pl.chunk
    for i, (bound, chunk) in enumerate(zip(bounds, chunks)):
        assert 1 <= bound <= cap
        assert chunk > 0 and chunk % gran == 0                      # whole key tiles and whole reference blocks
        assert pl.num_splits * chunk >= bound                       # the grid's split slots cover every length of the bucket
        assert -(-bound // chunk) <= pl.num_splits
        if i:
            assert bound * 2 <= bounds[i - 1] * 3 + 3 * gran        # steps of at most 3/2 (plus rounding to whole blocks)
        assert pl.chunk_for(bound) == chunks[bounds.index(bound)]   # equal bounds: the first entry serves
    assert pl.chunk_for(cap + 1) == pl.chunk and pl.chunk_for(0) == chunks[0]


def test_chunks_follow_the_lengths_not_the_capacity(fta_lib):
    """A cache far larger than the sequences in it (or a wide page table) must not leave the
    grid idle: for the headline shape with 8192 live keys the cut is the one a cache of
    exactly 8192 gets, whatever the capacity, and one sequence still spreads over the machine."""
    st, exact = plan(fta_lib, base_args())
    assert st == 0 and (exact.num_splits, exact.chunk) == (4, 2112)
    for capacity in (8192, 12288, 16384, 65536, 131072):
        st, pl = plan(fta_lib, base_args(cache_len=capacity, v_cache_len=capacity))
        assert st == 0
        live = _live_workgroups(pl, [8192] * 8, 8)
        assert 192 <= live <= 256, (capacity, pl.num_splits, pl.chunk_for(8192), live)
        assert pl.chunk_for(8192) <= 2 * 2112
    st, one = plan(fta_lib, base_args(bsz=1, cache_len=131072, v_cache_len=131072))
    st2, one_exact = plan(fta_lib, base_args(bsz=1))
    assert st == 0 and st2 == 0
    assert _live_workgroups(one, [8192], 8) >= 0.6 * _live_workgroups(one_exact, [8192], 8)
    # and a short batch in the big cache is not shredded either: chunks stay at four key tiles or more
    assert one.chunk_for(700) >= 256


def test_plan_of_the_64_row_wave_loop(fta_lib):
    """The hand-scheduled loop is a choice of the caller: units of 256 rows on contiguous caches,
    head_dim 64 or 128. Asked for anywhere else it is refused, never silently replaced."""
    wide = dict(num_q_heads=32, num_kv_heads=8, cur_heads=8, q_len=64, force_kernel=_lib.KERNEL_MFMA_WIDE)
    st, pl = plan(fta_lib, base_args(**wide))
    assert st == 0 and pl.kernel == _lib.KERNEL_MFMA and pl.rows_per_wg == 256 and pl.mfma_loop == 1
    # cut like the 8-wave loop until a timing of its tree phase says otherwise (FTA_TREE_TILE_WEIGHT sets the weight for such a run)
    assert (pl.num_splits, pl.chunk) == (4, 2112)
    st, pl = plan(fta_lib, base_args(**{**wide, "force_kernel": _lib.KERNEL_MFMA}))
    assert st == 0 and pl.rows_per_wg == 256 and pl.mfma_loop == 0
    if not os.environ.get("FTA_WIDE_LOOP"):
        st, pl = plan(fta_lib, base_args(**{**wide, "force_kernel": -1}))
        assert st == 0 and pl.mfma_loop == 0
    assert plan(fta_lib, base_args(**{**wide, "q_len": 8}))[0] == -9              # 32-row units
    assert plan(fta_lib, base_args(**{**wide, "head_dim": 256}))[0] == -9
    assert plan(fta_lib, base_args(**{**wide, "dtype": _lib.FTA_F32}))[0] == -9
    a = base_args(**wide)                                                         # paged caches: 64 pages of 128 positions per sequence
    table = (C.c_int32 * (8 * 64))()
    a.block_table, a.block_table_stride, a.page_size = C.cast(table, C.c_void_p), 64, 128
    a.k_stride[0] = a.v_stride[0] = 8 * 128 * 128
    a.k_stride[1] = a.v_stride[1] = 128 * 128
    assert fta_lib.fta_validate(C.byref(a)) == 0 and plan(fta_lib, a)[0] == -9

    a.force_kernel = -1
    st, pl = plan(fta_lib, a)
    assert st == 0 and pl.rows_per_wg == 256 and pl.mfma_loop == 0
    # a paged cache of no positions has no pages to name: rejected as a shape error
    a.cache_len = a.v_cache_len = 0
    assert fta_lib.fta_validate(C.byref(a)) == -7


def test_plan_reports_key_halves_only_when_asked_and_refuses_them_where_they_do_not_exist(fta_lib):
    """FTA_KERNEL_MFMA_SPLIT_KEYS: units of at most 64 rows, head_dim 64 / 128, any cache layout. Reported as the MFMA
    kernel with 64-row workgroups and mfma_loop = 2; the cut is the 4-wave variant's (same cost model)."""
    small = dict(num_q_heads=32, num_kv_heads=32, cur_heads=32, q_len=26, dtype=_lib.FTA_F16, force_kernel=_lib.KERNEL_MFMA_SPLIT_KEYS)
    st, pl = plan(fta_lib, base_args(**small))
    assert st == 0 and pl.kernel == _lib.KERNEL_MFMA and (pl.rows_per_wg, pl.row_blocks, pl.mfma_loop) == (64, 1, 2)
    st, plain = plan(fta_lib, base_args(**{**small, "force_kernel": _lib.KERNEL_MFMA}))
    assert st == 0 and (plain.rows_per_wg, plain.mfma_loop) == (128, 0)
    assert (pl.num_splits, pl.chunk, pl.num_workgroups) == (plain.num_splits, plain.chunk, plain.num_workgroups)
    if not os.environ.get("FTA_SPLIT_KEYS"):
        st, auto = plan(fta_lib, base_args(**{**small, "force_kernel": -1}))
        assert st == 0 and (auto.rows_per_wg, auto.mfma_loop) == (128, 0)
    st, pl = plan(fta_lib, base_args(**{**small, "num_kv_heads": 8, "cur_heads": 8, "q_len": 16}))     # GQA 4 x 16 = 64 rows
    assert st == 0 and pl.rows_per_wg == 64
    assert plan(fta_lib, base_args(**{**small, "num_kv_heads": 8, "cur_heads": 8, "q_len": 17}))[0] == -9   # 68 rows
    assert plan(fta_lib, base_args(**{**small, "head_dim": 256}))[0] == -9
    assert plan(fta_lib, base_args(**{**small, "dtype": _lib.FTA_F32}))[0] == -9
    assert plan(fta_lib, base_args(**{**small, "force_kernel": 4}))[0] == -9


def test_python_wrapper_rejects_cpu_tensors():
    """No CPU fallback: the product path refuses CPU tensors outright."""
    import torch
    from flash_tree_attn_amd import flash_decoding_attention
    q = torch.zeros(1, 2, 4, 64)
    kv = torch.zeros(1, 2, 16, 64)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        flash_decoding_attention(q, kv, kv, q, q, torch.zeros(4, 4), torch.tensor([16]))


# ---------------------------------------------------------------- the heuristic against measured split sweeps
def _regrets(fta_lib, fixture):
    """For every shape of a measured sweep (time of the whole call per forced split count, MI355X,
    bf16, head_dim 128, tests/golden/split_sweep_*.json): time at the plan's own split count over the
    best measured time. Counts between two measured ones are interpolated."""
    import json
    rows = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", fixture)))
    out = []
    for r in rows:
        st, pl = plan(fta_lib, base_args(bsz=r["bsz"], num_q_heads=r["hq"], num_kv_heads=r["hkv"], cur_heads=r["hkv"], q_len=r["L"],
                                         cache_len=r["T"], v_cache_len=r["T"]))
        assert st == 0
        pts = sorted((int(k), v) for k, v in r["us"].items())
        s = min(max(pl.num_splits, pts[0][0]), pts[-1][0])
        lo = max(p for p in pts if p[0] <= s)
        hi = min(p for p in pts if p[0] >= s)
        t = lo[1] if hi[0] == lo[0] else lo[1] + (hi[1] - lo[1]) * (s - lo[0]) / (hi[0] - lo[0])
        out.append(t / min(v for _, v in pts))
    return out


def test_split_heuristic_against_measured_sweeps(fta_lib):
    """A regression guard for changes of the cost model: on 112 shapes with full-length sequences the
    plan's split count must stay within 5 % of the best measured one on average (it is at 3.3 %), on 76
    shapes with log-uniform lengths within 6 % (it is at 3.9 %; lengths are not known to the plan)."""
    uniform = _regrets(fta_lib, "split_sweep_uniform.json")
    ragged = _regrets(fta_lib, "split_sweep_ragged.json")
    assert len(uniform) == 112 and len(ragged) == 76
    assert sum(uniform) / len(uniform) < 1.05 and max(uniform) < 1.35
    assert sum(ragged) / len(ragged) < 1.06 and max(ragged) < 1.40


def test_scratch_the_caller_brought_bounds_the_split_count(fta_lib):
    """A caller of the reference sizes mid_output from the batch's longest sequence
    (flash_tree_attn.py:274-281) and may pass no length bound: the plan, cut for the cache
    capacity, must then stay within those slots instead of asking for more."""
    big = dict(bsz=1, cache_len=131072, v_cache_len=131072)
    st, free = plan(fta_lib, base_args(**big))
    assert st == 0 and free.num_splits > 8
    a = base_args(**big)
    a.mid_o = a.mid_lse = 0x1000
    a.mid_splits = 8
    st, pl = plan(fta_lib, a)
    assert st == 0 and 1 < pl.num_splits <= 8 and pl.num_splits * pl.chunk >= 131072
    assert all(-(-b // c) <= pl.num_splits for b, c in zip(pl.len_bound, pl.chunk_by_len))
    a.mid_splits = 1
    st, pl = plan(fta_lib, a)
    assert st == 0 and pl.num_splits == 1
    a.force_splits = 4                      # a pinned count is the caller's word: it is planned, and fta_decode refuses the scratch
    st, pl = plan(fta_lib, a)
    assert st == 0 and pl.num_splits == 4


@pytest.mark.parametrize("kw", CASES)
def test_plan_with_its_own_scratch_filled_in_is_stable(fta_lib, kw):
    """A caller plans, allocates the slots the plan names, fills them in: the plan that fta_decode then makes from
    those arguments is the same plan. Fewer slots bound it."""
    a = base_args(**kw)
    st, first = plan(fta_lib, a)
    assert st == 0
    a.mid_o = a.mid_lse = 0x1000
    a.mid_splits = first.num_splits
    st, second = plan(fta_lib, a)
    assert st == 0 and bytes(second) == bytes(first)
    a.mid_splits = max(1, first.num_splits - 1)              # one slot short: the plan shrinks to fit, and stays there
    st, third = plan(fta_lib, a)
    assert st == 0 and third.num_splits <= a.mid_splits
    st, fourth = plan(fta_lib, a)
    assert bytes(fourth) == bytes(third)
