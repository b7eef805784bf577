"""The device functions that decide which workgroup does what (csrc/fta_device.h: decode_work,
item_by_order, batch_chunk, block_max, chunk_for) compiled for the HOST and run as written, one host
thread per GPU thread (tests/host_block/: std::barrier for __syncthreads, an exchange array per wave
for __shfl_xor), for every workgroup id of a launch. Checked against the contract the kernels and the
plan share: every workgroup of both stages derives the same chunk from the batch's longest sequence (the
plan's table entry), every (sequence, split) that has keys is handed out exactly once per (unit, row
block), heaviest first, and nothing else is."""
import ctypes as C
import os
import random
import subprocess

import pytest

from flash_tree_attn_amd import _lib
from flash_tree_attn_amd import build as fta_build
from test_abi import base_args, plan

HERE = os.path.dirname(os.path.abspath(__file__))
CLANG = os.path.join(os.path.dirname(fta_build.HIPCC), "..", "llvm", "bin", "clang++")


@pytest.fixture(scope="module")
def runner(tmp_path_factory):
    if not os.path.exists(CLANG):
        pytest.skip("no host clang++")
    exe = str(tmp_path_factory.mktemp("host_block") / "dispatch_host")
    cmd = [CLANG, "-std=c++20", "-O1", "-pthread", "-I", os.path.join(HERE, "host_block"), "-I", fta_build.INCLUDE, "-I", fta_build.CSRC,
           os.path.join(HERE, "host_block", "dispatch_main.cpp"), "-o", exe]
    subprocess.run(cmd, check=True, capture_output=True)

    def run(cases):
        text = "\n".join(" ".join(str(x) for x in c) for c in cases) + "\n"
        r = subprocess.run([exe], input=text, capture_output=True, text=True, timeout=600)
        assert r.returncode == 0, (r.stdout[-500:], r.stderr[-500:])
        out, cur = [], None
        for line in r.stdout.splitlines():
            if line.startswith("case"):
                cur = []
                out.append(cur)
            else:
                cur.append([int(x) for x in line.split()])
        return out
    return run


def make_case(fta_lib, lens, threads, units=1, row_blocks=1, **kw):
    a = base_args(bsz=len(lens), **kw)
    st, pl = plan(fta_lib, a)
    assert st == 0
    line = [len(lens), pl.num_splits, units, row_blocks, a.cache_len, threads, *lens, *pl.len_bound, *pl.chunk_by_len]
    return line, pl, a.cache_len


def check(rows, lens, pl, cache_len, units, row_blocks):
    clamped = [min(max(t, 0), cache_len) for t in lens]
    chunk = pl.chunk_for(max(clamped))
    S = pl.num_splits
    live_splits = [min(S, max(1, -(-t // chunk))) for t in clamped]
    assert len(rows) == S * units * len(lens) * row_blocks
    seen = {}
    for wid, live, b, split, length, got_chunk, unit, rb, stage2_chunk in rows:
        assert got_chunk == chunk and stage2_chunk == chunk, (wid, got_chunk, stage2_chunk, chunk)
        assert 0 <= unit < units and 0 <= rb < row_blocks
        if not live:
            continue
        assert 0 <= b < len(lens) and length == clamped[b]
        if split >= live_splits[b]:
            continue                                   # the kernel returns at once: identity order hands out empty splits too
        key = (unit, rb, b, split)
        assert key not in seen, key                    # ... exactly once
        seen[key] = wid
    want = {(u, r, b, s) for u in range(units) for r in range(row_blocks) for b in range(len(lens)) for s in range(live_splits[b])}
    assert set(seen) == want
    if 1 < len(lens) <= 256:
        # heaviest first, per (unit, row block): every full chunk before any tail, tails by falling size
        for u in range(units):
            for r in range(row_blocks):
                mine = sorted((wid, b, s) for (uu, rr, b, s), wid in seen.items() if (uu, rr) == (u, r))
                work = [chunk if s < live_splits[b] - 1 else clamped[b] - (live_splits[b] - 1) * chunk for _, b, s in mine]
                full = [i for i, (_, b, s) in enumerate(mine) if s < live_splits[b] - 1]
                tails = [i for i, (_, b, s) in enumerate(mine) if s == live_splits[b] - 1]
                assert not full or not tails or max(full) < min(tails)
                assert [work[i] for i in tails] == sorted((work[i] for i in tails), reverse=True)


def test_dispatch_functions_as_compiled_cpp(fta_lib, runner):
    rng = random.Random(7)
    cases, meta = [], []

    def add(lens, threads, units=1, row_blocks=1, **kw):
        line, pl, cache_len = make_case(fta_lib, lens, threads, units, row_blocks, **kw)
        cases.append(line)
        meta.append((lens, pl, cache_len, units, row_blocks))

    add([8192] * 8, 512, units=2)                                                      # the headline batch: 8 waves per workgroup
    add([8192] * 8, 256, cache_len=131072, v_cache_len=131072)                         # ... in a cache sixteen times larger
    add([700, 300, 0, 699, 1], 256, cache_len=8192, v_cache_len=8192, force_splits=4, row_blocks=2)
    add([5000], 256, cache_len=65536, v_cache_len=65536)                               # one sequence: no ordering pass
    add([0], 512, cache_len=4096, v_cache_len=4096)
    add([4096, 9999, -5, 4095], 256, cache_len=4096, v_cache_len=4096, force_splits=3)  # clamped to the cache, negative = empty
    add([rng.randrange(0, 3000) for _ in range(19)], 64, cache_len=4096, v_cache_len=4096, force_splits=3)
    add([(37 * i) % 400 for i in range(257)], 64, cache_len=4096, v_cache_len=4096, force_splits=2)   # beyond the ordered limit
    add([rng.randrange(0, 33000) for _ in range(64)], 64, cache_len=32768, v_cache_len=32768, force_splits=2)    # the largest batch a wave orders by itself
    add([rng.randrange(0, 3000) for _ in range(65)], 128, cache_len=4096, v_cache_len=4096, force_splits=3)      # the smallest that goes through LDS
    add([100] * 6, 256, cache_len=4096, v_cache_len=4096, force_splits=4)                  # equally long, one live split each: the closed form without full chunks
    add([0] * 3, 512, cache_len=4096, v_cache_len=4096, force_splits=2)                    # nothing cached anywhere
    add([4096] * 5, 512, cache_len=4096, v_cache_len=4096, force_splits=4, units=3)        # equally long at the cap, a grid that is no multiple of 8
    _, table = plan(fta_lib, base_args(bsz=2, cache_len=32768, v_cache_len=32768))
    for entry, delta in ((6, -1), (9, 0), (12, 1)):                                    # lengths on and next to a bound of the table
        add([min(table.len_bound[entry] + delta, 32768), 100], 256, cache_len=32768, v_cache_len=32768)
    results = runner(cases)
    assert len(results) == len(cases)
    for rows, (lens, pl, cache_len, units, row_blocks) in zip(results, meta):
        check(rows, lens, pl, cache_len, units, row_blocks)
    # the capacity case really is cut by the lengths: the same chunk as the exact-size cache
    assert results[1][0][5] == results[0][0][5] == 2112
