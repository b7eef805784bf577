"""The MFMA stage-1 kernel's SOURCE on host threads, against the oracle.

tests/host_block/stage1_mfma_host.cpp compiles flash_tree_attn_amd/csrc/stage1_mfma.hip for the host with
the instruction wrappers of csrc/gfx950_ops.h replaced by arithmetic stand-ins (gfx950_ops_host.h: the
32x32x16 matrix product in its lane layout, the transposing LDS read, the direct global->LDS load with
bounds-checked LDS addresses, ...), one host thread per GPU thread, and runs it through the library's own C
entry points. All three compiled loop variants run: 4 waves x 32 rows with rings of 2 (also head_dim 256),
and 8 waves x 32 rows software-pipelined over whole tiles. (The 64-row-wave kernel, whose loop is assembly, runs
in tests/test_host_block_wide.py with its statements interpreted.)

What this pins without a GPU: the work decomposition and addressing of the kernel (units, row blocks, splits,
chunk by the batch's longest sequence, strides, paged lookups, ragged and tree tiles, the ring slots), its
lane layouts, the online softmax with the deferred rescale, the compensated masked tiles, the epilogue, and
the merge inside the launch with counters. Time is modelled at its extremes only: global->LDS loads land when
issued, or (test_hand_counted_waits_...) as late as the kernel's vmcnt waits allow; LDS operand reads stay in
flight until the lgkmcnt wait that names their registers, and every such wait must land exactly the reads it
names (the stand-in aborts otherwise). Not shown: the last bits of the hardware's accumulation order, and speed.

TEST INFRASTRUCTURE ONLY: nothing under flash_tree_attn_amd/ knows of this build."""
import ctypes as C
import math
import os
import subprocess

import pytest
import torch

from flash_tree_attn_amd import _lib
from flash_tree_attn_amd import build as fta_build
from flash_tree_attn_amd.tree_mask import pack_mask
from oracle.tree_attn_oracle import tree_attention_oracle
from test_host_block_kernels import CLANG, HERE, SOURCES, TOL, HostCall, make, oracle
from test_zz_stage_entries_gpu import expected_partials, live_splits

MFMA = _lib.KERNEL_MFMA


@pytest.fixture(scope="module")
def host_lib(tmp_path_factory):
    if not os.path.exists(CLANG):
        pytest.skip("no host clang++")
    out = tmp_path_factory.mktemp("host_block_mfma")
    flags = ["-x", "c++", "-std=c++20", "-O1", "-fPIC", "-pthread", "-I", os.path.join(HERE, "host_block"), "-I", fta_build.INCLUDE, "-I", fta_build.CSRC]
    srcs = [os.path.join(fta_build.CSRC, s) for s in SOURCES] + [os.path.join(HERE, "host_block", "stage1_mfma_host.cpp")]
    procs, objs = [], []
    for src in srcs:
        obj = str(out / (os.path.basename(src) + ".o"))
        level = ["-O0"] if src.endswith("stage1_mfma_host.cpp") else []     # twenty instantiations: half a minute to optimise
        procs.append(subprocess.Popen([CLANG, *flags, *level, "-c", src, "-o", obj], stdout=subprocess.PIPE, stderr=subprocess.STDOUT))
        objs.append(obj)
    for proc in procs:
        log = proc.communicate()[0]
        assert proc.returncode == 0, log.decode()[-3000:]
    path = str(out / "libfta_host_mfma.so")
    subprocess.run([CLANG, "-shared", "-pthread", *objs, "-o", path], check=True, capture_output=True)
    lib = C.CDLL(path)
    for name in ("fta_decode", "fta_decode_stage1", "fta_decode_stage2"):
        getattr(lib, name).argtypes = [C.POINTER(_lib.FtaArgs), C.c_void_p]
    lib.fta_plan.argtypes = [C.POINTER(_lib.FtaArgs), C.c_int, C.POINTER(_lib.FtaPlanOut)]
    lib.host_block_loads_land_late.argtypes = [C.c_int]
    assert lib.fta_abi_version() == _lib.ABI_VERSION
    return lib


@pytest.fixture(autouse=True)
def loads_land_when_issued(host_lib):
    host_lib.host_block_loads_land_late(0)
    yield
    host_lib.host_block_loads_land_late(0)


def clamped(x, lens, tmax):
    return dict(x, kv_seq_len=torch.tensor([min(max(t, 0), tmax) for t in lens]))


@pytest.mark.parametrize("shape", [
    # bsz hq hkv L  D    tmax dtype           lens         splits rows_per_wg
    (2, 4, 2, 5, 64, 300, torch.bfloat16, [200, 77], 2, 128),        # 4 waves, rings of 2; ragged last tiles; one wave holds rows
    (1, 8, 1, 20, 128, 512, torch.float16, [470], 1, 256),           # 8 waves pipelined, 8 tiles through rings of 3 and 5, 160 rows, straight to `out`
    (2, 4, 1, 70, 64, 256, torch.bfloat16, [256, 64], 2, 256),       # 280 rows: two row blocks, the second nearly empty; two tree tiles; a split of whole tiles only
    (1, 2, 2, 3, 256, 256, torch.float16, [100], 1, 128),            # head_dim 256
    (3, 4, 2, 7, 128, 320, torch.bfloat16, [0, 999, -5], 3, 128),    # an empty cache, a length beyond the cache (clamped), a negative one (empty)
    (2, 2, 2, 33, 128, 192, torch.float16, [65, 1], 2, 128),         # 33 rows: the second wave holds one row; one key in the cache
])
def test_whole_call(host_lib, shape):
    bsz, hq, hkv, L, D, tmax, dtype, lens, splits, rows_per_wg = shape
    x = make(11, bsz, hq, hkv, L, D, tmax, dtype, lens)
    call = HostCall(host_lib, x, splits=splits, kernel=MFMA)
    assert call.plan.kernel == MFMA and call.plan.rows_per_wg == rows_per_wg and not call.plan.mfma_loop
    host_lib.host_block_loads_land_late(bsz % 2)          # the odd batches with loads that land as late as the waits allow
    out = call.run()
    assert torch.isfinite(out).all()
    torch.testing.assert_close(out.float(), oracle(clamped(x, lens, tmax)), **TOL[dtype])


@pytest.mark.parametrize("dtype,D", [(torch.bfloat16, 128), (torch.float16, 64)])
def test_stage1_alone_fills_the_slots_the_oracle_predicts(host_lib, dtype, D):
    """A cache far larger than the sequences: the kernel itself takes the chunk from the batch's longest sequence.
    Every live slot against the oracle's partial of that split (the owner of a sequence's end also holds the tree
    block); slots that a sequence does not reach stay untouched."""
    lens, tmax, S = [700, 130, 0], 8192, 4
    x = make(5, 3, 4, 2, 6, D, tmax, dtype, lens)
    call = HostCall(host_lib, x, splits=S, kernel=MFMA)
    assert call.plan.num_splits == S
    chunk = call.plan.chunk_for(max(lens))
    assert chunk < call.plan.chunk and chunk % 64 == 0
    call.run("fta_decode_stage1")
    assert torch.isnan(call.out).all()
    for b, t_b in enumerate(lens):
        parts = expected_partials(x, b, chunk, S)
        assert len(parts) == live_splits(t_b, chunk, S)
        for s, (o_ref, lse_ref) in enumerate(parts):
            torch.testing.assert_close(call.lse[b, :, s], lse_ref, atol=2e-3, rtol=1e-3)
            torch.testing.assert_close(call.mid[b, :, s], o_ref, **TOL[dtype])
        for s in range(len(parts), S):
            assert torch.isnan(call.mid[b, :, s]).all() and torch.isnan(call.lse[b, :, s]).all()
    out = call.run("fta_decode_stage2")
    torch.testing.assert_close(out.float(), oracle(x), **TOL[dtype])


@pytest.mark.parametrize("rows_per_wg", [128, 256])
def test_merge_inside_the_launch(host_lib, rows_per_wg):
    """With counters the workgroup that finishes a (sequence, unit, row block) last merges the partials itself and
    leaves the counters at zero; the result is that of the two-launch path bit for bit."""
    hq, L = (4, 6) if rows_per_wg == 128 else (8, 20)
    lens, tmax = [300, 64, 0], 320
    x = make(13, 3, hq, 1, L, 128, tmax, torch.bfloat16, lens)
    two = HostCall(host_lib, x, splits=3, kernel=MFMA)
    assert two.plan.rows_per_wg == rows_per_wg
    ref = two.run().clone()
    one = HostCall(host_lib, x, splits=3, kernel=MFMA, counters=True)
    assert one.plan.counter_elems > 0
    out = one.run()                             # fta_decode launches stage 1 only
    assert torch.isnan(one.mid[2]).all()        # (the empty sequence has one split and goes straight to `out`)
    torch.testing.assert_close(out.float(), oracle(x), **TOL[torch.bfloat16])
    assert torch.equal(out, ref)
    assert (one.counters == 0).all()
    out.fill_(float("nan"))
    assert torch.equal(one.run(), ref)          # and again, on the counters it left


def test_paged_caches_and_packed_mask(host_lib):
    lens, tmax, page = [300, 33], 384, 16
    x = make(7, 2, 4, 2, 6, 128, tmax, torch.float16, lens)
    per_seq = tmax // page
    g = torch.Generator().manual_seed(2)
    perm = torch.randperm(2 * per_seq + 3, generator=g)[: 2 * per_seq].view(2, per_seq)
    kp = torch.full((2 * per_seq + 3, 2, page, 128), float("nan"), dtype=torch.float16)
    vp = torch.full_like(kp, float("nan"))
    for b in range(2):
        for pg in range(per_seq):
            kp[perm[b, pg]] = x["k_cache"][b, :, pg * page:(pg + 1) * page]
            vp[perm[b, pg]] = x["v_cache"][b, :, pg * page:(pg + 1) * page]
    tables = torch.zeros(2, 96, dtype=torch.int32)             # a table four times wider than the sequences need
    tables[:, :per_seq] = perm.to(torch.int32)
    plain = HostCall(host_lib, x, splits=2, hint=tmax, kernel=MFMA).run().clone()
    paged = HostCall(host_lib, x, splits=2, hint=tmax, tables=tables, pools=(kp, vp), mask=pack_mask(x["mask"]), kernel=MFMA).run()
    torch.testing.assert_close(paged.float(), oracle(x), **TOL[torch.float16])
    assert torch.equal(paged, plain)                           # where rows come from changes nothing of what is computed


def test_paged_pipelined(host_lib):
    """The 8-wave loop fetches the next tile's pages ahead of its barrier: pages of 64 keys (one per tile) and of
    16 keys (the smallest the library takes), in a pool whose unused pages hold NaN."""
    lens, tmax = [448], 512
    x = make(17, 1, 8, 1, 20, 128, tmax, torch.bfloat16, lens)
    ref = oracle(x)
    for page in (64, 16):
        n = tmax // page
        perm = torch.randperm(n + 5, generator=torch.Generator().manual_seed(page))[:n]
        kp = torch.full((n + 5, 1, page, 128), float("nan"), dtype=torch.bfloat16)
        vp = torch.full_like(kp, float("nan"))
        for pg in range(n):
            kp[perm[pg]] = x["k_cache"][0, :, pg * page:(pg + 1) * page]
            vp[perm[pg]] = x["v_cache"][0, :, pg * page:(pg + 1) * page]
        tables = perm.to(torch.int32).view(1, n).contiguous()
        call = HostCall(host_lib, x, splits=2, hint=tmax, tables=tables, pools=(kp, vp), kernel=MFMA)
        assert call.plan.rows_per_wg == 256
        torch.testing.assert_close(call.run().float(), ref, **TOL[torch.bfloat16])


def test_peaked_logits_take_the_rescale_path(host_lib):
    """Scores that grow along the sequence raise the running maximum in nearly every tile (the rescale of O that
    is deferred behind the next P.V product), and a mask row that admits only the token itself."""
    lens, tmax, D = [384], 384, 128
    x = make(19, 1, 8, 1, 20, D, tmax, torch.float16, lens)
    ramp = torch.linspace(0.2, 3.0, tmax).view(1, 1, tmax, 1)
    x["k_cache"] = (x["q"][:, :1, :1, :].float() * ramp).to(torch.float16)       # keys ever more aligned with the first query row
    call = HostCall(host_lib, x, splits=1, kernel=MFMA)
    assert call.plan.rows_per_wg == 256
    torch.testing.assert_close(call.run().float(), oracle(x), **TOL[torch.float16])


# ---- key halves: units of at most 64 rows, two waves per 32-row block ---------------------------------------------
SPLIT_KEYS = _lib.KERNEL_MFMA_SPLIT_KEYS


@pytest.mark.parametrize("shape", [
    # bsz hq hkv L  D    tmax dtype           lens           splits
    (2, 4, 2, 5, 64, 300, torch.bfloat16, [200, 77], 2),          # 10 rows: one pair of waves computes; ragged last tiles
    (3, 4, 4, 26, 128, 320, torch.float16, [300, 64, 0], 3),      # 26 rows per head (MHA); an empty cache; a whole-tile split
    (2, 4, 1, 16, 128, 256, torch.bfloat16, [256, 31], 2),        # 64 rows: both pairs compute; fewer keys than half a tile
    (2, 8, 2, 1, 128, 256, torch.bfloat16, [256, 100], 2),        # plain decode, 4 rows
    (1, 2, 1, 20, 64, 192, torch.float16, [33], 1),               # 40 rows: the second pair holds 8; one key in the upper half of a tile; straight to `out`
    (2, 2, 2, 40, 64, 128, torch.bfloat16, [999, -5], 2),         # a tree whose second half tile is partly filled; clamped and negative lengths
])
def test_key_halves_whole_call(host_lib, shape):
    bsz, hq, hkv, L, D, tmax, dtype, lens, splits = shape
    x = make(23, bsz, hq, hkv, L, D, tmax, dtype, lens)
    call = HostCall(host_lib, x, splits=splits, kernel=SPLIT_KEYS)
    assert call.plan.kernel == MFMA and call.plan.rows_per_wg == 64 and call.plan.mfma_loop == 2 and call.plan.row_blocks == 1
    out = call.run()
    assert torch.isfinite(out).all()
    torch.testing.assert_close(out.float(), oracle(clamped(x, lens, tmax)), **TOL[dtype])


def test_key_halves_partials_counters_and_pages(host_lib):
    """The partial of every live split (the two waves' states merged before the epilogue), then the same call with the
    merge inside the launch, then on paged caches with the packed mask (bit-equal to the contiguous call)."""
    lens, tmax, S, page = [300, 130, 0], 1024, 4, 16
    x = make(29, 3, 4, 2, 12, 128, tmax, torch.bfloat16, lens)
    call = HostCall(host_lib, x, splits=S, kernel=SPLIT_KEYS)
    chunk = call.plan.chunk_for(max(lens))
    assert call.plan.num_splits == S and chunk < call.plan.chunk
    call.run("fta_decode_stage1")
    for b, t_b in enumerate(lens):
        parts = expected_partials(x, b, chunk, S)
        for s, (o_ref, lse_ref) in enumerate(parts):
            torch.testing.assert_close(call.lse[b, :, s], lse_ref, atol=2e-3, rtol=1e-3)
            torch.testing.assert_close(call.mid[b, :, s], o_ref, **TOL[torch.bfloat16])
        for s in range(len(parts), S):
            assert torch.isnan(call.mid[b, :, s]).all() and torch.isnan(call.lse[b, :, s]).all()
    ref = call.run("fta_decode_stage2").clone()
    torch.testing.assert_close(ref.float(), oracle(x), **TOL[torch.bfloat16])
    fused = HostCall(host_lib, x, splits=S, kernel=SPLIT_KEYS, counters=True)
    out = fused.run()                                          # sums the four partials in another order: equal to the last bit or two
    torch.testing.assert_close(out.float(), ref.float(), atol=1e-3, rtol=8e-3)
    assert (out == ref).float().mean() > 0.98 and (fused.counters == 0).all()
    per_seq = 320 // page                                      # pages for the first 320 positions only: nothing beyond is read
    perm = torch.randperm(3 * per_seq, generator=torch.Generator().manual_seed(3)).view(3, per_seq)
    kp = torch.full((3 * per_seq, 2, page, 128), float("nan"), dtype=torch.bfloat16)
    vp = torch.full_like(kp, float("nan"))
    for b in range(3):
        for pg in range(per_seq):
            kp[perm[b, pg]] = x["k_cache"][b, :, pg * page:(pg + 1) * page]
            vp[perm[b, pg]] = x["v_cache"][b, :, pg * page:(pg + 1) * page]
    tables = torch.zeros(3, tmax // page, dtype=torch.int32)
    tables[:, :per_seq] = perm.to(torch.int32)
    paged = HostCall(host_lib, x, splits=S, tables=tables, pools=(kp, vp), mask=pack_mask(x["mask"]), kernel=SPLIT_KEYS)
    assert paged.plan.chunk_for(max(lens)) == chunk
    assert torch.equal(paged.run(), ref)


def test_key_halves_are_refused_where_they_do_not_exist(host_lib):
    for hq, L, D in ((4, 20, 128), (2, 3, 256)):               # 80 rows per unit; head_dim 256
        x = make(1, 1, hq, 1, L, D, 64, torch.float16, [64])
        with pytest.raises(AssertionError):
            HostCall(host_lib, x, kernel=SPLIT_KEYS)


@pytest.mark.parametrize("shape", [
    # bsz hq hkv L  D    tmax dtype           lens         splits kernel      rows_per_wg
    (1, 8, 1, 20, 128, 512, torch.float16, [470], 1, MFMA, 256),                 # the 8-wave pipeline: K 3 tiles ahead in 4 stages, V ring 5, waits of 1 .. 4 tiles
    (1, 8, 1, 20, 128, 256, torch.bfloat16, [70], 1, MFMA, 256),                 # the same with fewer tiles than its rings hold
    (2, 4, 4, 26, 128, 320, torch.float16, [300, 64], 3, SPLIT_KEYS, 64),        # key halves
])
def test_hand_counted_waits_hold_when_loads_land_as_late_as_they_may(host_lib, shape):
    """The kernel waits for its tile loads by count (s_waitcnt vmcnt(N) with N from the ring's state). Here a
    load lands only when such a wait forces it to (not even __syncthreads counts): a count that allows one load too many
    leaves NaN patterns where the products read. (Checked by hand: with the wait for "one younger tile" allowing
    two, this fails and the default mode does not.) Contiguous, then paged: the table lookups sit between the requests
    and the waits. test_whole_call runs its odd batches in this mode as well (rings of 2, head_dim 256)."""
    bsz, hq, hkv, L, D, tmax, dtype, lens, splits, kernel, rows_per_wg = shape
    x = make(31, bsz, hq, hkv, L, D, tmax, dtype, lens)
    call = HostCall(host_lib, x, splits=splits, kernel=kernel)
    assert call.plan.rows_per_wg == rows_per_wg
    host_lib.host_block_loads_land_late(1)
    out = call.run()
    torch.testing.assert_close(out.float(), oracle(x), **TOL[dtype])
    if True:
        page, per_seq = 64, tmax // 64
        perm = torch.randperm(bsz * per_seq, generator=torch.Generator().manual_seed(5)).view(bsz, per_seq)
        kp = torch.empty((bsz * per_seq, hkv, page, D), dtype=dtype)
        vp = torch.empty_like(kp)
        for b in range(bsz):
            for pg in range(per_seq):
                kp[perm[b, pg]] = x["k_cache"][b, :, pg * page:(pg + 1) * page]
                vp[perm[b, pg]] = x["v_cache"][b, :, pg * page:(pg + 1) * page]
        paged = HostCall(host_lib, x, splits=splits, hint=tmax, tables=perm.to(torch.int32).contiguous(), pools=(kp, vp), kernel=kernel)
        torch.testing.assert_close(paged.run().float(), oracle(x), **TOL[dtype])
