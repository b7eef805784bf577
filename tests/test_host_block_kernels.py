"""The library's host side and those of its kernels that use no matrix instructions or inline assembly
(stage 1 wavefront-shuffle, stage 2 merge, KV append), compiled for the HOST from the product sources
and run one host thread per GPU thread (tests/host_block/hip/hip_runtime.h stands in for the few HIP
names they use; hipLaunchKernel = run the grid workgroup by workgroup), through the same C entry points,
against the oracle.

This is a test of the SOURCE where no GPU is at hand, not a way to use the library: the host build is
made in a temporary directory by this test, nothing under flash_tree_attn_amd/ knows of it, and the
package still raises on CPU tensors. It covers argument marshalling, the plan (including the table of
cuts by length), the dispatch order, the kernels' addressing (strides, paged caches, packed masks,
lengths clamped to the cache), the chunk choice from the batch's longest sequence in both stages, and
the stage entry points used separately."""
import ctypes as C
import math
import os
import subprocess

import pytest
import torch

from flash_tree_attn_amd import _lib
from flash_tree_attn_amd import build as fta_build
from flash_tree_attn_amd.tree_mask import additive_mask_from_parents, pack_mask, random_tree_parents
from oracle.kv_append_oracle import append_accepted_kv_oracle
from oracle.tree_attn_oracle import stage2_merge_oracle, tree_attention_oracle
from test_zz_stage_entries_gpu import expected_partials, live_splits

HERE = os.path.dirname(os.path.abspath(__file__))
CLANG = os.path.join(os.path.dirname(fta_build.HIPCC), "..", "llvm", "bin", "clang++")
SOURCES = ["fta_host.cpp", "stage1_shuffle.hip", "stage2_merge.hip", "append_kv.hip"]
DTYPES = {torch.float32: _lib.FTA_F32, torch.float16: _lib.FTA_F16, torch.bfloat16: _lib.FTA_BF16}
TOL = {torch.float16: dict(atol=2e-3, rtol=1e-2), torch.bfloat16: dict(atol=2e-3, rtol=1e-2), torch.float32: dict(atol=2e-5, rtol=1e-4)}


@pytest.fixture(scope="module")
def host_lib(tmp_path_factory):
    if not os.path.exists(CLANG):
        pytest.skip("no host clang++")
    out = tmp_path_factory.mktemp("host_block")
    flags = ["-x", "c++", "-std=c++20", "-O1", "-fPIC", "-pthread", "-I", os.path.join(HERE, "host_block"), "-I", fta_build.INCLUDE, "-I", fta_build.CSRC]
    objs = []
    for src in [os.path.join(fta_build.CSRC, s) for s in SOURCES] + [os.path.join(HERE, "host_block", "mfma_stub.cpp")]:
        obj = str(out / (os.path.basename(src) + ".o"))
        subprocess.run([CLANG, *flags, "-c", src, "-o", obj], check=True, capture_output=True)
        objs.append(obj)
    path = str(out / "libfta_host_block.so")
    subprocess.run([CLANG, "-shared", "-pthread", *objs, "-o", path], check=True, capture_output=True)
    lib = C.CDLL(path)
    for name in ("fta_decode", "fta_decode_stage1", "fta_decode_stage2"):
        getattr(lib, name).argtypes = [C.POINTER(_lib.FtaArgs), C.c_void_p]
    lib.fta_plan.argtypes = [C.POINTER(_lib.FtaArgs), C.c_int, C.POINTER(_lib.FtaPlanOut)]
    lib.fta_append_kv.argtypes = [C.POINTER(_lib.FtaAppendArgs), C.c_void_p]
    assert lib.fta_abi_version() == _lib.ABI_VERSION
    # This copy of the library runs stage 2's shared walk where it applies (the product only does on request): the
    # knobs are read once, by the first plan, so the request only has to stand until then.
    os.environ["FTA_STAGE2_SHARED_WALK"] = "1"
    try:
        HostCall(lib, make(0, 1, 1, 1, 1, 32, 64, torch.float32, [64]))
    finally:
        del os.environ["FTA_STAGE2_SHARED_WALK"]
    return lib


def make(seed, bsz, hq, hkv, L, D, tmax, dtype, lens, cur_heads=None):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g).to(dtype)
    ch = hkv if cur_heads is None else cur_heads      # tree K/V per cache head (the default) or per query head
    x = dict(q=r(bsz, hq, L, D), k_cache=r(bsz, hkv, tmax, D), v_cache=r(bsz, hkv, tmax, D), current_k=r(bsz, ch, L, D), current_v=r(bsz, ch, L, D))
    x["mask"] = additive_mask_from_parents(random_tree_parents(L, g), device="cpu")
    x["kv_seq_len"] = torch.as_tensor(lens, dtype=torch.int64)
    x["kv_group_num"] = hq // hkv
    return x


class HostCall:
    """fta_args over CPU tensors (what flash_decoding.prepare does for device tensors), planned, with scratch."""

    def __init__(self, lib, x, splits=0, hint=0, mask=None, tables=None, pools=None, kernel=_lib.KERNEL_SHUFFLE, counters=False, block_size=64, len32=False):
        self.lib, self.x = lib, x
        q = x["q"]
        bsz, hq, L, D = q.shape
        k, v = pools if pools is not None else (x["k_cache"], x["v_cache"])
        mask = x["mask"] if mask is None else mask
        a = _lib.FtaArgs()
        self.out = torch.full((bsz, hq, L, D), float("nan"), dtype=q.dtype)
        lens = x["kv_seq_len"].int() if len32 else x["kv_seq_len"]
        self.keep = (q, k, v, x["current_k"], x["current_v"], mask, lens, tables)
        a.q, a.k_cache, a.v_cache, a.cur_k, a.cur_v = q.data_ptr(), k.data_ptr(), v.data_ptr(), x["current_k"].data_ptr(), x["current_v"].data_ptr()
        a.mask, a.kv_seq_len, a.out = mask.data_ptr(), lens.data_ptr(), self.out.data_ptr()
        a.bsz, a.num_q_heads, a.num_kv_heads, a.cur_heads, a.q_len, a.head_dim = bsz, hq, k.size(1), x["current_k"].size(1), L, D
        if tables is not None:
            a.page_size = k.size(2)
            a.cache_len = a.v_cache_len = tables.size(1) * k.size(2)
            a.block_table, a.block_table_stride = tables.data_ptr(), tables.stride(0)
        else:
            a.cache_len = a.v_cache_len = k.size(2)
        a.block_size, a.max_seq_len_hint, a.dtype, a.len_dtype = block_size, hint, DTYPES[q.dtype], _lib.FTA_I32 if len32 else _lib.FTA_I64
        a.force_splits, a.force_kernel, a.sm_scale = splits, kernel, 1.0 / math.sqrt(D)
        for name, t in (("q_stride", q), ("k_stride", k), ("v_stride", v), ("ck_stride", x["current_k"]), ("cv_stride", x["current_v"]), ("out_stride", self.out)):
            getattr(a, name)[:] = t.stride()[:3]
        if mask.dtype == torch.int64:
            a.mask_kind = _lib.MASK_PACKED_U64
            a.mask_stride[:] = [0, 0, mask.stride(-2)]
        else:
            a.mask_stride[:] = [0, 0, L]
        self.plan = _lib.FtaPlanOut()
        assert lib.fta_plan(C.byref(a), 256, C.byref(self.plan)) == 0
        S = self.plan.num_splits
        self.mid = torch.full((bsz, hq, S, L, D), float("nan"))
        self.lse = torch.full((bsz, hq, S, L), float("nan"))
        a.mid_o, a.mid_lse, a.mid_splits = self.mid.data_ptr(), self.lse.data_ptr(), S
        a.mid_o_stride[:] = self.mid.stride()[:4]
        a.mid_lse_stride[:] = self.lse.stride()[:3]
        if counters:      # zeroed once by the caller, left at zero by every call: stage 1 then merges in its own launch
            self.counters = torch.zeros(bsz * hq * 4, dtype=torch.int32)
            a.counters, a.counter_elems = self.counters.data_ptr(), self.counters.numel()
        self.args = a

    def run(self, entry="fta_decode"):
        status = getattr(self.lib, entry)(C.byref(self.args), None)
        assert status == 0, status
        return self.out


def oracle(x):
    return tree_attention_oracle(x["q"], x["k_cache"], x["v_cache"], x["current_k"], x["current_v"], x["mask"], x["kv_seq_len"], None, x["kv_group_num"])


@pytest.mark.parametrize("shape", [
    # bsz hq hkv L  D   tmax  dtype           lens            splits
    (2, 4, 2, 5, 64, 300, torch.float32, [300, 77], 2),
    (3, 4, 2, 3, 32, 2048, torch.bfloat16, [130, 0, 64], 0),          # a cache far larger than the sequences; an empty cache
    (1, 2, 2, 9, 64, 200, torch.float16, [200], 1),                   # one split: straight to `out`, no scratch
    (2, 2, 1, 4, 32, 256, torch.float32, [999, -3], 3),               # a length beyond the cache is clamped, a negative one is empty
    (70, 1, 1, 2, 32, 192, torch.float32, [(53 * i) % 193 for i in range(70)], 2),   # more than 64 sequences: the ordering pass through LDS, both stages
])
def test_whole_call_on_host_threads(host_lib, shape):
    bsz, hq, hkv, L, D, tmax, dtype, lens, splits = shape
    x = make(3, bsz, hq, hkv, L, D, tmax, dtype, lens)
    call = HostCall(host_lib, x, splits=splits)
    out = call.run()
    x_ref = dict(x, kv_seq_len=torch.tensor([min(max(t, 0), tmax) for t in lens]))
    torch.testing.assert_close(out.float(), oracle(x_ref), **TOL[dtype])
    if max(lens) * 4 < tmax and call.plan.num_splits > 1:
        assert call.plan.chunk_for(max(lens)) < call.plan.chunk       # ... cut by the lengths


def test_stage_entries_on_host_threads(host_lib):
    """fta_decode_stage1 alone fills exactly the slots the oracle predicts (chunks chosen on the 'device' from the
    batch's longest sequence), fta_decode_stage2 alone merges them."""
    lens, tmax = [700, 130, 0], 4096
    x = make(5, 3, 4, 2, 4, 32, tmax, torch.float32, lens)
    call = HostCall(host_lib, x, splits=4)
    S = call.plan.num_splits
    chunk = call.plan.chunk_for(max(lens))
    assert S == 4 and chunk < call.plan.chunk
    call.run("fta_decode_stage1")
    assert torch.isnan(call.out).all()
    for b, t_b in enumerate(lens):
        parts = expected_partials(x, b, chunk, S)
        assert len(parts) == live_splits(t_b, chunk, S)
        for s, (o_ref, lse_ref) in enumerate(parts):
            torch.testing.assert_close(call.lse[b, :, s], lse_ref, atol=1e-4, rtol=1e-5)
            torch.testing.assert_close(call.mid[b, :, s], o_ref, atol=2e-5, rtol=1e-4)
        for s in range(len(parts), S):
            assert torch.isnan(call.mid[b, :, s]).all() and torch.isnan(call.lse[b, :, s]).all()
    # stage 2 alone, on partials of the oracle's making (dead splits, a row without any live split, NaN in unused slots)
    g = torch.Generator().manual_seed(1)
    s_of = [live_splits(t, chunk, S) for t in lens]
    mid, lse = torch.randn(call.mid.shape, generator=g), torch.randn(call.lse.shape, generator=g) * 3
    dead = torch.rand(lse.shape, generator=g) < 0.2
    dead[0, 0, :, 0] = True
    lse[dead], mid[dead] = -math.inf, 0.0
    for b in range(3):
        mid[b, :, s_of[b]:], lse[b, :, s_of[b]:] = float("nan"), float("nan")
    call.mid.copy_(mid), call.lse.copy_(lse)
    call.run("fta_decode_stage2")
    for b in range(3):
        ref, _ = stage2_merge_oracle([mid[b, :, s].double() for s in range(s_of[b])], [lse[b, :, s].double() for s in range(s_of[b])])
        torch.testing.assert_close(call.out[b].double(), ref, atol=2e-5, rtol=1e-4)
    assert call.out[0, 0, 0].abs().max() == 0


@pytest.mark.parametrize("dtype,D,L", [(torch.float32, 32, 3), (torch.bfloat16, 64, 5)])
def test_stage2_with_the_walk_shared_by_four_threads(host_lib, dtype, D, L):
    """Many splits, few rows (one long sequence): four threads share each row's walk over the splits and add
    their partial sums in LDS. Rows that do not fill the last workgroup, dead splits, slots the sequence does
    not reach, a row with no live split."""
    bsz, hq, hkv, tmax, lens = 2, 2, 1, 2048, [2000, 700]
    x = make(9, bsz, hq, hkv, L, D, tmax, dtype, lens)
    call = HostCall(host_lib, x, splits=16)
    S = call.plan.num_splits
    assert S >= 8 and bsz * hq * L * (D // 4) // 64 < 16 * 256          # the launch takes the shared walk
    chunk = call.plan.chunk_for(max(lens))
    s_of = [live_splits(t, chunk, S) for t in lens]
    assert s_of[0] == S and 1 < s_of[1] < S
    whole = call.run().clone()                                          # stage 1 + stage 2 through it
    torch.testing.assert_close(whole.float(), oracle(x), **TOL[dtype])
    g = torch.Generator().manual_seed(6)
    mid, lse = torch.randn(call.mid.shape, generator=g), torch.randn(call.lse.shape, generator=g) * 3
    dead = torch.rand(lse.shape, generator=g) < 0.2
    dead[1, 1, :, L - 1] = True
    lse[dead], mid[dead] = -math.inf, 0.0
    for b in range(bsz):
        mid[b, :, s_of[b]:], lse[b, :, s_of[b]:] = float("nan"), float("nan")
    call.mid.copy_(mid), call.lse.copy_(lse)
    call.out.fill_(float("nan"))
    call.run("fta_decode_stage2")
    for b in range(bsz):
        ref, _ = stage2_merge_oracle([mid[b, :, s].double() for s in range(s_of[b])], [lse[b, :, s].double() for s in range(s_of[b])])
        torch.testing.assert_close(call.out[b].double(), ref, **TOL[dtype])
    assert call.out[1, 1, L - 1].abs().max() == 0


def test_paged_caches_and_packed_mask_on_host_threads(host_lib):
    lens, tmax, page = [150, 33], 192, 16
    x = make(7, 2, 4, 2, 6, 32, tmax, torch.float16, lens)
    per_seq = tmax // page
    g = torch.Generator().manual_seed(2)
    perm = torch.randperm(2 * per_seq + 3, generator=g)[: 2 * per_seq].view(2, per_seq)
    kp = torch.full((2 * per_seq + 3, 2, page, 32), float("nan"), dtype=torch.float16)
    vp = torch.full_like(kp, float("nan"))
    for b in range(2):
        for pg in range(per_seq):
            kp[perm[b, pg]] = x["k_cache"][b, :, pg * page:(pg + 1) * page]
            vp[perm[b, pg]] = x["v_cache"][b, :, pg * page:(pg + 1) * page]
    tables = torch.zeros(2, 64, dtype=torch.int32)             # a table four times wider than the sequences need
    tables[:, :per_seq] = perm.to(torch.int32)
    plain = HostCall(host_lib, x, splits=2, hint=tmax).run().clone()
    paged = HostCall(host_lib, x, splits=2, hint=tmax, tables=tables, pools=(kp, vp), mask=pack_mask(x["mask"])).run()
    torch.testing.assert_close(paged.float(), oracle(x), **TOL[torch.float16])
    assert torch.equal(paged, plain)                           # where rows come from changes nothing of what is computed


def test_kv_append_on_host_threads(host_lib):
    g = torch.Generator().manual_seed(4)
    bsz, hkv, L, D, tmax = 3, 2, 6, 32, 40
    r = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16)
    k, v, ck, cv = r(bsz, hkv, tmax, D), r(bsz, hkv, tmax, D), r(bsz, hkv, L, D), r(bsz, hkv, L, D)
    idx = torch.tensor([[0, 2, 5, 1], [3, 3, 9, 0], [1, 0, 2, 4]], dtype=torch.int32)     # 9: outside the tree, dropped but counted
    acc = torch.tensor([3, 4, 2])
    lens = torch.tensor([10, 38, 0])                                                      # the second runs into the end of its cache
    k_ref, v_ref, n_ref = append_accepted_kv_oracle(k, v, ck, cv, idx, acc, lens)
    a = _lib.FtaAppendArgs()
    a.k_cache, a.v_cache, a.cur_k, a.cur_v = k.data_ptr(), v.data_ptr(), ck.data_ptr(), cv.data_ptr()
    a.accept_idx, a.accept_len, a.kv_seq_len, a.kv_seq_len_out = idx.data_ptr(), acc.data_ptr(), lens.data_ptr(), lens.data_ptr()
    a.bsz, a.num_kv_heads, a.q_len, a.head_dim, a.cache_len, a.max_accept = bsz, hkv, L, D, tmax, idx.size(1)
    a.dtype, a.len_dtype = _lib.FTA_BF16, _lib.FTA_I64
    for name, t in (("k_stride", k), ("v_stride", v), ("ck_stride", ck), ("cv_stride", cv)):
        getattr(a, name)[:] = t.stride()[:3]
    a.accept_idx_stride = idx.stride(0)
    assert host_lib.fta_append_kv(C.byref(a), None) == 0
    assert torch.equal(k, k_ref) and torch.equal(v, v_ref) and torch.equal(lens, n_ref)


def test_the_package_still_refuses_cpu_tensors():
    from flash_tree_attn_amd import flash_decoding_attention
    x = make(1, 1, 2, 2, 4, 32, 16, torch.float32, [16])
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        flash_decoding_attention(x["q"], x["k_cache"], x["v_cache"], x["current_k"], x["current_v"], x["mask"], x["kv_seq_len"])
