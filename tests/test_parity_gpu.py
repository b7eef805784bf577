"""GPU parity: the HIP path (through the C ABI) against the oracle on the same seeded
inputs. Tolerance for fp16/bf16 is the one the target states: atol 2e-3, rtol 1e-2
against the fp32 oracle; fp32 inputs are held to atol 2e-5, rtol 1e-4."""
import math
import os

import numpy as np
import pytest
import torch

from flash_tree_attn_amd import FtaAssertionError, _lib, flash_decoding_attention
from flash_tree_attn_amd.synthetic import CONFIGS, make_inputs
from flash_tree_attn_amd.tree_mask import additive_mask_from_parents, chain_parents, random_tree_parents
from oracle.tree_attn_oracle import tree_attention_oracle, two_stage_oracle

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TOL = {torch.float16: dict(atol=2e-3, rtol=1e-2), torch.bfloat16: dict(atol=2e-3, rtol=1e-2),
       torch.float32: dict(atol=2e-5, rtol=1e-4)}
DEV = "cuda"


@pytest.fixture(scope="module", autouse=True)
def _library_is_loaded():
    _lib.load()  # raises if libfta.so is missing: no silent fallback


def make(seed, bsz, hq, hkv, L, D, tmax, dtype, lens=None, cur_heads=None, tree="random"):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g).to(dtype).to(DEV)
    ch = hkv if cur_heads is None else cur_heads
    x = dict(q=r(bsz, hq, L, D), k_cache=r(bsz, hkv, tmax, D), v_cache=r(bsz, hkv, tmax, D),
             current_k=r(bsz, ch, L, D), current_v=r(bsz, ch, L, D))
    parents = chain_parents(L) if tree == "chain" else random_tree_parents(L, g)
    x["mask"] = additive_mask_from_parents(parents, device=DEV)
    if lens is None:
        lens = torch.randint(0, tmax + 1, (bsz,), generator=g)
    x["kv_seq_len"] = torch.as_tensor(lens, dtype=torch.int64).to(DEV)
    x["kv_group_num"] = hq // hkv
    return x


def oracle(x, sm_scale=None, dtype=torch.float32):
    return tree_attention_oracle(x["q"], x["k_cache"], x["v_cache"], x["current_k"], x["current_v"], x["mask"],
                                 x["kv_seq_len"], sm_scale, x["kv_group_num"], dtype=dtype)


def run(x, block_size=64, sm_scale=None, **kw):
    return flash_decoding_attention(x["q"], x["k_cache"], x["v_cache"], x["current_k"], x["current_v"], x["mask"],
                                    x["kv_seq_len"], block_size, sm_scale=sm_scale, kv_group_num=x["kv_group_num"], **kw)


def check(out, ref, dtype):
    assert out.dtype == dtype
    assert torch.isfinite(out).all()
    torch.testing.assert_close(out.float(), ref.float(), **TOL[dtype])


# ---------------------------------------------------------------- fixtures
def test_golden_cfg1_fp32_chain():
    """Workload cfg1_plumbing_fp32 (bsz 1, 8 MHA heads, D 64, L 4, chain mask, T 256, fp32)."""
    x = make_inputs(CONFIGS["cfg1_plumbing_fp32"], seed=0, device=DEV)
    out = run(x)
    check(out, oracle(x), torch.float32)
    data = np.load(os.path.join(GOLDEN, "cfg1_seed0.npz"))
    import hashlib
    h = hashlib.sha256()
    for t in (x["q"], x["k_cache"], x["v_cache"], x["current_k"], x["current_v"]):
        h.update(t.cpu().contiguous().numpy().tobytes())
    if h.hexdigest() == str(data["input_digest"]):
        torch.testing.assert_close(out.cpu().double(), torch.from_numpy(data["out"]), atol=2e-5, rtol=1e-4)
    for splits in (1, 2, 4):
        check(run(x, _force_splits=splits), oracle(x), torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_golden_tiny_gqa_ragged(dtype):
    d = np.load(os.path.join(GOLDEN, "tiny_gqa_ragged.npz"))
    t = lambda n: torch.from_numpy(d[n]).to(DEV)
    c = lambda n: t(n).to(dtype)
    out = flash_decoding_attention(c("q"), c("k"), c("v"), c("ck"), c("cv"), t("mask"), t("lens"), 16, kv_group_num=2)
    if dtype != torch.bfloat16:  # stored values are fp16-representable
        check(out, t("out"), dtype)
    else:
        ref = tree_attention_oracle(c("q"), c("k"), c("v"), c("ck"), c("cv"), t("mask"), t("lens"), None, 2)
        check(out, ref, dtype)


# ---------------------------------------------------------------- workloads cfg2 .. cfg5 at full size
def test_cfg2_medusa_fp16_ragged():
    cfg = CONFIGS["cfg2_medusa_7b_fp16"]
    x = make_inputs(cfg, seed=0, device=DEV)
    check(run(x), oracle(x), cfg.dtype)


def test_cfg3_gqa_bf16_full_size():
    cfg = CONFIGS["cfg3_gqa_8b_bf16"]
    x = make_inputs(cfg, seed=0, device=DEV, gen_device=DEV)
    ref = oracle(x)
    check(run(x), ref, cfg.dtype)
    for splits in (1, 3, 16):
        check(run(x, _force_splits=splits), ref, cfg.dtype)


def test_cfg4_long_context_bf16_full_size():
    cfg = CONFIGS["cfg4_long_ctx_bf16"]
    x = make_inputs(cfg, seed=0, device=DEV, gen_device=DEV)
    check(run(x), oracle(x), cfg.dtype)


def test_cfg5_ragged_70b_bf16_full_size():
    cfg = CONFIGS["cfg5_ragged_70b_bf16"]
    x = make_inputs(cfg, seed=0, device=DEV, gen_device=DEV)
    out = run(x)
    check(out, oracle(x), cfg.dtype)
    # the hint only shrinks the grid
    out_hint = run(x, max_seq_len_in_batch=int(x["kv_seq_len"].max()))
    check(out_hint, out, cfg.dtype)


def test_reference_test_shape_fp16():
    """The reference's single test (flash_tree_attn.py:416-440): Z 32, H 32, N_CTX 4096,
    D 128, q_len 128, fp16, block 128, a {1,-inf} mask, tree K/V with num_heads heads,
    checked there with atol 1e-2."""
    g = torch.Generator(device=DEV).manual_seed(20)
    n = lambda *s, std=1.0: (torch.randn(*s, generator=g, device=DEV) * std).half()
    q, k, v = n(32, 32, 128, 128, std=0.5), n(32, 32, 4096, 128, std=0.5), n(32, 32, 4096, 128, std=0.5)
    ck, cv = n(32, 32, 128, 128), n(32, 32, 128, 128)
    allowed = torch.rand(128, 128, generator=g, device=DEV) < 0.5
    allowed |= torch.eye(128, dtype=torch.bool, device=DEV)
    mask = torch.where(allowed, torch.ones((), device=DEV), torch.full((), -math.inf, device=DEV))
    lens = torch.full((32,), 4096, dtype=torch.int64, device=DEV)
    out = flash_decoding_attention(q, k, v, ck, cv, mask, lens, 128)
    ref = tree_attention_oracle(q, k, v, ck, cv, mask, lens, None, 1)
    check(out, ref, torch.float16)


# ---------------------------------------------------------------- shape / dtype sweep
SWEEP = [
    # bsz hq hkv  L   D   tmax dtype            lens
    (2, 4, 4, 1, 64, 100, torch.float16, [100, 33]),          # plain decode, one row
    (2, 8, 2, 3, 128, 300, torch.bfloat16, [300, 1]),         # rows 12 < 16: MFMA kernel, rows past the unit's end blanked
    (1, 8, 2, 4, 128, 200, torch.bfloat16, [200]),            # rows 16 -> MFMA
    (3, 6, 3, 16, 64, 257, torch.float16, [0, 64, 257]),      # T=0, T multiple, T odd
    (2, 4, 1, 26, 128, 513, torch.float16, [513, 129]),       # rows 104, padded block
    (2, 16, 2, 40, 128, 700, torch.bfloat16, [700, 699]),     # rows 320 -> two row blocks
    (1, 2, 2, 128, 64, 90, torch.bfloat16, [90]),             # L 128: two tree tiles
    (1, 2, 1, 130, 128, 10, torch.float16, [10]),             # rows 260, ragged tree tiles
    (2, 4, 2, 8, 32, 150, torch.float16, [150, 20]),          # D 32 -> shuffle
    (1, 4, 2, 8, 256, 150, torch.bfloat16, [131]),            # D 256: MFMA kernel, 128-row workgroups
    (2, 4, 2, 20, 256, 80, torch.float32, [80, 7]),           # fp32, D 256
    (1, 2, 2, 33, 32, 64, torch.float32, [64]),               # fp32, D 32, 3 row blocks of 16
]


@pytest.mark.parametrize("case", SWEEP, ids=lambda c: f"b{c[0]}h{c[1]}kv{c[2]}L{c[3]}D{c[4]}T{c[5]}{str(c[6])[6:]}")
def test_sweep(case):
    bsz, hq, hkv, L, D, tmax, dtype, lens = case
    x = make(7, bsz, hq, hkv, L, D, tmax, dtype, lens)
    ref = oracle(x)
    check(run(x), ref, dtype)
    check(run(x, block_size=16, _force_splits=3), ref, dtype)
    if dtype != torch.float32:
        # both stage-1 kernels agree with the oracle on the same inputs
        check(run(x, _force_kernel=_lib.KERNEL_SHUFFLE), ref, dtype)


@pytest.mark.parametrize("splits", [1, 2, 5, 13])
def test_split_count_independence(splits):
    x = make(11, 3, 8, 2, 24, 128, 1000, torch.bfloat16, [1000, 517, 64])
    check(run(x, _force_splits=splits), oracle(x), torch.bfloat16)


# ---------------------------------------------------------------- argument contract
def test_mask_forms():
    x = make(13, 2, 4, 2, 18, 128, 120, torch.float16, [120, 50])
    ref = oracle(x)
    base = x["mask"]
    for m in (base, base[None, None], base[None, None].expand(2, 4, 18, 18).contiguous(),
              base[None, None].expand(2, 1, 18, 18).contiguous(), torch.isfinite(base), base.half()):
        x["mask"] = m
        check(run(x), ref, torch.float16)
    # per-batch, per-head masks really are indexed per batch and head
    g = torch.Generator().manual_seed(5)
    per = torch.stack([torch.stack([additive_mask_from_parents(random_tree_parents(18, g)) for _ in range(4)])
                       for _ in range(2)]).to(DEV)
    x["mask"] = per
    check(run(x), oracle(x), torch.float16)
    # additive semantics: {1,-inf} like the reference's generator (flash_tree_attn.py:403-414)
    x["mask"] = torch.where(torch.isfinite(base), torch.ones_like(base), base)
    check(run(x), oracle(x), torch.float16)
    # arbitrary finite bias
    x["mask"] = torch.randn(18, 18, generator=g).to(DEV)
    check(run(x), oracle(x), torch.float16)


@pytest.mark.parametrize("L,hq,hkv,D,dtype", [(64, 32, 8, 128, torch.bfloat16), (26, 4, 4, 128, torch.float16),
                                              (130, 2, 1, 128, torch.float16), (5, 4, 2, 64, torch.float32),
                                              (3, 8, 2, 128, torch.bfloat16)])
def test_packed_mask_equals_additive_mask(L, hq, hkv, D, dtype):
    """A 0 / -inf additive mask and its packed bit form (one uint64 word per row and 64
    tree keys) must give identical results, in every broadcast form and in both kernels."""
    from flash_tree_attn_amd.tree_mask import pack_mask
    bsz = 3
    x = make(71, bsz, hq, hkv, L, D, 300, dtype, [300, 17, 128])
    g = torch.Generator().manual_seed(5)
    allowed = (torch.rand(bsz, hq, L, L, generator=g) < 0.5) | torch.eye(L, dtype=torch.bool)
    for view in (allowed[0, 0], allowed[:, :1], allowed):
        add = torch.where(view, torch.zeros(()), torch.full((), -math.inf)).to(DEV)
        xa, xp = dict(x, mask=add), dict(x, mask=pack_mask(view).to(DEV))
        ref = oracle(xa)
        out_add, out_packed = run(xa), run(xp)
        check(out_packed, ref, dtype)
        assert torch.equal(out_add, out_packed)
        if dtype != torch.float32:
            assert torch.equal(run(xa, _force_kernel=_lib.KERNEL_SHUFFLE), run(xp, _force_kernel=_lib.KERNEL_SHUFFLE))
    with pytest.raises(ValueError):
        run(dict(x, mask=torch.zeros(L, (L + 63) // 64 + 1, dtype=torch.int64, device=DEV)))


def test_fully_masked_rows_and_empty_cache():
    x = make(17, 2, 4, 2, 20, 128, 64, torch.bfloat16, [0, 40])
    x["mask"] = x["mask"].clone()
    x["mask"][3, :] = -math.inf
    ref = oracle(x)
    assert torch.all(ref[0, :, 3] == 0)
    for kern in (-1, _lib.KERNEL_SHUFFLE):
        out = run(x, _force_kernel=kern)
        check(out, ref, torch.bfloat16)
        assert torch.all(out[0, :, 3] == 0)


def test_tree_heads_per_query_head():
    """current_k/current_v with num_heads heads (flash_tree_attn.py:424-425) under GQA."""
    x = make(19, 2, 8, 2, 16, 128, 200, torch.float16, [200, 77], cur_heads=8)
    check(run(x), oracle(x), torch.float16)


def test_strided_views_like_reference_benchmark():
    """flash_tree_attn.py:471-483 passes k[:, :, :N] and k[:, :, N:] of one buffer."""
    g = torch.Generator().manual_seed(23)
    Z, H, N, L, D = 2, 4, 192, 16, 128
    q = torch.randn(Z, H, L, D, generator=g).half().to(DEV)
    k = torch.randn(Z, H, N + L, D, generator=g).half().to(DEV)
    v = torch.randn(Z, H, N + L, D, generator=g).half().to(DEV)
    mask = additive_mask_from_parents(random_tree_parents(L, g), device=DEV)
    lens = torch.tensor([N] * Z, device=DEV)
    out = flash_decoding_attention(q, k[:, :, :N], v[:, :, :N], k[:, :, N:], v[:, :, N:], mask, lens,
                                   block_size=64, sm_scale=0.11)
    ref = tree_attention_oracle(q, k[:, :, :N], v[:, :, :N], k[:, :, N:], v[:, :, N:], mask, lens, 0.11, 1)
    check(out, ref, torch.float16)
    # a transposed (inner stride != 1) q is copied, not rejected
    qt = q.transpose(2, 3).contiguous().transpose(2, 3)
    check(flash_decoding_attention(qt, k[:, :, :N], v[:, :, :N], k[:, :, N:], v[:, :, N:], mask, lens, sm_scale=0.11),
          ref, torch.float16)


def test_user_buffers_reference_sized():
    """output / mid_output / mid_output_lse shaped as the reference allocates them
    (flash_tree_attn.py:276-284) are accepted; output receives the final result."""
    x = make(29, 2, 8, 2, 32, 128, 2048, torch.bfloat16, [2048, 1000])
    kv_max_split = -(-2048 // 64)
    out = torch.empty(2, 8, 32, 128, dtype=torch.bfloat16, device=DEV)
    mid = torch.empty(2, 8, kv_max_split, 32, 128, dtype=torch.float32, device=DEV)
    lse = torch.empty(2, 8, kv_max_split, 32, dtype=torch.float32, device=DEV)
    ret = run(x, output=out, mid_output=mid, mid_output_lse=lse, max_seq_len_in_batch=2048)
    assert ret.data_ptr() == out.data_ptr()
    check(out, oracle(x), torch.bfloat16)
    # scratch too small for the planned splits -> the reference's assert (flash_tree_attn.py:286-288)
    with pytest.raises(AssertionError):
        run(x, mid_output=mid[:, :, :1], mid_output_lse=lse[:, :, :1], _force_splits=4)


def test_errors_like_reference_asserts():
    x = make(31, 1, 2, 2, 4, 64, 32, torch.float16, [32])
    with pytest.raises(AssertionError):
        run(x, block_size=48)                       # flash_tree_attn.py:268
    bad = dict(x)
    bad["v_cache"] = x["v_cache"][:, :, :16]
    with pytest.raises(AssertionError):
        run(bad)                                    # flash_tree_attn.py:264
    bad = make(31, 1, 2, 2, 4, 64, 32, torch.float16, [32])
    for name in ("q", "k_cache", "v_cache", "current_k", "current_v"):
        bad[name] = torch.cat([bad[name], bad[name][..., :32]], dim=-1)
    with pytest.raises(AssertionError):
        run(bad)                                    # head_dim 96: flash_tree_attn.py:263


def test_int32_lengths_scale_override_and_negative_scale():
    x = make(37, 2, 4, 2, 16, 64, 99, torch.float16, [99, 12])
    ref = oracle(x, sm_scale=0.05)
    check(run(x, sm_scale=0.05), ref, torch.float16)
    x32 = dict(x)
    x32["kv_seq_len"] = x["kv_seq_len"].int()
    check(run(x32, sm_scale=0.05), ref, torch.float16)
    check(run(x, sm_scale=-0.07), oracle(x, sm_scale=-0.07), torch.float16)


def test_lengths_beyond_cache_are_clamped_and_padding_is_ignored():
    x = make(41, 2, 4, 2, 16, 128, 128, torch.bfloat16, [100, 128])
    ref = oracle(x)
    # poison the padding past kv_seq_len: it must never be read into the result
    x["k_cache"][0, :, 100:] = float("nan")
    x["v_cache"][0, :, 100:] = float("inf")
    check(run(x), ref, torch.bfloat16)


@pytest.mark.parametrize("bsz,splits", [(37, 1), (37, 3), (37, 4), (64, 8), (65, 3), (200, 2), (300, 2)])
def test_ragged_batch_dispatch_order(bsz, splits):
    """Stage 1 resolves its workgroups longest-first from the batch's lengths; every
    (sequence, split) must still be computed exactly once whatever the order: ties, empty
    caches, lengths that are exact multiples of the chunk; batches a wave orders by itself
    (up to 64), batches ordered through LDS (65 .. 256) and batches beyond the limit of the
    ordered dispatch (identity order)."""
    g = torch.Generator().manual_seed(bsz * 31 + splits)
    tmax = 512
    lens = torch.randint(0, tmax + 1, (bsz,), generator=g).tolist()
    lens[0], lens[1], lens[2], lens[3] = 0, tmax, tmax, 0
    chunk = -(-tmax // splits // 64) * 64
    for i, mult in enumerate(range(1, splits + 1)):
        if 4 + i < bsz and mult * chunk <= tmax:
            lens[4 + i] = mult * chunk
    x = make(51, bsz, 4, 2, 8, 64, tmax, torch.float16, lens)
    ref = oracle(x)
    check(run(x, _force_splits=splits), ref, torch.float16)
    check(run(x, _force_splits=splits, _force_kernel=_lib.KERNEL_SHUFFLE), ref, torch.float16)


@pytest.mark.parametrize("shape", [
    # bsz hq hkv  L   D   tmax  lens                      splits
    (8, 32, 8, 64, 128, 2048, None, 4),                    # headline layout: 256 rows, 4 splits
    (5, 16, 2, 16, 128, 1500, [1500, 700, 64, 0, 1499], 5),  # 128 rows, ragged: 1..5 live splits
    (3, 12, 3, 40, 64, 900, [900, 450, 1], 3),             # D 64, padded row block
    (2, 16, 2, 40, 128, 700, [700, 300], 4),               # two row blocks per group
])
def test_single_launch_merge_matches_two_launches(shape):
    """With counters, the workgroup that finishes a sequence last merges the partials
    inside stage 1. Same result as stage 1 + stage 2, on repeated calls (the counters
    must be left zero), and the counters really are zero afterwards."""
    from flash_tree_attn_amd import flash_decoding as fd
    bsz, hq, hkv, L, D, tmax, lens, splits = shape
    x = make(61, bsz, hq, hkv, L, D, tmax, torch.bfloat16, lens if lens is not None else [tmax] * bsz)
    ref = oracle(x)
    pc = fd.prepare(x["q"], x["k_cache"], x["v_cache"], x["current_k"], x["current_v"], x["mask"], x["kv_seq_len"],
                 64, None, None, None, None, None, x["kv_group_num"], _force_splits=splits)
    assert pc.plan.kernel == _lib.KERNEL_MFMA and pc.plan.num_splits == splits and pc.plan.counter_elems > 0
    two = pc.run_two_launches().clone()
    check(two, ref, torch.bfloat16)
    for _ in range(3):
        pc.output.fill_(float("nan"))
        one = pc.run_single_launch().clone()
        check(one, ref, torch.bfloat16)
        torch.testing.assert_close(one.float(), two.float(), atol=1e-5, rtol=2 ** -7)
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream().cuda_stream
    buf = fd._counters[(x["q"].device.index, stream)]
    assert int(buf.abs().sum()) == 0


def to_pages(x, page_size, seed, spare_pages=3):
    """Scatters the contiguous caches of `x` into a shuffled page pool; returns
    (k_pages, v_pages, block_tables). Unused pool pages and the rows past each length
    hold NaN: they must never reach the result."""
    k, v = x["k_cache"], x["v_cache"]
    bsz, hkv, tmax, D = k.shape
    per_seq = -(-tmax // page_size)
    n_pages = bsz * per_seq + spare_pages
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(n_pages, generator=g)[: bsz * per_seq].view(bsz, per_seq)
    kp = torch.full((n_pages, hkv, page_size, D), float("nan"), dtype=k.dtype, device=k.device)
    vp = torch.full_like(kp, float("nan"))
    for b in range(bsz):
        t_b = int(x["kv_seq_len"][b])
        for pg in range(per_seq):
            lo, hi = pg * page_size, min((pg + 1) * page_size, tmax, t_b)
            if hi > lo:
                kp[perm[b, pg], :, : hi - lo] = k[b, :, lo:hi]
                vp[perm[b, pg], :, : hi - lo] = v[b, :, lo:hi]
    return kp, vp, perm.to(torch.int32).to(k.device)


@pytest.mark.parametrize("page_size", [16, 32, 64, 128])
@pytest.mark.parametrize("shape", [
    # bsz hq hkv  L   D   tmax  dtype           lens              splits
    (3, 16, 4, 64, 128, 1000, torch.bfloat16, [1000, 517, 63], 0),     # 256 rows: pipelined MFMA variant
    (2, 8, 2, 16, 128, 700, torch.float16, [700, 129], 3),             # 128-row plain variant, 3 splits
    (2, 4, 4, 3, 64, 300, torch.float32, [300, 0], 2),                 # shuffle kernel, an empty cache
])
def test_paged_caches_equal_contiguous_caches(page_size, shape):
    """Block-table addressing (flash_tree_attn.py:17-18,233 describe that layout) changes
    where rows are fetched from, not what is computed: the paged call must reproduce the
    contiguous call bit for bit, and the oracle within tolerance."""
    bsz, hq, hkv, L, D, tmax, dtype, lens, splits = shape
    x = make(81, bsz, hq, hkv, L, D, tmax, dtype, lens)
    ref = oracle(x)
    # the same length cap for both calls, so that both cut the same chunks (the paged
    # capacity is a whole number of pages)
    out = run(x, _force_splits=splits, max_seq_len_in_batch=tmax)
    kp, vp, tables = to_pages(x, page_size, seed=page_size)
    xp = dict(x, k_cache=kp, v_cache=vp)
    out_paged = run(xp, _force_splits=splits, block_tables=tables, max_seq_len_in_batch=tmax)
    check(out_paged, ref, dtype)
    assert torch.equal(out_paged, out)


def test_paged_pool_beyond_4_gib():
    """Page offsets are 64-bit: the pages in use sit at the far end of a 5 GiB pool."""
    bsz, hq, hkv, L, D, tmax, page = 2, 16, 8, 8, 128, 2048, 16
    x = make(83, bsz, hq, hkv, L, D, tmax, torch.bfloat16, [2048, 999])
    page_bytes = hkv * page * D * 2
    n_pages = (5 << 30) // page_bytes
    kp = torch.empty((n_pages, hkv, page, D), dtype=torch.bfloat16, device=DEV)
    vp = torch.empty_like(kp)
    per_seq = tmax // page
    g = torch.Generator().manual_seed(7)
    tables = (n_pages - 1 - torch.randperm(bsz * per_seq, generator=g)).view(bsz, per_seq)
    for b in range(bsz):
        kp[tables[b]] = x["k_cache"][b].view(hkv, per_seq, page, D).transpose(0, 1)
        vp[tables[b]] = x["v_cache"][b].view(hkv, per_seq, page, D).transpose(0, 1)
    assert int(tables.min()) * page_bytes > (4 << 30)
    out = run(dict(x, k_cache=kp, v_cache=vp), block_tables=tables.to(torch.int32).to(DEV))
    check(out, oracle(x), torch.bfloat16)
    assert torch.equal(out, run(x))


@pytest.mark.parametrize("case", [
    (1, 1, 4, 4, 1, 128, 300, torch.bfloat16, [300], None, 1),       # plain decode, one row per unit
    (2, 2, 8, 2, 1, 128, 777, torch.float16, [777, 123], None, 3),   # GQA 4, one token: 4 rows
    (3, 3, 8, 8, 4, 64, 500, torch.bfloat16, [0, 1, 500], None, 2),
    (4, 2, 8, 1, 1, 64, 1000, torch.float16, None, None, 4),         # GQA 8: 8 rows
    (5, 2, 6, 2, 5, 128, 650, torch.bfloat16, None, None, 0),        # 15 rows
    (6, 2, 8, 2, 3, 128, 400, torch.float16, None, 8, 2),            # tree heads = query heads: 3 rows
    (7, 4, 4, 4, 13, 64, 900, torch.bfloat16, None, None, 0),
    (8, 2, 8, 2, 2, 128, 4096, torch.bfloat16, [4096, 4000], None, 8),
])
def test_units_below_one_mfma_tile(case):
    """Units of 1-15 query rows (plain decode, tiny trees) take the MFMA kernel with most
    rows of its tile blanked; the shuffle kernel on the same inputs must agree with the oracle too."""
    from flash_tree_attn_amd import flash_decoding as fd
    from flash_tree_attn_amd.tree_mask import pack_mask
    seed, bsz, hq, hkv, L, D, tmax, dtype, lens, cur_heads, splits = case
    x = make(seed, bsz, hq, hkv, L, D, tmax, dtype, lens=lens, cur_heads=cur_heads)
    ref = oracle(x)
    pc = fd.prepare(x["q"], x["k_cache"], x["v_cache"], x["current_k"], x["current_v"], x["mask"], x["kv_seq_len"], 64,
                 None, None, None, None, None, x["kv_group_num"])
    assert pc.plan.kernel == _lib.KERNEL_MFMA and pc.plan.rows_per_group < 16
    out = run(x, _force_splits=splits)
    check(out, ref, dtype)
    check(run(x, _force_splits=splits, _force_kernel=_lib.KERNEL_SHUFFLE), ref, dtype)
    assert torch.equal(out, run(dict(x, mask=pack_mask(x["mask"].cpu()).to(DEV)), _force_splits=splits))


def test_repeat_calls_take_the_remembered_signature(monkeypatch):
    """The drop-in function keeps the validated arguments and plan of a call signature and
    only refreshes pointers on the next call with the same signature: new data, same shapes
    must give that data's result, without going through prepare() again; a changed signature,
    a mask that needs conversion or a misaligned tensor must take the full path."""
    from flash_tree_attn_amd import flash_decoding as fd
    fd._fast.__dict__.pop("entries", None)
    shape = (2, 8, 2, 16, 128, 2000, torch.bfloat16)
    x1 = make(71, *shape, lens=[2000, 1500])
    x2 = make(72, *shape, lens=[1, 1999])
    for splits in (1, 3):   # direct output, and partials + merge with scratch from the allocator
        out1 = run(x1, _force_splits=splits)
        assert len(fd._fast.entries) >= 1
        check(out1, oracle(x1), torch.bfloat16)
        with monkeypatch.context() as mp:
            mp.setattr(fd, "prepare", lambda *a, **k: pytest.fail("a repeat call went through prepare()"))
            out2 = run(x2, _force_splits=splits)
            again = run(x1, _force_splits=splits)
        check(out2, oracle(x2), torch.bfloat16)
        assert torch.equal(again, out1)
    # caller's buffers: same signature -> remembered, results land in the given output
    outbuf = torch.empty_like(x1["q"])
    mid = torch.empty(2, 8, 4, 16, 128, dtype=torch.float32, device=DEV)
    lse = torch.empty(2, 8, 4, 16, dtype=torch.float32, device=DEV)
    for x in (x1, x2, x1):
        got = run(x, output=outbuf, mid_output=mid, mid_output_lse=lse, _force_splits=4)
        assert got.data_ptr() == outbuf.data_ptr()
        check(got, oracle(x), torch.bfloat16)
    # another signature in between (strided views of one buffer), then the first one again
    big = torch.randn(2, 2, 2100, 128, device=DEV).to(torch.bfloat16)
    xs = dict(x1, k_cache=big[:, :, :2000], current_k=big[:, :, 2000:2016])
    for x in (xs, x2, xs):
        check(run(x), oracle(x), torch.bfloat16)
    # a bool mask is converted on every call and never remembered; a q whose rows are not 16-byte
    # aligned falls back to the full path (which copies it) although its signature is known
    n = len(fd._fast.entries)
    xb = dict(x1, mask=torch.isfinite(x1["mask"]))
    for _ in range(2):
        check(run(xb), oracle(x1), torch.bfloat16)
    assert len(fd._fast.entries) == n
    flat = torch.empty(x2["q"].numel() + 4, dtype=torch.bfloat16, device=DEV)
    q_off = flat[4:].view(x2["q"].shape)
    q_off.copy_(x2["q"])
    assert q_off.data_ptr() % 16 == 8 and q_off.stride() == x2["q"].stride()
    check(run(dict(x2, q=q_off)), oracle(x2), torch.bfloat16)


def test_calls_follow_the_current_stream():
    """The library launches on torch's current stream (as the reference's Triton launches do):
    calls issued under `torch.cuda.stream(side)` must be ordered with other work of that stream,
    on the full path, on the remembered path and with the merge inside stage 1 (whose counter
    buffer is kept per stream)."""
    from flash_tree_attn_amd import flash_decoding as fd
    fd._fast.__dict__.pop("entries", None)
    x = make(91, 2, 8, 2, 16, 128, 3000, torch.bfloat16, lens=[3000, 2500])
    ref = oracle(x)
    pc = fd.prepare(x["q"], x["k_cache"], x["v_cache"], x["current_k"], x["current_v"], x["mask"], x["kv_seq_len"], 64,
                    None, None, None, None, None, x["kv_group_num"], _force_splits=2)
    assert pc.plan.single_launch == 1
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    outs = []
    with torch.cuda.stream(side):
        scale = torch.full((1,), 2.0, device=DEV, dtype=torch.bfloat16)
        for _ in range(3):                      # full path once, then the remembered signature
            q2 = x["q"] * scale                 # produced on the side stream right before the call
            outs.append(run(dict(x, q=q2), _force_splits=2, sm_scale=0.5 / math.sqrt(128)))
            outs.append(run(dict(x, q=q2), _force_splits=1, sm_scale=0.5 / math.sqrt(128)) * 1.0)   # consumed on it right after
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for o in outs:
        check(o, ref, torch.bfloat16)
    assert any(k[1] == side.cuda_stream for k in fd._counters)


@pytest.mark.parametrize("splits", [1, 3])
def test_call_under_graph_capture_and_replay(splits):
    """A serving loop captures its decode step in a HIP graph: the call (one kernel, or stage 1 +
    stage 2 with the caller's scratch) is captured once and replayed with new data in the same
    buffers; every replay, with eager work and synchronisations in between, must equal the oracle."""
    x = make(95, 2, 8, 2, 16, 128, 2048, torch.bfloat16, lens=[2048, 900])
    out = torch.empty_like(x["q"])
    mid = torch.empty(2, 8, 4, 16, 128, dtype=torch.float32, device=DEV)
    lse = torch.empty(2, 8, 4, 16, dtype=torch.float32, device=DEV)
    call = lambda: run(x, output=out, mid_output=mid, mid_output_lse=lse, _force_splits=splits)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):            # warm-up outside the capture (first-call set-up, remembered signature)
        for _ in range(3):
            call()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    check(out, oracle(x), torch.bfloat16)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    g = torch.Generator().manual_seed(7)
    for rep in range(4):
        x["q"].copy_(torch.randn(x["q"].shape, generator=g).to(torch.bfloat16))            # eager work between replays
        x["k_cache"][:, :, :64].copy_(torch.randn(2, 2, 64, 128, generator=g).to(torch.bfloat16))
        x["kv_seq_len"].copy_(torch.tensor([2048 - 100 * rep, 1 + 300 * rep]))
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        check(out, oracle(x), torch.bfloat16)


def test_paged_argument_errors():
    x = make(82, 2, 4, 2, 8, 128, 128, torch.float16, [128, 5])
    kp, vp, tables = to_pages(x, 32, seed=1)
    xp = dict(x, k_cache=kp, v_cache=vp)
    with pytest.raises(ValueError):
        run(xp, block_tables=tables.long())                       # must be int32
    with pytest.raises(ValueError):
        run(xp, block_tables=tables[:1])                          # one row per sequence
    bad = dict(x, k_cache=kp[:, :, :24].contiguous(), v_cache=vp[:, :, :24].contiguous())
    with pytest.raises(FtaAssertionError):
        run(bad, block_tables=tables)                             # page size 24 is not a block size


def _random_case(rng):
    """One random configuration of everything the entry point accepts."""
    dtype = [torch.bfloat16, torch.float16, torch.float32][rng.randrange(3)]
    D = [32, 64, 128, 256][rng.randrange(4)] if dtype == torch.float32 else [64, 128, 128, 128, 32, 256][rng.randrange(6)]
    hkv = [1, 2, 3, 4][rng.randrange(4)]
    G = [1, 2, 4, 8][rng.randrange(4)]
    L = [1, 2, 5, 8, 16, 17, 31, 32, 48, 64, 65, 100][rng.randrange(12)]
    if G * L > 512:
        L = 512 // G
    bsz = rng.randrange(1, 6)
    tmax = [64, 100, 257, 600, 1500][rng.randrange(5)]
    lens = [rng.choice([0, 1, tmax, rng.randrange(0, tmax + 1)]) for _ in range(bsz)]
    splits = rng.choice([0, 0, 1, 2, 3, 7])
    cur_heads = hkv if rng.random() < 0.7 else hkv * G
    return dict(dtype=dtype, D=D, hkv=hkv, hq=hkv * G, L=L, bsz=bsz, tmax=tmax, lens=lens, splits=splits, cur_heads=cur_heads,
                page=rng.choice([0, 0, 16, 32, 64, 128]), packed=rng.random() < 0.4, len32=rng.random() < 0.3,
                block=rng.choice([16, 32, 64, 128]), shuffle=rng.random() < 0.2)


@pytest.mark.parametrize("seed", range(48))
def test_random_configurations_against_the_oracle(seed):
    """Seeded random draws over dtype, head_dim, GQA factor, tree size, lengths (incl. 0, 1
    and full), split count, block size, tree heads, paged or contiguous caches, packed or
    additive mask, int32 or int64 lengths, either stage-1 kernel."""
    import random
    from flash_tree_attn_amd.tree_mask import pack_mask
    c = _random_case(random.Random(1000 + seed))
    x = make(2000 + seed, c["bsz"], c["hq"], c["hkv"], c["L"], c["D"], c["tmax"], c["dtype"], c["lens"], cur_heads=c["cur_heads"])
    ref = oracle(x)
    kw = dict(_force_splits=c["splits"])
    if c["shuffle"]:
        kw["_force_kernel"] = _lib.KERNEL_SHUFFLE
    if c["packed"]:
        x["mask"] = pack_mask(x["mask"].cpu()).to(DEV)
    if c["len32"]:
        x["kv_seq_len"] = x["kv_seq_len"].int()
    if c["page"]:
        x["k_cache"], x["v_cache"], kw["block_tables"] = to_pages(x, c["page"], seed)
    out = run(x, block_size=c["block"], **kw)
    check(out, ref, c["dtype"])


# ---------------------------------------------------------------- size-independent properties
def test_properties_at_headline_size():
    cfg = CONFIGS["cfg3_gqa_8b_bf16"]
    x = make_inputs(cfg, seed=1, device=DEV, gen_device=DEV)
    # constant V -> constant output, whatever the logits are
    xc = dict(x)
    xc["v_cache"] = torch.full_like(x["v_cache"], 0.75)
    xc["current_v"] = torch.full_like(x["current_v"], 0.75)
    out = run(xc)
    torch.testing.assert_close(out.float(), torch.full_like(out, 0.75).float(), atol=4e-3, rtol=0)
    # q = 0 -> mean over cache and allowed tree values
    xz = dict(x)
    xz["q"] = torch.zeros_like(x["q"])
    out = run(xz).float()
    allowed = torch.isfinite(x["mask"]).float()                          # [L, L]
    num = x["v_cache"].float().sum(2)[:, :, None] + torch.einsum("ij,bhjd->bhid", allowed, x["current_v"].float())
    mean = (num / (cfg.cache_len + allowed.sum(1))[None, None, :, None]).repeat_interleave(cfg.kv_group_num, dim=1)
    torch.testing.assert_close(out, mean, atol=2e-3, rtol=1e-2)
    # output is linear in V for fixed q, k
    x2 = dict(x)
    x2["v_cache"], x2["current_v"] = x["v_cache"] * 2, x["current_v"] * 2
    torch.testing.assert_close(run(x2).float(), run(x).float() * 2, atol=2e-3, rtol=1e-2)
