"""More of the MFMA stage-1 kernel's SOURCE on host threads (the harness of tests/test_host_block_mfma.py, in a file of
its own so that the CPU suite's worker processes share the load): draws of the entry point's whole argument space, and
rows that a few keys carry (keys of more spread than N(0, 1)), where the rounding of P to the 16-bit type would show
without the compensating product of stage1_mfma_kernel.h (kHeavyShare).

TEST INFRASTRUCTURE ONLY: nothing under flash_tree_attn_amd/ knows of this build."""
import pytest
import torch

from flash_tree_attn_amd import _lib
from flash_tree_attn_amd.tree_mask import pack_mask
from test_host_block_kernels import TOL, HostCall, make, oracle
from test_host_block_mfma import MFMA, host_lib, loads_land_when_issued  # noqa: F401  (fixtures: this module gets its own build)


# Draws of the GPU suite's random-configuration generator (tests/test_parity_gpu.py: _random_case, steered towards
# 16-bit inputs and larger units), kept here as literals: everything the entry point accepts, combined at random.
# 158 such draws (and the 48 of the GPU test itself, most of which take the shuffle kernel) were run on host threads
# once; these are six quick ones that between them take every compiled loop, pages, the packed mask, 32-bit lengths,
# tree heads per query head, block sizes other than 64, forced and free split counts and the merge inside the launch.
RANDOM_DRAWS = [
    # seed dtype            D    hq hkv cur L    bsz tmax lens                splits page packed len32 block kernel      counters rows loop
    (112, torch.bfloat16, 64, 3, 3, 3, 130, 1, 257, [257], 1, 128, False, True, 16, MFMA, False, 256, 0),
    (118, torch.bfloat16, 128, 2, 1, 2, 70, 1, 600, [299], 0, 0, False, False, 32, MFMA, True, 128, 0),
    (120, torch.float16, 128, 4, 4, 4, 16, 2, 100, [0, 1], 2, 32, False, False, 16, _lib.KERNEL_MFMA_SPLIT_KEYS, True, 64, 2),
    (123, torch.bfloat16, 128, 1, 1, 1, 130, 3, 257, [196, 257, 228], 3, 32, False, False, 64, MFMA, True, 256, 0),
    (145, torch.float16, 64, 12, 3, 3, 65, 3, 257, [0, 1, 79], 2, 32, False, True, 64, MFMA, True, 256, 0),
    (151, torch.float16, 64, 8, 2, 2, 65, 5, 600, [282, 1, 1, 272, 1], 1, 0, True, False, 16, MFMA, False, 256, 0),
]


def scattered_pages(x, page, seed, spare=3):
    """The contiguous caches of `x` scattered into a shuffled page pool; unused pages and rows past a length hold NaN."""
    k, v = x["k_cache"], x["v_cache"]
    bsz, hkv, tmax, D = k.shape
    per_seq = -(-tmax // page)
    perm = torch.randperm(bsz * per_seq + spare, generator=torch.Generator().manual_seed(seed))[: bsz * per_seq].view(bsz, per_seq)
    kp = torch.full((bsz * per_seq + spare, hkv, page, D), float("nan"), dtype=k.dtype)
    vp = torch.full_like(kp, float("nan"))
    for b in range(bsz):
        for pg in range(per_seq):
            lo, hi = pg * page, min((pg + 1) * page, tmax, int(x["kv_seq_len"][b]))
            if hi > lo:
                kp[perm[b, pg], :, : hi - lo], vp[perm[b, pg], :, : hi - lo] = k[b, :, lo:hi], v[b, :, lo:hi]
    return kp, vp, perm.to(torch.int32).contiguous()


@pytest.mark.parametrize("draw", RANDOM_DRAWS, ids=lambda d: f"draw{d[0]}")
def test_random_draws_of_everything_the_entry_point_accepts(host_lib, draw):
    seed, dtype, D, hq, hkv, cur, L, bsz, tmax, lens, splits, page, packed, len32, block, kernel, counters, rows_per_wg, loop = draw
    x = make(2000 + seed, bsz, hq, hkv, L, D, tmax, dtype, lens, cur_heads=cur)
    ref = oracle(x)
    kw = dict(splits=splits, kernel=kernel, counters=counters, block_size=block, len32=len32, mask=pack_mask(x["mask"]) if packed else None)
    if page:
        kp, vp, tables = scattered_pages(x, page, seed)
        kw.update(tables=tables, pools=(kp, vp))
    call = HostCall(host_lib, x, **kw)
    assert call.plan.kernel == MFMA and call.plan.rows_per_wg == rows_per_wg and call.plan.mfma_loop == loop
    host_lib.host_block_loads_land_late(seed % 2)
    out = call.run()
    assert torch.isfinite(out).all()
    torch.testing.assert_close(out.float(), ref, **TOL[dtype])
    if counters and call.plan.counter_elems:
        assert (call.counters == 0).all()


def share_of_tolerance(out, ref, atol=2e-3, rtol=1e-2):
    """Largest error as a share of atol + rtol * |ref| (1.0 = at the line), and how many elements are beyond it."""
    err = (out.float() - ref).abs()
    tol = atol + rtol * ref.abs()
    return (err / tol).max().item(), int((err > tol).sum())


def spread_keys(x, scale_k):
    """The same inputs with keys of `scale_k` times the spread: logits ~ N(0, scale_k^2), so a few keys carry a row."""
    return dict(x, k_cache=(x["k_cache"].float() * scale_k).to(x["k_cache"].dtype))


# Logits with more spread than N(0, 1): a handful of keys carry each row, and the rounding of their probabilities to
# bf16 (2^-9 relative, flash_tree_attn.py:117 rounds P to V's type as well) reaches the output undamped. Full tiles with
# such a key take the compensating residue product (stage1_mfma_kernel.h: kHeavyShare). Without it the 8-wave loop
# measured 1.18 of the tolerance at four times the spread (seed 0, 512 keys); the bars here are 1.0 there and half the
# tolerance at twice the spread, for every compiled loop.
PEAKED = [(scale_k, seed, keys) for scale_k in (4.0, 2.0) for seed in (0, 3, 75) for keys in (512, 1024)]


@pytest.mark.parametrize("scale_k,seed,keys", PEAKED)
def test_peaked_logits_8_wave_loop(host_lib, scale_k, seed, keys):
    x = spread_keys(make(seed, 1, 4, 1, 64, 128, keys, torch.bfloat16, [keys]), scale_k)
    call = HostCall(host_lib, x, splits=1, kernel=MFMA)
    assert call.plan.rows_per_wg == 256 and call.plan.mfma_loop == 0
    share, bad = share_of_tolerance(call.run(), oracle(x))
    assert bad == 0 and share <= (1.0 if scale_k > 2 else 0.5), (share, bad)


@pytest.mark.parametrize("scale_k,seed", [(4.0, 0), (4.0, 3), (2.0, 0), (2.0, 3)])
@pytest.mark.parametrize("form", ["4 waves", "key halves", "head_dim 256"])
def test_peaked_logits_other_loops(host_lib, form, scale_k, seed):
    hq, L, D, kernel, rows, loop = {"4 waves": (2, 64, 128, MFMA, 128, 0), "key halves": (1, 64, 128, _lib.KERNEL_MFMA_SPLIT_KEYS, 64, 2),
                                    "head_dim 256": (2, 32, 256, MFMA, 128, 0)}[form]
    x = spread_keys(make(seed, 1, hq, 1, L, D, 512, torch.bfloat16, [512]), scale_k)
    call = HostCall(host_lib, x, splits=2, kernel=kernel)
    assert call.plan.rows_per_wg == rows and call.plan.mfma_loop == loop
    share, bad = share_of_tolerance(call.run(), oracle(x))
    assert bad == 0 and share <= (1.0 if scale_k > 2 else 0.5), (share, bad)


def test_one_unit_of_the_headline_workload(host_lib):
    """One cache head of one sequence of the headline workload (4 query heads x 64 tree tokens = 256 rows, 8192 cached
    keys, bf16), cut as the plan cuts the whole workload on 256 CUs: 4 splits of 2112 keys, 33 tiles through the fused
    loop per workgroup, the tree tile on the last. Well inside the tolerance on N(0, 1) data."""
    x = make(0, 1, 4, 1, 64, 128, 8192, torch.bfloat16, [8192])
    call = HostCall(host_lib, x, splits=4, kernel=MFMA)
    assert (call.plan.num_splits, call.plan.chunk, call.plan.rows_per_wg, call.plan.mfma_loop) == (4, 2112, 256, 0)
    share, bad = share_of_tolerance(call.run(), oracle(x))
    assert bad == 0 and share <= 0.25, share
