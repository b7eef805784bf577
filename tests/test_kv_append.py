"""Accepted-path KV append (`fta_append_kv`, include/fta.h): the oracle against torch's
own indexing on CPU, argument errors of the C entry point without a GPU, and bit-exact
GPU parity (it is a copy: no tolerance)."""
import ctypes as C

import pytest
import torch

from flash_tree_attn_amd import _lib
from oracle.kv_append_oracle import append_accepted_kv_oracle

DEV = "cuda"


def make(seed, bsz, hkv, L, D, cache_len, dtype, lens, acc, max_accept, len_dtype=torch.int64):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g).to(dtype)
    x = dict(k_cache=r(bsz, hkv, cache_len, D), v_cache=r(bsz, hkv, cache_len, D), current_k=r(bsz, hkv, L, D),
             current_v=r(bsz, hkv, L, D))
    idx = torch.stack([torch.randperm(L, generator=g)[:max_accept] if L >= max_accept
                       else torch.randint(0, L, (max_accept,), generator=g) for _ in range(bsz)]).to(torch.int32)
    x["accept_idx"] = idx
    x["accept_len"] = torch.tensor(acc, dtype=len_dtype)
    x["kv_seq_len"] = torch.tensor(lens, dtype=len_dtype)
    return x


# ---------------------------------------------------------------- CPU
def test_oracle_equals_torch_indexing():
    x = make(1, 3, 2, 10, 8, 40, torch.float32, [5, 38, 0], [4, 4, 0], 4)
    k, v, n = append_accepted_kv_oracle(**x)
    for b, (t, a) in enumerate(zip([5, 38, 0], [4, 4, 0])):
        room = min(a, 40 - t)
        sel = x["accept_idx"][b, :room].long()
        exp_k = x["k_cache"][b].clone()
        exp_k[:, t:t + room] = x["current_k"][b].index_select(1, sel)
        exp_v = x["v_cache"][b].clone()
        exp_v[:, t:t + room] = x["current_v"][b].index_select(1, sel)
        assert torch.equal(k[b], exp_k) and torch.equal(v[b], exp_v)
    assert n.tolist() == [9, 40, 0]


def base_args(**kw):
    a = _lib.FtaAppendArgs()
    for f in ("k_cache", "v_cache", "cur_k", "cur_v", "accept_idx", "accept_len", "kv_seq_len", "kv_seq_len_out"):
        setattr(a, f, 0x1000)
    cfg = dict(bsz=2, num_kv_heads=4, q_len=8, head_dim=128, cache_len=64, max_accept=4, dtype=_lib.FTA_BF16,
               len_dtype=_lib.FTA_I64)
    cfg.update(kw)
    for k, v in cfg.items():
        setattr(a, k, v)
    D, L, T, H = a.head_dim, a.q_len, a.cache_len, a.num_kv_heads
    a.k_stride[:] = [H * T * D, T * D, D]
    a.v_stride[:] = a.k_stride[:]
    a.ck_stride[:] = [H * L * D, L * D, D]
    a.cv_stride[:] = a.ck_stride[:]
    a.accept_idx_stride = a.max_accept
    return a


def test_append_argument_errors_without_touching_the_gpu(fta_lib):
    assert fta_lib.fta_append_kv(None, None) == -1
    a = base_args()
    a.accept_idx = None
    assert fta_lib.fta_append_kv(C.byref(a), None) == -1
    assert fta_lib.fta_append_kv(C.byref(base_args(head_dim=100)), None) == -2
    assert fta_lib.fta_append_kv(C.byref(base_args(dtype=9)), None) == -6
    assert fta_lib.fta_append_kv(C.byref(base_args(bsz=0)), None) == -7
    a = base_args()
    a.k_stride[2] = 100
    assert fta_lib.fta_append_kv(C.byref(a), None) == -8
    a = base_args()
    a.cur_v = 0x1008
    assert fta_lib.fta_append_kv(C.byref(a), None) == -8
    if not torch.cuda.is_available():
        assert fta_lib.fta_append_kv(C.byref(base_args()), None) == -11


def test_python_wrapper_rejects_cpu_tensors():
    from flash_tree_attn_amd import append_accepted_kv
    x = make(2, 1, 1, 4, 32, 8, torch.float16, [2], [1], 2)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        append_accepted_kv(**x)


# ---------------------------------------------------------------- GPU
def gpu_run(x, out_of_place=False):
    from flash_tree_attn_amd import append_accepted_kv
    d = {k: v.to(DEV) for k, v in x.items()}
    out = torch.full_like(d["kv_seq_len"], -7) if out_of_place else None
    old = d["kv_seq_len"].clone()
    ret = append_accepted_kv(**d, out_kv_seq_len=out)
    if out_of_place:
        assert torch.equal(d["kv_seq_len"], old) and ret is out
    else:
        assert ret is d["kv_seq_len"]
    return d["k_cache"].cpu(), d["v_cache"].cpu(), ret.cpu()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("out_of_place", [False, True])
def test_append_matches_oracle_bit_for_bit(dtype, out_of_place):
    # ragged accept lengths incl. 0, a sequence that hits the cache capacity, an empty cache
    x = make(3, 5, 3, 16, 128, 96, dtype, [10, 93, 0, 96, 50], [6, 6, 1, 3, 0], 6)
    k, v, n = append_accepted_kv_oracle(**x)
    gk, gv, gn = gpu_run(x, out_of_place)
    assert torch.equal(gk, k) and torch.equal(gv, v) and torch.equal(gn, n)
    assert n.tolist() == [16, 96, 1, 96, 50]


@pytest.mark.gpu
def test_repeat_appends_refresh_pointers_only():
    """The second call with the same signature reuses the remembered arguments: other data,
    other tensors, same shapes must still match the oracle; non-contiguous index rows (copied
    by the full path) are never remembered."""
    from flash_tree_attn_amd import flash_decoding as fd
    fd._fast.__dict__.pop("entries", None)
    for seed, lens, acc in ((11, [10, 93, 0], [6, 2, 1]), (12, [0, 1, 90], [1, 6, 6]), (13, [5, 5, 5], [0, 0, 3])):
        x = make(seed, 3, 2, 16, 128, 96, torch.bfloat16, lens, acc, 6)
        k, v, n = append_accepted_kv_oracle(**x)
        gk, gv, gn = gpu_run(x, out_of_place=True)
        assert torch.equal(gk, k) and torch.equal(gv, v) and torch.equal(gn, n)
        assert sum(1 for key in fd._fast.entries if key[0] == "append") == 1
    x = make(14, 3, 2, 16, 128, 96, torch.bfloat16, [10, 20, 30], [2, 2, 2], 6)
    wide = torch.zeros(3, 12, dtype=torch.int32)
    wide[:, ::2] = x["accept_idx"]
    from flash_tree_attn_amd import append_accepted_kv
    k, v, n = append_accepted_kv_oracle(**x)
    for _ in range(2):
        d = {name: t.to(DEV) for name, t in x.items()}
        d["accept_idx"] = wide.to(DEV)[:, ::2]
        assert d["accept_idx"].stride(1) == 2
        gn = append_accepted_kv(**d)
        assert torch.equal(d["k_cache"].cpu(), k) and torch.equal(d["v_cache"].cpu(), v) and torch.equal(gn.cpu(), n)
    assert sum(1 for key in fd._fast.entries if key[0] == "append") == 1


@pytest.mark.gpu
def test_append_edge_cases():
    # int32 lengths, head_dim 32 and 256, out-of-range tree positions are dropped but counted,
    # accept_len beyond max_accept and negative lengths are clamped
    for D in (32, 256):
        x = make(4, 3, 2, 5, D, 20, torch.float16, [3, 7, -2], [9, 2, 3], 4, len_dtype=torch.int32)
        x["accept_idx"][1, 0] = 5
        x["accept_idx"][1, 1] = -1
        k, v, n = append_accepted_kv_oracle(**x)
        gk, gv, gn = gpu_run(x)
        assert torch.equal(gk, k) and torch.equal(gv, v) and torch.equal(gn, n)
        assert n.tolist() == [7, 9, 3] and gn.dtype == torch.int32
        assert torch.equal(gk[1], x["k_cache"][1])   # nothing valid to copy for sequence 1


@pytest.mark.gpu
def test_append_into_strided_cache_views():
    from flash_tree_attn_amd import append_accepted_kv
    x = make(5, 2, 2, 8, 64, 32, torch.bfloat16, [4, 30], [3, 3], 3)
    kv = torch.zeros(2, 2, 2, 32, 64, dtype=torch.bfloat16)   # [bsz, K|V, heads, T, D], as the reference benchmark slices
    kv[:, 0], kv[:, 1] = x["k_cache"], x["v_cache"]
    d = {k: v.to(DEV) for k, v in x.items()}
    kvd = kv.to(DEV)
    d["k_cache"], d["v_cache"] = kvd[:, 0], kvd[:, 1]
    append_accepted_kv(**d)
    k, v, n = append_accepted_kv_oracle(**x)
    assert torch.equal(kvd[:, 0].cpu(), k) and torch.equal(kvd[:, 1].cpu(), v) and torch.equal(d["kv_seq_len"].cpu(), n)


@pytest.mark.gpu
def test_decode_and_append_in_one_graph():
    """The verification step and the cache update captured together in one HIP graph and
    replayed: each replay attends to the cache as the previous replays left it, appends the
    accepted rows and advances the lengths in place; an eager loop over the oracle on copies
    must see the same outputs, caches and lengths after every replay."""
    from flash_tree_attn_amd import append_accepted_kv, flash_decoding_attention
    from flash_tree_attn_amd.tree_mask import additive_mask_from_parents, chain_parents
    from oracle.tree_attn_oracle import tree_attention_oracle
    g = torch.Generator().manual_seed(21)
    bsz, hq, hkv, L, D, cap = 2, 8, 2, 8, 128, 512
    r = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(DEV)
    k_cache, v_cache = r(bsz, hkv, cap, D), r(bsz, hkv, cap, D)
    q, ck, cv = r(bsz, hq, L, D), r(bsz, hkv, L, D), r(bsz, hkv, L, D)
    lens = torch.tensor([300, 17], dtype=torch.int64, device=DEV)
    mask = additive_mask_from_parents(chain_parents(L), device=DEV)
    idx = torch.arange(L, dtype=torch.int32).repeat(bsz, 1).to(DEV)      # a chain: the first n rows are the accepted path
    n_acc = torch.tensor([3, 5], dtype=torch.int64, device=DEV)
    out = torch.empty_like(q)

    def step():
        flash_decoding_attention(q, k_cache, v_cache, ck, cv, mask, lens, kv_group_num=hq // hkv, output=out)
        append_accepted_kv(k_cache, v_cache, ck, cv, idx, n_acc, lens)

    keep = (k_cache.clone(), v_cache.clone(), lens.clone())
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                                         # warm-up, then put the state back
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    k_cache.copy_(keep[0]); v_cache.copy_(keep[1]); lens.copy_(keep[2])
    ref_k, ref_v, ref_lens = (t.clone() for t in keep)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    k_cache.copy_(keep[0]); v_cache.copy_(keep[1]); lens.copy_(keep[2])  # capture does not run the step, but be explicit
    for rep in range(4):
        q.copy_(r(bsz, hq, L, D)); ck.copy_(r(bsz, hkv, L, D)); cv.copy_(r(bsz, hkv, L, D))
        n_acc.copy_(torch.tensor([1 + rep, 5 - rep]))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ref = tree_attention_oracle(q, ref_k, ref_v, ck, cv, mask, ref_lens, None, hq // hkv)
        torch.testing.assert_close(out.float(), ref, atol=2e-3, rtol=1e-2)
        ref_k, ref_v, ref_lens = (t.to(DEV) for t in append_accepted_kv_oracle(ref_k, ref_v, ck, cv, idx, n_acc, ref_lens))
        assert torch.equal(lens, ref_lens) and torch.equal(k_cache, ref_k) and torch.equal(v_cache, ref_v)


@pytest.mark.gpu
def test_speculative_loop_decode_append_decode():
    """Two verification steps with an append in between equal the oracle run on a cache
    that was extended by hand."""
    from flash_tree_attn_amd import append_accepted_kv, flash_decoding_attention
    from flash_tree_attn_amd.tree_mask import additive_mask_from_parents, random_tree_parents
    from oracle.tree_attn_oracle import tree_attention_oracle
    g = torch.Generator().manual_seed(9)
    bsz, hq, hkv, L, D, cap = 2, 8, 2, 12, 128, 256
    r = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(DEV)
    k_cache, v_cache = r(bsz, hkv, cap, D), r(bsz, hkv, cap, D)
    lens = torch.tensor([100, 37], dtype=torch.int64, device=DEV)
    ref_k, ref_v, ref_lens = k_cache.clone(), v_cache.clone(), lens.clone()
    for step in range(2):
        parents = random_tree_parents(L, g)
        mask = additive_mask_from_parents(parents, device=DEV)
        q, ck, cv = r(bsz, hq, L, D), r(bsz, hkv, L, D), r(bsz, hkv, L, D)
        out = flash_decoding_attention(q, k_cache, v_cache, ck, cv, mask, lens, kv_group_num=hq // hkv)
        ref = tree_attention_oracle(q, ref_k, ref_v, ck, cv, mask, ref_lens, None, hq // hkv)
        torch.testing.assert_close(out.float(), ref, atol=2e-3, rtol=1e-2)
        # accept a root-to-node path: walk up from a random node
        paths = []
        for b in range(bsz):
            node, path = int(torch.randint(0, L, (1,), generator=g)), []
            while node >= 0:
                path.append(node)
                node = int(parents[node])
            paths.append(path[::-1])
        n_acc = torch.tensor([len(p) for p in paths], dtype=torch.int64, device=DEV)
        idx = torch.zeros(bsz, L, dtype=torch.int32)
        for b, pth in enumerate(paths):
            idx[b, :len(pth)] = torch.tensor(pth, dtype=torch.int32)
        append_accepted_kv(k_cache, v_cache, ck, cv, idx.to(DEV), n_acc, lens)
        for b, pth in enumerate(paths):
            t = int(ref_lens[b])
            ref_k[b, :, t:t + len(pth)] = ck[b][:, pth]
            ref_v[b, :, t:t + len(pth)] = cv[b][:, pth]
            ref_lens[b] = t + len(pth)
        assert torch.equal(lens, ref_lens) and torch.equal(k_cache, ref_k) and torch.equal(v_cache, ref_v)


@pytest.mark.gpu
@pytest.mark.parametrize("page_size", [16, 64])
def test_append_into_paged_caches(page_size):
    """The same append through a block table: gathering the pages back gives the
    contiguous result, bit for bit; pool pages of other sequences are untouched."""
    from flash_tree_attn_amd import append_accepted_kv
    bsz, hkv, L, D, cap = 3, 2, 10, 128, 128
    x = make(6, bsz, hkv, L, D, cap, torch.bfloat16, [15, 126, 64], [5, 5, 3], 5)
    k_ref, v_ref, n_ref = append_accepted_kv_oracle(**x)
    per_seq = cap // page_size
    g = torch.Generator().manual_seed(page_size)
    n_pages = bsz * per_seq + 4
    tables = torch.randperm(n_pages, generator=g)[: bsz * per_seq].view(bsz, per_seq)
    to_pool = lambda c: c.view(bsz, hkv, per_seq, page_size, D).permute(0, 2, 1, 3, 4).reshape(bsz * per_seq, hkv, page_size, D)
    kp = torch.full((n_pages, hkv, page_size, D), 7.0, dtype=torch.bfloat16)
    vp = torch.full_like(kp, -7.0)
    kp[tables.view(-1)], vp[tables.view(-1)] = to_pool(x["k_cache"]), to_pool(x["v_cache"])
    d = {k: v.to(DEV) for k, v in x.items()}
    kpd, vpd = kp.to(DEV), vp.to(DEV)
    d["k_cache"], d["v_cache"] = kpd, vpd
    ret = append_accepted_kv(**d, block_tables=tables.to(torch.int32).to(DEV))
    from_pool = lambda pool: pool.cpu()[tables.view(-1)].view(bsz, per_seq, hkv, page_size, D).permute(0, 2, 1, 3, 4).reshape(bsz, hkv, cap, D)
    assert torch.equal(from_pool(kpd), k_ref) and torch.equal(from_pool(vpd), v_ref) and torch.equal(ret.cpu(), n_ref)
    spare = torch.ones(n_pages, dtype=torch.bool)
    spare[tables.view(-1)] = False
    assert bool((kpd.cpu()[spare] == 7.0).all()) and bool((vpd.cpu()[spare] == -7.0).all())
