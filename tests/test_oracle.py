"""Pins the CPU oracle without the reference: against torch's SDPA (a library
routine), closed forms, invariants and brute force. A dropped term, wrong sign,
transposed operand or wrong head mapping in the oracle fails at least one of these."""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from flash_tree_attn_amd.synthetic import CONFIGS, make_inputs
from flash_tree_attn_amd.tree_mask import (additive_mask_from_parents, ancestor_matrix, chain_parents,
                                           random_tree_parents)
from oracle import tree_attn_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def rand_case(seed, bsz=2, hq=4, hkv=2, L=6, D=16, tmax=40, lens=None, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=dtype)
    q, k, v = r(bsz, hq, L, D), r(bsz, hkv, tmax, D), r(bsz, hkv, tmax, D)
    ck, cv = r(bsz, hkv, L, D), r(bsz, hkv, L, D)
    mask = additive_mask_from_parents(random_tree_parents(L, g)).to(dtype)
    if lens is None:
        lens = torch.randint(1, tmax + 1, (bsz,), generator=g)
    return q, k, v, ck, cv, mask, torch.as_tensor(lens, dtype=torch.int64)


def sdpa_reference(q, k, v, ck, cv, mask, lens, scale, G):
    """torch.nn.functional.scaled_dot_product_attention per sequence on [cache[:T]; tree]."""
    bsz, hq, L, D = q.shape
    outs = []
    for b in range(bsz):
        T = int(lens[b])
        kk = torch.cat([k[b, :, :T], ck[b]], dim=1).repeat_interleave(G, dim=0)
        vv = torch.cat([v[b, :, :T], cv[b]], dim=1).repeat_interleave(G, dim=0)
        am = torch.cat([torch.zeros(L, T, dtype=q.dtype), mask], dim=1)
        outs.append(F.scaled_dot_product_attention(q[b][None], kk[None], vv[None], attn_mask=am, scale=scale)[0])
    return torch.stack(outs)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_whole_path_equals_sdpa(seed):
    q, k, v, ck, cv, mask, lens = rand_case(seed)
    scale = 0.37
    ref = sdpa_reference(q, k, v, ck, cv, mask, lens, scale, 2)
    out = O.tree_attention_oracle(q, k, v, ck, cv, mask, lens, scale, 2, dtype=torch.float64)
    torch.testing.assert_close(out, ref, atol=1e-12, rtol=1e-10)


def test_chain_tree_is_causal_attention():
    """Chain tree (the mask of workload cfg1_plumbing_fp32) == SDPA is_causal on the last L positions."""
    q, k, v, ck, cv, _, _ = rand_case(3, bsz=1, hq=2, hkv=2, L=4, D=8, tmax=12)
    lens = torch.tensor([12])
    mask = additive_mask_from_parents(chain_parents(4)).double()
    out = O.tree_attention_oracle(q, k, v, ck, cv, mask, lens, None, 1, dtype=torch.float64)
    kk, vv = torch.cat([k, ck], dim=2), torch.cat([v, cv], dim=2)
    qfull = torch.cat([torch.zeros(1, 2, 12, 8, dtype=torch.float64), q], dim=2)
    ref = F.scaled_dot_product_attention(qfull, kk, vv, is_causal=True)[:, :, -4:]
    torch.testing.assert_close(out, ref, atol=1e-12, rtol=1e-10)


def test_zero_mask_is_plain_attention():
    q, k, v, ck, cv, _, lens = rand_case(4)
    out = O.tree_attention_oracle(q, k, v, ck, cv, torch.zeros(6, 6, dtype=torch.float64), lens, None, 2, dtype=torch.float64)
    ref = sdpa_reference(q, k, v, ck, cv, torch.zeros(6, 6, dtype=torch.float64), lens, 1 / math.sqrt(16), 2)
    torch.testing.assert_close(out, ref, atol=1e-12, rtol=1e-10)


def test_constant_v_gives_constant_output():
    q, k, v, ck, cv, mask, lens = rand_case(5)
    v = torch.full_like(v, 2.5)
    cv = torch.full_like(cv, 2.5)
    out = O.tree_attention_oracle(q, k, v, ck, cv, mask, lens, None, 2, dtype=torch.float64)
    torch.testing.assert_close(out, torch.full_like(out, 2.5), atol=1e-12, rtol=0)


def test_zero_q_gives_mean_of_allowed_values():
    q, k, v, ck, cv, mask, lens = rand_case(6, bsz=1, hq=2, hkv=1, L=5)
    q = torch.zeros_like(q)
    out = O.tree_attention_oracle(q, k, v, ck, cv, mask, lens, None, 2, dtype=torch.float64)
    T = int(lens[0])
    for i in range(5):
        allowed = torch.isfinite(mask[i])
        mean = (v[0, 0, :T].sum(0) + cv[0, 0][allowed].sum(0)) / (T + int(allowed.sum()))
        torch.testing.assert_close(out[0, 0, i], mean, atol=1e-12, rtol=1e-10)
        torch.testing.assert_close(out[0, 1, i], mean, atol=1e-12, rtol=1e-10)


def test_gqa_equals_mha_on_expanded_kv():
    q, k, v, ck, cv, mask, lens = rand_case(7)
    out = O.tree_attention_oracle(q, k, v, ck, cv, mask, lens, None, 2, dtype=torch.float64)
    e = lambda x: x.repeat_interleave(2, dim=1)
    out_mha = O.tree_attention_oracle(q, e(k), e(v), e(ck), e(cv), mask, lens, None, 1, dtype=torch.float64)
    torch.testing.assert_close(out, out_mha, atol=1e-13, rtol=0)
    # tree K/V may also come with one head per query head (flash_tree_attn.py:424-425)
    out_hq_tree = O.tree_attention_oracle(q, k, v, e(ck), e(cv), mask, lens, None, 2, dtype=torch.float64)
    torch.testing.assert_close(out, out_hq_tree, atol=1e-13, rtol=0)


def test_mask_is_additive_not_boolean():
    """The reference's generator emits {1, -inf} (flash_tree_attn.py:403-414): allowed tree
    logits get +1. Equivalent to a {0,-inf} mask with every cache logit lowered by 1, i.e.
    scale*q.(k) - 1 -> append a constant feature."""
    q, k, v, ck, cv, mask, lens = rand_case(8, bsz=1, hq=2, hkv=2, L=4, D=8, tmax=10)
    lens = torch.tensor([10])
    plus_one = torch.where(torch.isfinite(mask), torch.ones_like(mask), mask)
    out = O.tree_attention_oracle(q, k, v, ck, cv, plus_one, lens, 1.0, 1, dtype=torch.float64)
    # extra feature: q gets 1, cache keys get -1, tree keys get 0  -> cache logits shift by -1
    q2 = torch.cat([q, torch.ones(1, 2, 4, 1, dtype=torch.float64)], -1)
    k2 = torch.cat([k, -torch.ones(1, 2, 10, 1, dtype=torch.float64)], -1)
    ck2 = torch.cat([ck, torch.zeros(1, 2, 4, 1, dtype=torch.float64)], -1)
    ref = sdpa_reference(q2, k2, v, ck2, cv, mask, lens, 1.0, 1)
    torch.testing.assert_close(out, ref, atol=1e-12, rtol=1e-10)


def test_bool_mask_means_allowed():
    q, k, v, ck, cv, mask, lens = rand_case(9)
    out_f = O.tree_attention_oracle(q, k, v, ck, cv, mask, lens, None, 2, dtype=torch.float64)
    out_b = O.tree_attention_oracle(q, k, v, ck, cv, torch.isfinite(mask), lens, None, 2, dtype=torch.float64)
    torch.testing.assert_close(out_f, out_b, atol=0, rtol=0)


def test_brute_force_tiny():
    q, k, v, ck, cv, mask, lens = rand_case(10, bsz=1, hq=2, hkv=1, L=3, D=2, tmax=8, lens=[5])
    out = O.tree_attention_oracle(q, k, v, ck, cv, mask, lens, 0.8, 2, dtype=torch.float64)
    ref = O.brute_force_oracle(q, k, v, ck, cv, mask, lens, 0.8, 2)
    torch.testing.assert_close(out, ref, atol=1e-13, rtol=1e-12)


def test_stage1_partial_closed_form():
    g = torch.Generator().manual_seed(11)
    qb, kb, vb = (torch.randn(3, 5, 8, generator=g, dtype=torch.float64), torch.randn(3, 20, 8, generator=g, dtype=torch.float64),
                  torch.randn(3, 20, 8, generator=g, dtype=torch.float64))
    acc, lse = O.stage1_partial_oracle(qb, kb, vb, 4, 13, 0.5)
    ref = F.scaled_dot_product_attention(qb[None], kb[None, :, 4:13], vb[None, :, 4:13], scale=0.5)[0]
    torch.testing.assert_close(acc, ref, atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(lse, torch.logsumexp(0.5 * qb @ kb[:, 4:13].transpose(1, 2), dim=-1), atol=1e-12, rtol=1e-10)


def test_stage2_merge_invariants():
    g = torch.Generator().manual_seed(12)
    qb, kb, vb = (torch.randn(2, 4, 8, generator=g, dtype=torch.float64), torch.randn(2, 30, 8, generator=g, dtype=torch.float64),
                  torch.randn(2, 30, 8, generator=g, dtype=torch.float64))
    full, full_lse = O.stage1_partial_oracle(qb, kb, vb, 0, 30, 0.3)
    for cuts in ([0, 30], [0, 7, 30], [0, 1, 2, 29, 30], [0, 10, 20, 30]):
        parts = [O.stage1_partial_oracle(qb, kb, vb, a, b, 0.3) for a, b in zip(cuts[:-1], cuts[1:])]
        for order in (parts, parts[::-1]):
            o, lse = O.stage2_merge_oracle([p[0] for p in order], [p[1] for p in order])
            torch.testing.assert_close(o, full, atol=1e-12, rtol=1e-10)
            torch.testing.assert_close(lse, full_lse, atol=1e-12, rtol=1e-10)
    # duplicate partial: same output, lse + ln 2
    o, lse = O.stage2_merge_oracle([full, full], [full_lse, full_lse])
    torch.testing.assert_close(o, full, atol=1e-13, rtol=0)
    torch.testing.assert_close(lse, full_lse + math.log(2), atol=1e-12, rtol=0)
    # a dead partial (lse = -inf) is ignored
    o, lse = O.stage2_merge_oracle([torch.zeros_like(full), full], [torch.full_like(full_lse, -math.inf), full_lse])
    torch.testing.assert_close(o, full, atol=1e-13, rtol=0)


def test_final_merge_is_exp_weighted_mean():
    g = torch.Generator().manual_seed(13)
    oa, ob = torch.randn(3, 4, 8, generator=g, dtype=torch.float64), torch.randn(3, 4, 8, generator=g, dtype=torch.float64)
    la, lb = torch.randn(3, 4, generator=g, dtype=torch.float64) * 3, torch.randn(3, 4, generator=g, dtype=torch.float64) * 3
    out = O.final_merge_oracle(oa, la, ob, lb)
    wa, wb = torch.exp(la)[..., None], torch.exp(lb)[..., None]
    torch.testing.assert_close(out, (wa * oa + wb * ob) / (wa + wb), atol=1e-12, rtol=1e-10)


@pytest.mark.parametrize("block", [16, 64])
def test_two_stage_restatement_equals_whole_path(block):
    q, k, v, ck, cv, mask, lens = rand_case(14, tmax=150, lens=[150, 37])
    a = O.tree_attention_oracle(q, k, v, ck, cv, mask, lens, None, 2, dtype=torch.float64)
    b = O.two_stage_oracle(q, k, v, ck, cv, mask, lens, block, None, 2, dtype=torch.float64)
    torch.testing.assert_close(a, b, atol=1e-12, rtol=1e-10)


def test_edge_conventions():
    q, k, v, ck, cv, mask, _ = rand_case(15)
    # T_b = 0: tree-only attention
    lens = torch.tensor([0, 3])
    out = O.tree_attention_oracle(q, k, v, ck, cv, mask, lens, None, 2, dtype=torch.float64)
    tree_only = F.scaled_dot_product_attention(q[0][None], ck[0].repeat_interleave(2, 0)[None], cv[0].repeat_interleave(2, 0)[None], attn_mask=mask)[0]
    torch.testing.assert_close(out[0], tree_only, atol=1e-12, rtol=1e-10)
    # fully masked tree row with T_b > 0: cache-only attention; with T_b = 0: zeros
    dead = mask.clone()
    dead[2, :] = -math.inf
    out = O.tree_attention_oracle(q, k, v, ck, cv, dead, lens, None, 2, dtype=torch.float64)
    assert torch.all(out[0, :, 2] == 0) and torch.isfinite(out).all()
    cache_only = F.scaled_dot_product_attention(q[1][None], k[1, :, :3].repeat_interleave(2, 0)[None], v[1, :, :3].repeat_interleave(2, 0)[None])[0]
    torch.testing.assert_close(out[1, :, 2], cache_only[:, 2], atol=1e-12, rtol=1e-10)
    b2 = O.two_stage_oracle(q, k, v, ck, cv, dead, lens, 16, None, 2, dtype=torch.float64)
    torch.testing.assert_close(out, b2, atol=1e-12, rtol=1e-10)


def test_tree_mask_builders():
    anc = ancestor_matrix([-1, 0, 0, 1, 3, 2])
    expect = torch.tensor([[1, 0, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0], [1, 0, 1, 0, 0, 0], [1, 1, 0, 1, 0, 0],
                           [1, 1, 0, 1, 1, 0], [1, 0, 1, 0, 0, 1]], dtype=torch.bool)
    assert torch.equal(anc, expect)
    assert torch.equal(ancestor_matrix(chain_parents(5)), torch.ones(5, 5).tril().bool())
    with pytest.raises(ValueError):
        ancestor_matrix([-1, 1])


def test_golden_cfg1_seed0():
    data = np.load(os.path.join(GOLDEN, "cfg1_seed0.npz"))
    import hashlib
    x = make_inputs(CONFIGS["cfg1_plumbing_fp32"], seed=0)
    h = hashlib.sha256()
    for t in (x["q"], x["k_cache"], x["v_cache"], x["current_k"], x["current_v"]):
        h.update(t.contiguous().numpy().tobytes())
    if h.hexdigest() != str(data["input_digest"]):
        pytest.skip("torch's CPU generator stream differs from the one the fixture was drawn with")
    out = O.tree_attention_oracle(x["q"], x["k_cache"], x["v_cache"], x["current_k"], x["current_v"], x["mask"],
                                  x["kv_seq_len"], x["sm_scale"], 1, dtype=torch.float32)
    torch.testing.assert_close(out.double(), torch.from_numpy(data["out"]), atol=2e-6, rtol=1e-5)
    two = O.two_stage_oracle(x["q"], x["k_cache"], x["v_cache"], x["current_k"], x["current_v"], x["mask"],
                             x["kv_seq_len"], 64, x["sm_scale"], 1, dtype=torch.float32)
    torch.testing.assert_close(two.double(), torch.from_numpy(data["out"]), atol=2e-6, rtol=1e-5)


def test_golden_tiny_gqa_ragged():
    d = np.load(os.path.join(GOLDEN, "tiny_gqa_ragged.npz"))
    t = lambda n: torch.from_numpy(d[n])
    out = O.tree_attention_oracle(t("q"), t("k"), t("v"), t("ck"), t("cv"), t("mask"), t("lens"), None, 2, dtype=torch.float32)
    torch.testing.assert_close(out.double(), t("out"), atol=2e-6, rtol=1e-5)
    ref = sdpa_reference(t("q").double(), t("k").double(), t("v").double(), t("ck").double(), t("cv").double(),
                         t("mask").double(), t("lens"), 1 / math.sqrt(32), 2)
    torch.testing.assert_close(ref, t("out"), atol=1e-12, rtol=1e-10)
