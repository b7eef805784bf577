"""Writes the golden fixtures of tests/golden/ from the fp64 oracle.

The reference holds no golden vectors for this path (its only test draws unseeded
random inputs, flash_tree_attn.py:416-440), so these vectors come from this repo's
own oracle, which tests/test_oracle.py pins against torch's SDPA, closed forms and
brute force. Run from the repo root:  python tests/golden/make_golden.py
"""
import hashlib
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from flash_tree_attn_amd.synthetic import CONFIGS, make_inputs  # noqa: E402
from flash_tree_attn_amd.tree_mask import additive_mask_from_parents, random_tree_parents  # noqa: E402
from oracle.tree_attn_oracle import tree_attention_oracle  # noqa: E402


def digest(*tensors) -> str:
    h = hashlib.sha256()
    for t in tensors:
        h.update(t.contiguous().cpu().numpy().tobytes())
    return h.hexdigest()


def cfg1():
    """Workload cfg1_plumbing_fp32 at seed 0: inputs are re-drawn from the seed by the test
    (their digest is stored), the expected fp64 output is stored in full."""
    cfg = CONFIGS["cfg1_plumbing_fp32"]
    x = make_inputs(cfg, seed=0)
    out = tree_attention_oracle(x["q"], x["k_cache"], x["v_cache"], x["current_k"], x["current_v"], x["mask"],
                                x["kv_seq_len"], x["sm_scale"], x["kv_group_num"], dtype=torch.float64)
    np.savez(os.path.join(HERE, "cfg1_seed0.npz"), out=out.numpy(),
             input_digest=np.array(digest(x["q"], x["k_cache"], x["v_cache"], x["current_k"], x["current_v"])))


def tiny_gqa_ragged():
    """A small ragged GQA case stored with its inputs (fp16-representable values)."""
    g = torch.Generator().manual_seed(1234)
    bsz, hq, hkv, L, D, tmax = 2, 4, 2, 5, 32, 24
    rnd = lambda *s: torch.randn(*s, generator=g).half().float()
    q, k, v = rnd(bsz, hq, L, D), rnd(bsz, hkv, tmax, D), rnd(bsz, hkv, tmax, D)
    ck, cv = rnd(bsz, hkv, L, D), rnd(bsz, hkv, L, D)
    parents = random_tree_parents(L, g)
    mask = additive_mask_from_parents(parents)
    lens = torch.tensor([7, 19], dtype=torch.int64)
    out = tree_attention_oracle(q, k, v, ck, cv, mask, lens, None, hq // hkv, dtype=torch.float64)
    np.savez(os.path.join(HERE, "tiny_gqa_ragged.npz"), q=q.numpy(), k=k.numpy(), v=v.numpy(), ck=ck.numpy(),
             cv=cv.numpy(), mask=mask.numpy(), lens=lens.numpy(), parents=parents.numpy(), out=out.numpy())


if __name__ == "__main__":
    cfg1()
    tiny_gqa_ragged()
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
