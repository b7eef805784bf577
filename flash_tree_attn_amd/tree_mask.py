"""Tree-mask builders for speculative-decoding verification.

The reference's own generator (flash_tree_attn.py:403-414) draws an unseeded random
{1, -inf} matrix that is not a tree; real callers (Medusa / EAGLE style drafts) hold
a parent array. These helpers turn a parent array into the ADDITIVE mask the op
consumes (flash_tree_attn.py:368): 0 where column j is an ancestor of, or equal to,
row i, and -inf elsewhere.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch


def random_tree_parents(q_len: int, generator: Optional[torch.Generator] = None) -> torch.Tensor:
    """parent[0] = -1 (root), parent[i] ~ Uniform{0..i-1}: a random draft tree in
    topological order."""
    parents = torch.full((q_len,), -1, dtype=torch.int64)
    for i in range(1, q_len):
        parents[i] = int(torch.randint(0, i, (1,), generator=generator))
    return parents


def chain_parents(q_len: int) -> torch.Tensor:
    """A chain: token i's parent is i-1; its ancestor mask is the causal mask."""
    return torch.arange(-1, q_len - 1, dtype=torch.int64)


def ancestor_matrix(parents: Sequence[int]) -> torch.Tensor:
    """Boolean [L, L]: entry (i, j) is True iff j is i or an ancestor of i. Parents
    must precede their children (parent[i] < i), roots carry -1."""
    p = [int(x) for x in parents]
    L = len(p)
    anc = torch.zeros(L, L, dtype=torch.bool)
    for i in range(L):
        if not (-1 <= p[i] < i):
            raise ValueError(f"parent[{i}] = {p[i]} is not in [-1, {i})")
        if p[i] >= 0:
            anc[i] = anc[p[i]]
        anc[i, i] = True
    return anc


def additive_mask_from_parents(parents: Sequence[int], device=None, dtype=torch.float32) -> torch.Tensor:
    """[L, L] additive mask: 0 on ancestor-or-self, -inf elsewhere."""
    anc = ancestor_matrix(parents)
    mask = torch.full(anc.shape, float("-inf"), dtype=dtype)
    mask[anc] = 0.0
    return mask.to(device) if device is not None else mask
