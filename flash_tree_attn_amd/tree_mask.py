"""Tree-mask builders for speculative-decoding verification.

The reference's own generator (flash_tree_attn.py:403-414) draws an unseeded random
{1, -inf} matrix that is not a tree; real callers (Medusa / EAGLE style drafts) hold
a parent array, or a list of paths from which one follows (`parents_from_paths`). These
helpers turn a parent array into the ADDITIVE mask the op
consumes (flash_tree_attn.py:368): 0 where column j is an ancestor of, or equal to,
row i, and -inf elsewhere; or into the PACKED form, one bit per (row, tree key) in
64-bit words (8 bytes per row and 64 keys instead of 256), which the kernels expand to
0 / -inf themselves.
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


def parents_from_paths(paths: Sequence[Sequence[int]]) -> torch.Tensor:
    """Parent array of a draft tree given the way Medusa-style drafts describe it: one entry per
    non-root node, the tuple of child ranks that leads to it from the root ((0,), (0, 0), (1,),
    (0, 1), ...). Node 0 is the root (the last accepted token); the other nodes follow in order of
    (depth, path), so parents precede their children and siblings are ordered by rank. Every
    proper prefix of a path must be a path of the list itself."""
    nodes = sorted({tuple(int(c) for c in path) for path in paths}, key=lambda path: (len(path), path))
    if any(len(path) == 0 for path in nodes):
        raise ValueError("the empty path is the root and is not listed")
    index = {(): 0}
    parents = [-1]
    for path in nodes:
        if path[:-1] not in index:
            raise ValueError(f"path {list(path)} has no parent {list(path[:-1])} in the list")
        index[path] = len(parents)
        parents.append(index[path[:-1]])
    return torch.tensor(parents, dtype=torch.int64)


def path_to_node(parents: Sequence[int], node: int) -> list:
    """Tree positions from the root to `node`, both included: the accepted path whose K/V rows
    `append_accepted_kv` moves into the cache once verification has picked `node`."""
    p = [int(x) for x in parents]
    if not 0 <= int(node) < len(p):
        raise ValueError(f"node {node} is not in [0, {len(p)})")
    path, j = [], int(node)
    while j >= 0:
        if len(path) > len(p):
            raise ValueError("the parent array has a cycle")
        path.append(j)
        j = p[j]
    return path[::-1]


def accepted_paths(parents: Sequence[int], nodes: Sequence[int], device=None):
    """(accept_idx int32 [bsz, longest path], accept_len int64 [bsz]) for `append_accepted_kv`: row b
    holds the positions from the root to nodes[b], padded with zeros behind accept_len[b]."""
    paths = [path_to_node(parents, n) for n in nodes]
    width = max(len(path) for path in paths)
    idx = torch.zeros(len(paths), width, dtype=torch.int32)
    for b, path in enumerate(paths):
        idx[b, : len(path)] = torch.tensor(path, dtype=torch.int32)
    lens = torch.tensor([len(path) for path in paths], dtype=torch.int64)
    return (idx.to(device), lens.to(device)) if device is not None else (idx, lens)


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


def pack_mask(allowed: torch.Tensor) -> torch.Tensor:
    """Packs a boolean "may attend" tensor [..., L, L] (or an additive mask: finite =
    attend) into int64 words [..., L, ceil(L/64)]: bit (j % 64) of word j // 64 of row i
    is set iff row i attends tree key j. The words are uint64 bit patterns stored in
    int64 (the dtype torch can index and move); `flash_decoding_attention` takes an int64
    mask to be this form. Additive values other than 0 / -inf cannot be packed."""
    if allowed.dtype != torch.bool:
        finite = torch.isfinite(allowed)
        if bool(((allowed != 0) & finite).any()):
            raise ValueError("only 0 / -inf additive masks can be packed")
        allowed = finite
    L = allowed.size(-1)
    if allowed.dim() < 2 or allowed.size(-2) != L:
        raise ValueError(f"mask must be [..., q_len, q_len], got {tuple(allowed.shape)}")
    words = (L + 63) // 64
    pad = words * 64 - L
    a = torch.nn.functional.pad(allowed, (0, pad)).reshape(*allowed.shape[:-1], words, 64).to(torch.int64)
    weights = torch.ones(64, dtype=torch.int64, device=allowed.device) << torch.arange(64, device=allowed.device)
    return (a * weights).sum(-1)   # bit 63 wraps into the sign bit: the intended bit pattern


def unpack_mask(packed: torch.Tensor, q_len: int) -> torch.Tensor:
    """Inverse of pack_mask: boolean [..., q_len, q_len]."""
    shifts = torch.arange(64, device=packed.device)
    bits = ((packed.unsqueeze(-1) >> shifts) & 1).bool()
    return bits.reshape(*packed.shape[:-1], packed.size(-1) * 64)[..., :q_len]


def packed_mask_from_parents(parents: Sequence[int], device=None) -> torch.Tensor:
    """[L, ceil(L/64)] packed ancestor-or-self mask of a parent array."""
    m = pack_mask(ancestor_matrix(parents))
    return m.to(device) if device is not None else m
