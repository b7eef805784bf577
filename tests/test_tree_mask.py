"""CPU checks of the tree-mask builders: parent array -> ancestor matrix -> additive
mask / packed bit words (the mask the op adds at flash_tree_attn.py:368)."""
import pytest
import torch

from flash_tree_attn_amd.tree_mask import (accepted_paths, additive_mask_from_parents, ancestor_matrix, chain_parents, pack_mask,
                                           packed_mask_from_parents, parents_from_paths, path_to_node, random_tree_parents,
                                           unpack_mask)


def brute_ancestors(parents):
    L = len(parents)
    anc = torch.zeros(L, L, dtype=torch.bool)
    for i in range(L):
        j = i
        while j >= 0:
            anc[i, j] = True
            j = int(parents[j])
    return anc


@pytest.mark.parametrize("L", [1, 2, 7, 26, 64, 100])
def test_ancestor_matrix_is_the_transitive_parent_walk(L):
    g = torch.Generator().manual_seed(L)
    parents = random_tree_parents(L, g)
    anc = ancestor_matrix(parents)
    assert torch.equal(anc, brute_ancestors(parents))
    add = additive_mask_from_parents(parents)
    assert torch.equal(torch.isfinite(add), anc) and bool((add[anc] == 0).all())


def test_chain_is_causal():
    assert torch.equal(ancestor_matrix(chain_parents(9)), torch.tril(torch.ones(9, 9, dtype=torch.bool)))


def test_bad_parent_array_is_rejected():
    with pytest.raises(ValueError):
        ancestor_matrix([-1, 1])      # a node cannot be its own parent
    with pytest.raises(ValueError):
        ancestor_matrix([-1, 2, 0])   # parents must precede their children


@pytest.mark.parametrize("L", [1, 5, 63, 64, 65, 128, 130])
def test_pack_unpack_round_trip(L):
    g = torch.Generator().manual_seed(100 + L)
    allowed = torch.rand(3, 2, L, L, generator=g) < 0.4
    packed = pack_mask(allowed)
    assert packed.dtype == torch.int64 and packed.shape == (3, 2, L, (L + 63) // 64)
    assert torch.equal(unpack_mask(packed, L), allowed)
    # bit j of word j // 64, checked one bit at a time in plain Python
    i, j = L - 1, L - 1
    word = int(packed[1, 1, i, j // 64]) & 0xFFFFFFFFFFFFFFFF
    assert bool((word >> (j % 64)) & 1) == bool(allowed[1, 1, i, j])
    # bits past q_len are clear
    if L % 64:
        assert bool((unpack_mask(packed, ((L + 63) // 64) * 64)[..., L:] == 0).all())


def test_packing_takes_additive_masks_and_refuses_biases():
    parents = random_tree_parents(70, torch.Generator().manual_seed(3))
    add = additive_mask_from_parents(parents)
    assert torch.equal(pack_mask(add), pack_mask(ancestor_matrix(parents)))
    assert torch.equal(packed_mask_from_parents(parents), pack_mask(add))
    with pytest.raises(ValueError):
        pack_mask(torch.where(torch.isfinite(add), torch.ones(()), add))   # the reference's {1, -inf} form is a bias
    full = pack_mask(torch.ones(64, 64, dtype=torch.bool))
    assert bool((full == -1).all())   # all 64 bits set, sign bit included


def test_paths_give_the_parent_array_of_the_tree_they_describe():
    # a small Medusa-style description: two candidates for the first draft position, three below the better one, ...
    paths = [[0], [1], [0, 0], [0, 1], [0, 2], [1, 0], [0, 0, 0]]
    parents = parents_from_paths(paths)
    #        root  [0] [1] [0,0] [0,1] [0,2] [1,0] [0,0,0]
    assert parents.tolist() == [-1, 0, 0, 1, 1, 1, 2, 3]
    anc = ancestor_matrix(parents)
    # node i attends node j iff j's path is a prefix of i's: the definition, node by node
    nodes = [()] + sorted((tuple(q) for q in paths), key=lambda q: (len(q), q))
    for i, pi in enumerate(nodes):
        for j, pj in enumerate(nodes):
            assert bool(anc[i, j]) == (pi[: len(pj)] == pj)
    # the order of the list does not matter, duplicates are one node, a missing parent is an error
    assert torch.equal(parents_from_paths(paths[::-1] + [[1]]), parents)
    with pytest.raises(ValueError):
        parents_from_paths([[0], [1, 0]])
    with pytest.raises(ValueError):
        parents_from_paths([[0], []])
    assert parents_from_paths([]).tolist() == [-1]                     # the root alone
    assert torch.equal(parents_from_paths([[0] * d for d in range(1, 6)]), chain_parents(6))


@pytest.mark.parametrize("L", [1, 9, 64])
def test_accepted_path_is_the_row_of_the_ancestor_matrix(L):
    parents = random_tree_parents(L, torch.Generator().manual_seed(7 * L))
    anc = ancestor_matrix(parents)
    for node in range(L):
        path = path_to_node(parents, node)
        assert path == torch.nonzero(anc[node]).flatten().tolist()      # ancestors in topological order, node last
        assert path[0] == 0 and path[-1] == node
    nodes = [L - 1, 0, L // 2]
    idx, lens = accepted_paths(parents, nodes)
    assert idx.dtype == torch.int32 and lens.dtype == torch.int64 and idx.shape == (3, int(lens.max()))
    for b, node in enumerate(nodes):
        assert idx[b, : lens[b]].tolist() == path_to_node(parents, node) and bool((idx[b, lens[b]:] == 0).all())
    with pytest.raises(ValueError):
        path_to_node(parents, L)


def test_accepted_paths_feed_the_append_as_defined():
    """The pair (accept_idx, accept_len) built from picked nodes, through the append's definition (the oracle): the rows
    that land behind each sequence's end are the tree rows of the path, root first."""
    from oracle.kv_append_oracle import append_accepted_kv_oracle
    g = torch.Generator().manual_seed(5)
    parents = parents_from_paths([[0], [1], [0, 0], [0, 1], [1, 0], [0, 0, 0]])
    L, bsz, hkv, T, D = len(parents), 3, 2, 16, 8
    k, v = torch.randn(bsz, hkv, T, D, generator=g), torch.randn(bsz, hkv, T, D, generator=g)
    ck, cv = torch.randn(bsz, hkv, L, D, generator=g), torch.randn(bsz, hkv, L, D, generator=g)
    lens = torch.tensor([3, 0, 9])
    nodes = [6, 0, 5]                                   # [0, 0, 0], the root alone, [1, 0]
    idx, n_acc = accepted_paths(parents, nodes)
    assert n_acc.tolist() == [4, 1, 3] and idx[0].tolist() == [0, 1, 3, 6] and idx[2, :3].tolist() == [0, 2, 5]
    k2, v2, new_lens = append_accepted_kv_oracle(k, v, ck, cv, idx, n_acc, lens)
    assert new_lens.tolist() == [7, 1, 12]
    for b, node in enumerate(nodes):
        path = path_to_node(parents, node)
        t = int(lens[b])
        assert torch.equal(k2[b, :, t:t + len(path)], ck[b][:, path]) and torch.equal(v2[b, :, t:t + len(path)], cv[b][:, path])
        assert torch.equal(k2[b, :, :t], k[b, :, :t]) and torch.equal(k2[b, :, t + len(path):], k[b, :, t + len(path):])
