"""CPU checks of the tree-mask builders: parent array -> ancestor matrix -> additive
mask / packed bit words (the mask the op adds at flash_tree_attn.py:368)."""
import pytest
import torch

from flash_tree_attn_amd.tree_mask import (additive_mask_from_parents, ancestor_matrix, chain_parents, pack_mask,
                                           packed_mask_from_parents, random_tree_parents, unpack_mask)


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
