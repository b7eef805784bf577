"""MI355X-native tree-attention decode: `flash_decoding_attention` on gfx950.

The public function mirrors NonvolatileMemory/flash_tree_attn's
`flash_decoding_attention` (flash_tree_attn.py:216-231) and calls hand-written HIP
kernels through the C ABI declared in include/fta.h.
"""
from .flash_decoding import FtaAssertionError, PreparedCall, flash_decoding_attention, prepare
from .kv_append import append_accepted_kv
from .tree_mask import (accepted_paths, additive_mask_from_parents, ancestor_matrix, chain_parents, pack_mask,
                        packed_mask_from_parents, parents_from_paths, path_to_node, random_tree_parents, unpack_mask)

__all__ = [
    "flash_decoding_attention", "prepare", "PreparedCall", "FtaAssertionError", "append_accepted_kv",
    "additive_mask_from_parents", "ancestor_matrix", "chain_parents", "random_tree_parents",
    "pack_mask", "unpack_mask", "packed_mask_from_parents", "parents_from_paths", "path_to_node", "accepted_paths",
]
