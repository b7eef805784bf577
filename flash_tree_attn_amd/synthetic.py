"""Seeded synthetic inputs for the five benchmark / parity configurations (and two plain-decode shapes).

Values are drawn in fp32 and cast, the tree comes from `tree_mask`, lengths are
int64 like the reference's test (flash_tree_attn.py:434). Small configurations are
drawn on the CPU so a CPU checker and the GPU see identical values; the large ones
(`gen_device="cuda"`) are drawn on the device to keep generation in seconds.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, Optional

import torch

from .tree_mask import additive_mask_from_parents, chain_parents, random_tree_parents


@dataclass(frozen=True)
class Config:
    name: str
    bsz: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    q_len: int
    cache_len: int
    dtype: torch.dtype
    lengths: str        # "full" | "uniform:lo:hi" | "loguniform:lo:hi"
    tree: str           # "chain" | "random"
    block_size: int = 64

    @property
    def kv_group_num(self) -> int:
        return self.num_heads // self.num_kv_heads


CONFIGS: Dict[str, Config] = {
    "cfg1_plumbing_fp32": Config("cfg1_plumbing_fp32", 1, 8, 8, 64, 4, 256, torch.float32, "full", "chain"),
    "cfg2_medusa_7b_fp16": Config("cfg2_medusa_7b_fp16", 4, 32, 32, 128, 26, 4096, torch.float16, "uniform:1024:4096", "random"),
    "cfg3_gqa_8b_bf16": Config("cfg3_gqa_8b_bf16", 8, 32, 8, 128, 64, 8192, torch.bfloat16, "full", "random"),
    "cfg4_long_ctx_bf16": Config("cfg4_long_ctx_bf16", 1, 32, 8, 128, 64, 131072, torch.bfloat16, "full", "random"),
    "cfg5_ragged_70b_bf16": Config("cfg5_ragged_70b_bf16", 64, 64, 8, 128, 16, 32768, torch.bfloat16, "loguniform:512:32768", "random"),
    # units below one MFMA tile (not BASELINE configurations): plain decode, one row per unit, and one token on a GQA-4 model
    "decode1_mha_fp16": Config("decode1_mha_fp16", 8, 32, 32, 128, 1, 32768, torch.float16, "full", "chain"),
    "decode1_gqa4_bf16": Config("decode1_gqa4_bf16", 64, 32, 8, 128, 1, 4096, torch.bfloat16, "full", "chain"),
    # the shape of the reference's own test (flash_tree_attn.py:416,435: Z 32, H 32, N_CTX 4096, D 128, q_len 128, block 128)
    "reftest_mha_fp16": Config("reftest_mha_fp16", 32, 32, 32, 128, 128, 4096, torch.float16, "full", "random", 128),
    # the headline shape inside a cache allocated for 64K positions: the lengths, not the capacity, must set the cut
    "cfg3_in_64k_cache_bf16": Config("cfg3_in_64k_cache_bf16", 8, 32, 8, 128, 64, 65536, torch.bfloat16, "uniform:8192:8192", "random"),
    # head_dim 256 (two query heads per cache head), tree of 64
    "d256_gqa2_bf16": Config("d256_gqa2_bf16", 8, 16, 8, 256, 64, 8192, torch.bfloat16, "full", "random"),
}


def sample_lengths(cfg: Config, gen: torch.Generator) -> torch.Tensor:
    if cfg.lengths == "full":
        return torch.full((cfg.bsz,), cfg.cache_len, dtype=torch.int64)
    kind, lo, hi = cfg.lengths.split(":")
    lo, hi = int(lo), int(hi)
    u = torch.rand(cfg.bsz, generator=gen, dtype=torch.float64)
    if kind == "uniform":
        t = lo + torch.floor(u * (hi - lo + 1))
    elif kind == "loguniform":
        t = torch.floor(torch.exp(math.log(lo) + u * (math.log(hi) - math.log(lo))))
    else:
        raise ValueError(cfg.lengths)
    return t.clamp(lo, hi).to(torch.int64)


def make_inputs(cfg: Config, seed: int = 0, device: str = "cpu", gen_device: Optional[str] = None,
                kv_sets: int = 1) -> dict:
    """Returns q, k_cache, v_cache, current_k, current_v, mask, kv_seq_len, sm_scale, ...
    With kv_sets > 1, `k_caches` / `v_caches` hold that many independent caches (for
    rotating buffers in a benchmark); k_cache / v_cache are the first."""
    cpu_gen = torch.Generator().manual_seed(seed)
    gen_device = gen_device or "cpu"
    if gen_device == "cpu":
        vgen = cpu_gen
    else:
        vgen = torch.Generator(device=gen_device).manual_seed(seed)

    def normal(*shape):
        x = torch.randn(*shape, generator=vgen, device=gen_device, dtype=torch.float32)
        return x.to(cfg.dtype).to(device)

    parents = chain_parents(cfg.q_len) if cfg.tree == "chain" else random_tree_parents(cfg.q_len, cpu_gen)
    lens = sample_lengths(cfg, cpu_gen)
    q = normal(cfg.bsz, cfg.num_heads, cfg.q_len, cfg.head_dim)
    cur_k = normal(cfg.bsz, cfg.num_kv_heads, cfg.q_len, cfg.head_dim)
    cur_v = normal(cfg.bsz, cfg.num_kv_heads, cfg.q_len, cfg.head_dim)
    k_caches = [normal(cfg.bsz, cfg.num_kv_heads, cfg.cache_len, cfg.head_dim) for _ in range(kv_sets)]
    v_caches = [normal(cfg.bsz, cfg.num_kv_heads, cfg.cache_len, cfg.head_dim) for _ in range(kv_sets)]
    return {
        "q": q, "k_cache": k_caches[0], "v_cache": v_caches[0], "current_k": cur_k, "current_v": cur_v,
        "k_caches": k_caches, "v_caches": v_caches,
        "mask": additive_mask_from_parents(parents, device=device),
        "kv_seq_len": lens.to(device), "parents": parents,
        "sm_scale": 1.0 / math.sqrt(cfg.head_dim), "block_size": cfg.block_size,
        "kv_group_num": cfg.kv_group_num,
    }


def algorithmic_bytes(cfg: Config, kv_seq_len: torch.Tensor, mask: torch.Tensor) -> int:
    """Bytes the path must move at minimum: K/V cache rows below kv_seq_len, current
    k/v, q, the output, the mask and the lengths. Scratch and padding do not count."""
    esz = torch.empty((), dtype=cfg.dtype).element_size()
    total_t = int(kv_seq_len.sum())
    kv = 2 * cfg.num_kv_heads * total_t * cfg.head_dim * esz
    cur = 2 * cfg.bsz * cfg.num_kv_heads * cfg.q_len * cfg.head_dim * esz
    qo = 2 * cfg.bsz * cfg.num_heads * cfg.q_len * cfg.head_dim * esz
    return kv + cur + qo + mask.numel() * mask.element_size() + cfg.bsz * 8


def flops(cfg: Config, kv_seq_len: torch.Tensor) -> int:
    total = int(kv_seq_len.sum()) + cfg.bsz * cfg.q_len
    return 4 * cfg.num_heads * cfg.q_len * total * cfg.head_dim
