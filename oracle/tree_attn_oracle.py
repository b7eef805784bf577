"""CPU oracle for `flash_decoding_attention` (tree-attention decode).

TEST INFRASTRUCTURE ONLY: the shipped package never imports this module. It is
used by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg as
the checker / CPU baseline.

All functions are plain torch and run on whatever device their inputs live on
(CPU for the baseline and the CPU test-suite; the GPU parity tests may also feed
them device tensors so that full-size configurations finish in seconds).

Two independent restatements live here, plus a brute-force loop version:

* `tree_attention_oracle`  - the definition of "correct" for the whole path:
  softmax attention of the L tree queries over [cache[:T_b] ; tree keys] with the
  additive tree mask on the tree-key block. This is what the reference's own test
  asserts against (flash_tree_attn.py:388-397, :431, :440), written per sequence
  so that ragged kv_seq_len never reads cache padding.
* `two_stage_oracle`       - a restatement of the reference *algorithm*:
  per-split normalised partials + lse (flash_tree_attn.py:49-144), the streaming
  LSE merge (flash_tree_attn.py:174-211), the eager tree block
  (flash_tree_attn.py:367-371) and the sigmoid merge (flash_tree_attn.py:373),
  all in one chosen float type instead of the reference's mixed fp16 rounding.
* `brute_force_oracle`     - pure-Python float loops for tiny shapes.

Pinning (see tests/test_oracle.py): whole path == torch SDPA per sequence with
the mask pasted on the bottom-right corner; chain tree == causal attention;
stage-1 lse == torch.logsumexp of the slice; merge invariants (partition
independence, S=1 identity, duplicate partial => lse + ln 2); sigmoid merge ==
exp-weighted mean in fp64; V == const => output const; q == 0 => mean of allowed
V rows; GQA == MHA on expanded KV; {1,-inf} mask == {0,-inf} mask with cache
logits shifted; brute force on tiny shapes. The reference holds no golden
vectors for this path (its one test is unseeded, flash_tree_attn.py:416-440), so
the committed fixtures under tests/golden/ come from this oracle in fp64.

Conventions that the reference leaves undefined (it yields NaN there) and this
oracle fixes: a query row whose every logit is -inf returns zeros; T_b == 0 is
tree-only attention.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import torch


def _expand_heads(x: torch.Tensor, num_q_heads: int) -> torch.Tensor:
    """[Hx, T, D] -> [Hq, T, D]; Hx may be Hkv (each KV head serves G consecutive
    query heads, flash_tree_attn.py:71) or already Hq (flash_tree_attn.py:424)."""
    hx = x.shape[0]
    if hx == num_q_heads:
        return x
    assert num_q_heads % hx == 0
    return x.repeat_interleave(num_q_heads // hx, dim=0)


def _mask_for(mask: torch.Tensor, b: int, bsz: int, hq: int, L: int, dtype) -> torch.Tensor:
    """Additive mask of sequence b broadcast to [Hq, L, L] (flash_tree_attn.py:368)."""
    if mask.dtype == torch.bool:
        m = torch.zeros(mask.shape, dtype=dtype, device=mask.device)
        m.masked_fill_(~mask, float("-inf"))
    else:
        m = mask.to(dtype)
    m = m.expand(bsz, hq, L, L) if m.dim() == 4 else m.expand(hq, L, L).unsqueeze(0).expand(bsz, hq, L, L)
    return m[b]


def _safe_softmax_av(s: torch.Tensor, v: torch.Tensor):
    """softmax(s) @ v and logsumexp(s) with all -inf rows -> zeros / -inf."""
    m = s.max(dim=-1, keepdim=True).values
    m_safe = torch.where(torch.isinf(m) & (m < 0), torch.zeros_like(m), m)
    p = torch.exp(s - m_safe)
    l = p.sum(dim=-1, keepdim=True)
    o = torch.matmul(p, v) / torch.where(l == 0, torch.ones_like(l), l)
    lse = torch.where(l == 0, torch.full_like(l, float("-inf")), m_safe + torch.log(l))
    return o, lse.squeeze(-1)


def tree_attention_oracle(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    current_k: torch.Tensor,
    current_v: torch.Tensor,
    mask: torch.Tensor,
    kv_seq_len: torch.Tensor,
    sm_scale: Optional[float] = None,
    kv_group_num: int = 1,
    dtype: torch.dtype = torch.float32,
    return_lse: bool = False,
):
    """Whole-path oracle in `dtype` (fp32 for parity, fp64 for fixtures).

    Definition (flash_tree_attn.py:388-397): logits = scale * q @ [K;k_cur]^T with
    `mask` ADDED to the last L columns (flash_tree_attn.py:391-392), softmax over
    all T_b + L columns, times [V;v_cur]. Returns [bsz, Hq, L, D] in `dtype`.
    """
    bsz, hq, L, D = q.shape
    assert hq % kv_group_num == 0 and k_cache.shape[1] * kv_group_num == hq
    scale = 1.0 / math.sqrt(D) if sm_scale is None else float(sm_scale)
    out = torch.zeros(bsz, hq, L, D, dtype=dtype, device=q.device)
    lse_out = torch.zeros(bsz, hq, L, dtype=dtype, device=q.device)
    lens = [int(t) for t in kv_seq_len.tolist()]
    for b in range(bsz):
        T = lens[b]
        qb = q[b].to(dtype)
        kb = torch.cat([_expand_heads(k_cache[b, :, :T].to(dtype), hq), _expand_heads(current_k[b].to(dtype), hq)], dim=1)
        vb = torch.cat([_expand_heads(v_cache[b, :, :T].to(dtype), hq), _expand_heads(current_v[b].to(dtype), hq)], dim=1)
        s = torch.matmul(qb, kb.transpose(1, 2)) * scale
        s[:, :, T:] += _mask_for(mask, b, bsz, hq, L, dtype)
        o, lse = _safe_softmax_av(s, vb)
        out[b] = o
        lse_out[b] = lse
    return (out, lse_out) if return_lse else out


# --------------------------------------------------------------------------- #
# Restatement of the reference's two-stage algorithm
# --------------------------------------------------------------------------- #

def stage1_partial_oracle(qb, kb, vb, start: int, end: int, scale: float):
    """One split of stage 1 for one sequence (flash_tree_attn.py:49-144).

    qb [Hq, L, D]; kb, vb [Hq, T, D] already head-expanded; keys [start, end).
    Returns the NORMALISED partial (acc / l, flash_tree_attn.py:121) and
    lse = m + log l (flash_tree_attn.py:144)."""
    s = torch.matmul(qb, kb[:, start:end].transpose(1, 2)) * scale   # :110-112
    m = s.max(dim=-1, keepdim=True).values                             # :113
    p = torch.exp(s - m)                                               # :114-115
    l = p.sum(dim=-1, keepdim=True)                                    # :116
    acc = torch.matmul(p, vb[:, start:end]) / l                        # :120-121
    return acc, (m + torch.log(l)).squeeze(-1)                         # :144


def stage2_merge_oracle(mid_o: Sequence[torch.Tensor], mid_lse: Sequence[torch.Tensor]):
    """Streaming LSE merge over splits (flash_tree_attn.py:189-211).

    mid_o[s] [..., D] normalised partials, mid_lse[s] [...]. Returns (O, LSE)."""
    m_i = torch.full_like(mid_lse[0], float("-inf"))                  # :189
    l_i = torch.zeros_like(mid_lse[0])                                 # :190
    acc = torch.zeros_like(mid_o[0])                                   # :191
    for o_s, lse_s in zip(mid_o, mid_lse):                             # :195
        m_ij = torch.maximum(m_i, lse_s)                               # :198
        dead = torch.isinf(m_ij) & (m_ij < 0)
        m_safe = torch.where(dead, torch.zeros_like(m_ij), m_ij)
        scale = torch.exp(m_i - m_safe)                                # :199
        w = torch.exp(lse_s - m_safe)                                  # :201-202
        acc = acc * scale.unsqueeze(-1) + w.unsqueeze(-1) * o_s        # :200,:203
        l_i = scale * l_i + w                                          # :204
        m_i = m_ij                                                     # :205
    l_safe = torch.where(l_i == 0, torch.ones_like(l_i), l_i)
    out = acc / l_safe.unsqueeze(-1)                                   # :207
    lse = torch.where(l_i == 0, torch.full_like(l_i, float("-inf")), m_i + torch.log(l_safe))  # :208
    return out, lse


def tree_block_oracle(qb, ckb, cvb, mask_b, scale: float):
    """Eager tree block (flash_tree_attn.py:367-371): p = q k_cur^T scale + mask."""
    p = torch.matmul(qb, ckb.transpose(1, 2)) * scale                  # :367
    p = p + mask_b                                                     # :368
    return _safe_softmax_av(p, cvb)                                    # :369-371


def final_merge_oracle(o_cache, lse_cache, o_cur, lse_cur):
    """out = O - sigmoid(lse_cur - lse_cache) * (O - O_cur) (flash_tree_attn.py:373).
    -inf on either side degenerates to the other operand."""
    d = lse_cur - lse_cache
    d = torch.where(torch.isnan(d), torch.zeros_like(d), d)           # (-inf) - (-inf)
    w = torch.sigmoid(d).unsqueeze(-1)
    return o_cache - w * (o_cache - o_cur)


def two_stage_oracle(q, k_cache, v_cache, current_k, current_v, mask, kv_seq_len,
                     block_size: int = 64, sm_scale: Optional[float] = None,
                     kv_group_num: int = 1, dtype: torch.dtype = torch.float32):
    """The reference pipeline restated: stage 1 over ceil(T_b / block_size) splits
    (flash_tree_attn.py:185, :274), stage 2, tree block, sigmoid merge."""
    bsz, hq, L, D = q.shape
    scale = 1.0 / math.sqrt(D) if sm_scale is None else float(sm_scale)
    out = torch.zeros(bsz, hq, L, D, dtype=dtype, device=q.device)
    lens = [int(t) for t in kv_seq_len.tolist()]
    for b in range(bsz):
        T = lens[b]
        qb = q[b].to(dtype)
        kb = _expand_heads(k_cache[b, :, :T].to(dtype), hq)
        vb = _expand_heads(v_cache[b, :, :T].to(dtype), hq)
        parts = [stage1_partial_oracle(qb, kb, vb, s0, min(s0 + block_size, T), scale)
                 for s0 in range(0, T, block_size)]
        if parts:
            o_cache, lse_cache = stage2_merge_oracle([p[0] for p in parts], [p[1] for p in parts])
        else:
            o_cache = torch.zeros(hq, L, D, dtype=dtype, device=q.device)
            lse_cache = torch.full((hq, L), float("-inf"), dtype=dtype, device=q.device)
        o_cur, lse_cur = tree_block_oracle(qb, _expand_heads(current_k[b].to(dtype), hq),
                                           _expand_heads(current_v[b].to(dtype), hq),
                                           _mask_for(mask, b, bsz, hq, L, dtype), scale)
        out[b] = final_merge_oracle(o_cache, lse_cache, o_cur, lse_cur)
    return out


# --------------------------------------------------------------------------- #
# Brute force (tiny shapes only)
# --------------------------------------------------------------------------- #

def brute_force_oracle(q, k_cache, v_cache, current_k, current_v, mask, kv_seq_len,
                       sm_scale: Optional[float] = None, kv_group_num: int = 1):
    """Pure-Python float (fp64) loops; mask must be [L, L] float. Tiny shapes only."""
    bsz, hq, L, D = q.shape
    scale = 1.0 / math.sqrt(D) if sm_scale is None else float(sm_scale)
    cur_group = hq // current_k.shape[1]
    out = torch.zeros(bsz, hq, L, D, dtype=torch.float64)
    for b in range(bsz):
        T = int(kv_seq_len[b])
        for h in range(hq):
            hk = h // kv_group_num
            hc = h // cur_group
            for i in range(L):
                logits, values = [], []
                for t in range(T):
                    logits.append(scale * sum(float(q[b, h, i, d]) * float(k_cache[b, hk, t, d]) for d in range(D)))
                    values.append([float(v_cache[b, hk, t, d]) for d in range(D)])
                for j in range(L):
                    logits.append(scale * sum(float(q[b, h, i, d]) * float(current_k[b, hc, j, d]) for d in range(D))
                                  + float(mask[i, j]))
                    values.append([float(current_v[b, hc, j, d]) for d in range(D)])
                mx = max(logits)
                if mx == float("-inf"):
                    continue
                w = [math.exp(x - mx) for x in logits]
                z = sum(w)
                for d in range(D):
                    out[b, h, i, d] = sum(wi * vi[d] for wi, vi in zip(w, values)) / z
    return out
