"""CPU restatement of the accepted-path KV append (TEST INFRASTRUCTURE ONLY: imported by
tests/, never by the product).

The reference has no code for this step (README.md:63-64 names cache management as the
caller's job), so there is nothing of the reference to follow; the definition is the
one in include/fta.h, restated as plain loops:
    k_cache[b, h, T_b + a] = current_k[b, h, accept_idx[b, a]]  for a < accept_len[b]
    new_len[b] = min(T_b + accept_len[b], cache_len)
Pinned by: it is a gather/scatter of whole rows, so tests compare against torch's own
index_select / slice assignment on the same inputs, bit for bit.
"""
import torch


def append_accepted_kv_oracle(k_cache, v_cache, current_k, current_v, accept_idx, accept_len, kv_seq_len):
    """Returns (k_cache', v_cache', new_len) as new CPU tensors; inputs are not modified."""
    k, v = k_cache.detach().cpu().clone(), v_cache.detach().cpu().clone()
    ck, cv = current_k.detach().cpu(), current_v.detach().cpu()
    idx, n_acc, lens = accept_idx.cpu(), accept_len.cpu(), kv_seq_len.cpu()
    bsz, _, cache_len, _ = k.shape
    q_len = ck.size(2)
    new_len = lens.clone()
    for b in range(bsz):
        t = min(max(int(lens[b]), 0), cache_len)
        n = min(max(int(n_acc[b]), 0), idx.size(1))
        for a in range(n):
            src = int(idx[b, a])
            if t + a >= cache_len or not (0 <= src < q_len):
                continue
            k[b, :, t + a] = ck[b, :, src]
            v[b, :, t + a] = cv[b, :, src]
        new_len[b] = min(t + n, cache_len)
    return k, v, new_len
