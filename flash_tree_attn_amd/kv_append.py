"""`append_accepted_kv`: writes the accepted path of the draft tree into the KV cache.

The step that follows `flash_decoding_attention` in a speculative-decoding loop; the
reference leaves it to its caller (README.md:63-64). Runs a gfx950 copy kernel through
the C ABI (`fta_append_kv`, include/fta.h); GPU tensors only, no fallback.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from . import _lib
from .flash_decoding import _DTYPES, _FAST_MAX_ENTRIES, _as_rows, _check, _current_stream, _fast, _rows_ok, _sig


def append_accepted_kv(k_cache: torch.Tensor, v_cache: torch.Tensor, current_k: torch.Tensor, current_v: torch.Tensor,
                       accept_idx: torch.Tensor, accept_len: torch.Tensor, kv_seq_len: torch.Tensor,
                       out_kv_seq_len: Optional[torch.Tensor] = None,
                       block_tables: Optional[torch.Tensor] = None) -> torch.Tensor:
    """For every sequence b and a < accept_len[b]:
        k_cache[b, :, kv_seq_len[b] + a] = current_k[b, :, accept_idx[b, a]]   (same for v)
    and the returned lengths are kv_seq_len + accept_len (clamped to the cache capacity;
    rows past it are dropped). `k_cache` / `v_cache` are updated in place; the lengths go
    to `out_kv_seq_len`, or in place into `kv_seq_len` when it is None.

      k_cache / v_cache   [bsz, num_kv_heads, cache_len, head_dim]
      current_k / _v      [bsz, num_kv_heads, q_len, head_dim]
      accept_idx          int32 [bsz, max_accept]: tree positions of the accepted path, root first
      accept_len          [bsz], dtype of kv_seq_len (int32 or int64)
    Paged caches: pass `block_tables` int32 [bsz, pages per sequence]; k_cache / v_cache are then the page
    pools [num_pages, num_kv_heads, page_size, head_dim] of `flash_decoding_attention(block_tables=...)`,
    and the capacity of a sequence is pages per sequence * page_size.
    """
    lib = _lib.load()
    # Repeat calls: the filled arguments of a call signature (shape, strides, dtype, device of every
    # tensor) are kept per thread, as in flash_decoding_attention; a repeat only refreshes the pointers.
    try:
        key = ("append", _sig(k_cache), _sig(v_cache), _sig(current_k), _sig(current_v), _sig(accept_idx), _sig(accept_len),
               _sig(kv_seq_len), _sig(out_kv_seq_len), _sig(block_tables))
        entry = _fast.__dict__.get("entries", {}).get(key)
    except (AttributeError, TypeError):
        key = entry = None
    if entry is not None and torch.cuda.current_device() == entry[2]:
        a, ref, index = entry
        out = kv_seq_len if out_kv_seq_len is None else out_kv_seq_len
        pk, pv, pck, pcv = k_cache.data_ptr(), v_cache.data_ptr(), current_k.data_ptr(), current_v.data_ptr()
        if not (pk | pv | pck | pcv) & 15:
            a.k_cache, a.v_cache, a.cur_k, a.cur_v = pk, pv, pck, pcv
            a.accept_idx, a.accept_len = accept_idx.data_ptr(), accept_len.data_ptr()
            a.kv_seq_len, a.kv_seq_len_out = kv_seq_len.data_ptr(), out.data_ptr()
            if block_tables is not None:
                a.block_table = block_tables.data_ptr()
            status = lib.fta_append_kv(ref, _current_stream(index))
            if status:
                _check(status)
            return out
    dev = k_cache.device
    if dev.type != "cuda":
        raise RuntimeError("append_accepted_kv runs on the GPU only; there is no CPU fallback")
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape:
        raise ValueError("k_cache / v_cache must be [bsz, num_kv_heads, cache_len, head_dim] and alike")
    paged = block_tables is not None
    tables_given = block_tables
    _, hkv, cache_len, D = k_cache.shape
    bsz = current_k.size(0) if current_k.dim() == 4 else -1
    if paged:
        if block_tables.dim() != 2 or block_tables.size(0) != bsz or block_tables.dtype != torch.int32 or block_tables.device != dev:
            raise ValueError("block_tables must be an int32 tensor [bsz, pages per sequence] on the caches' device")
        if block_tables.stride(1) != 1 and block_tables.size(1) > 1:
            block_tables = block_tables.contiguous()
    elif k_cache.size(0) != bsz:
        raise ValueError("k_cache / v_cache must hold one cache per sequence of current_k")
    if k_cache.dtype not in _DTYPES:
        raise ValueError(f"unsupported dtype {k_cache.dtype}")
    if current_k.shape != current_v.shape or current_k.dim() != 4 or current_k.size(0) != bsz or current_k.size(3) != D:
        raise ValueError("current_k / current_v must be [bsz, num_kv_heads, q_len, head_dim]")
    if current_k.size(1) != hkv:
        raise ValueError("only tree K/V with num_kv_heads heads can be appended to the cache")
    for t in (v_cache, current_k, current_v):
        if t.dtype != k_cache.dtype or t.device != dev:
            raise ValueError("caches and tree K/V must share dtype and device")
    for name, t in (("k_cache", k_cache), ("v_cache", v_cache)):
        if not _rows_ok(t):
            raise ValueError(f"{name} needs unit inner stride and 16-byte aligned rows (it is updated in place)")
    originals = (current_k, current_v, accept_idx, accept_len, tables_given)
    current_k, current_v = _as_rows(current_k), _as_rows(current_v)
    if accept_idx.dim() != 2 or accept_idx.size(0) != bsz or accept_idx.dtype != torch.int32 or accept_idx.device != dev:
        raise ValueError("accept_idx must be an int32 tensor [bsz, max_accept] on the caches' device")
    if accept_idx.stride(1) != 1 and accept_idx.size(1) > 1:
        accept_idx = accept_idx.contiguous()
    if kv_seq_len.dtype not in (torch.int32, torch.int64) or kv_seq_len.numel() != bsz or kv_seq_len.device != dev:
        raise ValueError("kv_seq_len must be an int32/int64 tensor of bsz elements on the caches' device")
    if accept_len.dtype != kv_seq_len.dtype or accept_len.numel() != bsz or accept_len.device != dev:
        raise ValueError("accept_len must match kv_seq_len in dtype, size and device")
    if not kv_seq_len.is_contiguous():
        raise ValueError("kv_seq_len must be contiguous (it is updated in place)")
    accept_len = accept_len.contiguous().view(-1)
    out = kv_seq_len if out_kv_seq_len is None else out_kv_seq_len
    if out.dtype != kv_seq_len.dtype or out.numel() != bsz or out.device != dev or not out.is_contiguous():
        raise ValueError("out_kv_seq_len must match kv_seq_len in dtype, size and device, and be contiguous")

    a = _lib.FtaAppendArgs()
    a.k_cache, a.v_cache, a.cur_k, a.cur_v = k_cache.data_ptr(), v_cache.data_ptr(), current_k.data_ptr(), current_v.data_ptr()
    a.accept_idx, a.accept_len = accept_idx.data_ptr(), accept_len.data_ptr()
    a.kv_seq_len, a.kv_seq_len_out = kv_seq_len.data_ptr(), out.data_ptr()
    a.bsz, a.num_kv_heads, a.q_len, a.head_dim = bsz, hkv, current_k.size(2), D
    a.cache_len, a.max_accept = cache_len, accept_idx.size(1)
    if paged:
        a.page_size, a.cache_len = cache_len, block_tables.size(1) * cache_len
        a.block_table, a.block_table_stride = block_tables.data_ptr(), block_tables.stride(0)
    a.dtype = _DTYPES[k_cache.dtype]
    a.len_dtype = _lib.FTA_I64 if kv_seq_len.dtype == torch.int64 else _lib.FTA_I32
    a.k_stride[:] = k_cache.stride()[:3]
    a.v_stride[:] = v_cache.stride()[:3]
    a.ck_stride[:] = current_k.stride()[:3]
    a.cv_stride[:] = current_v.stride()[:3]
    a.accept_idx_stride = accept_idx.stride(0)
    with torch.cuda.device(dev):
        _check(lib.fta_append_kv(C.byref(a), C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)))
    used = (current_k, current_v, accept_idx, accept_len, block_tables)
    if key is not None and entry is None and dev.index is not None and all(
            (o is None and u is None) or (o is not None and u is not None and o.data_ptr() == u.data_ptr())
            for o, u in zip(originals, used)):
        cache = _fast.__dict__.setdefault("entries", {})
        if len(cache) >= _FAST_MAX_ENTRIES:
            cache.clear()
        cache[key] = (a, C.byref(a), dev.index)
    return out
