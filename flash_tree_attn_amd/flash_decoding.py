"""`flash_decoding_attention`: drop-in for the reference function of the same name
(flash_tree_attn.py:216-376), running hand-written gfx950 kernels through the C ABI
of libfta.so. PyTorch is used for device memory and the current stream only.

Differences from the reference that a caller can observe (all deliberate):
* `output=`, when given, receives the FINAL result and is returned; the reference
  leaves the cache-only attention there and returns a new tensor
  (flash_tree_attn.py:373-376).
* `mid_output` / `mid_output_lse` are scratch for at most `plan.num_splits` splits
  (never more than ceil(max_len / block_size), so reference-sized buffers fit).
* No host sync: `kv_seq_len.max().item()` (flash_tree_attn.py:272) is not needed.
  `max_seq_len_in_batch` (any upper bound of the lengths) or, without it, the cache
  capacity bounds the grid and the scratch; how the keys are cut into chunks follows
  the real lengths, which the kernels read themselves.
* fp16, bf16 and fp32 inputs; `current_k/current_v` with num_kv_heads or num_heads
  heads; any q_len >= 1; `mask` float (additive, flash_tree_attn.py:368), bool, or int64
  bit words from `tree_mask.pack_mask` (8 bytes per row and 64 tree keys).
* A query row whose every logit is -inf yields zeros (the reference yields NaN).
There is no CPU or eager fallback: CPU tensors and a missing library raise.
"""
from __future__ import annotations

import ctypes as C
import threading
from typing import Optional

import torch

from . import _lib

_DTYPES = {torch.float32: _lib.FTA_F32, torch.float16: _lib.FTA_F16, torch.bfloat16: _lib.FTA_BF16}


class FtaAssertionError(ValueError, AssertionError):
    """Raised where the reference trips a bare `assert` (flash_tree_attn.py:263-291)."""


_ASSERT_STATUSES = {-2, -3, -4, -5}
_cu_count = {}
_counters = {}           # (device index, stream handle) -> the int32 counter buffer calls on that stream use
_retired_counters = []   # buffers a larger one replaced: kept alive, an earlier launch or a captured graph may still name them
_suspect_counters = set()   # keys whose last launch returned an error: cleared before the next use


def _counters_for(device: torch.device, stream: int, elems: int) -> Optional[torch.Tensor]:
    """Zeroed int32 counters for the single-launch merge, or None where the call has to take two
    launches. The kernel leaves the counters zero again, so one buffer per (device, stream)
    serves every call issued on that stream; calls on different streams may overlap in time and
    get buffers of their own. A buffer, once handed out, lives until the process ends. While
    the stream is capturing a graph the answer is None: a graph would keep the buffer's
    address for as long as it is replayed, next to eager calls that count in the same memory."""
    if torch.cuda.is_current_stream_capturing():
        return None
    key = (device.index, stream)
    buf = _counters.get(key)
    if buf is None or buf.numel() < elems:
        if buf is not None:
            _retired_counters.append(buf)
        buf = torch.zeros(max(elems, 4096), dtype=torch.int32, device=device)
        _counters[key] = buf
        _suspect_counters.discard(key)
    elif key in _suspect_counters:
        buf.zero_()   # a launch that failed may have left counts behind: every later merge would wait for ever-missing partials
        _suspect_counters.discard(key)
    return buf


def _launch_failed(device: torch.device, stream: int) -> None:
    if (device.index, stream) in _counters:
        _suspect_counters.add((device.index, stream))


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _current_stream(index: int) -> int:
    """Handle of torch's current stream on device `index` (the reference launches on it too)."""
    if _raw_stream is not None:
        return _raw_stream(index)
    return torch.cuda.current_stream(index).cuda_stream


def _check(status: int) -> None:
    if status == 0:
        return
    text = _lib.load().fta_strerror(status).decode()
    if status in _ASSERT_STATUSES:
        raise FtaAssertionError(f"fta status {status}: {text}")
    _lib.check(status)


def _rows_ok(t: torch.Tensor) -> bool:
    vec = 16 // t.element_size()
    return (t.stride(-1) == 1 and all(s % vec == 0 and s >= 0 for s in t.stride()[:-1])
            and t.data_ptr() % 16 == 0)


def _as_rows(t: torch.Tensor) -> torch.Tensor:
    """128-bit row access needs unit inner stride and 16-byte aligned rows; anything
    else is copied once (the reference honours arbitrary strides, flash_tree_attn.py:311-330)."""
    if _rows_ok(t):
        return t
    t = t.contiguous()
    return t if t.data_ptr() % 16 == 0 else t.clone()   # contiguous but at an odd offset of its storage


def _num_cus(device: torch.device) -> int:
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if idx not in _cu_count:
        _cu_count[idx] = torch.cuda.get_device_properties(idx).multi_processor_count
    return _cu_count[idx]


def _prepare_mask(mask: torch.Tensor, bsz: int, hq: int, L: int, device) -> torch.Tensor:
    if mask.device != device:
        raise ValueError("mask must live on the same device as q")
    if mask.dtype == torch.int64:   # packed bits (tree_mask.pack_mask): [..., L, ceil(L/64)]
        words = (L + 63) // 64
        if mask.dim() > 4 or mask.dim() < 2 or mask.size(-1) != words or mask.size(-2) != L:
            raise ValueError(f"a packed mask must be [..., q_len, ceil(q_len/64)] = [..., {L}, {words}], got {tuple(mask.shape)}")
        while mask.dim() < 4:
            mask = mask.unsqueeze(0)
        try:
            mask = mask.expand(bsz, hq, L, words)
        except RuntimeError as e:
            raise ValueError(f"mask of shape {tuple(mask.shape)} does not broadcast to {(bsz, hq, L, words)}") from e
        return mask if mask.stride(3) == 1 or words == 1 else mask.contiguous()
    if mask.dtype == torch.bool:
        m = torch.zeros(mask.shape, dtype=torch.float32, device=device)
        m.masked_fill_(~mask, float("-inf"))
        mask = m
    elif mask.dtype != torch.float32:
        mask = mask.float()
    if mask.dim() > 4 or mask.dim() < 2:
        raise ValueError(f"mask must be [q_len, q_len] up to [bsz, num_heads, q_len, q_len], got {tuple(mask.shape)}")
    while mask.dim() < 4:
        mask = mask.unsqueeze(0)
    try:
        mask = mask.expand(bsz, hq, L, L)
    except RuntimeError as e:
        raise ValueError(f"mask of shape {tuple(mask.shape)} does not broadcast to {(bsz, hq, L, L)}") from e
    if mask.stride(3) != 1 and L > 1:
        mask = mask.contiguous()
    return mask


def build_args(q, k_cache, v_cache, current_k, current_v, mask, kv_seq_len, block_size,
               max_seq_len_in_batch, sm_scale, kv_group_num, force_splits=0, force_kernel=-1, block_tables=None):
    """Validates tensors on the Python side and fills an FtaArgs (without out/scratch).
    Returns (args, keepalive) where keepalive holds every tensor the pointers refer to."""
    if q.dim() != 4:
        raise ValueError(f"q must be [bsz, num_heads, q_len, head_dim], got {tuple(q.shape)}")
    bsz, hq, L, D = q.shape
    dev = q.device
    if dev.type != "cuda":
        raise RuntimeError("flash_decoding_attention runs on the GPU only; there is no CPU fallback")
    if q.dtype not in _DTYPES:
        raise ValueError(f"unsupported dtype {q.dtype}")
    paged = block_tables is not None
    for name, t in (("k_cache", k_cache), ("v_cache", v_cache), ("current_k", current_k), ("current_v", current_v)):
        if t.dim() != 4:
            raise ValueError(f"{name} must be 4-dimensional, got {tuple(t.shape)}")
        if t.dtype != q.dtype or t.device != dev:
            raise ValueError(f"{name} must have q's dtype and device")
        pool = paged and name.endswith("cache")   # [num_pages, num_kv_heads, page_size, head_dim]
        if (t.size(0) != bsz and not pool) or t.size(3) != D:
            raise ValueError(f"{name} has shape {tuple(t.shape)}, incompatible with q {tuple(q.shape)}")
    if paged:
        if block_tables.dim() != 2 or block_tables.size(0) != bsz or block_tables.dtype != torch.int32 or block_tables.device != dev:
            raise ValueError("block_tables must be an int32 tensor [bsz, pages per sequence] on q's device")
        if block_tables.stride(1) != 1 and block_tables.size(1) > 1:
            block_tables = block_tables.contiguous()
        if k_cache.shape != v_cache.shape:
            raise FtaAssertionError("paged k_cache and v_cache must have the same shape")
    hkv = k_cache.size(1)
    if v_cache.size(1) != hkv or hkv * int(kv_group_num) != hq:
        raise ValueError(f"num_heads {hq} != num_kv_heads {hkv} * kv_group_num {kv_group_num}")
    if current_k.shape != current_v.shape or current_k.size(2) != L:
        raise ValueError("current_k/current_v must be [bsz, num_kv_heads (or num_heads), q_len, head_dim]")
    if kv_seq_len.device != dev or kv_seq_len.dtype not in (torch.int32, torch.int64) or kv_seq_len.numel() != bsz:
        raise ValueError("kv_seq_len must be an int32/int64 tensor of bsz elements on q's device")

    q, k_cache, v_cache = _as_rows(q), _as_rows(k_cache), _as_rows(v_cache)
    current_k, current_v = _as_rows(current_k), _as_rows(current_v)
    kv_seq_len = kv_seq_len.contiguous().view(-1)
    mask = _prepare_mask(mask, bsz, hq, L, dev)

    a = _lib.FtaArgs()
    a.q, a.k_cache, a.v_cache = q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr()
    a.cur_k, a.cur_v = current_k.data_ptr(), current_v.data_ptr()
    a.mask, a.kv_seq_len = mask.data_ptr(), kv_seq_len.data_ptr()
    a.bsz, a.num_q_heads, a.num_kv_heads, a.cur_heads = bsz, hq, hkv, current_k.size(1)
    a.q_len, a.head_dim = L, D
    if paged:   # logical capacity per sequence; the pools' dim 2 is the page size
        a.page_size = k_cache.size(2)
        a.cache_len = a.v_cache_len = block_tables.size(1) * k_cache.size(2)
        a.block_table, a.block_table_stride = block_tables.data_ptr(), block_tables.stride(0)
    else:
        a.cache_len, a.v_cache_len = k_cache.size(2), v_cache.size(2)
    a.block_size = int(block_size)
    a.max_seq_len_hint = 0 if max_seq_len_in_batch is None else max(int(max_seq_len_in_batch), 1)
    a.dtype = _DTYPES[q.dtype]
    a.len_dtype = _lib.FTA_I64 if kv_seq_len.dtype == torch.int64 else _lib.FTA_I32
    a.force_splits, a.force_kernel = int(force_splits), int(force_kernel)
    a.sm_scale = float(1.0 / (D ** 0.5) if sm_scale is None else sm_scale)
    a.q_stride[:] = q.stride()[:3]
    a.k_stride[:] = k_cache.stride()[:3]
    a.v_stride[:] = v_cache.stride()[:3]
    a.ck_stride[:] = current_k.stride()[:3]
    a.cv_stride[:] = current_v.stride()[:3]
    a.mask_stride[:] = mask.stride()[:3]
    a.mask_kind = _lib.MASK_PACKED_U64 if mask.dtype == torch.int64 else _lib.MASK_ADDITIVE_F32
    return a, (q, k_cache, v_cache, current_k, current_v, mask, kv_seq_len, block_tables)


def plan_for(args: "_lib.FtaArgs", num_cus: int) -> "_lib.FtaPlanOut":
    pl = _lib.FtaPlanOut()
    _check(_lib.load().fta_plan(C.byref(args), int(num_cus), C.byref(pl)))
    return pl


class PreparedCall:
    """One validated, planned call: the filled fta_args, its output and scratch tensors.
    `run()` launches the whole path on the current stream; `run_stage1()` / `run_stage2()`
    launch the halves (a profiler or a KV-sequence-sharded caller uses those). The tensors
    it was prepared from must stay alive and unmoved while it is in use."""

    def __init__(self, args, plan, output, mid_output, mid_output_lse, keep, device):
        self.args, self.plan, self.output = args, plan, output
        self.mid_output, self.mid_output_lse = mid_output, mid_output_lse
        self._keep, self._device = keep, device
        self._lib = _lib.load()
        self._ref = C.byref(args)

    def _launch(self, fn, single_launch=False):
        index = self._device.index
        if index is not None and torch.cuda.current_device() != index:
            with torch.cuda.device(index):
                return self._launch(fn, single_launch)
        stream = _current_stream(torch.cuda.current_device())
        buf = _counters_for(self._device, stream, self.plan.counter_elems) if single_launch and self.plan.counter_elems > 0 else None
        if buf is not None:
            self.args.counters, self.args.counter_elems = buf.data_ptr(), buf.numel()
        else:
            self.args.counters, self.args.counter_elems = None, 0
        status = fn(self._ref, stream)
        if status:
            if buf is not None:
                _launch_failed(self._device, stream)
            _check(status)
        return self.output

    def run(self):
        """The whole path: one launch where the plan advises the merge inside stage 1
        (few splits), else stage 1 + stage 2."""
        return self._launch(self._lib.fta_decode, single_launch=bool(self.plan.single_launch))

    def run_single_launch(self):
        """The whole path in one launch wherever the plan has counters, advised or not."""
        return self._launch(self._lib.fta_decode, single_launch=True)

    def run_two_launches(self):
        """The whole path as stage 1 + stage 2 kernels (what a caller without counters gets)."""
        return self._launch(self._lib.fta_decode)

    def run_stage1(self):
        return self._launch(self._lib.fta_decode_stage1)

    def run_stage2(self):
        return self._launch(self._lib.fta_decode_stage2)


def prepare(q, k_cache, v_cache, current_k, current_v, mask, kv_seq_len, block_size=64,
            max_seq_len_in_batch=None, output=None, mid_output=None, mid_output_lse=None,
            sm_scale=None, kv_group_num=1, _force_splits=0, _force_kernel=-1, block_tables=None) -> PreparedCall:
    """Validates, plans and allocates once; the returned PreparedCall can be launched
    repeatedly (a decode loop that reuses its buffers pays the Python checks once)."""
    _lib.load()
    args, keep = build_args(q, k_cache, v_cache, current_k, current_v, mask, kv_seq_len, block_size,
                            max_seq_len_in_batch, sm_scale, kv_group_num, _force_splits, _force_kernel, block_tables)
    bsz, hq, L, D = q.shape
    dev = q.device
    # scratch the caller brought is known to the plan: it bounds the split count the heuristic may pick
    user_mid = mid_output is not None and mid_output_lse is not None
    for name, t, nd in (("mid_output", mid_output, 5), ("mid_output_lse", mid_output_lse, 4)):
        if t is None:
            continue
        if t.dim() != nd or t.dtype != torch.float32 or t.device != dev or t.stride(-1) != 1:
            raise FtaAssertionError(f"{name} must be a float32 tensor with {nd} dims on q's device")
        if t.size(0) < bsz or t.size(1) != hq or t.size(3) != L or (nd == 5 and t.size(4) != D):
            raise FtaAssertionError(f"{name} has incompatible shape {tuple(t.shape)}")
    if user_mid:
        args.mid_o, args.mid_lse = mid_output.data_ptr(), mid_output_lse.data_ptr()
        args.mid_splits = min(mid_output.size(2), mid_output_lse.size(2))
    pl = plan_for(args, _num_cus(dev))

    if output is None:
        output = torch.empty((bsz, hq, L, D), dtype=q.dtype, device=dev)
    else:
        if output.shape != (bsz, hq, L, D) or output.dtype != q.dtype or output.device != dev:
            raise FtaAssertionError("output must be [bsz, num_heads, q_len, head_dim] with q's dtype and device")
        if not _rows_ok(output):
            raise ValueError("output needs unit inner stride and 16-byte aligned rows")
    args.out = output.data_ptr()
    args.out_stride[:] = output.stride()[:3]

    if pl.num_splits > 1:
        if mid_output is None:
            mid_output = torch.empty((bsz, hq, pl.num_splits, L, D), dtype=torch.float32, device=dev)
        if mid_output_lse is None:
            mid_output_lse = torch.empty((bsz, hq, pl.num_splits, L), dtype=torch.float32, device=dev)
        args.mid_o, args.mid_lse = mid_output.data_ptr(), mid_output_lse.data_ptr()
        args.mid_splits = min(mid_output.size(2), mid_output_lse.size(2))
        args.mid_o_stride[:] = mid_output.stride()[:4]
        args.mid_lse_stride[:] = mid_output_lse.stride()[:3]
        if args.mid_splits < pl.num_splits:
            _check(-5)
    return PreparedCall(args, pl, output, mid_output, mid_output_lse, keep, dev)


# ---- repeat calls of the drop-in function --------------------------------------------
# A decode loop calls flash_decoding_attention with the same shapes, strides and dtypes
# over and over, and at short contexts the Python checks above cost more than the kernel.
# The first call with a given signature goes through prepare(); if it needed no copies or
# conversions, its filled fta_args and plan are kept (per thread), and later calls with
# the same signature only refresh the pointers, allocate the output and launch. Whatever
# depends on tensor VALUES stays on the device (lengths, mask, block table), so the
# signature is: shape, strides, dtype and device of every tensor plus the scalar arguments.
_fast = threading.local()
_FAST_MAX_ENTRIES = 128


class _FastEntry:
    __slots__ = ("args", "ref", "plan", "out_shape", "dtype", "device", "index", "mid_o_shape", "mid_lse_shape", "decode")


def _sig(t):
    return None if t is None else (t.shape, t.stride(), t.dtype, t.device)


def _fast_key(q, k_cache, v_cache, current_k, current_v, mask, kv_seq_len, block_size, max_seq_len_in_batch, output,
              mid_output, mid_output_lse, sm_scale, kv_group_num, block_tables, force_splits, force_kernel):
    return (q.shape, q.stride(), q.dtype, q.device, _sig(k_cache), _sig(v_cache), _sig(current_k), _sig(current_v),
            _sig(mask), _sig(kv_seq_len), block_size, max_seq_len_in_batch, _sig(output), _sig(mid_output),
            _sig(mid_output_lse), sm_scale, kv_group_num, _sig(block_tables), force_splits, force_kernel)


def _remember(key, pc, originals, user_mid):
    """Keeps a prepared call for its signature if the kernels read the caller's tensors as they came."""
    for orig, kept in zip(originals, pc._keep):
        if orig is None and kept is None:
            continue
        if orig is None or kept is None or kept.dtype != orig.dtype or kept.data_ptr() != orig.data_ptr():
            return   # copied or converted: such calls take the full path every time
    if pc._device.index is None or user_mid == "partial":
        return
    e = _FastEntry()
    e.args, e.ref, e.plan = pc.args, C.byref(pc.args), pc.plan
    e.out_shape, e.dtype, e.device, e.index = tuple(pc.output.shape), pc.output.dtype, pc._device, pc._device.index
    own_mid = pc.plan.num_splits > 1 and not user_mid
    e.mid_o_shape = tuple(pc.mid_output.shape) if own_mid else None
    e.mid_lse_shape = tuple(pc.mid_output_lse.shape) if own_mid else None
    e.decode = pc._lib.fta_decode
    cache = _fast.__dict__.setdefault("entries", {})
    if len(cache) >= _FAST_MAX_ENTRIES:
        cache.clear()
    cache[key] = e


def _run_remembered(e, q, k_cache, v_cache, current_k, current_v, mask, kv_seq_len, output, mid_output, mid_output_lse,
                    block_tables):
    """Launch from a remembered signature; None sends the call down the full path."""
    if torch.cuda.current_device() != e.index:
        return None
    if output is None:
        output = torch.empty(e.out_shape, dtype=e.dtype, device=e.device)
    a = e.args
    pq, pk, pv, pck, pcv, pout = (q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), current_k.data_ptr(),
                                  current_v.data_ptr(), output.data_ptr())
    if (pq | pk | pv | pck | pcv | pout) & 15:
        return None   # rows not 16-byte aligned: the full path copies them
    a.q, a.k_cache, a.v_cache, a.cur_k, a.cur_v, a.out = pq, pk, pv, pck, pcv, pout
    a.mask, a.kv_seq_len = mask.data_ptr(), kv_seq_len.data_ptr()
    if block_tables is not None:
        a.block_table = block_tables.data_ptr()
    plan = e.plan
    if plan.num_splits > 1:
        if e.mid_o_shape is not None:   # scratch of the planned size, from torch's caching allocator
            mid_output = torch.empty(e.mid_o_shape, dtype=torch.float32, device=e.device)
            mid_output_lse = torch.empty(e.mid_lse_shape, dtype=torch.float32, device=e.device)
        a.mid_o, a.mid_lse = mid_output.data_ptr(), mid_output_lse.data_ptr()
    stream = _current_stream(e.index)
    buf = _counters_for(e.device, stream, plan.counter_elems) if plan.single_launch else None
    if buf is not None:
        a.counters, a.counter_elems = buf.data_ptr(), buf.numel()
    else:
        a.counters, a.counter_elems = None, 0
    status = e.decode(e.ref, stream)
    if status:
        if buf is not None:
            _launch_failed(e.device, stream)
        _check(status)
    return output


def flash_decoding_attention(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    current_k: torch.Tensor,
    current_v: torch.Tensor,
    mask: torch.Tensor,
    kv_seq_len: torch.Tensor,
    block_size: int = 64,
    max_seq_len_in_batch: Optional[int] = None,
    output: Optional[torch.Tensor] = None,
    mid_output: Optional[torch.Tensor] = None,
    mid_output_lse: Optional[torch.Tensor] = None,
    sm_scale: Optional[float] = None,
    kv_group_num: int = 1,
    *,
    block_tables: Optional[torch.Tensor] = None,
    _force_splits: int = 0,
    _force_kernel: int = -1,
) -> torch.Tensor:
    """Tree-attention decode (speculative-decoding verification).

    Same parameters, order and defaults as the reference (flash_tree_attn.py:216-231):
      q [bsz, num_heads, q_len, head_dim]; k_cache / v_cache [bsz, num_kv_heads, ctx, head_dim];
      current_k / current_v [bsz, num_kv_heads, q_len, head_dim]; mask [q_len, q_len] or
      [bsz, num_heads, q_len, q_len], ADDED to the tree logits; kv_seq_len [bsz].
    Paged caches (the layout the reference's comments describe, flash_tree_attn.py:17-18,233):
      pass `block_tables` int32 [bsz, pages per sequence]; k_cache / v_cache are then page pools
      [num_pages, num_kv_heads, page_size, head_dim] with page_size in {16, 32, 64, 128}, and position
      j of sequence b is row j % page_size of page block_tables[b, j // page_size].
    Returns [bsz, num_heads, q_len, head_dim] in q's dtype.
    """
    key = None
    try:
        key = _fast_key(q, k_cache, v_cache, current_k, current_v, mask, kv_seq_len, block_size, max_seq_len_in_batch,
                        output, mid_output, mid_output_lse, sm_scale, kv_group_num, block_tables, _force_splits, _force_kernel)
        entry = _fast.__dict__.get("entries", {}).get(key)
    except (AttributeError, TypeError):   # not tensors / unhashable scalars: let the full path report it
        entry = None
    if entry is not None:
        out = _run_remembered(entry, q, k_cache, v_cache, current_k, current_v, mask, kv_seq_len, output, mid_output,
                              mid_output_lse, block_tables)
        if out is not None:
            return out
    pc = prepare(q, k_cache, v_cache, current_k, current_v, mask, kv_seq_len, block_size,
                 max_seq_len_in_batch, output, mid_output, mid_output_lse, sm_scale, kv_group_num,
                 _force_splits, _force_kernel, block_tables)
    out = pc.run()
    if key is not None and entry is None:
        _remember(key, pc, (q, k_cache, v_cache, current_k, current_v, mask, kv_seq_len, block_tables),
                  "partial" if (mid_output is None) != (mid_output_lse is None) else mid_output is not None)
    return out
