"""Host-side logic of the Python drop-in that needs no GPU: the call signature under which
validated arguments are remembered, and the rule for what may be remembered."""
import types

import torch

from flash_tree_attn_amd import _lib
from flash_tree_attn_amd import flash_decoding as fd


def _tensors(L=4, T=32, D=64, dtype=torch.float16):
    q = torch.zeros(2, 4, L, D, dtype=dtype)
    k = torch.zeros(2, 2, T, D, dtype=dtype)
    v = torch.zeros(2, 2, T, D, dtype=dtype)
    ck = torch.zeros(2, 2, L, D, dtype=dtype)
    cv = torch.zeros(2, 2, L, D, dtype=dtype)
    mask = torch.zeros(L, L)
    lens = torch.zeros(2, dtype=torch.int64)
    return [q, k, v, ck, cv, mask, lens]


def _key(ts, block_size=64, max_len=None, output=None, mid=None, lse=None, scale=None, group=2, tables=None, fs=0, fk=-1):
    return fd._fast_key(*ts, block_size, max_len, output, mid, lse, scale, group, tables, fs, fk)


def test_signature_is_shape_stride_dtype_and_scalars_not_data():
    a, b = _tensors(), _tensors()
    b[0].fill_(3.0)                                   # other storage, other values: same signature
    assert _key(a) == _key(b) and hash(_key(a)) == hash(_key(b))
    assert _key(a) != _key(_tensors(T=33))            # shape
    assert _key(a) != _key(_tensors(dtype=torch.bfloat16))
    big = torch.zeros(2, 2, 40, 64, dtype=torch.float16)
    c = _tensors()
    c[1] = big[:, :, :32]                             # same shape, other strides (a slice of a larger cache)
    assert c[1].shape == a[1].shape and _key(a) != _key(c)
    d = _tensors()
    d[6] = d[6].int()                                 # int32 lengths
    assert _key(a) != _key(d)
    for kw in (dict(block_size=32), dict(max_len=20), dict(scale=0.5), dict(fs=3), dict(fk=0),
               dict(output=torch.zeros(2, 4, 4, 64, dtype=torch.float16)),
               dict(tables=torch.zeros(2, 2, dtype=torch.int32))):
        assert _key(a) != _key(a, **kw), kw


def _fake_call(ts, keep=None, splits=1, mid=None, lse=None):
    plan = _lib.FtaPlanOut()
    plan.num_splits = splits
    out = torch.zeros_like(ts[0])
    return types.SimpleNamespace(args=_lib.FtaArgs(), plan=plan, output=out, mid_output=mid, mid_output_lse=lse,
                                 _keep=tuple(keep if keep is not None else ts) + (None,), _device=torch.device("cuda", 0),
                                 _lib=types.SimpleNamespace(fta_decode=None))


def test_only_calls_that_used_the_callers_tensors_are_remembered():
    fd._fast.__dict__.pop("entries", None)
    ts = _tensors()
    fd._remember("plain", _fake_call(ts), tuple(ts) + (None,), False)
    assert "plain" in fd._fast.entries
    e = fd._fast.entries["plain"]
    assert e.out_shape == (2, 4, 4, 64) and e.dtype == torch.float16 and e.index == 0 and e.mid_o_shape is None

    copied = list(ts)
    copied[0] = ts[0].clone()                         # the full path had to copy q
    fd._remember("copied", _fake_call(ts, keep=copied), tuple(ts) + (None,), False)
    converted = list(ts)
    converted[5] = ts[5].double()                     # ... or convert the mask
    fd._remember("converted", _fake_call(ts, keep=converted), tuple(ts) + (None,), False)
    fd._remember("partial", _fake_call(ts, splits=2, mid=torch.zeros(2, 4, 2, 4, 64), lse=torch.zeros(2, 4, 2, 4)),
                 tuple(ts) + (None,), "partial")        # only one of the two scratch buffers came from the caller
    assert set(fd._fast.entries) == {"plain"}

    mid, lse = torch.zeros(2, 4, 2, 4, 64), torch.zeros(2, 4, 2, 4)
    fd._remember("own scratch", _fake_call(ts, splits=2, mid=mid, lse=lse), tuple(ts) + (None,), False)
    assert fd._fast.entries["own scratch"].mid_o_shape == (2, 4, 2, 4, 64)
    assert fd._fast.entries["own scratch"].mid_lse_shape == (2, 4, 2, 4)
    fd._remember("caller's scratch", _fake_call(ts, splits=2, mid=mid, lse=lse), tuple(ts) + (None,), True)
    assert fd._fast.entries["caller's scratch"].mid_o_shape is None

    for i in range(fd._FAST_MAX_ENTRIES + 5):         # bounded: the table is dropped when full
        fd._remember(("k", i), _fake_call(ts), tuple(ts) + (None,), False)
    assert len(fd._fast.entries) <= fd._FAST_MAX_ENTRIES
    fd._fast.__dict__.pop("entries", None)


def test_misaligned_contiguous_tensor_is_cloned():
    flat = torch.zeros(64 * 4 + 4, dtype=torch.float16)
    t = flat[4:].view(4, 64)
    assert t.is_contiguous() and t.data_ptr() % 16 == 8
    r = fd._as_rows(t)
    assert r.data_ptr() % 16 == 0 and torch.equal(r, t)
    ok = torch.zeros(4, 64, dtype=torch.float16)
    assert fd._as_rows(ok) is ok


def test_counter_buffers_are_never_dropped_and_are_cleared_after_a_failed_launch(monkeypatch):
    """The single-launch merge counts arrivals in a buffer the wrapper keeps per (device, stream).
    An earlier launch may still be running on a buffer when a larger one replaces it, so replaced
    buffers stay alive; a capturing stream gets none (the graph would keep its address); a launch
    that returned an error may have left counts behind, so the buffer is cleared before its next use."""
    capturing = [False]
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: capturing[0])
    monkeypatch.setattr(fd, "_counters", {})
    monkeypatch.setattr(fd, "_retired_counters", [])
    monkeypatch.setattr(fd, "_suspect_counters", set())
    dev = torch.device("cpu")
    a = fd._counters_for(dev, 7, 100)
    assert a.dtype == torch.int32 and a.numel() >= 100 and int(a.abs().sum()) == 0
    assert fd._counters_for(dev, 7, 50) is a                       # reused while it is large enough
    other = fd._counters_for(dev, 8, 50)
    assert other is not a                                          # a buffer per stream
    big = fd._counters_for(dev, 7, a.numel() + 1)
    assert big is not a and big.numel() > a.numel()
    assert any(r is a for r in fd._retired_counters)               # the replaced one is kept alive
    assert fd._counters[(None, 7)] is big

    capturing[0] = True
    assert fd._counters_for(dev, 7, 10) is None                    # even though this stream has a buffer
    assert fd._counters_for(dev, 9, 10) is None and (None, 9) not in fd._counters
    capturing[0] = False

    big[:5] = 3                                                    # what a launch that died half-way leaves behind
    fd._launch_failed(dev, 7)
    again = fd._counters_for(dev, 7, 10)
    assert again is big and int(big.abs().sum()) == 0
    big[0] = 1                                                     # not suspect any more: the wrapper does not touch it
    assert fd._counters_for(dev, 7, 10) is big and int(big[0]) == 1
    fd._launch_failed(dev, 12345)                                  # a stream without a buffer: nothing to remember
    assert (None, 12345) not in fd._suspect_counters
