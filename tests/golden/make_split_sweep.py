"""Regenerates split_sweep_uniform.json / split_sweep_ragged.json on an MI355X:
    python tests/golden/make_split_sweep.py uniform|ragged
For a grid of shapes (bf16, head_dim 128) it times the whole call of flash_decoding_attention
at every forced split count of a fixed set and writes microseconds per call. `uniform` takes
every sequence at the full cache length; `ragged` draws log-uniform lengths over a 16x range
(seeded) with the first sequence at full length. tests/test_abi.py compares the plan's own
split count with these measurements."""
import itertools
import json
import math
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from flash_tree_attn_amd import prepare  # noqa: E402
from flash_tree_attn_amd.tree_mask import additive_mask_from_parents, random_tree_parents  # noqa: E402

SPLITS = (1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64)


def timed(calls, n):
    for i in range(max(4, n // 4)):
        calls[i % len(calls)].run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(n):
        calls[i % len(calls)].run()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / n


def main(kind):
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(0)
    cg = torch.Generator().manual_seed(1)
    r = lambda *s: torch.randn(*s, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    batches = (1, 4, 16, 64) if kind == "uniform" else (4, 16, 64)
    out = []
    for bsz, (hq, hkv), L, T in itertools.product(batches, ((32, 32), (32, 8), (64, 8)), (1, 8, 26, 64), (1024, 8192, 65536)):
        kv_bytes = 2 * bsz * hkv * T * 128 * 2
        if kv_bytes > 3 << 30:
            continue
        sets = 2 if kv_bytes > (256 << 20) else 4   # rotate over several caches: no reuse out of the last-level cache
        q, ck, cv = r(bsz, hq, L, 128), r(bsz, hkv, L, 128), r(bsz, hkv, L, 128)
        kvs = [(r(bsz, hkv, T, 128), r(bsz, hkv, T, 128)) for _ in range(sets)]
        mask = additive_mask_from_parents(random_tree_parents(L), device=dev)
        if kind == "uniform":
            lens = torch.full((bsz,), T, dtype=torch.int64)
        else:
            lens = torch.exp(torch.rand(bsz, generator=cg) * math.log(16.0)).mul(T / 16.0).long().clamp(1, T)
            lens[0] = T
        lens = lens.to(dev)
        us = {}
        for s in SPLITS:
            if s > max(1, T // 256):
                continue
            calls = [prepare(q, k, v, ck, cv, mask, lens, 64, kv_group_num=hq // hkv, _force_splits=s) for k, v in kvs]
            n = 40 if kv_bytes < (1 << 30) else 12
            us[str(s)] = round(min(timed(calls, n), timed(calls, n)), 1)
            del calls
        out.append(dict(bsz=bsz, hq=hq, hkv=hkv, L=L, T=T, us=us))
        print(out[-1], flush=True)
        del kvs, q, ck, cv
        torch.cuda.empty_cache()
    with open(os.path.join(HERE, f"split_sweep_{kind}.json"), "w") as f:
        f.write("[\n" + ",\n".join(json.dumps(o, separators=(",", ":")) for o in out) + "\n]\n")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "uniform")
