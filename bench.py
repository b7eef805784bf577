#!/usr/bin/env python3
"""Benchmark of the tree-attention decode hot path on one MI355X.

A step is one call of `flash_decoding_attention` (stage 1 + LSE merge) on one batch of
synthetic input already resident in HBM. Steps rotate over several independent KV-cache
sets so the footprint exceeds the 256 MB Infinity Cache. Before the warm-up steps the
call runs untimed for --settle-ms so that the card's clocks have settled. Prints ONE JSON line:
value = achieved GB/s over the whole call (algorithmic bytes / time per call),
`roofline` = the dominant kernel (stage 1) timed alone with HIP events on the launch
stream, `cpu_baseline` = the fp32 PyTorch eager oracle on the host cores (a bounded
sample), timed in the same run.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
MFMA_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 / fp16 MFMA rate (the co-constraint of the headline shape)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--settle-ms", type=float, default=150.0,
                    help="run the call untimed for this long before the warm-up steps: the card raises its clocks over the "
                         "first tens of milliseconds of load (a 110 us call measures 102 us once they have settled)")
    ap.add_argument("--config", default="cfg3_gqa_8b_bf16", help="workload name (flash_tree_attn_amd.synthetic.CONFIGS)")
    ap.add_argument("--kv-sets", type=int, default=0, help="independent KV caches to rotate over (0 = enough for >1 GiB)")
    ap.add_argument("--splits", type=int, default=0, help="pin the split count (0 = heuristic)")
    ap.add_argument("--kernel", default="auto", choices=["auto", "mfma", "mfma_wide", "mfma_split_keys", "shuffle"],
                    help="pin the stage-1 kernel (auto = the plan's choice); for comparing them on one workload. mfma_wide = the "
                         "MFMA kernel with 64-row waves and the hand-scheduled half-tile loop (256-row units, contiguous caches); mfma_split_keys = "
                         "the MFMA kernel with two waves per 32-row block, each taking half of a tile's keys (units of at most 64 rows)")
    ap.add_argument("--op", default="decode", choices=["decode", "append_kv"],
                    help="decode = the tree-attention call (the headline); append_kv = the accepted-path KV append that follows it")
    ap.add_argument("--accept", type=int, default=8, help="accepted tree rows per sequence for --op append_kv")
    ap.add_argument("--paged", type=int, default=0, metavar="PAGE",
                    help="run on paged caches: pages of PAGE positions (16/32/64/128), shuffled in one pool, with a block table")
    ap.add_argument("--packed-mask", action="store_true", help="pass the tree mask as packed bit words instead of float32")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--reference-sweep", action="store_true",
                    help="only run the sweep of the reference's own benchmark (flash_tree_attn.py:442-487: bsz 2, 32 MHA heads, "
                         "D 128, fp16, q_len 16..128 x context 64..256, K/V passed as slices of one buffer) through the drop-in "
                         "call, next to an eager torch attention on the GPU, and print the table as one JSON line")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run plain device copies of a known size (reference point for rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline sample")
    ap.add_argument("--compare", default="", metavar="K1,K2,...",
                    help="only time the call with each of these stage-1 kernels (names as for --kernel) on the same inputs, in one "
                         "process and one warm card, and print the medians side by side as one JSON line")
    return ap.parse_args()


def traffic_from_profiles(config_name):
    """HBM bytes per stage-1 launch from the committed rocprofv3 --pmc summary, if any."""
    path = os.path.join(ROOT, "profiles", f"stage1_{config_name}_pmc.txt")
    if not os.path.exists(path):
        return None
    m = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", open(path).read(), flags=re.M)
    return float(m.group(1)) if m else None


def cpu_baseline(cfg, x, budget_s):
    """fp32 eager oracle on the host cores over as many whole sequences of the batch as
    fit the time budget; reported in the metric's unit (algorithmic GB/s)."""
    import torch
    from flash_tree_attn_amd.synthetic import algorithmic_bytes
    from oracle.tree_attn_oracle import tree_attention_oracle

    cpu = {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in x.items() if k not in ("k_caches", "v_caches")}

    def run(nseq):
        sl = slice(0, nseq)
        t0 = time.perf_counter()
        tree_attention_oracle(cpu["q"][sl], cpu["k_cache"][sl], cpu["v_cache"][sl], cpu["current_k"][sl],
                              cpu["current_v"][sl], cpu["mask"], cpu["kv_seq_len"][sl], cpu["sm_scale"],
                              cpu["kv_group_num"])
        return time.perf_counter() - t0

    run(1)  # warm-up (thread pool, allocator)
    t1 = run(1)
    nseq = int(max(1, min(cfg.bsz, budget_s / 2 / max(t1, 1e-6))))
    reps, times = 0, []
    t_start = time.perf_counter()
    while reps < 5 and (reps < 1 or time.perf_counter() - t_start < budget_s):
        times.append(run(nseq))
        reps += 1
    t = sorted(times)[len(times) // 2]
    sample_cfg_bytes = algorithmic_bytes(cfg, cpu["kv_seq_len"][:nseq], cpu["mask"]) * 1.0
    # per-sequence terms scale with nseq; recompute q/out/current terms for the sample
    esz = cpu["q"].element_size()
    per_seq_fixed = (2 * cfg.num_kv_heads + 2 * cfg.num_heads) * cfg.q_len * cfg.head_dim * esz + 8
    sample_bytes = sample_cfg_bytes - (cfg.bsz - nseq) * per_seq_fixed
    return {
        "value": sample_bytes / t / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"{nseq} of {cfg.bsz} sequences of {cfg.name}, fp32 eager oracle, median of {reps} run(s), "
                  f"{t * 1e6 / nseq * cfg.bsz:.0f} us/call extrapolated to the full batch, os.cpu_count()={os.cpu_count()}",
        "us_per_call_extrapolated": t * 1e6 / nseq * cfg.bsz,
    }


def reference_sweep(dev):
    """The reference's in-file benchmark (flash_tree_attn.py:442-487), shape for shape and
    call for call: Z 2, H 32, HEAD_DIM 128, fp16 normal(0, 0.5) inputs, block 64, the cache
    and the tree block passed as slices of one [Z, H, N_CTX + q_len, D] buffer, a fresh
    call of the drop-in function per step (wrapper included, as its `triton` provider
    does); the `torch` provider is eager masked attention on the GPU over the
    concatenated keys, as the reference's torch_tree_attention (flash_tree_attn.py:380-397). Median of
    event-timed batches, in milliseconds like the reference prints."""
    import torch
    from flash_tree_attn_amd import flash_decoding_attention
    from flash_tree_attn_amd.tree_mask import additive_mask_from_parents, random_tree_parents
    Z, H, D, blk = 2, 32, 128, 64
    sm_scale = 1.0 / D ** 0.5
    g = torch.Generator().manual_seed(0)

    def timed(fn, batches=15, per_batch=20):
        for _ in range(30):
            fn()
        torch.cuda.synchronize()
        ts = []
        for _ in range(batches):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(per_batch):
                fn()
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1) / per_batch)
        return sorted(ts)[len(ts) // 2]

    rows = []
    for q_len in (16, 32, 64, 128):
        for n_ctx in (64, 128, 256):
            q = (torch.randn(Z, H, q_len, D, generator=g) * 0.5).half().to(dev)
            k = (torch.randn(Z, H, n_ctx + q_len, D, generator=g) * 0.5).half().to(dev)
            v = (torch.randn(Z, H, n_ctx + q_len, D, generator=g) * 0.5).half().to(dev)
            mask = additive_mask_from_parents(random_tree_parents(q_len, g), device=dev)
            lens = torch.tensor([n_ctx] * Z, device=dev)
            full_mask = torch.cat([torch.zeros(q_len, n_ctx, device=dev), mask], dim=1).half()

            def eager():
                p = torch.matmul(q, k.transpose(2, 3)) * sm_scale + full_mask
                return torch.matmul(torch.softmax(p.float(), dim=-1).half(), v)

            def ours():
                return flash_decoding_attention(q, k[:, :, :n_ctx], v[:, :, :n_ctx], k[:, :, n_ctx:], v[:, :, n_ctx:], mask, lens,
                                                block_size=blk, sm_scale=sm_scale)

            torch.testing.assert_close(ours().float(), eager().float(), atol=1e-2, rtol=0)   # the reference test's tolerance (flash_tree_attn.py:440)
            nbytes = (q.numel() + k.numel() + v.numel()) * 2                                 # the reference's byte count (flash_tree_attn.py:484)
            ms_ours, ms_eager = timed(ours), timed(eager)
            rows.append({"q_len": q_len, "n_ctx": n_ctx, "ms": round(ms_ours, 5), "torch_eager_ms": round(ms_eager, 5),
                         "gbs": round(nbytes / ms_ours * 1e-6, 1)})
    print(json.dumps({"reference_sweep": {"shape": "Z 2, H 32, D 128, fp16, block 64", "timing": "median of 15 batches of 20 calls, "
                      "each a fresh call of flash_decoding_attention (Python wrapper included)", "rows": rows}}))


def bench_append(args, cfg, dev):
    """Times the accepted-path KV append at the workload's shapes: `--accept` rows of the
    tree per sequence go to the end of each cache; lengths are written out of place so
    that every step does the same work. Checked against the CPU oracle first."""
    import torch
    from flash_tree_attn_amd import append_accepted_kv
    from flash_tree_attn_amd.synthetic import make_inputs
    from oracle.kv_append_oracle import append_accepted_kv_oracle

    x = make_inputs(cfg, seed=0, device=dev, gen_device=dev, kv_sets=1)
    n_acc = min(args.accept, cfg.q_len)
    g = torch.Generator().manual_seed(0)
    idx = torch.stack([torch.randperm(cfg.q_len, generator=g)[:n_acc].sort().values for _ in range(cfg.bsz)]).to(torch.int32).to(dev)
    acc = torch.full((cfg.bsz,), n_acc, dtype=torch.int64, device=dev)
    lens = (x["kv_seq_len"] - n_acc).clamp_(min=0)
    out_lens = torch.empty_like(lens)
    small = slice(0, min(cfg.bsz, 2))   # oracle check on two sequences
    kc, vc = x["k_cache"][small].clone(), x["v_cache"][small].clone()
    ref = append_accepted_kv_oracle(kc, vc, x["current_k"][small], x["current_v"][small], idx[small], acc[small], lens[small])
    got_lens = append_accepted_kv(kc, vc, x["current_k"][small], x["current_v"][small], idx[small], acc[small], lens[small].clone())
    assert torch.equal(kc.cpu(), ref[0]) and torch.equal(vc.cpu(), ref[1]) and torch.equal(got_lens.cpu(), ref[2])

    run = lambda: append_accepted_kv(x["k_cache"], x["v_cache"], x["current_k"], x["current_v"], idx, acc, lens, out_lens)
    for _ in range(args.warmup):
        run()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(args.steps):
        run()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / args.steps
    esz = x["k_cache"].element_size()
    nbytes = 2 * 2 * cfg.bsz * cfg.num_kv_heads * n_acc * cfg.head_dim * esz + cfg.bsz * (n_acc * 4 + 24)   # rows read + written, indices, lengths
    print(json.dumps({
        "metric": "accepted-path KV append us/call", "value": round(ms * 1e3, 2), "unit": "us", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8 (row copies)", "data": "synthetic, resident in HBM",
        "config": {"workload": cfg.name + " / append_kv", "bsz": cfg.bsz, "kv_heads": cfg.num_kv_heads, "head_dim": cfg.head_dim,
                   "accepted_rows": n_acc, "algorithmic_bytes": nbytes},
        "roofline": {"bound": "hbm", "kernel": "append_kv", "achieved": round(nbytes / (ms * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 6), "traffic": None,
                     "note": "launch-bound: one small kernel per call"},
    }))


def compare_kernels(args, cfg, x, mask_arg, names, kernel_ids):
    """Times the whole call and stage 1 alone with each named stage-1 kernel on the same contiguous inputs: one settle
    phase, then per kernel a warm-up and event-timed batches of 25 calls, kernels taking turns batch by batch so that a
    drift of the card's clocks hits all of them alike. Each kernel's result is checked against the first one's."""
    import torch
    from flash_tree_attn_amd import prepare
    from flash_tree_attn_amd.synthetic import algorithmic_bytes
    for n in names:
        if n not in kernel_ids:
            raise SystemExit(f"--compare: no kernel named {n!r}")
    kv_sets = len(x["k_caches"])
    calls = {n: [prepare(x["q"], kc, vc, x["current_k"], x["current_v"], mask_arg, x["kv_seq_len"], cfg.block_size, None, None, None, None,
                         x["sm_scale"], cfg.kv_group_num, _force_splits=args.splits, _force_kernel=kernel_ids[n])
                 for kc, vc in zip(x["k_caches"], x["v_caches"])] for n in names}
    tol = dict(atol=2e-3, rtol=1e-2) if cfg.dtype != torch.float32 else dict(atol=2e-5, rtol=1e-4)
    first = calls[names[0]][0].run().float().clone()
    for n in names[1:]:
        torch.testing.assert_close(calls[n][0].run().float(), first, **tol)
    stream = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def batch(n, fn_name, steps=25):
        torch.cuda.synchronize()
        e0.record(stream)
        for i in range(steps):
            getattr(calls[n][i % kv_sets], fn_name)()
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps * 1e3   # us per call

    t_settle = time.perf_counter()
    while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
        for n in names:
            batch(n, "run", 8)
    rounds = max(1, args.steps // 25)
    whole, stage1 = {n: [] for n in names}, {n: [] for n in names}
    for _ in range(rounds):
        for n in names:
            whole[n].append(batch(n, "run"))
        for n in names:
            stage1[n].append(batch(n, "run_stage1"))
    med = lambda v: sorted(v)[len(v) // 2]
    nbytes = algorithmic_bytes(cfg, x["kv_seq_len"].cpu(), mask_arg)
    rows = {}
    for n in names:
        pl = calls[n][0].plan
        rows[n] = {"us_per_call": round(med(whole[n]), 2), "stage1_us": round(med(stage1[n]), 2), "gbs": round(nbytes / med(whole[n]) / 1e3, 1),
                   "plan": f"{pl.num_splits} x {pl.chunk_for(int(x['kv_seq_len'].max()))}", "rows_per_wg": pl.rows_per_wg, "mfma_loop": pl.mfma_loop}
    print(json.dumps({"compare": {"workload": cfg.name, "batches_of_25_per_kernel": rounds, "kernels": rows}}))


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if args.steps < 1 or args.warmup < 0:
        print("bench.py: --steps must be at least 1 and --warmup not negative", file=sys.stderr)
        sys.exit(2)
    import torch
    from flash_tree_attn_amd import _lib, prepare
    from flash_tree_attn_amd.synthetic import CONFIGS, algorithmic_bytes, flops, make_inputs

    _lib.load()  # no fallback: fail loudly if the HIP library is missing
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    cfg = CONFIGS[args.config]
    dev = "cuda:0"
    torch.cuda.set_device(0)
    if args.reference_sweep:
        return reference_sweep(dev)
    if args.copy_calibration:
        nbytes_copy = 1 << 30
        src = torch.empty(nbytes_copy // 2, dtype=torch.bfloat16, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(max(args.steps, 1)):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": True, "bytes_read_per_copy": nbytes_copy, "bytes_written_per_copy": nbytes_copy,
                          "copies": max(args.steps, 1)}))
        return
    if args.op == "append_kv":
        return bench_append(args, cfg, dev)
    esz = torch.empty((), dtype=cfg.dtype).element_size()
    kv_bytes = 2 * cfg.bsz * cfg.num_kv_heads * cfg.cache_len * cfg.head_dim * esz
    kv_sets = args.kv_sets or max(2, min(8, -(-(1 << 30) // kv_bytes)))
    small = kv_bytes * kv_sets < (64 << 20)
    x = make_inputs(cfg, seed=0, device=dev, gen_device="cpu" if small else dev, kv_sets=kv_sets)

    mask_arg = x["mask"]
    if args.packed_mask:
        from flash_tree_attn_amd.tree_mask import pack_mask
        mask_arg = pack_mask(x["mask"])
    def paged(kc, vc, seed):
        """The same cache as a pool of shuffled pages plus its block table."""
        bsz, hkv, t, d = kc.shape
        pg, per_seq = args.paged, kc.shape[2] // args.paged
        perm = torch.randperm(bsz * per_seq, generator=torch.Generator().manual_seed(seed)).to(dev)
        pool = lambda c: c.view(bsz, hkv, per_seq, pg, d).permute(0, 2, 1, 3, 4).reshape(bsz * per_seq, hkv, pg, d)
        kp, vp = torch.empty_like(pool(kc)), torch.empty_like(pool(vc))
        kp[perm], vp[perm] = pool(kc), pool(vc)
        return kp, vp, perm.view(bsz, per_seq).to(torch.int32)

    kernel_ids = {"auto": -1, "mfma": _lib.KERNEL_MFMA, "mfma_wide": _lib.KERNEL_MFMA_WIDE, "mfma_split_keys": _lib.KERNEL_MFMA_SPLIT_KEYS,
                  "shuffle": _lib.KERNEL_SHUFFLE}
    if args.compare:
        return compare_kernels(args, cfg, x, mask_arg, [k.strip() for k in args.compare.split(",")], kernel_ids)
    calls = []
    for i, (kc, vc) in enumerate(zip(x["k_caches"], x["v_caches"])):
        tables = None
        if args.paged:
            assert cfg.cache_len % args.paged == 0
            kc, vc, tables = paged(kc, vc, i)
            if i == 0:
                x["k_cache_paged"], x["v_cache_paged"], x["tables"] = kc, vc, tables
        calls.append(prepare(x["q"], kc, vc, x["current_k"], x["current_v"], mask_arg, x["kv_seq_len"], cfg.block_size,
                             None, None, None, None, x["sm_scale"], cfg.kv_group_num, _force_splits=args.splits,
                             _force_kernel=kernel_ids[args.kernel],
                             block_tables=tables))
    if args.paged:   # the contiguous copies are no longer needed, except set 0 for the self-check
        x["k_caches"], x["v_caches"] = x["k_caches"][:1], x["v_caches"][:1]
    plan = calls[0].plan
    nbytes = algorithmic_bytes(cfg, x["kv_seq_len"].cpu(), mask_arg)
    nflops = flops(cfg, x["kv_seq_len"].cpu())

    # quick self-check of the measured path against the oracle on one sequence
    from oracle.tree_attn_oracle import tree_attention_oracle
    out = calls[0].run()
    ref = tree_attention_oracle(x["q"][:1], x["k_cache"][:1], x["v_cache"][:1], x["current_k"][:1], x["current_v"][:1],
                                x["mask"], x["kv_seq_len"][:1], x["sm_scale"], cfg.kv_group_num)
    tol = dict(atol=2e-3, rtol=1e-2) if cfg.dtype != torch.float32 else dict(atol=2e-5, rtol=1e-4)
    torch.testing.assert_close(out[:1].float(), ref, **tol)

    stream = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def timed(fn_name, steps):
        torch.cuda.synchronize()
        e0.record(stream)
        for i in range(steps):
            getattr(calls[i % kv_sets], fn_name)()
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps  # ms per step

    # settle phase: steady-state clocks before anything is timed (see --settle-ms)
    t_settle = time.perf_counter()
    while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
        for i in range(32):
            calls[i % kv_sets].run()
        torch.cuda.synchronize()
    for i in range(args.warmup):
        calls[i % kv_sets].run()
    # the timed region: exactly --steps calls, event-timed in batches (25 calls each from 50 steps on, 5 each from 10
    # on, one batch below that; the last batch takes what is left). With three batches or more the headline is the
    # median batch, so that one disturbed batch (a clock dip, another tenant of the host) does not move it; with
    # fewer it is the mean over all calls, and the line says which. The mean is reported beside it either way.
    per_batch = 25 if args.steps >= 50 else 5 if args.steps >= 10 else args.steps
    sizes = [per_batch] * (args.steps // per_batch) + ([args.steps % per_batch] if args.steps % per_batch else [])
    batch_ms = [timed("run", n) for n in sizes]
    ms_mean = sum(b * n for b, n in zip(batch_ms, sizes)) / args.steps
    full = sorted(b for b, n in zip(batch_ms, sizes) if n == per_batch)   # a short last batch takes no part in the median
    use_median = len(full) >= 3
    ms = full[len(full) // 2] if use_median else ms_mean
    batch_sorted = sorted(batch_ms)
    single_launch = bool(plan.single_launch)   # the merge runs inside the stage-1 kernel
    ms_two = timed("run_two_launches", args.steps) if single_launch else ms
    ms_stage1_alone = timed("run_stage1", args.steps)
    ms_stage2 = timed("run_stage2", args.steps) if plan.num_splits > 1 else 0.0
    # the dominant kernel as launched in the timed region: with the merge inside, the call IS that kernel
    ms_stage1 = ms if single_launch else ms_stage1_alone

    gbs = nbytes / (ms * 1e-3) / 1e9
    gbs_s1 = nbytes / (ms_stage1 * 1e-3) / 1e9
    result = {
        "metric": "tree-attn us/call + achieved HBM GB/s (% peak), 8B GQA q_len=64 @8K ctx",
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "settle_ms": args.settle_ms, "ms_per_step": ms, "us_per_call": ms * 1e3,
        "ms_per_step_is": ("median of the event-timed batches of the --steps calls" if use_median else
                           "mean over the --steps calls (fewer than three full batches: no median taken)"), "ms_per_step_mean": ms_mean,
        "us_per_call_batches": {"median": round(full[len(full) // 2] * 1e3, 2) if use_median else None, "min": round(batch_sorted[0] * 1e3, 2),
                                "max": round(batch_sorted[-1] * 1e3, 2), "batches": len(sizes), "calls_per_batch": per_batch,
                                "calls_in_last_batch": sizes[-1]},
        "pct_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}[cfg.dtype],
        "data": "synthetic (seed 0, N(0,1) q/k/v, random tree mask), inputs resident in HBM",
        "config": {"workload": cfg.name, "bsz": cfg.bsz, "q_heads": cfg.num_heads, "kv_heads": cfg.num_kv_heads,
                   "head_dim": cfg.head_dim, "q_len": cfg.q_len, "cache_len": cfg.cache_len, "lengths": cfg.lengths,
                   "block_size": cfg.block_size, "mask": "packed u64" if args.packed_mask else "additive f32",
                   "kv_layout": f"paged, {args.paged} positions per page, shuffled pool" if args.paged else "contiguous per sequence", "kv_sets_rotated": kv_sets, "num_splits": plan.num_splits,
                   "chunk": plan.chunk, "chunk_for_these_lengths": plan.chunk_for(int(x["kv_seq_len"].max())), "stage1_kernel": ("mfma", "mfma_wide", "mfma_split_keys")[plan.mfma_loop] if plan.kernel == _lib.KERNEL_MFMA else "shuffle",
                   "stage1_workgroups": plan.num_workgroups, "algorithmic_bytes": nbytes, "flops": nflops},
        "tflops": nflops / (ms * 1e-3) / 1e12,
        "roofline": {"bound": "hbm", "kernel": "stage1", "achieved": round(gbs_s1, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(gbs_s1 / HBM_PEAK_GBS, 4), "traffic": traffic_from_profiles(cfg.name),
                     "traffic_source": None if traffic_from_profiles(cfg.name) is None else f"profiles/stage1_{cfg.name}_pmc.txt (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE of an "
                                       "earlier run of this command, scaled by a plain copy; not measured in this run)",
                     "us_per_launch": ms_stage1 * 1e3, "single_launch": single_launch,
                     "two_launch_call_us": ms_two * 1e3, "stage1_without_merge_us": ms_stage1_alone * 1e3,
                     "stage2_us_per_launch": ms_stage2 * 1e3,
                     "mfma_tflops": nflops / (ms_stage1 * 1e-3) / 1e12,
                     "mfma_frac_of_dense_peak": round(nflops / (ms_stage1 * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4)},
    }
    # context for the datasheet peak: what a plain device copy of 1 GiB streams on this box (read + write bytes)
    src = torch.empty(1 << 29, dtype=torch.bfloat16, device=dev).normal_()
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    e0.record(stream)
    for _ in range(10):
        dst.copy_(src)
    e1.record(stream)
    torch.cuda.synchronize()
    copy_gbs = 10 * 2 * src.numel() * 2 / (e0.elapsed_time(e1) * 1e-3) / 1e9
    del src, dst
    result["measured_copy_gbs"] = round(copy_gbs, 1)
    result["roofline"]["frac_of_measured_copy"] = round(gbs_s1 / copy_gbs, 4)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(cfg, x, args.cpu_seconds)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
