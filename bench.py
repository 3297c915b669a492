#!/usr/bin/env python3
"""Benchmarks of the paged-attention hot path on one MI355X.

Default (the headline line): paged decode, Llama-7B layer shape, batch 64.
One step = one pass of the decode hot path over one batch for one transformer
layer: KV append of the new K/V rows (one per sequence), then paged attention
of the query tokens against the block KV cache (32 q heads, 32 kv heads,
head_dim 128, bf16, block 16, context lengths uniform in [512, 4096], randomly
permuted block tables, q/K/V ~ N(0,1)).  Several layers' pools are resident
and the steps rotate over them, as a decoder's layers do, so no step re-reads
bytes the previous one left in cache.

With no `--workload` (or `--workload all`) all five configurations run, each
under the same gates, and appear in the line's `workloads` object (the headline
fields are the Llama-7B ones).  Every workload's parity gate runs first (its
CPU oracle keeps the GPU idle for seconds), then the timed regions follow each
other without a gap: the first milliseconds of GPU work after an idle gap run in
a power transient (`after_idle` shows it launch by launch), which is not the
state a serving loop is in.  `--workload llama70b | grpo` run the GQA and the shared-prefix decode shapes
the same way; `--workload prefill` runs chunked prefill + KV append (16
sequences, cached prefix uniform in [0, 4096], 512 new tokens each) and
reports TFLOP/s against the dense bf16 MFMA peak.  `--workload gpt2` runs the
configuration the reference itself can run on a CPU, end to end: GPT-2 small,
random-init fp32, batch 4, prompts of 128 token ids, greedy decode of 64 tokens
through the block KV cache (one step = one whole generation), tokens/s =
4 * 64 / wall, tokens checked against the CPU oracle's loop, with the oracle's
paged loop and its full-recompute loop (examples/generate_text.py:24-40) timed
beside it.

Prints ONE JSON line.  For decode `value` is achieved HBM GB/s of the whole
step (algorithmic bytes / wall time per step), with decode tokens/s beside it;
`roofline` describes the dominant call (decode: main kernel + its split-K
reduce; prefill: the MFMA kernel) timed with events on the launch stream in a
pass of its own after the wall-timed steps (EVENT_LAUNCHES launches, each
bracketed by an event pair); `cpu_baseline` is the CPU oracle (the
reference's dense attention arithmetic driven through the block table) timed
on the host cores on the same workload.  Before anything is timed every
sequence of the batch is checked against the oracle (max-abs 2e-2, bf16) and
the appended rows are compared with the pool bit for bit.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, vendor figure
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 matrix, vendor figure

EVENT_LAUNCHES = 40         # event-bracketed launches of the dominant call behind `roofline`
PARITY_BAR = 2e-2           # max-abs against the oracle, bf16 (the bar the target states)
ROOT = os.path.dirname(os.path.abspath(__file__))
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def measured_traffic(workload, seed):
    """HBM bytes per launch of the workload's dominant kernel as the profiler's
    FETCH_SIZE / WRITE_SIZE counters gave them (profiles/traffic.json holds
    the counter readings, the scale factors from a copy of known size and a
    digest of the kernel sources they were measured on).  A figure measured
    on other sources than the ones that are about to run is not reported:
    returns (bytes or None, stale flag)."""
    from ironcore_amd import build as ic_build
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None, False
    ent = rec.get("workloads", {}).get(workload)
    if ent is None or ent.get("seed", 0) != seed:
        return None, False
    if rec.get("csrc_sha256") != ic_build.csrc_digest():
        return None, True
    return int(ent["hbm_bytes_per_launch"]), False


DOMINANT_KERNEL = {"llama7b": "paged_decode_mfma_kernel", "llama70b": "paged_decode_mfma_kernel",
                   "grpo": "paged_decode_mfma_kernel", "prefill": "paged_prefill_kernel"}
COPY_BYTES = 1 << 30


def traffic_record(prof_dir, seed):
    """profiles/traffic.json from counter runs of this file (one counter per
    run, --copy-calibration on): per workload, the dominant kernel's
    FETCH_SIZE and WRITE_SIZE per dispatch (KiB, mean over its dispatches),
    each scaled by what the same counter read for the 1 GiB device copy
    (which reads and writes 1 GiB), as HBM bytes per launch."""
    import csv
    import glob
    from ironcore_amd import build as ic_build

    def per_dispatch(run_dir, counter, kernel):
        files = glob.glob(os.path.join(run_dir, "**", "*counter_collection.csv"), recursive=True)
        if not files:
            return None, None
        mine, copies = [], []
        for row in csv.DictReader(open(files[0])):
            if row["Counter_Name"] != counter:
                continue
            name, val = row["Kernel_Name"], float(row["Counter_Value"])
            if kernel in name:
                mine.append(val)
            elif "copy" in name.lower():
                copies.append(val)
        if not mine or not copies:
            return None, None
        # the calibration copies move 2^20 KiB each way; the counter reads that, or half of it (it
        # counts in larger units on some paths), to within a percent
        kib = COPY_BYTES / 1024.0
        cal = [v for v in copies if abs(v / kib - 1) < 0.01 or abs(2 * v / kib - 1) < 0.01]
        if not cal:
            return None, None
        return sum(mine) / len(mine), sum(cal) / len(cal)

    rec = {"csrc_sha256": ic_build.csrc_digest(), "unit": "KiB per dispatch", "copy_bytes": COPY_BYTES,
           "workloads": {}}
    for workload, kernel in DOMINANT_KERNEL.items():
        ent = {"kernel": kernel, "seed": seed}
        total = 0.0
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            k, c = per_dispatch(os.path.join(prof_dir, f"pmc_{counter}_{workload}"), counter, kernel)
            if k is None:
                ent = None
                break
            scale = (COPY_BYTES / 1024.0) / c  # counter units per KiB actually moved by the copy
            ent[counter] = round(k, 1)
            ent[counter + "_copy"] = round(c, 1)
            ent[counter + "_scale"] = round(scale, 4)
            total += k * scale * 1024.0
        if ent is not None:
            ent["hbm_bytes_per_launch"] = int(round(total))
            rec["workloads"][workload] = ent
    os.makedirs(os.path.dirname(TRAFFIC_FILE), exist_ok=True)
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(rec, f, indent=1, sort_keys=True)
        f.write("\n")
    return rec


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default 200; gpt2: 5)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps (default 20; gpt2: 1)")
    ap.add_argument("--layers", type=int, default=4, help="resident layer pools the steps rotate over")
    ap.add_argument("--min-chunk-tokens", type=int, default=0, help="smallest split-K share (0 = library default)")
    ap.add_argument("--workload", default="all",
                    choices=["all", "llama7b", "llama70b", "grpo", "prefill", "gpt2"],
                    help="all = the headline line (llama7b) with the other four configurations under `workloads`")
    ap.add_argument("--cohort-size", type=int, default=0,
                    help="shared-prefix cohort size for decode (0 = the samples per prompt of the workload, else 1)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--zero-operands", action="store_true",
                    help="prefill: replace q, K and V by zeros (same kernel, same instructions, same bytes; shows "
                         "how much of the launch time is the clock the device holds under toggling operands)")
    ap.add_argument("--no-mfma-probe", action="store_true",
                    help="prefill: skip the 2 s measurement of the matrix rate the device sustains")
    ap.add_argument("--no-after-idle", action="store_true",
                    help="prefill: skip the pass that profiles the first launches after an idle gap (counter runs: "
                         "its launches would enter the per-dispatch averages)")
    ap.add_argument("--cpu-seconds", type=float, default=6.0, help="CPU baseline time budget per workload")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy (known traffic) so a counter run can be scaled")
    ap.add_argument("--traffic-from", metavar="DIR", default=None,
                    help="no benchmark: read the rocprofv3 counter runs under DIR (pmc_FETCH_SIZE_<workload>/, "
                         "pmc_WRITE_SIZE_<workload>/, each made with --copy-calibration) and write "
                         "profiles/traffic.json, stamped with the digest of the kernel sources")
    args = ap.parse_args()
    args.gpt2_steps = args.steps if args.workload == "gpt2" and args.steps else 5
    args.gpt2_warmup = args.warmup if args.workload == "gpt2" and args.warmup is not None else 1
    if args.steps is None:
        args.steps = 200
    if args.warmup is None:
        args.warmup = 20
    return args


def cpu_info():
    import torch
    try:
        model = next(l.split(":", 1)[1].strip() for l in open("/proc/cpuinfo") if l.startswith("model name"))
    except Exception:
        model = "unknown"
    return {"cores": torch.get_num_threads(), "host_cpu_count": os.cpu_count(), "cpu_model": model}


def copy_calibration(torch, dev):
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()


def time_steps(torch, step, steps, warmup, event_launches=EVENT_LAUNCHES):
    """Run `warmup` untimed steps, then exactly `steps` timed ones bracketed by
    synchronisations (no events inside: an event costs a step a launch slot),
    then a pass of `event_launches` further steps each of which records an
    event pair around its dominant call.  `step(i, ev)` enqueues step i and
    records `ev[0]` before and `ev[1]` after the dominant call when `ev` is not
    None.  Returns (ms per step by wall clock, per-call ms of the dominant
    call)."""
    for i in range(warmup):
        step(i, None)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i, None)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall * 1e3 / steps, event_pass(torch, step, steps, event_launches)


def event_pass(torch, step, first, n):
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for i, pair in enumerate(ev):
        step(first + i, pair)
    torch.cuda.synchronize()
    return [a.elapsed_time(b) for a, b in ev]


def after_idle(torch, step, idle_s, warmup, steps):
    """What the first launches after an idle GPU cost.  The wall-timed steps
    follow the parity gate, during which the CPU oracle runs for seconds and
    the GPU does nothing; with the driver's counts (5 + 20 steps) they are the
    first few milliseconds of work after that gap.  This pass repeats the
    situation (GPU idle for `idle_s`, then `n` steps, every call bracketed by
    events) so that the line can say how much of a step's wall time beyond its
    kernels' steady-state time is the device still raising its clock."""
    torch.cuda.synchronize()
    time.sleep(idle_s)
    n = min(warmup + steps, 60)
    dom = event_pass(torch, step, 0, n)
    window = dom[warmup:] if warmup < n else dom
    return {"idle_s": round(idle_s, 2), "launches": n, "dominant_call_ms": [round(x, 4) for x in dom],
            "mean_of_timed_window_ms": round(sum(window) / len(window), 5),
            "what": "the dominant call by events for the first launches after the GPU sat idle as long as "
                    "during the parity gate's CPU oracle; the wall-timed steps start in the same state, and "
                    "mean_of_timed_window_ms (launches warmup .. warmup+steps-1 of this pass) is what the "
                    "dominant call cost inside them: after an idle gap the device runs its first millisecond "
                    "of work at a high clock, then drops below its steady clock for a few milliseconds and "
                    "recovers over tens of milliseconds, so a timed region of a few milliseconds right after "
                    "the gate sits in that transient, while the steady-state event times behind `roofline` "
                    "do not"}


def timed_oracle(fn, budget_s):
    """The parity gate's oracle call doubles as the CPU baseline: run it once
    (result kept for the gate), then again while the budget lasts (at most two
    more), and report the median.  Returns (result, seconds, runs)."""
    t0 = time.perf_counter()
    ref = fn()
    times = [time.perf_counter() - t0]
    while len(times) < 3 and sum(times) + times[-1] <= budget_s:
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return ref, statistics.median(times), len(times)


def bench_decode(args, torch, dev, workload):
    from ironcore_amd import paged_ops, workloads
    from oracle import paged as oracle_paged
    make = {"llama7b": workloads.llama7b_decode, "llama70b": workloads.llama70b_gqa_decode,
            "grpo": workloads.qwen7b_grpo_decode}[workload]
    wl = make(device=dev, seed=args.seed)
    b, hn, gn, hd, bs = wl.batch, wl.hn, wl.gn, wl.hd, wl.block_size
    pools = [(wl.k_pool, wl.v_pool)]          # one pool pair per resident layer
    for layer in range(1, args.layers):
        g = torch.Generator(device=dev)
        g.manual_seed(args.seed + 100 + layer)
        pools.append(tuple(torch.randn(wl.k_pool.shape, generator=g, device=dev, dtype=torch.float32)
                           .to(wl.k_pool.dtype) for _ in range(2)))
    # the step's new K/V rows go to the slot of each sequence's last token
    last = wl.context_lens.long() - 1
    slot_mapping = (wl.block_tables.long().gather(1, (last // bs).unsqueeze(1)).squeeze(1) * bs + last % bs)
    g = torch.Generator(device=dev)
    g.manual_seed(args.seed + 7)
    k_new = torch.randn(b, gn, hd, generator=g, device=dev, dtype=torch.float32).to(wl.k_pool.dtype)
    v_new = torch.randn(b, gn, hd, generator=g, device=dev, dtype=torch.float32).to(wl.k_pool.dtype)
    out = torch.empty(b, hn * hd, dtype=wl.query.dtype, device=dev)
    # sequences that alias prefix blocks (GRPO samples of one prompt) are decoded in
    # cohorts that stream the shared blocks once; the sharing is a property of the
    # block tables, found on the host once, outside the timed region
    cohort = args.cohort_size if args.cohort_size > 0 else int(wl.extra.get("n_samples", 1))
    shared = None
    if cohort > 1:
        shared = torch.from_numpy(paged_ops.shared_prefix_blocks(
            wl.block_tables.cpu().numpy(), wl.context_lens.cpu().numpy(), bs, cohort)).to(dev)

    def step(i, ev):
        kp, vp = pools[i % len(pools)]
        paged_ops.kv_append(k_new, v_new, kp, vp, slot_mapping)
        if ev:
            ev[0].record()
        paged_ops.paged_decode(wl.query, kp, vp, wl.block_tables, wl.context_lens,
                               wl.max_context_len, out=out, min_chunk_tokens=args.min_chunk_tokens,
                               cohort_size=cohort, cohort_shared_blocks=shared)
        if ev:
            ev[1].record()

    # parity gate on the tensors that are about to be timed: EVERY sequence of the batch against
    # the oracle, and the appended rows against the pool bit for bit
    step(0, None)
    torch.cuda.synchronize()
    kp_cpu, vp_cpu = pools[0][0].cpu(), pools[0][1].cpu()
    q_cpu, bt_cpu, cl_cpu = wl.query.cpu(), wl.block_tables.cpu(), wl.context_lens.cpu()
    ref, cpu_s, cpu_runs = timed_oracle(
        lambda: oracle_paged.paged_decode(q_cpu, kp_cpu, vp_cpu, bt_cpu, cl_cpu),
        0.0 if args.no_cpu_baseline else args.cpu_seconds)
    parity = (out.float().cpu() - ref.float()).abs().max().item()
    if not parity <= PARITY_BAR:
        sys.exit(f"parity gate failed ({wl.name}): max|out - oracle| = {parity} > {PARITY_BAR}")
    sm = slot_mapping.cpu()
    for pool_cpu, new in ((kp_cpu, k_new), (vp_cpu, v_new)):
        got = pool_cpu[sm // bs, :, sm % bs, :]
        if not torch.equal(got.view(torch.int16), new.cpu().view(torch.int16)):
            sys.exit(f"parity gate failed ({wl.name}): appended rows differ from the pool")
    del kp_cpu, vp_cpu, ref
    yield None          # the gate is passed; everything below is measurement
    if args.copy_calibration:
        copy_calibration(torch, dev)

    ms_per_step, decode_ms = time_steps(torch, step, args.steps, args.warmup)
    decode_ms_avg = sum(decode_ms) / len(decode_ms)

    def append_only(i, ev):
        if ev:
            ev[0].record()
        paged_ops.kv_append(k_new, v_new, pools[0][0], pools[0][1], slot_mapping)
        if ev:
            ev[1].record()
    append_ms_avg = statistics.mean(event_pass(torch, append_only, 0, 20))
    es = wl.query.element_size()
    decode_bytes = wl.algorithmic_bytes()
    append_bytes = 2 * (2 * b * gn * hd * es) + 8 * b
    value = (decode_bytes + append_bytes) / (ms_per_step * 1e-3) / 1e9
    achieved = decode_bytes / (decode_ms_avg * 1e-3) / 1e9
    traffic, stale = measured_traffic(workload, args.seed)
    result = {
        "metric": "paged_decode_hbm_gbps", "value": round(value, 1), "unit": "GB/s",
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "decode_tokens_per_s_per_layer": round(b / (ms_per_step * 1e-3), 1),
        "decode_tokens_per_s_32_layers": round(b / (32 * ms_per_step * 1e-3), 1),
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": wl.name, "batch": b, "q_heads": hn, "kv_heads": gn, "head_dim": hd,
                   "block_size": bs, "sum_context": wl.logical_tokens, "unique_tokens": wl.unique_tokens,
                   "resident_layers": len(pools), "cohort_size": cohort,
                   "step": f"kv_append({b} rows) + paged_decode, one layer"},
        "parity_max_abs_vs_oracle": parity,
        # wall time of a step beyond its two calls' steady-state event times.  An event pair adds a few
        # microseconds to what it brackets (for the 64-row append more than the 4.5 us the kernel takes by
        # the profiler), so a step without launch gaps reads below zero here
        "append_ms": round(append_ms_avg, 5),
        "step_minus_kernels_ms": round(ms_per_step - decode_ms_avg - append_ms_avg, 5),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic,
                     "kernel": "paged_decode_mfma_kernel (+ paged_decode_reduce_kernel)",
                     "bytes_per_launch": decode_bytes, "avg_launch_ms": round(decode_ms_avg, 5),
                     "median_launch_ms": round(statistics.median(decode_ms), 5),
                     "n_event_samples": len(decode_ms)},
    }
    if stale:
        result["roofline"]["traffic_stale"] = True
    if wl.logical_tokens != wl.unique_tokens:
        logical = wl.logical_tokens * wl.kv_bytes_per_token()
        result["logical_kv_gbps"] = round(logical / (decode_ms_avg * 1e-3) / 1e9, 1)
    if not args.no_cpu_baseline:
        tokens = wl.logical_tokens
        result["cpu_baseline"] = {
            "value": round(tokens * wl.kv_bytes_per_token() / cpu_s / 1e9, 3), "unit": "GB/s", "kind": "port",
            "sample": f"all {b} sequences of the same batch, one layer, median of {cpu_runs} run(s) of the "
                      f"oracle (gather through the block table + dense attention); {tokens} context tokens",
            "tokens_per_s_per_layer": round(b / cpu_s, 2), **cpu_info()}
    yield result


def bench_prefill(args, torch, dev):
    from ironcore_amd import paged_ops, workloads
    from oracle import paged as oracle_paged
    wl = workloads.llama7b_chunked_prefill(device=dev, seed=args.seed)
    if args.zero_operands:
        for t in (wl.query, wl.k_new, wl.v_new, wl.k_pool, wl.v_pool):
            t.zero_()
    out = torch.empty(wl.query.shape[0], wl.hn * wl.hd, dtype=wl.query.dtype, device=dev)

    def step(i, ev):
        paged_ops.kv_append(wl.k_new, wl.v_new, wl.k_pool, wl.v_pool, wl.slot_mapping)
        if ev:
            ev[0].record()
        paged_ops.paged_prefill(wl.query, wl.k_pool, wl.v_pool, wl.block_tables, wl.context_lens,
                                wl.cu_seqlens_q, wl.max_chunk_len, causal=True, out=out)
        if ev:
            ev[1].record()

    # parity gate: ALL sequences, all heads, against the oracle; the appended rows against the
    # pool bit for bit
    step(0, None)
    torch.cuda.synchronize()
    cpu = (wl.query.cpu(), wl.k_pool.cpu(), wl.v_pool.cpu(), wl.block_tables.cpu(), wl.context_lens.cpu(),
           wl.cu_seqlens_q.cpu())
    ref, cpu_s, cpu_runs = timed_oracle(lambda: oracle_paged.paged_prefill(*cpu),
                                        0.0 if args.no_cpu_baseline else args.cpu_seconds)
    parity = (out.float().cpu() - ref.float()).abs().max().item()
    if not parity <= PARITY_BAR:
        sys.exit(f"parity gate failed ({wl.name}): max|out - oracle| = {parity} > {PARITY_BAR}")
    sm = wl.slot_mapping.cpu()
    for pool_cpu, new in ((cpu[1], wl.k_new), (cpu[2], wl.v_new)):
        got = pool_cpu[sm // wl.block_size, :, sm % wl.block_size, :]
        if not torch.equal(got.view(torch.int16), new.cpu().view(torch.int16)):
            sys.exit(f"parity gate failed ({wl.name}): appended rows differ from the pool")
    del cpu, ref
    yield None          # the gate is passed; everything below is measurement
    if args.copy_calibration:
        copy_calibration(torch, dev)

    ms_per_step, call_ms = time_steps(torch, step, args.steps, args.warmup)
    call_avg = sum(call_ms) / len(call_ms)
    idle = None if args.no_after_idle else after_idle(torch, step, min(max(cpu_s * cpu_runs, 0.5), 6.0),
                                                      args.warmup, args.steps)
    flops = wl.flops()
    es = wl.query.element_size()
    append_bytes = 2 * 2 * wl.k_new.numel() * es
    tflops = flops / (call_avg * 1e-3) / 1e12
    n_tok = wl.query.shape[0]
    traffic, stale = measured_traffic("prefill", args.seed)

    def append_only(i, ev):
        if ev:
            ev[0].record()
        paged_ops.kv_append(wl.k_new, wl.v_new, wl.k_pool, wl.v_pool, wl.slot_mapping)
        if ev:
            ev[1].record()
    _, app_ms = time_steps(torch, append_only, 5, 5)
    app_in_step_avg = statistics.mean(app_ms)

    # the same append with rotary embedding fused in (Q rotated in place, K rotated
    # into the pool, V copied), timed the same way on a scratch copy of the query
    from ironcore_amd.layers.rotary import RotaryPositionalEmbedding
    rope = RotaryPositionalEmbedding(wl.hd, max_seq_len=8192).to(dev)
    cos_t, sin_t = rope.cos_emb, rope.sin_emb
    q_rot = wl.query.clone()
    pos = torch.cat([torch.arange(pf, pf + c, dtype=torch.int32) for pf, c in zip(wl.prefix_lens, wl.chunk_lens)]
                    ).to(dev)

    def rope_append_only(i, ev):
        if ev:
            ev[0].record()
        paged_ops.rope_kv_append(q_rot, wl.k_new, wl.v_new, wl.k_pool, wl.v_pool, wl.slot_mapping, pos,
                                 cos_t, sin_t)
        if ev:
            ev[1].record()
    _, rope_ms = time_steps(torch, rope_append_only, 5, 5)
    rope_bytes = append_bytes + 2 * wl.query.numel() * es
    paged_ops.kv_append(wl.k_new, wl.v_new, wl.k_pool, wl.v_pool, wl.slot_mapping)  # leave the pool unrotated

    # the matrix rate the device sustains once its clock has settled under load: a register-only
    # MFMA loop on every SIMD, launched back to back for over a second, the last launches timed
    sustained = None
    if not args.no_mfma_probe:
        sink = torch.zeros(16, dtype=torch.float32, device=dev)
        iters = 20000  # about 6 ms per launch
        t_end = time.perf_counter() + 1.5
        probe_flops = 0
        while time.perf_counter() < t_end:
            for _ in range(10):
                probe_flops = paged_ops.mfma_probe(iters, sink)
            torch.cuda.synchronize()
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(20)]
        for a, b in ev:
            a.record()
            paged_ops.mfma_probe(iters, sink)
            b.record()
        torch.cuda.synchronize()
        probe_ms = statistics.mean(a.elapsed_time(b) for a, b in ev)
        sustained = probe_flops / (probe_ms * 1e-3) / 1e12

    result = {
        "metric": "paged_prefill_mfma_tflops", "value": round(flops / (ms_per_step * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s", "prefill_tokens_per_s_per_layer": round(n_tok / (ms_per_step * 1e-3), 1),
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic, all-zero operands (a clock probe, not the benchmark workload)" if args.zero_operands
                else "synthetic",
        "config": {"workload": wl.name, "n_seqs": len(wl.chunk_lens), "chunk": wl.max_chunk_len,
                   "sum_prefix": sum(wl.prefix_lens), "q_heads": wl.hn, "kv_heads": wl.gn,
                   "head_dim": wl.hd, "block_size": wl.block_size,
                   "step": "kv_append(chunk rows) + paged_prefill, one layer"},
        "parity_max_abs_vs_oracle": parity,
        "append_ms": round(app_in_step_avg, 5),
        "step_minus_kernels_ms": round(ms_per_step - call_avg - app_in_step_avg, 5),
        **({"after_idle": idle} if idle is not None else {}),
        "append_hbm_gbps": round(append_bytes / (statistics.mean(app_ms) * 1e-3) / 1e9, 1),
        "rope_append_hbm_gbps": round(rope_bytes / (statistics.mean(rope_ms) * 1e-3) / 1e9, 1),
        "roofline": {"bound": "mfma", "achieved": round(tflops, 2), "peak": MFMA_BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": traffic,
                     "kernel": "paged_prefill_kernel", "flops_per_launch": flops,
                     "avg_launch_ms": round(call_avg, 5), "median_launch_ms": round(statistics.median(call_ms), 5),
                     "n_event_samples": len(call_ms)},
    }
    if stale:
        result["roofline"]["traffic_stale"] = True
    if sustained is not None:
        # not the roofline's peak (that is the vendor's figure): what a bare MFMA loop reaches on
        # this box, and the kernel's rate as a fraction of it
        result["roofline"]["sustained_mfma"] = {
            "value": round(sustained, 1), "unit": "TFLOP/s",
            "what": "independent v_mfma_f32_32x32x16_bf16, register operands, one wave per SIMD, after 1.5 s of "
                    "back-to-back launches (ic_mfma_probe)",
            "frac_of_peak": round(sustained / MFMA_BF16_PEAK_TFLOPS, 4),
            "kernel_frac_of_sustained": round(tflops / sustained, 4)}
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = {"value": round(flops / cpu_s / 1e12, 4), "unit": "TFLOP/s", "kind": "port",
                                  "sample": f"all {len(wl.chunk_lens)} sequences of the batch, all heads, median of "
                                            f"{cpu_runs} run(s) of the oracle (gather through the block table + dense "
                                            "attention under the shifted causal mask)",
                                  **cpu_info()}
    yield result


def bench_gpt2(args, torch, dev):
    """GPT-2 small end to end (12 layers, 12 heads, head_dim 64, vocab 50257,
    configs/model/gpt2-small.yaml:1-9), fp32, batch 4, 128 + 64 tokens, block 16."""
    from ironcore_amd import config as ic_config
    from ironcore_amd import generation
    from oracle import gpt2 as oracle_gpt2
    batch, prompt, new = 4, 128, 64
    cfg = ic_config.gpt2_small_config("fp32")
    torch.manual_seed(args.seed)
    model = generation.LanguageModel(cfg, vocab_size=50257)
    weights = {k: v.detach().clone() for k, v in model.state_dict().items()}
    ids = torch.randint(0, 50257, (batch, prompt), generator=torch.Generator().manual_seed(args.seed))
    model = model.to(dev)
    ids_dev = ids.to(dev)
    m = cfg.model
    dims = oracle_gpt2.Dims(m.num_layers, m.num_attention_heads, m.num_attention_groups, m.d_model, m.ln_eps)

    def timed(fn, steps, warmup):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            out = fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps, out

    # parity gate: one generation on the GPU against the CPU oracle's loops (which are also the CPU baseline)
    got = generation.generate(model, ids_dev, new, use_graph=True)
    torch.cuda.synchronize()
    cpu = None
    if not args.no_cpu_baseline:
        t0 = time.perf_counter()
        want, margins = oracle_gpt2.generate_paged(weights, dims, ids, new, return_margins=True)
        t_paged = time.perf_counter() - t0
        if not torch.equal(got.cpu(), want):
            sys.exit(f"parity gate failed: greedy tokens differ from the oracle's (min margin {margins.min().item():.3e})")
        t0 = time.perf_counter()
        full = oracle_gpt2.generate_full_recompute(weights, dims, ids, new)
        t_full = time.perf_counter() - t0
        cpu = {"value": round(batch * new / t_paged, 1), "unit": "tokens/s", "kind": "port",
               "sample": "the whole workload, once: the oracle's block-KV-cache loop",
               "full_recompute_tokens_per_s": round(batch * new / t_full, 1),
               "full_recompute_equals_paged": bool(torch.equal(full, want)), **cpu_info()}
        min_margin = margins.min().item()
    yield None          # the gate is passed; everything below is measurement

    sec, got = timed(lambda: generation.generate(model, ids_dev, new, use_graph=True), args.gpt2_steps, args.gpt2_warmup)
    sec_eager, got_eager = timed(lambda: generation.generate(model, ids_dev, new), args.gpt2_steps, args.gpt2_warmup)
    sec_full, got_full = timed(lambda: generation.generate_full_recompute(model, ids_dev, new), 1, 0)
    if not torch.equal(got, got_eager):
        sys.exit("parity gate failed: the graph-replay loop and the step-by-step loop chose different tokens")
    if cpu is not None and not torch.equal(got.cpu(), want):
        sys.exit("parity gate failed: a timed generation chose other tokens than the gated one")
    result = {
        "metric": "generate_tokens_per_s", "value": round(batch * new / sec, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.gpt2_steps, "warmup": args.gpt2_warmup, "ms_per_step": round(sec * 1e3, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "gpt2-small end to end: random-init fp32, batch 4, prompt 128, greedy 64 new tokens, "
                               "block 16",
                   "step": "one generation: prefill of the prompts, 63 cached decode steps (one eager, one "
                           "captured into a HIP graph, 61 replays of it; capture is inside the timed region)"},
        "step_by_step_tokens_per_s_gpu": round(batch * new / sec_eager, 1),
        "full_recompute_tokens_per_s_gpu": round(batch * new / sec_full, 1),
        "paged_equals_full_recompute_gpu": bool(torch.equal(got, got_full)),
        # every kernel of a step is far below its roofline at this size (a decode step streams
        # 12 layers x 4 sequences x <= 192 tokens of K/V): the step is bound by launches
        "roofline": None,
    }
    if cpu is not None:
        result["tokens_identical_to_oracle"] = True
        result["min_top1_top2_margin"] = min_margin
        result["cpu_baseline"] = cpu
    yield result


def main():
    args = parse()
    if args.traffic_from:
        rec = traffic_record(args.traffic_from, args.seed)
        print(json.dumps({"traffic_record": TRAFFIC_FILE, "workloads": sorted(rec["workloads"]),
                          "csrc_sha256": rec["csrc_sha256"]}))
        return
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the paged-attention path is single-GPU "
                 "(sequences and KV heads shard without communication); run with --gpus 1")
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (the paged path has no CPU implementation)")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    def start(workload):
        """The workload's generator: its first step builds the inputs and passes the parity gate
        (GPU result against the CPU oracle, which is timed as the CPU baseline), its second
        measures and returns the result."""
        if workload == "prefill":
            gen = bench_prefill(args, torch, dev)
        elif workload == "gpt2":
            gen = bench_gpt2(args, torch, dev)
        else:
            gen = bench_decode(args, torch, dev, workload)
        next(gen)
        return gen

    if args.workload != "all":
        print(json.dumps(next(start(args.workload))))
        return
    t0 = time.perf_counter()
    # Every workload's gate first (seconds of CPU oracle each, the GPU idle), then the timed regions
    # back to back: a timed region then follows GPU work, not an idle gap, and measures the state a
    # serving loop is in.  (After an idle gap the first milliseconds of work run in a power
    # transient, see `after_idle` in the prefill entry.)  All five workloads are resident together
    # (about 25 GB).  The end-to-end workload runs first: its half second of small launches is what
    # the headline workload's warm-up steps follow.
    order = ("gpt2", "llama7b", "llama70b", "grpo", "prefill")
    gens = {w: start(w) for w in ("llama7b", "llama70b", "grpo", "prefill", "gpt2")}
    gates_s = time.perf_counter() - t0
    results = {w: next(gens[w]) for w in order}
    result = results["llama7b"]
    # the other configurations, each gated and measured the same way; an entry keeps the fields
    # that describe a measurement and drops the ones that repeat the top-level line's
    keep = ("metric", "value", "unit", "ms_per_step", "steps", "warmup", "dtype", "config", "roofline",
            "cpu_baseline", "parity_max_abs_vs_oracle", "pct_of_hbm_peak", "decode_tokens_per_s_per_layer",
            "logical_kv_gbps", "prefill_tokens_per_s_per_layer", "append_hbm_gbps", "rope_append_hbm_gbps",
            "append_ms", "step_minus_kernels_ms", "after_idle",
            "tokens_identical_to_oracle", "step_by_step_tokens_per_s_gpu", "full_recompute_tokens_per_s_gpu",
            "paged_equals_full_recompute_gpu", "min_top1_top2_margin")
    result["workloads"] = {w: {k: results[w][k] for k in keep if k in results[w]}
                           for w in ("llama7b", "llama70b", "grpo", "prefill", "gpt2")}
    result["run_order"] = {"gates": ["llama7b", "llama70b", "grpo", "prefill", "gpt2"], "gates_s": round(gates_s, 1),
                           "timed": list(order)}
    result["bench_wall_s"] = round(time.perf_counter() - t0, 1)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
