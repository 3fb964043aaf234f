#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2|c1|c3|c4|c5|idx|all]

Default (what the driver runs): configuration 2 of BASELINE.json — Llama-3-8B-shape GQA
flash-decode, batch 64, every sequence at context 4096, bf16 paged KV cache with block size 128,
plus the reshape-and-cache (`rope_and_cache`) of the 64 new tokens. One step = one
`rope_and_cache` + one `attention` call over that batch, inputs resident in HBM. Prints ONE JSON
line; `value` is KV bytes read per second over the whole step. `roofline` prices the dominant
kernel (the decode attention kernel) against the 8 TB/s HBM peak; `cpu_baseline` times the CPU
oracle on a bounded sample of the same workload on the host cores.

Other configurations (`--config`) print the same kind of line for their own workload; `all`
prints one line per configuration (the first line is still configuration 2).
"""
import argparse
import json
import os
import sys
import time

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE runs of this
# script scaled by the same counters' readings for a plain 1 GiB copy (see --calibrate-copy); None
# where no counter run has been taken.
MEASURED_TRAFFIC_BYTES = {"c2": 1080233210, "c3": 302337768, "c4": 325291619, "c5": 1623718207}


def _events(torch):
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


def _time_region(torch, fn, iters):
    """Average milliseconds per call of `fn` over `iters` back-to-back asynchronous calls, from HIP
    events recorded on the stream the kernels are launched on (torch's current stream)."""
    a, b = _events(torch)
    torch.cuda.synchronize()
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


def _launch_dist(torch, fn, launches=100):
    """Median, 10th and 90th percentile (ms) of `launches` back-to-back calls of `fn`, each between its own
    pair of HIP events on the stream the kernels are launched on."""
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(launches + 1)]
    torch.cuda.synchronize()
    ev[0].record()
    for i in range(launches):
        fn()
        ev[i + 1].record()
    torch.cuda.synchronize()
    t = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(launches))
    pick = lambda q: round(t[min(launches - 1, int(q * launches))], 4)
    return {"median": pick(0.5), "p10": pick(0.1), "p90": pick(0.9), "launches": launches}


def _cpu_info():
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return model


def _cpu_threads(torch):
    n = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    n = max(1, min(n, os.cpu_count() or 1))
    torch.set_num_threads(n)
    return n


def bench_gqa_decode(args, torch, rt, name, shape, ctx, seed, int8=False, with_rope=True):
    from gvirt_amd import workloads as W
    from gvirt_amd import _C
    dev = "cuda:0"
    w = W.gqa_decode(shape, ctx, seed, device=dev, int8_kv=int8)
    r = W.rope_inputs(shape, w, seed) if with_rope and not int8 else None
    s = shape
    B = w["batch"]
    rt.blocking = False
    pristine = r["inout"].clone() if r is not None else None

    def rope():
        _C.rope_and_cache(rt, r["inout"], w["k_cache"], w["v_cache"], r["position"], r["cosin"], r["slot_mapping"],
                          s.n_heads, s.n_kv_heads, s.head_dim, s.head_dim, s.block_size, True)

    def attn():
        _C.attention(rt, r["inout"] if r is not None else w["qkv"], w["k_cache"], w["v_cache"], w["output"],
                     w["query_start_loc"], w["lens"], w["cached_lens"], w["block_tables"], s.n_heads, s.n_kv_heads,
                     s.head_dim, s.block_size, B, w["max_num_block"], k_scale=w["k_scale"], v_scale=w["v_scale"])

    def step():
        if r is not None:
            rope()
        attn()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    run_step = step
    if args.graph:
        # the step captured once into a HIP graph and replayed: what a launch-bound serving loop would do
        # (the library only enqueues kernels; its scratch pool was grown by the warm-up)
        graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                step()
        torch.cuda.synchronize()
        run_step = graph.replay
        for _ in range(3):
            run_step()
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run_step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # dominant kernel alone: back-to-back launches of the attention op between two events
    ms_kernel = _time_region(torch, attn, max(args.steps, 20))
    ms_rope = _time_region(torch, rope, max(args.steps, 20)) if r is not None else 0.0

    kv_bytes = w["kv_bytes"]
    qo_bytes = 2 * B * s.n_heads * s.head_dim * 2 + sum((c + s.block_size - 1) // s.block_size for c in ctx) * 4
    alg_bytes = kv_bytes + qo_bytes
    achieved = alg_bytes / (ms_kernel * 1e-3) / 1e9

    # parity spot check through the oracle (the checker, not the thing measured). rope_and_cache
    # rotates its rows in place, so the timed steps kept re-rotating the same buffer (same work,
    # drifting values); one more step from the pristine rows gives the output that is checked.
    if r is not None:
        r["inout"].copy_(pristine)
    step()
    torch.cuda.synchronize()
    cpu = None
    if not args.no_cpu:
        sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
        from oracle import xlite_oracle as O
        ncpu = _cpu_threads(torch)
        n_sample = min(B, 64)   # every sequence of the headline batch; the timed runs below add up to about 10 s
        sample = list(range(0, B, max(1, B // n_sample)))[:n_sample]
        wc = {k: (v.cpu() if isinstance(v, torch.Tensor) else v) for k, v in w.items()}
        qkv_c = (r["inout"] if r is not None else w["qkv"]).cpu()
        got = w["output"].float().cpu()

        def run_oracle():
            return O.attention_ref(qkv_c, wc["k_cache"], wc["v_cache"], wc["query_start_loc"], wc["lens"],
                                   wc["cached_lens"], wc["block_tables"], s.n_heads, s.n_kv_heads, s.head_dim,
                                   s.block_size, B, w["max_num_block"], wc["k_scale"], wc["v_scale"], seqs=sample)
        ref = run_oracle()  # warm-up + parity
        err = (got[sample] - ref[sample]).abs()
        tol = 5e-2 if int8 else 2e-2
        if float(err.max()) > tol:
            raise SystemExit("parity check failed in bench: max abs err %g" % float(err.max()))
        reps, t_cpu = 0, 0.0
        while reps < 3 or (t_cpu < 10.0 and reps < 20):
            t1 = time.perf_counter()
            run_oracle()
            t_cpu += time.perf_counter() - t1
            reps += 1
        per_elt = 1 if int8 else 2
        sample_bytes = sum(ctx[i] for i in sample) * s.n_kv_heads * s.head_dim * 2 * per_elt
        cpu = {"value": round(sample_bytes / (t_cpu / reps) / 1e9, 3), "unit": "GB/s", "cores": ncpu, "kind": "port",
               "sample": "%d of %d sequences (indices %s), %d timed runs of the PyTorch oracle, %s" %
                         (len(sample), B, sample if len(sample) <= 8 else "%d..%d step %d" % (sample[0], sample[-1], sample[1] - sample[0]),
                          reps, _cpu_info()),
               "max_abs_err_vs_gpu": float(err.max())}

    tokens_per_s = B / (ms_step * 1e-3)
    return {
        "metric": "decode attn KV-read GB/s (% of HBM peak) + prefill TFLOP/s, 1 MI355X",
        "value": round(kv_bytes / (ms_step * 1e-3) / 1e9, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8" if int8 else "bf16", "data": "synthetic",
        "config": {"workload": name, "batch": B, "n_heads": s.n_heads, "n_kv_heads": s.n_kv_heads,
                   "head_dim": s.head_dim, "block_size": s.block_size, "ctx_total": int(sum(ctx)),
                   "ctx_max": int(max(ctx)), "kv_bytes_per_step": int(kv_bytes),
                   "launch": "graph replay" if args.graph else "eager"},
        "pct_of_hbm_peak": round(100.0 * kv_bytes / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
        "tokens_per_s": round(tokens_per_s, 1),
        "kernel_ms": {"attention": round(ms_kernel, 4), "rope_and_cache": round(ms_rope, 4)},
        "attention_ms_dist": _launch_dist(torch, attn),
        "roofline": {"bound": "hbm", "kernel": "decode_dma_kernel / decode_mfma_kernel (+ merge_meta_kernel)", "achieved": round(achieved, 2),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES.get(name.split()[0]),
                     "algorithmic_bytes_per_launch": int(alg_bytes)},
        "cpu_baseline": cpu,
    }


def bench_prefill(args, torch, rt):
    from gvirt_amd import workloads as W
    from gvirt_amd import _C
    shape = W.QWEN25_7B
    lens = W.c3_total_lengths()
    dev = "cuda:0"
    rt.blocking = False
    chunks, caches, ci = [], None, 0
    while True:
        w = W.gqa_prefill_chunk(shape, lens, ci, 2048, W.SEED_BASE + 3, device=dev, caches=caches)
        if w is None:
            break
        caches = w["caches"]
        chunks.append(w)
        ci += 1

    def step():
        for w in chunks:
            _C.attention(rt, w["qkv"], w["k_cache"], w["v_cache"], w["output"], w["query_start_loc"], w["lens"],
                         w["cached_lens"], w["block_tables"], shape.n_heads, shape.n_kv_heads, shape.head_dim,
                         shape.block_size, w["batch"], w["max_num_block"])

    for _ in range(max(1, args.warmup // 4)):
        step()
    steps = max(3, args.steps // 5)
    ms = _time_region(torch, step, steps)
    flops = sum(w["flops"] for w in chunks)
    tokens = sum(w["tokens"] for w in chunks)
    tf = flops / (ms * 1e-3) / 1e12
    cpu = None
    if not args.no_cpu:
        # the oracle on the shortest sequence's part of the first chunk: parity, then its rate
        sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
        from oracle import xlite_oracle as O
        ncpu = _cpu_threads(torch)
        torch.cuda.synchronize()
        w0 = chunks[0]
        c = {k: (v.cpu() if isinstance(v, torch.Tensor) else v) for k, v in w0.items() if k != "caches"}
        i = min(range(len(lens)), key=lambda j: lens[j])
        got = w0["output"].float().cpu()

        def run_oracle():
            return O.attention_ref(c["qkv"], c["k_cache"], c["v_cache"], c["query_start_loc"], c["lens"], c["cached_lens"],
                                   c["block_tables"], shape.n_heads, shape.n_kv_heads, shape.head_dim, shape.block_size,
                                   w0["batch"], w0["max_num_block"], seqs=[i])
        ref = run_oracle()
        r0, rl = int(c["query_start_loc"][i]), int(c["lens"][i])
        err = (got[r0:r0 + rl] - ref[r0:r0 + rl]).abs()
        if float(err.max()) > 2e-2:
            raise SystemExit("parity check failed in bench: max abs err %g" % float(err.max()))
        reps, t_cpu = 0, 0.0
        while reps < 3 and t_cpu < 20.0:
            t1 = time.perf_counter()
            run_oracle()
            t_cpu += time.perf_counter() - t1
            reps += 1
        sample_flops = 4 * shape.n_heads * shape.head_dim * (rl * (rl + 1) // 2)
        cpu = {"value": round(sample_flops / (t_cpu / reps) / 1e12, 4), "unit": "TFLOP/s", "cores": ncpu, "kind": "port",
               "sample": "sequence %d of the first chunk (%d rows, causal), %d timed runs of the PyTorch oracle, %s" %
                         (i, rl, reps, _cpu_info()),
               "max_abs_err_vs_gpu": float(err.max())}
    return {"metric": "decode attn KV-read GB/s (% of HBM peak) + prefill TFLOP/s, 1 MI355X", "value": round(tf, 2),
            "unit": "TFLOP/s", "n_gpus": 1, "steps": steps, "warmup": max(1, args.warmup // 4), "ms_per_step": round(ms, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "c3 qwen2.5-7b chunked causal prefill", "total_lens": lens, "chunk": 2048,
                       "calls_per_step": len(chunks)},
            "tokens_per_s": round(tokens / (ms * 1e-3), 1),
            "roofline": {"bound": "mfma", "kernel": "prefill_kernel", "achieved": round(tf, 2),
                         "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
                         "traffic": MEASURED_TRAFFIC_BYTES.get("c3"), "algorithmic_flops_per_step": int(flops)},
            "cpu_baseline": cpu}


def bench_mla(args, torch, rt):
    from gvirt_amd import workloads as W
    from gvirt_amd import _C
    s = W.MlaShape()
    ctx = W.c4_context_lengths()
    w = W.mla_decode(s, ctx, W.SEED_BASE + 4, device="cuda:0")
    rt.blocking = False

    def step():
        _C.mla_attention(rt, w["q_absorb"], w["qr"], w["k_cache"], w["pe_cache"], w["o_absorb"], w["query_start_loc"],
                         w["lens"], w["cached_lens"], w["block_tables"], s.n_heads, s.rope_head_dim, s.kv_lora_rank,
                         s.block_size, w["batch"], w["max_num_blocks"], s.scale)

    for _ in range(args.warmup):
        step()
    ms = _time_region(torch, step, args.steps)
    gbs = w["kv_bytes"] / (ms * 1e-3) / 1e9
    tf = w["flops"] / (ms * 1e-3) / 1e12
    cpu = None
    if not args.no_cpu:
        # the oracle (the checker, not the thing measured) on two of the sequences: parity, then its rate
        sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
        from oracle import xlite_oracle as O
        ncpu = _cpu_threads(torch)
        torch.cuda.synchronize()
        sample = [0, len(ctx) // 2]
        c = {k: (v.cpu() if isinstance(v, torch.Tensor) else v) for k, v in w.items()}
        mb = w["max_num_blocks"]
        sub_tables = torch.cat([c["block_tables"].view(len(ctx), mb)[i] for i in sample])
        sub = lambda t: torch.stack([t[i] for i in sample])

        def run_oracle():
            return O.mla_attention_ref(sub(c["q_absorb"]), sub(c["qr"]), c["k_cache"], c["pe_cache"],
                                       torch.arange(len(sample), dtype=torch.int32), torch.ones(len(sample), dtype=torch.int32),
                                       sub(c["cached_lens"]), sub_tables, s.n_heads, s.rope_head_dim, s.kv_lora_rank,
                                       s.block_size, len(sample), mb, s.scale)
        ref = run_oracle()
        got = sub(w["o_absorb"].float().cpu()).reshape(ref.shape)
        err = (got - ref).abs()
        if float(err.max()) > 2e-2:
            raise SystemExit("parity check failed in bench: max abs err %g" % float(err.max()))
        reps, t_cpu = 0, 0.0
        while reps < 3 and t_cpu < 20.0:
            t1 = time.perf_counter()
            run_oracle()
            t_cpu += time.perf_counter() - t1
            reps += 1
        sample_bytes = sum(ctx[i] for i in sample) * (s.kv_lora_rank + s.rope_head_dim) * 2
        cpu = {"value": round(sample_bytes / (t_cpu / reps) / 1e9, 3), "unit": "GB/s", "cores": ncpu, "kind": "port",
               "sample": "%d of %d sequences (indices %s), %d timed runs of the PyTorch oracle, %s" %
                         (len(sample), len(ctx), sample, reps, _cpu_info()),
               "max_abs_err_vs_gpu": float(err.max())}
    floor_ms = max(w["kv_bytes"] / (HBM_PEAK_GBS * 1e9), w["flops"] / (MFMA_BF16_PEAK_TFLOPS * 1e12)) * 1e3
    return {"metric": "decode attn KV-read GB/s (% of HBM peak) + prefill TFLOP/s, 1 MI355X", "value": round(gbs, 2),
            "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "c4 deepseek-r1 MLA absorbed decode", "batch": 32, "n_heads": 128, "ctx_total": int(sum(ctx)),
                       "kv_bytes_per_step": int(w["kv_bytes"]), "flops_per_step": int(w["flops"])},
            "tflops": round(tf, 2), "tokens_per_s": round(32 / (ms * 1e-3), 1), "attention_ms_dist": _launch_dist(torch, step),
            "roofline": {"bound": "hbm", "kernel": "mla_decode_kernel (+ merge_mla_kernel)", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS,
                         "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get("c4"),
                         "frac_of_max_floor": round(floor_ms / ms, 4), "mfma_frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4)},
            "cpu_baseline": cpu}


def bench_indexer(args, torch, rt):
    """DSA indexer on the decode batch of configuration 4 (64 indexer heads of 128, one key head): the
    `indexer_topk` operator (scores + selection of 2048 positions per row). Not a BASELINE configuration:
    printed only with --config idx."""
    import numpy as np
    from gvirt_amd import workloads as W
    from gvirt_amd import _C
    dev = "cuda:0"
    ctx = W.c4_context_lengths()
    nH, D, bs, top_k = 64, 128, 64, 2048
    batch = len(ctx)
    maxblk = max((c + bs - 1) // bs for c in ctx)
    NB = batch * maxblk + 1
    g = torch.Generator(device=dev).manual_seed(W.SEED_BASE + 6)
    q = torch.randn(batch, nH, D, generator=g, device=dev).bfloat16()
    wgt = torch.randn(batch, D + nH, generator=g, device=dev).bfloat16()
    kc = torch.randn(NB, bs, D, generator=g, device=dev).bfloat16()
    tables = torch.randperm(NB, generator=g, device=dev)[: batch * maxblk].int()
    qsl = torch.arange(batch, dtype=torch.int32, device=dev)
    lens = torch.ones(batch, dtype=torch.int32, device=dev)
    clens = torch.tensor([c - 1 for c in ctx], dtype=torch.int32, device=dev)
    idx = torch.arange(maxblk * bs, dtype=torch.int32, device=dev)
    out = torch.zeros(batch, top_k, dtype=torch.int32, device=dev)
    rt.blocking = False

    def step():
        _C.indexer_topk(rt, q, kc, wgt, idx, out, qsl, lens, clens, tables, nH, D, bs, batch, maxblk, top_k)

    for _ in range(args.warmup):
        step()
    ms = _time_region(torch, step, args.steps)
    kbytes = sum(ctx) * D * 2
    gbs = kbytes / (ms * 1e-3) / 1e9
    return {"metric": "decode attn KV-read GB/s (% of HBM peak) + prefill TFLOP/s, 1 MI355X", "value": round(gbs, 2),
            "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "idx DSA indexer_topk on the c4 decode batch", "batch": batch, "n_heads": nH, "head_dim": D,
                       "top_k": top_k, "ctx_total": int(sum(ctx)), "key_bytes_per_step": int(kbytes)},
            "roofline": {"bound": "hbm", "kernel": "indexer_scores_kernel (+ indexer_select_kernel)", "achieved": round(gbs, 2),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None},
            "cpu_baseline": None}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="c2")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU oracle leg")
    ap.add_argument("--graph", action="store_true",
                    help="decode configurations: time replays of the step captured into a HIP graph instead of eager calls")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain 1 GiB device-to-device copy kernel: under a counter run its "
                         "FETCH_SIZE / WRITE_SIZE readings give the scale of those counters")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU's share only (no collectives, no sharding); run with --gpus 1",
              file=sys.stderr)
        raise SystemExit(2)

    import torch
    if not torch.cuda.is_available():
        raise SystemExit("bench.py: no GPU visible")
    from gvirt_amd import workloads as W
    from gvirt_amd._C import Runtime
    rt = Runtime(0, 64)

    if args.calibrate_copy:
        src = torch.full((1 << 28,), 1.0, dtype=torch.float32, device="cuda:0")
        dst = torch.empty_like(src)
        dst.copy_(src)   # one elementwise copy kernel: reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    todo = ["c2", "c1", "c5", "c3", "c4"] if args.config == "all" else [args.config]
    for c in todo:
        if c == "c2":
            out = bench_gqa_decode(args, torch, rt, "c2 llama-3-8b GQA flash-decode + reshape_and_cache", W.LLAMA3_8B,
                                   [4096] * 64, W.SEED_BASE + 2)
        elif c == "c1":
            out = bench_gqa_decode(args, torch, rt, "c1 qwen2-0.5b GQA decode", W.QWEN2_05B, W.c1_context_lengths(),
                                   W.SEED_BASE + 1)
        elif c == "c5":
            out = bench_gqa_decode(args, torch, rt, "c5 llama-3-8b int8-KV decode", W.LLAMA3_8B, W.c5_context_lengths(),
                                   W.SEED_BASE + 5, int8=True)
        elif c == "c3":
            out = bench_prefill(args, torch, rt)
        elif c == "c4":
            out = bench_mla(args, torch, rt)
        elif c == "idx":
            out = bench_indexer(args, torch, rt)
        else:
            raise SystemExit("unknown config " + c)
        print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
