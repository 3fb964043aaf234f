#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config default|c2|c1|c3|c4|c5|idx|all]

Default (what the driver runs): configuration 2 of BASELINE.json — Llama-3-8B-shape GQA
flash-decode, batch 64, every sequence at context 4096, bf16 paged KV cache with block size 128,
plus the reshape-and-cache (`rope_and_cache`) of the 64 new tokens. One step = one
`rope_and_cache` + one `attention` call over that batch, inputs resident in HBM. Prints ONE JSON
line; `value` is KV bytes read per second over the whole step. `roofline` prices the dominant
kernel (the decode attention kernel) against the 8 TB/s HBM peak; `cpu_baseline` times the CPU
oracle on a bounded sample of the same workload on the host cores.

With no `--config` the same line also carries `other_configs`: configurations 1, 3, 4 and 5 measured in
the same run, each with its own value, roofline and CPU baseline, and beside configuration 4 the whole `mla_v2`
operator (`c4_mla_v2`), the attention over the indexer's position lists (`c4_dsa`), the indexer itself (`idx`) and
configuration 3 over an int8 cache (`c3_int8`).
`--config c1|c2|c3|c3_int8|c4|c5|idx` prints the line(s) of that workload alone; `all` prints one line per
configuration (the first is configuration 2).

Before its warm-up steps every configuration runs its step, untimed, for 80 ms of GPU time (`device_spin_up_ms`):
the part's clocks take tens of milliseconds of sustained load to settle, and each timed region follows an idle
GPU (data set-up, the previous configuration's CPU baseline).

Cache residency: configurations 2, 3 and 5 stream far more than the 256 MB of last-level cache per step.
Configuration 4 (233 MB of latent cache) rotates over four distinct cache sets (932 MB) so that no step finds
its cache resident; configuration 1 (0.8 MB) is timed step by step with a 1 GiB fill between the steps.
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
PEAK_CLOCK_GHZ = 2.4   # the engine clock the published MI355X matrix peaks are quoted at
MEASURED_TRAFFIC_BYTES = {"c2": 1080255689, "c3": 334666881, "c4": 274669317, "c5": 1623779956}
# where each constant comes from: the committed counter summary whose "HBM traffic per launch" line holds it
TRAFFIC_SOURCE = {"c2": "profiles/decode_dma_kernel_c2_llama3_8b_b64_ctx4096.md",
                  "c3": "profiles/prefill_kernel_c3_qwen25_7b_chunked.md",
                  "c4": "profiles/mla_decode_kernel_c4_deepseek_r1_b32.md",
                  "c5": "profiles/decode_dma8_kernel_int8_c5_llama3_8b_b128_ragged.md"}


def _traffic(key):
    return {"traffic": MEASURED_TRAFFIC_BYTES.get(key),
            "traffic_source": (TRAFFIC_SOURCE[key] + " (rocprofv3 --pmc runs of an earlier invocation of this command, "
                               "not measured by this run)") if key in MEASURED_TRAFFIC_BYTES else None}


def _events(torch):
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


def _clock_under_load(torch, rt, fn, iters=200):
    """Shader clock in GHz over `iters` back-to-back calls of `fn`, from the stamps workgroup 0 of the streaming MLA and
    prefill kernels leaves when a probe buffer is set (xlite_hip_set_clock_probe): shader-clock ticks over 100 MHz
    wall-clock ticks of the last launch."""
    import ctypes
    buf = torch.zeros(4, dtype=torch.int64, device="cuda:0")
    rt._lib.xlite_hip_set_clock_probe(ctypes.c_void_p(buf.data_ptr()))
    try:
        for _ in range(iters):
            fn()
        torch.cuda.synchronize()
    finally:
        rt._lib.xlite_hip_set_clock_probe(None)
    c0, w0, c1, w1 = [int(x) for x in buf.tolist()]
    return round((c1 - c0) / ((w1 - w0) * 10.0), 3) if w1 > w0 else None


def _clock_fields(clock_ghz, tflops):
    """The measured clock next to the one the published matrix peak assumes, and the matrix rate against the peak
    scaled to the measured clock (the published 2.5 PFLOP/s is 256 compute units at 2.4 GHz)."""
    if not clock_ghz:
        return {"shader_clock_ghz_under_load": None}
    return {"shader_clock_ghz_under_load": clock_ghz, "peak_clock_ghz": PEAK_CLOCK_GHZ,
            "mfma_frac_at_measured_clock": round(tflops / (MFMA_BF16_PEAK_TFLOPS * clock_ghz / PEAK_CLOCK_GHZ), 4)}


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


SPIN_UP_MS = 80.0


def _spin_up(torch, fn, min_ms=SPIN_UP_MS):
    """Untimed: calls `fn` until `min_ms` of GPU time have passed. The part is power-managed and takes tens of
    milliseconds of sustained load to settle its clocks (the MLA decode batch: 0.106 ms per call over the first 52
    calls after an idle second, 0.088 ms from about the 300th on); every configuration's timed region follows the CPU
    baseline of the one before, during which the GPU sits idle."""
    a, b = _events(torch)
    done = 0.0
    while done < min_ms:
        a.record()
        for _ in range(8):
            fn()
        b.record()
        torch.cuda.synchronize()
        done += a.elapsed_time(b)


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


def _flushed_steps(torch, fn, steps, flush):
    """Milliseconds of `steps` calls of `fn`, each between its own pair of HIP events on the launching stream,
    with `flush()` (untimed) before every one."""
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in ev:
        flush()
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return [a.elapsed_time(b) for a, b in ev]


def bench_gqa_decode(args, torch, rt, name, shape, ctx, seed, int8=False, with_rope=True, cold=False):
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
            # the pair as one call into the library (same kernels as rope() then attn())
            _C.decode_step(rt, r["inout"], w["k_cache"], w["v_cache"], w["output"], r["position"], r["cosin"],
                           r["slot_mapping"], w["query_start_loc"], w["lens"], w["cached_lens"], w["block_tables"],
                           s.n_heads, s.n_kv_heads, s.head_dim, s.head_dim, s.block_size, B, w["max_num_block"])
        else:
            attn()

    _spin_up(torch, step)
    if r is not None:
        r["inout"].copy_(pristine)   # (rope_and_cache rotates its rows in place)
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
    residency = "streams %.0f MB per step, far beyond the 256 MB last-level cache" % (w["kv_bytes"] / 1e6)
    if cold:
        # a working set that would sit in the last-level cache: every timed step follows a 1 GiB fill
        junk = torch.empty(1 << 28, dtype=torch.float32, device=dev)
        flush = lambda: junk.fill_(1.0)
        ms_step = sum(_flushed_steps(torch, run_step, args.steps, flush)) / args.steps
        t_attn = _flushed_steps(torch, attn, max(args.steps, 20), flush)
        ms_kernel = sum(t_attn) / len(t_attn)
        t_rope = _flushed_steps(torch, rope, max(args.steps, 20), flush) if r is not None else [0.0]
        ms_rope = sum(t_rope) / len(t_rope)
        residency = "cold: a 1 GiB fill runs (untimed) before every timed step; each step between its own events"
        del junk
    else:
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
                   "launch": "graph replay" if args.graph else "eager", "cache_residency": residency,
                   "device_spin_up_ms": SPIN_UP_MS},
        "pct_of_hbm_peak": round(100.0 * kv_bytes / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
        "tokens_per_s": round(tokens_per_s, 1),
        "kernel_ms": {"attention": round(ms_kernel, 4), "rope_and_cache": round(ms_rope, 4)},
        "attention_ms_dist": _launch_dist(torch, attn),
        "roofline": {"bound": "hbm", "kernel": "decode_dma_kernel / decode_dma8_kernel / decode_mfma_kernel (+ merge_meta_kernel)", "achieved": round(achieved, 2),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     **_traffic(name.split()[0]), "algorithmic_bytes_per_launch": int(alg_bytes)},
        "cpu_baseline": cpu,
    }


def bench_prefill(args, torch, rt, int8=False):
    """Configuration 3; `int8`: the same chunk calls over an int8 cache (one fp32 scale per token and kv head), which
    the operator serves by dequantising the visible blocks once per call into an fp16 copy."""
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
    ks = vs = None
    if int8:
        kq, ks = W.quantize_cache(caches["k_cache"], torch.int8)
        vq, vs = W.quantize_cache(caches["v_cache"], torch.int8)
        for w in chunks:
            w["k_cache"], w["v_cache"] = kq, vq
        caches["k_cache"] = caches["v_cache"] = None   # (the bf16 tensors are freed)

    def step():
        for w in chunks:
            _C.attention(rt, w["qkv"], w["k_cache"], w["v_cache"], w["output"], w["query_start_loc"], w["lens"],
                         w["cached_lens"], w["block_tables"], shape.n_heads, shape.n_kv_heads, shape.head_dim,
                         shape.block_size, w["batch"], w["max_num_block"], k_scale=ks, v_scale=vs)

    # a step is 2.2 ms: at least 3 warm-up steps and 10 timed ones whatever --steps says, so that the figure
    # does not hang on the clock ramp after the previous configuration
    warm = max(3, args.warmup // 4)
    _spin_up(torch, step)
    for _ in range(warm):
        step()
    steps = max(10, args.steps // 5)
    ms = _time_region(torch, step, steps)
    step_dist = _launch_dist(torch, step, 20)

    def call(w):
        return lambda: _C.attention(rt, w["qkv"], w["k_cache"], w["v_cache"], w["output"], w["query_start_loc"], w["lens"],
                                    w["cached_lens"], w["block_tables"], shape.n_heads, shape.n_kv_heads, shape.head_dim,
                                    shape.block_size, w["batch"], w["max_num_block"], k_scale=ks, v_scale=vs)
    per_call = []
    for w in chunks:
        d = _launch_dist(torch, call(w), 20)
        d["tflops_at_median"] = round(w["flops"] / (d["median"] * 1e-3) / 1e12, 1)
        per_call.append(d)
    # a short chunk over the same caches: 256 tokens of every sequence behind 2048 cached ones. Over the int8 cache
    # such chunks are read by the prefill kernel itself (no copy); the bf16 leg runs the same call for comparison.
    short = None
    if not args.no_extras:
        if int8:
            caches["k_cache"], caches["v_cache"] = kq, vq
        ws = W.gqa_prefill_chunk(shape, lens, 8, 256, W.SEED_BASE + 33, device=dev, caches=caches)
        short = _launch_dist(torch, call(ws), 20)
        short["tflops_at_median"] = round(ws["flops"] / (short["median"] * 1e-3) / 1e12, 1)
        short["workload"] = "%d sequences x 256 tokens behind 2048 cached" % ws["batch"]
        short["kernel"] = "prefill_kernel reading the int8 bytes and scales itself" if int8 else "prefill_kernel"
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
        ksc, vsc = (ks.cpu(), vs.cpu()) if int8 else (None, None)

        def run_oracle():
            return O.attention_ref(c["qkv"], c["k_cache"], c["v_cache"], c["query_start_loc"], c["lens"], c["cached_lens"],
                                   c["block_tables"], shape.n_heads, shape.n_kv_heads, shape.head_dim, shape.block_size,
                                   w0["batch"], w0["max_num_block"], ksc, vsc, seqs=[i])
        ref = run_oracle()
        r0, rl = int(c["query_start_loc"][i]), int(c["lens"][i])
        err = (got[r0:r0 + rl] - ref[r0:r0 + rl]).abs()
        if float(err.max()) > (5e-2 if int8 else 2e-2):
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
            "unit": "TFLOP/s", "n_gpus": 1, "steps": steps, "warmup": warm, "ms_per_step": round(ms, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8 cache, fp16 products" if int8 else "bf16",
            "data": "synthetic",
            "config": {"workload": "c3_int8 qwen2.5-7b chunked causal prefill over an int8 KV cache" if int8
                                   else "c3 qwen2.5-7b chunked causal prefill", "total_lens": lens, "chunk": 2048,
                       "calls_per_step": len(chunks)},
            "tokens_per_s": round(tokens / (ms * 1e-3), 1), "step_ms_dist": step_dist, "chunk_call_ms_dist": per_call,
            "short_chunk_call": short,
            "roofline": {"bound": "mfma", "kernel": "dequant_blocks_kernel + prefill_kernel" if int8 else "prefill_kernel",
                         "achieved": round(tf, 2),
                         "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
                         **(_traffic("c3") if not int8 else {"traffic": None}), "algorithmic_flops_per_step": int(flops),
                         **_clock_fields(_clock_under_load(torch, rt, step, iters=10), tf)},
            "cpu_baseline": cpu}


def bench_mla(args, torch, rt):
    from gvirt_amd import workloads as W
    from gvirt_amd import _C
    s = W.MlaShape()
    ctx = W.c4_context_lengths()
    # four distinct cache sets (same lengths, different contents, tables and queries), used in turn: 4 x 233 MB
    # cannot stay in the 256 MB last-level cache between the steps that use one set
    n_sets = 4
    sets = [W.mla_decode(s, ctx, W.SEED_BASE + 4 + 1000 * i, device="cuda:0") for i in range(n_sets)]
    w = sets[0]
    rt.blocking = False
    turn = [0]

    def run(x):
        _C.mla_attention(rt, x["q_absorb"], x["qr"], x["k_cache"], x["pe_cache"], x["o_absorb"], x["query_start_loc"],
                         x["lens"], x["cached_lens"], x["block_tables"], s.n_heads, s.rope_head_dim, s.kv_lora_rank,
                         s.block_size, x["batch"], x["max_num_blocks"], s.scale)

    def step():
        run(sets[turn[0] % n_sets])
        turn[0] += 1

    _spin_up(torch, step)
    for _ in range(max(args.warmup, n_sets)):
        step()
    steps = ((max(args.steps, n_sets) + n_sets - 1) // n_sets) * n_sets   # every set equally often
    ms = _time_region(torch, step, steps)
    ms_resident = _time_region(torch, lambda: run(w), steps)   # one set over and over, for comparison
    gbs = w["kv_bytes"] / (ms * 1e-3) / 1e9
    tf = w["flops"] / (ms * 1e-3) / 1e12
    dist = _launch_dist(torch, step)
    clock_ghz = _clock_under_load(torch, rt, step)

    # the two einsums of the mla_v2 operator around the attention (W_UK absorb, W_UV), reported separately
    g = torch.Generator(device="cuda:0").manual_seed(W.SEED_BASE + 44)
    B, H, C, N, V = w["batch"], s.n_heads, s.kv_lora_rank, s.nope_head_dim, s.v_head_dim
    q_nope = torch.randn(B, H, N + s.rope_head_dim, generator=g, device="cuda:0").bfloat16()
    wuk = [(torch.randn(H, N, C, generator=g, device="cuda:0") * N ** -0.5).bfloat16() for _ in range(n_sets * 4)]
    wuv = [(torch.randn(H, C, V, generator=g, device="cuda:0") * C ** -0.5).bfloat16() for _ in range(n_sets * 4)]
    q_abs = torch.empty(B, H * C, dtype=torch.bfloat16, device="cuda:0")
    o_v = torch.empty(B, H * V, dtype=torch.bfloat16, device="cuda:0")
    et = [0]

    def absorb():   # 16 weight sets of 16.8 MB in turn: 268 MB, not resident between uses
        _C._einsum(rt, "bench", q_nope, wuk[et[0] % len(wuk)], q_abs, B, H, N, C, False, False, t_stride=N + s.rope_head_dim)
        et[0] += 1

    def unabsorb():
        _C._einsum(rt, "bench", w["o_absorb"], wuv[et[0] % len(wuv)], o_v, B, H, C, V, False, False)
        et[0] += 1

    for f in (absorb, unabsorb):
        _spin_up(torch, f, 20.0)
    ms_abs = _time_region(torch, absorb, 32)
    ms_unabs = _time_region(torch, unabsorb, 32)
    wbytes = H * N * C * 2
    _C._einsum(rt, "bench", q_nope, wuk[0], q_abs, B, H, N, C, False, False, t_stride=N + s.rope_head_dim)
    torch.cuda.synchronize()
    ein_err = float((q_abs.view(B, H, C).float() - torch.einsum("mht,htd->mhd", q_nope[:, :, :N].float(), wuk[0].float())).abs().max())
    einsum = {"absorb_ms": round(ms_abs, 4), "unabsorb_ms": round(ms_unabs, 4), "weight_bytes_each": wbytes,
              "absorb_GBs": round((wbytes + q_nope.numel() * 2 + q_abs.numel() * 2) / (ms_abs * 1e-3) / 1e9, 1),
              "unabsorb_GBs": round((wbytes + q_abs.numel() * 2 + o_v.numel() * 2) / (ms_unabs * 1e-3) / 1e9, 1),
              "frac_of_hbm_peak": round((wbytes + q_nope.numel() * 2 + q_abs.numel() * 2) / (ms_abs * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
              "max_abs_err_vs_torch_fp32": ein_err,
              "note": "einsum_kernel, 16 weight sets used in turn; bound by the 16.8 MB weight read"}
    cpu = None
    if not args.no_cpu:
        # the oracle (the checker, not the thing measured) on two of the sequences: parity, then its rate
        sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
        from oracle import xlite_oracle as O
        ncpu = _cpu_threads(torch)
        run(w)
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
    extra = {"c4_mla_v2": _bench_mla_v2(args, torch, rt, s, ctx, sets, wuk, wuv, q_nope, steps),
             "c4_dsa": _bench_mla_dsa(args, torch, rt, s, ctx, sets, steps)}
    return {"extra_legs": extra,
            "metric": "decode attn KV-read GB/s (% of HBM peak) + prefill TFLOP/s, 1 MI355X", "value": round(gbs, 2),
            "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": max(args.warmup, n_sets), "ms_per_step": round(ms, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "c4 deepseek-r1 MLA absorbed decode", "batch": 32, "n_heads": 128, "ctx_total": int(sum(ctx)),
                       "kv_bytes_per_step": int(w["kv_bytes"]), "flops_per_step": int(w["flops"]),
                       "cache_residency": "%d distinct cache sets of %.0f MB used in turn (%.0f MB in all, beyond the 256 MB "
                                          "last-level cache); one set over and over takes %.4f ms per step" %
                                          (n_sets, w["kv_bytes"] / 1e6, n_sets * w["kv_bytes"] / 1e6, ms_resident)},
            "tflops": round(tf, 2), "tokens_per_s": round(32 / (ms * 1e-3), 1), "attention_ms_dist": dist,
            "ms_per_step_one_resident_set": round(ms_resident, 4), "einsums": einsum,
            "roofline": {"bound": "hbm", "kernel": "mla_decode_kernel (+ merge_mla_kernel)", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS,
                         "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4), **_traffic("c4"),
                         "frac_of_max_floor": round(floor_ms / ms, 4), "mfma_frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
                         **_clock_fields(clock_ghz, tf)},
            "cpu_baseline": cpu}


def _line(value, unit, steps, warmup, ms, dtype="bf16"):
    return {"metric": "decode attn KV-read GB/s (% of HBM peak) + prefill TFLOP/s, 1 MI355X", "value": value, "unit": unit,
            "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic"}


def _time_oracle(fn, budget_s=15.0, max_reps=3):
    reps, t = 0, 0.0
    while reps < max_reps and t < budget_s:
        t1 = time.perf_counter()
        fn()
        t += time.perf_counter() - t1
        reps += 1
    return t / reps, reps


def _bench_mla_v2(args, torch, rt, s, ctx, sets, wuk, wuv, q_nope, steps):
    """The operator the reference exposes (xlite/csrc/_C.cpp:1234-1301): W_UK absorb einsum + absorbed attention +
    W_UV einsum in one call, on the configuration-4 batch; cache sets and weight sets used in turn."""
    from gvirt_amd import _C
    B, H, C, N, V, R = len(ctx), s.n_heads, s.kv_lora_rank, s.nope_head_dim, s.v_head_dim, s.rope_head_dim
    out = torch.empty(B, H * V, dtype=torch.bfloat16, device="cuda:0")
    none = torch.zeros(1, dtype=torch.int32, device="cuda:0")
    turn = [0]

    def call(x, ku, kv):
        _C.mla_v2(rt, q_nope, x["qr"], x["k_cache"], x["pe_cache"], ku, kv, out, x["query_start_loc"], x["lens"],
                  x["cached_lens"], x["block_tables"], H, R, N, V, C, s.block_size, x["batch"], x["max_num_blocks"], s.scale,
                  none, 0)

    def step():
        i = turn[0]
        call(sets[i % len(sets)], wuk[i % len(wuk)], wuv[i % len(wuv)])
        turn[0] += 1

    _spin_up(torch, step)
    for _ in range(max(args.warmup, len(sets))):
        step()
    ms = _time_region(torch, step, steps)
    w = sets[0]
    wbytes = 2 * H * N * C * 2
    alg = w["kv_bytes"] + wbytes + q_nope.numel() * 2 + w["qr"].numel() * 2 + out.numel() * 2
    gbs = alg / (ms * 1e-3) / 1e9
    cpu = None
    if not args.no_cpu:
        from oracle import xlite_oracle as O
        ncpu = _cpu_threads(torch)
        call(w, wuk[0], wuv[0])
        torch.cuda.synchronize()
        sample = [0, len(ctx) // 2]
        c = {k: (v.cpu() if isinstance(v, torch.Tensor) else v) for k, v in w.items()}
        mb = w["max_num_blocks"]
        sub = lambda t: torch.stack([t[i] for i in sample])
        sub_tables = torch.cat([c["block_tables"].view(len(ctx), mb)[i] for i in sample])
        qn, ku, kv = q_nope.cpu(), wuk[0].cpu(), wuv[0].cpu()

        def run_oracle():
            return O.mla_v2_ref(sub(qn), sub(c["qr"]), c["k_cache"], c["pe_cache"], ku, kv,
                                torch.arange(len(sample), dtype=torch.int32), torch.ones(len(sample), dtype=torch.int32),
                                sub(c["cached_lens"]), sub_tables, H, R, N, V, C, s.block_size, len(sample), mb, s.scale)
        ref = run_oracle()
        got = sub(out.float().cpu()).reshape(ref.shape)
        err = float((got - ref).abs().max())
        if err > 2e-2:
            raise SystemExit("parity check failed in bench (mla_v2): max abs err %g" % err)
        t_cpu, reps = _time_oracle(run_oracle)
        sample_bytes = sum(ctx[i] for i in sample) * (C + R) * 2 + wbytes
        cpu = {"value": round(sample_bytes / t_cpu / 1e9, 3), "unit": "GB/s", "cores": ncpu, "kind": "port",
               "sample": "%d of %d sequences (indices %s) with both weight tensors, %d timed runs of the PyTorch oracle, %s" %
                         (len(sample), len(ctx), sample, reps, _cpu_info()), "max_abs_err_vs_gpu": err}
    o = _line(round(gbs, 2), "GB/s", steps, max(args.warmup, len(sets)), ms)
    o.update({"config": {"workload": "c4_mla_v2: the mla_v2 operator (absorb einsum + attention + W_UV einsum) on the c4 batch",
                         "batch": B, "n_heads": H, "ctx_total": int(sum(ctx)), "weight_bytes": int(wbytes),
                         "cache_residency": "%d cache sets and %d weight sets used in turn" % (len(sets), len(wuk))},
              "tokens_per_s": round(B / (ms * 1e-3), 1),
              "roofline": {"bound": "hbm", "kernel": "einsum_htd_kernel + mla_decode_kernel + merge_mla_kernel + einsum_kernel",
                           "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                           "traffic": None, "algorithmic_bytes_per_launch": int(alg)},
              "cpu_baseline": cpu})
    return o


def _bench_mla_dsa(args, torch, rt, s, ctx, sets, steps):
    """DeepSeek sparse attention on the configuration-4 batch: the indexer's lists of 2048 positions per row
    (indexer_topk on random index queries and keys, run once per cache set, untimed) consumed by mla_attention."""
    from gvirt_amd import workloads as W
    from gvirt_amd import _C
    dev = "cuda:0"
    B, H, C, R, bs, top_k, iH, iD = len(ctx), s.n_heads, s.kv_lora_rank, s.rope_head_dim, s.block_size, 2048, 64, 128
    g = torch.Generator(device=dev).manual_seed(W.SEED_BASE + 46)
    lists = []
    for x in sets:
        NB, mb = x["k_cache"].shape[0], x["max_num_blocks"]
        iq = torch.randn(B, iH, iD, generator=g, device=dev).bfloat16()
        iw = torch.randn(B, iD + iH, generator=g, device=dev).bfloat16()
        ik = torch.randn(NB, bs, iD, generator=g, device=dev).bfloat16()
        l = torch.full((B, top_k), -1, dtype=torch.int32, device=dev)
        _C.indexer_topk(rt, iq, ik, iw, torch.arange(mb * bs, dtype=torch.int32, device=dev), l, x["query_start_loc"],
                        x["lens"], x["cached_lens"], x["block_tables"], iH, iD, bs, B, mb, top_k)
        lists.append(l)
        del iq, iw, ik
    torch.cuda.synchronize()
    turn = [0]

    def call(x, l):
        _C.mla_attention(rt, x["q_absorb"], x["qr"], x["k_cache"], x["pe_cache"], x["o_absorb"], x["query_start_loc"],
                         x["lens"], x["cached_lens"], x["block_tables"], H, R, C, bs, x["batch"], x["max_num_blocks"],
                         s.scale, l, top_k)

    def step():
        i = turn[0] % len(sets)
        call(sets[i], lists[i])
        turn[0] += 1

    _spin_up(torch, step)
    for _ in range(max(args.warmup, len(sets))):
        step()
    ms = _time_region(torch, step, steps)
    n_pos = sum(min(c, top_k) for c in ctx)
    alg = n_pos * (C + R) * 2 + B * H * (C + R) * 2 + B * H * C * 2 + B * top_k * 4
    gbs = alg / (ms * 1e-3) / 1e9
    flops = n_pos * H * (2 * (C + R) + 2 * C)
    cpu = None
    if not args.no_cpu:
        from oracle import xlite_oracle as O
        ncpu = _cpu_threads(torch)
        w, l = sets[0], lists[0]
        call(w, l)
        torch.cuda.synchronize()
        sample = [0, len(ctx) // 2]
        c = {k: (v.cpu() if isinstance(v, torch.Tensor) else v) for k, v in w.items()}
        mb = w["max_num_blocks"]
        sub = lambda t: torch.stack([t[i] for i in sample])
        sub_tables = torch.cat([c["block_tables"].view(len(ctx), mb)[i] for i in sample])
        sub_lists = sub(l.cpu()).clamp(min=0)

        def run_oracle():
            return O.mla_attention_ref(sub(c["q_absorb"]), sub(c["qr"]), c["k_cache"], c["pe_cache"],
                                       torch.arange(len(sample), dtype=torch.int32), torch.ones(len(sample), dtype=torch.int32),
                                       sub(c["cached_lens"]), sub_tables, H, R, C, bs, len(sample), mb, s.scale, sub_lists, top_k)
        ref = run_oracle()
        got = sub(w["o_absorb"].float().cpu()).reshape(ref.shape)
        err = float((got - ref).abs().max())
        if err > 2e-2:
            raise SystemExit("parity check failed in bench (DSA): max abs err %g" % err)
        t_cpu, reps = _time_oracle(run_oracle)
        cpu = {"value": round(len(sample) * top_k * (C + R) * 2 / t_cpu / 1e9, 3), "unit": "GB/s", "cores": ncpu, "kind": "port",
               "sample": "%d of %d rows (indices %s) over their lists, %d timed runs of the PyTorch oracle, %s" %
                         (len(sample), len(ctx), sample, reps, _cpu_info()), "max_abs_err_vs_gpu": err}
    o = _line(round(gbs, 2), "GB/s", steps, max(args.warmup, len(sets)), ms)
    o.update({"config": {"workload": "c4_dsa: mla_attention over top-k position lists (2048 per row, from indexer_topk) on the c4 batch",
                         "batch": B, "n_heads": H, "top_k": top_k, "positions_per_step": int(n_pos),
                         "cache_residency": "%d cache sets used in turn" % len(sets)},
              "tflops": round(flops / (ms * 1e-3) / 1e12, 2), "tokens_per_s": round(B / (ms * 1e-3), 1),
              "roofline": {"bound": "hbm", "kernel": "mla_decode_kernel<lists> (+ merge_mla_kernel)", "achieved": round(gbs, 2),
                           "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                           "algorithmic_bytes_per_launch": int(alg),
                           "mfma_frac": round(flops / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)},
              "cpu_baseline": cpu})
    return o


def bench_indexer(args, torch, rt):
    """DSA indexer on the decode batch of configuration 4 (64 indexer heads of 128, one key head): the
    `indexer_topk` operator (scores + selection of 2048 positions per row). Not one of the five configurations of
    BASELINE.json: the line `idx` of `other_configs`, or alone with --config idx."""
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

    _spin_up(torch, step)
    for _ in range(args.warmup):
        step()
    ms = _time_region(torch, step, args.steps)
    kbytes = sum(ctx) * D * 2
    gbs = kbytes / (ms * 1e-3) / 1e9

    # the same operator's scores on a prefill chunk: 2048 rows of one sequence after 6144 cached positions (the rows of a
    # workgroup share the sequence's K rows through LDS), reported beside the decode figure
    p_rows, p_cached = 2048, 6144
    p_maxblk = (p_rows + p_cached + bs - 1) // bs
    pq = torch.randn(p_rows, nH, D, generator=g, device=dev).bfloat16()
    pw = torch.randn(p_rows, D + nH, generator=g, device=dev).bfloat16()
    pkc = torch.randn(p_maxblk + 1, bs, D, generator=g, device=dev).bfloat16()
    ptab = torch.randperm(p_maxblk + 1, generator=g, device=dev)[:p_maxblk].int()
    pscores = torch.zeros(p_rows, p_maxblk * bs, dtype=torch.bfloat16, device=dev)
    pz = torch.zeros(1, dtype=torch.int32, device=dev)
    plens = torch.full((1,), p_rows, dtype=torch.int32, device=dev)
    pcl = torch.full((1,), p_cached, dtype=torch.int32, device=dev)

    def pstep():
        _C.indexer_scores(rt, pq, pkc, pw, pscores, pz, plens, pcl, ptab, nH, D, bs, 1, p_maxblk)

    _spin_up(torch, pstep)
    pms = _time_region(torch, pstep, 10)
    pflops = 2.0 * p_rows * (p_rows + p_cached) * nH * D
    cpu = None
    if not args.no_cpu:
        # the oracle on two rows of the decode batch: its lists against the operator's (the reference test's 3 % bound)
        from oracle import xlite_oracle as O
        ncpu = _cpu_threads(torch)
        step()
        torch.cuda.synchronize()
        sample = [0, batch // 2]
        sub = lambda t: torch.stack([t[i] for i in sample])
        tb = torch.cat([tables.view(batch, maxblk)[i] for i in sample]).cpu()
        qc, wc, kcc, clc = sub(q.cpu()), sub(wgt.cpu()), kc.cpu(), sub(clens.cpu())

        def run_oracle():
            sc = O.indexer_scores_ref(qc, kcc, wc, torch.arange(len(sample), dtype=torch.int32),
                                      torch.ones(len(sample), dtype=torch.int32), clc, tb, nH, D, bs, len(sample), maxblk)
            return O.indexer_topk_ref(sc, top_k)
        want = run_oracle()
        got = sub(out.cpu())
        worst = 0.0
        for j, i in enumerate(sample):
            row = got[j, :min(top_k, ctx[i])].tolist()
            worst = max(worst, len(set(want[j][0]) - set(row)) / max(1, len(row)))
        if worst > 0.03:
            raise SystemExit("parity check failed in bench (indexer): %.1f %% of the oracle's list missing" % (100 * worst))
        t_cpu, reps = _time_oracle(run_oracle)
        cpu = {"value": round(sum(ctx[i] for i in sample) * D * 2 / t_cpu / 1e9, 3), "unit": "GB/s", "cores": ncpu, "kind": "port",
               "sample": "%d of %d rows (indices %s), %d timed runs of the PyTorch oracle (scores + selection), %s" %
                         (len(sample), batch, sample, reps, _cpu_info()),
               "list_fraction_missing_vs_gpu": round(worst, 5)}
    return {"metric": "decode attn KV-read GB/s (% of HBM peak) + prefill TFLOP/s, 1 MI355X", "value": round(gbs, 2),
            "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "idx DSA indexer_topk on the c4 decode batch", "batch": batch, "n_heads": nH, "head_dim": D,
                       "top_k": top_k, "ctx_total": int(sum(ctx)), "key_bytes_per_step": int(kbytes)},
            "prefill_scores": {"workload": "indexer_scores, %d rows of one sequence after %d cached positions" % (p_rows, p_cached),
                               "ms": round(pms, 4), "tflops": round(pflops / (pms * 1e-3) / 1e12, 1),
                               "frac_of_mfma_peak": round(pflops / (pms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                               "kernel": "indexer_scores_shared_kernel"},
            "roofline": {"bound": "hbm", "kernel": "indexer_scores_kernel (+ indexer_select_kernel)", "achieved": round(gbs, 2),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                         "algorithmic_bytes_per_launch": int(kbytes)},
            "cpu_baseline": cpu}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="default",
                    help="default: configuration 2 with the other configurations attached; c1..c5, idx: that one alone; "
                         "all: one line each")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU oracle leg")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the side measurements of a configuration (the prefill legs' short chunk call), so that a "
                         "profile of the command holds the configuration's own launches only")
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

    def run_config(c):
        if c == "c2":
            return bench_gqa_decode(args, torch, rt, "c2 llama-3-8b GQA flash-decode + reshape_and_cache", W.LLAMA3_8B,
                                    [4096] * 64, W.SEED_BASE + 2)
        if c == "c1":
            return bench_gqa_decode(args, torch, rt, "c1 qwen2-0.5b GQA decode", W.QWEN2_05B, W.c1_context_lengths(),
                                    W.SEED_BASE + 1, cold=True)
        if c == "c5":
            return bench_gqa_decode(args, torch, rt, "c5 llama-3-8b int8-KV decode", W.LLAMA3_8B, W.c5_context_lengths(),
                                    W.SEED_BASE + 5, int8=True)
        if c == "c3":
            return bench_prefill(args, torch, rt)
        if c == "c3_int8":
            return bench_prefill(args, torch, rt, int8=True)
        if c == "c4":
            return bench_mla(args, torch, rt)
        if c == "idx":
            return bench_indexer(args, torch, rt)
        raise SystemExit("unknown config " + c)

    if args.config == "default":
        # the headline line (configuration 2) carrying the other configurations measured in the same run
        out = run_config("c2")
        others = {}
        drop = ("metric", "n_gpus", "higher_is_better", "scaling", "vs_baseline", "data")
        for c in ("c1", "c3", "c3_int8", "c4", "c5", "idx"):
            try:
                o = run_config(c)
                for name, leg in (o.pop("extra_legs", None) or {}).items():   # c4: the whole mla_v2 operator, the DSA lists
                    others[name] = {k: v for k, v in leg.items() if k not in drop}
                for k in drop:
                    o.pop(k, None)
                others[c] = o
            except (Exception, SystemExit) as e:   # the headline line is printed whatever happens to the others
                others[c] = {"error": "%s: %s" % (type(e).__name__, e)}
            torch.cuda.empty_cache()
        out["other_configs"] = others
        failed = [c for c, o in others.items() if "error" in o]
        out["other_configs_failed"] = failed
        print(json.dumps(out), flush=True)
        if failed:
            raise SystemExit(1)   # the headline line is out; a broken configuration still fails the run
        return
    todo = ["c2", "c1", "c5", "c3", "c3_int8", "c4", "idx"] if args.config == "all" else [args.config]
    for c in todo:
        o = run_config(c)
        legs = o.pop("extra_legs", None) or {}
        print(json.dumps(o), flush=True)
        for leg in legs.values():
            print(json.dumps(leg), flush=True)
        torch.cuda.empty_cache()


if __name__ == "__main__":
    main()
