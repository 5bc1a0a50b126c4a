"""Benchmark of the token-sampling hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2]

A step is one batched sampling call over one [B, vocab] matrix of synthetic logits already
resident in HBM.  Steps walk a ring of distinct matrices larger than the 256 MB Infinity Cache so
that every step reads its logits from HBM.  Prints one JSON line: rows/s over exactly K steps, the
roofline of the step's launches (median of five repeats, HIP events on the launch stream), every
workload of the benchmark contract at its own shape, launch and read floors, and the reference's
CPU sampler timed on this box's host cores.

    python bench.py --parse-pmc FETCH_DIR WRITE_DIR --out profiles/NAME.json

turns two rocprofv3 --pmc runs of this script (FETCH_SIZE, then WRITE_SIZE, each with --copy-probe)
into the small JSON file the `roofline.traffic` figure is read from.
"""
from __future__ import annotations

import argparse
import csv
import glob
import json
import os
import platform
import statistics
import sys
import time
from concurrent.futures import ThreadPoolExecutor

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
COPY_PROBE_BYTES = 256 << 20
STEP_KERNELS = ("split_pass1_kernel", "split_pass2_kernel", "split_finish_kernel", "split_walk_kernel", "sample_rows_kernel")


def synth_logits_device(w, count, torch, dev):
    """`count` matrices of workload `w`'s distribution generated on the device (same shape,
    dtype and statistics as executorch_amd.workloads, torch's generator instead of numpy's)."""
    from executorch_amd import workloads as W

    tdt = {W.DTYPE_FLOAT: torch.float32, W.DTYPE_HALF: torch.float16, W.DTYPE_BFLOAT16: torch.bfloat16}[w.dtype]
    g = torch.Generator(device=dev).manual_seed(w.data_seed)
    ring = []
    for _ in range(count):
        if w.kind == "peaked":
            x = torch.randn((w.batch, w.vocab), generator=g, device=dev)
            ids = torch.rand((w.batch, w.vocab), generator=g, device=dev).topk(20, dim=1).indices
            x.scatter_add_(1, ids, torch.full_like(ids, 8.0, dtype=torch.float32))
        elif w.kind == "flat":
            x = torch.randn((w.batch, w.vocab), generator=g, device=dev) * 0.5
        elif w.kind == "normal2":
            x = torch.randn((w.batch, w.vocab), generator=g, device=dev) * 2.0
        elif w.kind == "normal15":
            x = torch.randn((w.batch, w.vocab), generator=g, device=dev) * 1.5
        elif w.kind == "mixed":
            x = torch.randn((w.batch, w.vocab), generator=g, device=dev)
            u = torch.rand((w.batch // 2, w.vocab), generator=g, device=dev).clamp_(1e-7, 1 - 1e-7)
            gum = -torch.log(-torch.log(u))
            hot = torch.randint(0, w.vocab, (w.batch // 2, 1), generator=g, device=dev)
            gum.scatter_add_(1, hot, torch.full_like(hot, 12.0, dtype=torch.float32))
            x[1::2] = gum
            del u, gum
        else:
            raise ValueError(w.kind)
        ring.append(x.to(tdt))
        del x
    return ring


def cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return platform.processor() or "unknown"


def physical_cores() -> int:
    try:
        seen = set()
        phys = core = None
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("physical id"):
                    phys = line.split(":")[1].strip()
                elif line.startswith("core id"):
                    core = line.split(":")[1].strip()
                elif not line.strip() and phys is not None and core is not None:
                    seen.add((phys, core))
                    phys = core = None
        if seen:
            return len(seen)
    except OSError:
        pass
    return os.cpu_count() or 1


def cpu_baseline(w, gpu_tokens, seconds_budget=12.0):
    """The reference sampler on this box's host cores, on a bounded sample of the workload:
    `sampler.cpp` itself (oracle/_ref) when it was built, else the oracle's restatement.  The same
    leg checks `gpu_tokens` (what the library returned for step 0 of the workload) against the
    oracle: this function is the only place where bench.py touches oracle/."""
    import numpy as np

    from executorch_amd import workloads as W
    from oracle import oracle as O

    rows = min(w.batch, 64)
    x = W.logits(w, 0, rows)
    want, _ = O.sample_rows(x, w.dtype, O.inv_temperature(w.temperature), w.topp, 0, W.coin_seeds(w, rows).copy(),
                            mode=O.MODE_UPCAST, tie=O.TIE_STABLE, threads=8)
    mismatches = int((np.asarray(gpu_tokens)[:rows] != want).sum())
    # worker threads: this job's share of the host (16 threads per GPU on the benchmark boxes), not
    # every core the machine reports
    cores = max(1, min(16, os.cpu_count() or 1))
    use_ref = O.have_ref()

    def one_row(b, reps):
        if use_ref:
            s = O.RefSampler(w.vocab, w.temperature, w.topp, w.coin_seed + b)
        else:
            s = O.Sampler(w.vocab, w.temperature, w.topp, w.coin_seed + b, mode=O.MODE_NATIVE)
        for _ in range(reps):
            s.sample(x[b].copy(), w.dtype)

    t0 = time.perf_counter()
    one_row(0, 3)
    per_row = (time.perf_counter() - t0) / 3
    reps = max(1, int(seconds_budget * cores / (per_row * rows)))
    reps = min(reps, 5000)
    t0 = time.perf_counter()
    with ThreadPoolExecutor(cores) as pool:
        list(pool.map(lambda b: one_row(b, reps), range(rows)))
    dt = time.perf_counter() - t0
    t0 = time.perf_counter()
    one_row(1 % rows, 5)
    one_core = 5 / (time.perf_counter() - t0)
    both = cpu_baseline_config(w, seconds=1.5)
    return {
        "value": rows * reps / dt,
        "unit": "rows/s",
        "cores": cores,
        "native_and_upcast": {k: both[k] for k in ("native", "upcast_fp32") if k in both},
        "kind": "reference" if use_ref else "port",
        "sample": f"{rows} rows of {w.name} step 0, each sampled {reps} times by its own Sampler, native "
                  f"{W.DTYPE_NAMES[w.dtype]} sample<T>, {cores} threads ({dt:.1f} s)",
        "rows_per_s_one_core": one_core,
        "cpu_model": cpu_model(),
        "physical_cores": physical_cores(),
        "logical_cpus": os.cpu_count(),
        "compiler": "g++ -std=c++17 -O2 (sampler.cpp as the reference builds it)" if use_ref else "g++ -std=c++17 -O2 (restatement)",
        "parity": {"rows_checked": rows, "token_mismatches_vs_oracle": mismatches},
    }


def cpu_baseline_config(w, seconds=1.2):
    """The reference sampler on this box's host cores for one workload of the contract, on a bounded
    sample of its rows (step 0): one core, one Sampler, rows one after the other (the literal
    reference usage); and every thread of this job's share of the host, a Sampler each.  16-bit
    workloads are timed twice: the native sample<T> instantiation, and sample<float> on the rows
    converted to fp32 beforehand (the arithmetic the GPU path reproduces; the conversion itself is
    not timed).  `sampler.cpp` itself (oracle/_ref) when it was built, else the oracle's restatement."""
    import numpy as np

    from executorch_amd import workloads as W
    from oracle import oracle as O

    cores = max(1, min(16, os.cpu_count() or 1))
    use_ref = O.have_ref()
    rows = cores
    if w.batch >= rows:
        x = W.logits(w, 0, rows)
    else:  # (a workload of one row per step: the rows of as many steps)
        x = np.concatenate([W.logits(w, step, w.batch) for step in range(-(-rows // w.batch))])[:rows]
    modes = [("native", x, w.dtype, O.MODE_NATIVE)]
    if w.dtype != W.DTYPE_FLOAT:
        modes.append(("upcast_fp32", np.ascontiguousarray(W.to_f32(x, w.dtype), dtype=np.float32), W.DTYPE_FLOAT, O.MODE_NATIVE))
    res = {"kind": "reference" if use_ref else "port", "cores": cores, "unit": "rows/s",
           "sample": f"{rows} rows of {w.name} (step 0; the first steps of a one-row workload), each sampled repeatedly by its own "
                     f"Sampler ({seconds:.1f} s per figure)"}

    def make(b):
        if use_ref:
            return O.RefSampler(w.vocab, w.temperature, w.topp, w.coin_seed + b)
        return O.Sampler(w.vocab, w.temperature, w.topp, w.coin_seed + b, mode=O.MODE_NATIVE)

    for label, data, dtype, _ in modes:
        def run(b, reps):
            smp = make(b)
            for _ in range(reps):
                smp.sample(data[b].copy(), dtype)  # (the sampler overwrites its input: a fresh copy per call)

        t0 = time.perf_counter()
        run(0, 2)
        per_row = max((time.perf_counter() - t0) / 2, 1e-6)
        reps = max(1, min(20000, int(seconds / per_row)))
        t0 = time.perf_counter()
        run(0, reps)
        one = reps / (time.perf_counter() - t0)
        t0 = time.perf_counter()
        with ThreadPoolExecutor(cores) as pool:
            list(pool.map(lambda b: run(b, reps), range(rows)))
        many = rows * reps / (time.perf_counter() - t0)
        res[label] = {"rows_per_s_one_core": one, "rows_per_s_all_threads": many, "threads": rows}
    return res


def timed_us(fn, reps, torch, repeats=1):
    """Duration of fn() in microseconds from events on the current stream: the mean over `reps`
    calls, or with repeats > 1 the median of that many such means."""
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    means = []
    for _ in range(repeats):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        means.append(e0.elapsed_time(e1) * 1e3 / reps)
    return statistics.median(means)


def bench_logit_chain(w, logits, torch, dev, s=None, out=None):
    """The device-side logit processors on a private copy of one batch of the workload: a chain of
    lists (repetition penalty over a 512-token history per row, then a 16-token mask), which touches
    a few hundred entries per row, and a chain of two whole-row processors, which has to read and
    write every entry once whatever its length (priced against the HBM peak)."""
    from executorch_amd.logit_processor import LogitChain

    work = logits.clone()
    g = torch.Generator(device=dev).manual_seed(7)
    history = torch.randint(0, w.vocab, (w.batch, 512), generator=g, device=dev, dtype=torch.int32)
    lengths = torch.full((w.batch,), 512, dtype=torch.int32, device=dev)
    lists = LogitChain().add_repetition_penalty(1.0009765625, history, lengths).add_mask(list(range(100, 116)))
    rows = LogitChain().add_scale(1.0).add_bias(0.0)
    lists_us = timed_us(lambda: lists.process(work), 50, torch)
    rows_us = timed_us(lambda: rows.process(work), 50, torch)
    moved = 2 * w.bytes_per_step  # the batch is read once and written once
    fused = {}
    if s is not None:
        # the same two whole-row processors applied while the sampler reads the rows, against the
        # sampler alone and against the two calls (all three on the same matrix)
        fused = {"sample_alone_us": timed_us(lambda: s.sample_batch(work, out=out), 100, torch, repeats=5),
                 "chain_then_sample_us": timed_us(lambda: (rows.process(work), s.sample_batch(work, out=out)), 100, torch, repeats=5),
                 "chain_fused_into_sample_us": timed_us(lambda: s.sample_batch_chain(work, rows, out=out), 100, torch, repeats=5)}
        fused["fused_over_alone"] = fused["chain_fused_into_sample_us"] / fused["sample_alone_us"]
    return {**fused, "lists_us": lists_us, "lists": "repetition penalty, 512-token history per row + mask of 16 ids",
            "whole_rows_us": rows_us, "whole_rows": "scale + bias", "whole_rows_algorithmic_bytes": moved,
            "whole_rows_gbs": moved / (rows_us * 1e-6) / 1e9, "whole_rows_frac_of_hbm_peak": moved / (rows_us * 1e-6) / 1e9 / HBM_PEAK_GBS}


def bench_host_buffers(w, s, logits, out, torch):
    """What the same step costs when the boundary is handed HOST memory: one batch copied from
    pinned host memory to the device and sampled (the PCIe-inclusive rate; never `value`), the
    reference-shaped single-row entry ets_sampler_sample() on a pageable host row, and
    logits_to_token() (util.h:64-71), which the reference calls once per decoded token."""
    import executorch_amd as ea

    host = torch.empty(logits.shape, dtype=logits.dtype, pin_memory=True)
    host.copy_(logits)
    staged = torch.empty_like(logits)

    def batch_step():
        staged.copy_(host, non_blocking=True)
        s.sample_batch(staged, out=out)

    batch_us = timed_us(batch_step, 20, torch)
    row = logits[0].cpu()
    one = type(s)(w.vocab, w.temperature, w.topp, 1)
    for _ in range(3):
        one.sample(row)
    t0 = time.perf_counter()
    for _ in range(50):
        one.sample(row)
    row_us = (time.perf_counter() - t0) * 1e6 / 50
    for _ in range(3):
        ea.logits_to_token(row, w.temperature)
    t0 = time.perf_counter()
    for _ in range(50):
        ea.logits_to_token(row, w.temperature)
    l2t_us = (time.perf_counter() - t0) * 1e6 / 50
    return {"batch_from_pinned_host_us": batch_us, "rows_per_s_pcie_inclusive": w.batch / (batch_us * 1e-6),
            "single_row_host_entry_us": row_us, "logits_to_token_us": l2t_us}


def bench_gumbel(w, s, ring, out, torch):
    """The Gumbel-max mode (one pass, no sequential sum) on the same ring with the library's own
    noise: one read of the logits, priced against the HBM peak."""
    state = {"i": 0}

    def step():
        s.gumbel_max_batch(ring[state["i"] % len(ring)], w.temperature, out=out)
        state["i"] += 1

    us = timed_us(step, 100, torch)
    gbs = w.bytes_per_step / (us * 1e-6) / 1e9
    return {"us_per_step": us, "rows_per_s": w.batch / (us * 1e-6), "algorithmic_bytes": w.bytes_per_step, "gbs": gbs,
            "frac_of_hbm_peak": gbs / HBM_PEAK_GBS}


def bench_greedy(w, ring, out, torch):
    """Temperature 0 (arg-max, sampler.cpp:44-56) on the same ring: one read of the logits."""
    import executorch_amd as ea

    g = ea.Sampler(w.vocab, 0.0, w.topp, 1, max_batch=w.batch)
    state = {"i": 0}

    def step():
        g.sample_batch(ring[state["i"] % len(ring)], out=out)
        state["i"] += 1

    us = timed_us(step, 100, torch)
    gbs = w.bytes_per_step / (us * 1e-6) / 1e9
    return {"us_per_step": us, "rows_per_s": w.batch / (us * 1e-6), "algorithmic_bytes": w.bytes_per_step, "gbs": gbs,
            "frac_of_hbm_peak": gbs / HBM_PEAK_GBS}


def bench_configs(w, s, ring, out, steps, torch):
    """ets_sampler_sample_batch_configs on the same ring: every row with the workload's own
    parameters, and a mix of four kinds of rows (one group of launches per kind)."""
    import numpy as np
    from executorch_amd.sampler import SAMPLING_CONFIG_DTYPE
    kinds = [(w.temperature, w.topp, 0, 0), (0.0, w.topp, 0, 0), (1.0, 1.0, 0, 0), (0.8, w.topp, 40, 0)]
    # (structured arrays, built once: a serving loop keeps its requests' parameters in this form)
    uniform = np.asarray([kinds[0]] * w.batch, dtype=SAMPLING_CONFIG_DTYPE)
    mixed = np.asarray([kinds[b % 4] for b in range(w.batch)], dtype=SAMPLING_CONFIG_DTYPE)
    state = {"i": 0}

    def run(cfg):
        def step():
            s.sample_batch_configs(ring[state["i"] % len(ring)], cfg, out=out)
            state["i"] += 1
        return step

    n = max(10, steps // 4)
    return {"uniform_us": timed_us(run(uniform), n, torch), "mixed_us": timed_us(run(mixed), n, torch),
            "mixed": "a quarter of the rows each: the workload's top-p, greedy, multinomial T=1, top-k 40 T=0.8"}


def bench_draw_modes(w, logits, out, torch):
    """The other element types and draws on the headline's shape and rows: the same matrix as
    fp16 / fp32, each with the workload's top-p, the multinomial draw (top-p 1) and top-k 40
    (microseconds per batch)."""
    import executorch_amd as ea

    res = {}
    for name, tdt in (("bf16", torch.bfloat16), ("fp16", torch.float16), ("fp32", torch.float32)):
        x = logits.to(tdt).contiguous()
        for mode, topp, topk in (("top_p", w.topp, 0), ("multinomial", 1.0, 0), ("top_k_40", w.topp, 40)):
            s = ea.Sampler(w.vocab, w.temperature, topp, w.coin_seed, max_batch=w.batch)
            s.set_topk(topk)
            res[f"{name}_{mode}_us"] = timed_us(lambda: s.sample_batch(x, out=out), 30, torch)
    return res


def bench_batch_sweep(w, torch, dev):
    """The headline's rows at other batch sizes."""
    import executorch_amd as ea

    res = {}
    g = torch.Generator(device=dev)
    g.manual_seed(11)
    for rows in (1, 8, 64, 256, 1024):
        x = torch.randn((rows, w.vocab), generator=g, device=dev, dtype=torch.float32)
        ids = torch.randint(0, w.vocab, (rows, 20), generator=g, device=dev)
        x.scatter_add_(1, ids, torch.full(ids.shape, 8.0, device=dev))
        x = x.to(torch.bfloat16).contiguous()
        s = ea.Sampler(w.vocab, w.temperature, w.topp, w.coin_seed, max_batch=rows)
        out = torch.empty(rows, dtype=torch.int32, device=dev)
        us = timed_us(lambda: s.sample_batch(x, out=out), 30, torch)
        gbs = rows * w.vocab * 2 / (us * 1e-6) / 1e9
        res[f"B{rows}"] = {"us_per_batch": us, "rows_per_s": rows / (us * 1e-6), "frac_of_hbm_peak": gbs / HBM_PEAK_GBS}
    return res


def bench_all_configs(torch, dev, with_cpu=True):
    """Every workload of the benchmark contract at its own batch, element type and parameters:
    microseconds per step (median of five repeats, device time), rows/s, and the step's algorithmic
    bytes (B x V x element size, read once) against the HBM peak.  Small rings (at least two
    matrices, more where they are cheap) keep this bounded; cfg1 also runs at temperature 0."""
    import dataclasses

    import executorch_amd as ea
    from executorch_amd import workloads as W

    res = {}
    for name in ("cfg1_greedy", "cfg1", "cfg2", "cfg3", "cfg4", "cfg5"):
        w = W.WORKLOADS[name]
        n_ring = max(2, min(40, (320 << 20) // w.bytes_per_step))
        ring = synth_logits_device(dataclasses.replace(w, data_seed=w.data_seed + 100), n_ring, torch, dev)
        s = ea.Sampler(w.vocab, w.temperature, w.topp, w.coin_seed, max_batch=w.batch)
        out = torch.empty(w.batch, dtype=torch.int32, device=dev)
        state = {"i": 0}

        def step():
            s.sample_batch(ring[state["i"] % n_ring], out=out)
            state["i"] += 1

        reps = 4 if name in ("cfg3", "cfg5") else 20
        us = timed_us(step, reps, torch, repeats=5)
        gbs = w.bytes_per_step / (us * 1e-6) / 1e9
        res[name] = {"vocab": w.vocab, "batch": w.batch, "dtype": W.DTYPE_NAMES[w.dtype], "temperature": w.temperature,
                     "top_p": w.topp, "us_per_step": us, "rows_per_s": w.batch / (us * 1e-6),
                     "algorithmic_bytes": w.bytes_per_step, "gbs": gbs, "frac_of_hbm_peak": gbs / HBM_PEAK_GBS,
                     "ring_matrices": n_ring, "steps_per_repeat": reps, "repeats": 5}
        if w.batch == 1:
            res[name]["note"] = ("one row per step: the ring's matrices stay in the caches, and a step is bound by the latency of "
                                 "its launches, not by bytes: read us_per_step, not the fraction of the HBM peak")
        if with_cpu:
            res[name]["cpu_baseline"] = cpu_baseline_config(w)
        del ring, s
        torch.cuda.empty_cache()
    return res


def bench_floors(w, ring, torch, dev):
    """What no kernel of this shape can beat on this box: an empty launch, and a kernel that only
    reads one step's logits (the ring keeps the reads in HBM), with as many workgroups as the step
    has rows and with enough to fill the chip."""
    import ctypes as C

    from executorch_amd import _capi

    L = _capi.hooks()
    stream = torch.cuda.current_stream(dev).cuda_stream
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    empty_us = timed_us(lambda: L.ets_test_empty_launch(stream), 200, torch, repeats=5)
    res = {"empty_launch_us": empty_us}
    state = {"i": 0}
    for wgs in (w.batch, 256, 1024, 4096):
        def step():
            x = ring[state["i"] % len(ring)]
            L.ets_test_read_floor(x.data_ptr(), C.c_int64(w.bytes_per_step), wgs, sink.data_ptr(), stream)
            state["i"] += 1
        us = timed_us(step, 100, torch, repeats=5)
        res[f"read_{wgs}_workgroups_us"] = us
        res[f"read_{wgs}_workgroups_gbs"] = w.bytes_per_step / (us * 1e-6) / 1e9
    # a hand-over between two workgroups through a word in device memory (release by one, bounded
    # polling by the other): microseconds per one-way signal, on another die and on the same one
    hops = 2000
    for label, partner in (("other_xcd", 1), ("same_xcd", 8)):
        words = torch.zeros(64, dtype=torch.int32, device=dev)
        res_w = torch.zeros(4, dtype=torch.int32, device=dev)
        st = L.ets_test_signal_floor(words.data_ptr(), hops, 1 << 16, partner, res_w.data_ptr(), stream)
        torch.cuda.synchronize()
        ticks = res_w.cpu().numpy().astype("uint32")
        ok = st == 0 and int(ticks[0]) == 0
        res[f"signal_{label}_us"] = float(ticks[1]) * 0.01 / (2 * hops) if ok else None  # (100 MHz clock)
    return res


def bench_graph(w, s, ring, out, torch, dev):
    """The same step captured into a HIP graph and replayed (the launches of one call as one graph
    launch), for the launch-bound batch of the headline.  One graph per ring matrix."""
    try:
        side = torch.cuda.Stream(device=dev)
        graphs = []
        n = min(len(ring), 8)
        with torch.cuda.stream(side):
            for i in range(n):
                s.sample_batch(ring[i], out=out)  # warm: buffers allocated, attributes set
            torch.cuda.synchronize()
            for i in range(n):
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=side):
                    s.sample_batch(ring[i], out=out)
                graphs.append(g)
        state = {"i": 0}

        def step():
            graphs[state["i"] % n].replay()
            state["i"] += 1

        us = timed_us(step, 50, torch, repeats=5)
        return {"us_per_step": us, "rows_per_s": w.batch / (us * 1e-6), "graphs": n}
    except Exception as e:  # capture is not supported by every runtime build
        return {"us_per_step": None, "error": str(e)[:200]}


def parse_pmc(fetch_dir, write_dir, out_path):
    """FETCH_SIZE / WRITE_SIZE (KiB per dispatch) of the step's kernels and of the 256 MiB copy probe
    from two rocprofv3 counter-collection runs -> HBM bytes per step."""
    def collect(path, counter):
        per = {}
        for f in glob.glob(os.path.join(path, "**", "*counter_collection.csv"), recursive=True):
            for r in csv.DictReader(open(f)):
                if r["Counter_Name"] != counter:
                    continue
                per.setdefault(r["Kernel_Name"], []).append(float(r["Counter_Value"]))
        return per

    fetch, write = collect(fetch_dir, "FETCH_SIZE"), collect(write_dir, "WRITE_SIZE")

    def mean_of(per, key):
        vals = [v for k, vs in per.items() if key in k for v in vs]
        return (sum(vals) / len(vals), len(vals)) if vals else (None, 0)

    copy_f, _ = mean_of(fetch, "copy_probe_kernel")
    copy_w, _ = mean_of(write, "copy_probe_kernel")
    probe_kib = COPY_PROBE_BYTES / 1024
    res = {"copy_probe_bytes": COPY_PROBE_BYTES, "copy_fetch_kib": copy_f, "copy_write_kib": copy_w,
           "fetch_factor": probe_kib / copy_f if copy_f else None, "write_factor": probe_kib / copy_w if copy_w else None,
           "kernels": {}}
    total = 0.0
    found = {k: (mean_of(fetch, k), mean_of(write, k)) for k in STEP_KERNELS}
    found = {k: v for k, v in found.items() if v[0][0] is not None or v[1][0] is not None}
    # a kernel that a step launches twice (multinomial rows: pass 2 and the walk kernel) counts twice
    steps_f = min((v[0][1] for v in found.values() if v[0][1]), default=0)
    steps_w = min((v[1][1] for v in found.values() if v[1][1]), default=0)
    for k, ((f, nf), (wv, nw)) in found.items():
        per_step = [round(nf / steps_f) if steps_f else 0, round(nw / steps_w) if steps_w else 0]
        res["kernels"][k] = {"fetch_kib": f, "write_kib": wv, "dispatches": [nf, nw], "launches_per_step": per_step}
        if f is not None and res["fetch_factor"]:
            total += f * per_step[0] * res["fetch_factor"] * 1024
        if wv is not None and res["write_factor"]:
            total += wv * per_step[1] * res["write_factor"] * 1024
    res["traffic_bytes_per_step"] = total
    with open(out_path, "w") as fo:
        json.dump(res, fo, indent=1)
        fo.write("\n")
    print(json.dumps(res))


def step_kernels_text(w):
    """Which launches make up one step of this workload (what the events of the timed loop bracket)."""
    if w.temperature == 0.0:
        return "one step = argmax_partial_kernel + argmax_finish_kernel (two launches)"
    if not 0.0 < w.topp < 1.0:
        return ("one step = split_pass1_kernel + split_pass2_kernel + split_walk_kernel + split_pass2_kernel + "
                "split_walk_kernel (multinomial rows, five launches; their summed duration is what the events bracket)")
    ns = (w.vocab + 511) // 512
    g = max(1, min(256 // w.batch if w.batch <= 256 else 1, (ns + 15) // 16, 64))
    fused = os.environ.get("ETS_FUSE", "1") != "0" and w.batch * g <= 256 and -(-ns // g) <= 64
    if fused:
        return ("one step = split_pass2_kernel with pass 1 inside (the workgroups of a row exchange maxima and sums "
                "through memory) + split_finish_kernel (two launches; their summed duration is what the events bracket)")
    return ("one step = split_pass1_kernel + split_pass2_kernel + split_finish_kernel (three launches; "
            "their summed duration is what the events bracket)")


def measured_traffic(name):
    """HBM bytes per step from the committed counter summary of this workload, or None."""
    path = os.path.join(ROOT, "profiles", f"traffic_{name}.json")
    try:
        with open(path) as f:
            return json.load(f).get("traffic_bytes_per_step"), os.path.relpath(path, ROOT)
    except (OSError, ValueError):
        return None, None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg2")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="only the headline loop (a profile of this command then holds its kernels only)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run five 256 MiB device copies: a kernel of known traffic that calibrates "
                         "FETCH_SIZE / WRITE_SIZE when this command runs under rocprofv3 --pmc")
    ap.add_argument("--parse-pmc", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"))
    ap.add_argument("--out", default=None)
    args = ap.parse_args()
    if args.parse_pmc:
        parse_pmc(args.parse_pmc[0], args.parse_pmc[1], args.out or os.path.join(ROOT, "profiles", f"traffic_{args.workload}.json"))
        return
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; rows are independent, so more GPUs would each take "
              "a slice of the batch with no communication.  Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import executorch_amd as ea
    from executorch_amd import workloads as W
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    w = W.WORKLOADS[args.workload]
    step_bytes = w.bytes_per_step
    ring_len = max(2, -(-(576 << 20) // step_bytes))  # >= 576 MiB of distinct logits
    ring = synth_logits_device(w, ring_len, torch, dev)
    s = ea.Sampler(w.vocab, w.temperature, w.topp, w.coin_seed, max_batch=w.batch)
    out = torch.empty(w.batch, dtype=torch.int32, device=dev)

    # step 0 of the workload from host-generated rows: the tokens the CPU leg checks
    rows = min(w.batch, 64)
    hx = W.logits(w, 0, rows)
    if w.dtype == W.DTYPE_BFLOAT16:
        dx = torch.from_numpy(hx.view(np.int16)).to(dev).view(torch.bfloat16)
    else:
        dx = torch.from_numpy(hx).to(dev)
    chk = ea.Sampler(w.vocab, w.temperature, w.topp, w.coin_seed, max_batch=rows)
    got = chk.sample_batch(dx).cpu().numpy()

    if args.copy_probe:
        src = torch.empty(COPY_PROBE_BYTES, dtype=torch.uint8, device=dev).random_()
        dst = torch.empty_like(src)
        for _ in range(5):
            from executorch_amd import _capi
            st = _capi.hooks().ets_test_copy_probe(src.data_ptr(), dst.data_ptr(), COPY_PROBE_BYTES, torch.cuda.current_stream().cuda_stream)
            assert st == 0
        torch.cuda.synchronize()
        del src, dst

    for i in range(args.warmup):
        s.sample_batch(ring[i % ring_len], out=out)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        s.sample_batch(ring[i % ring_len], out=out)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    # device time of a step's launches: events on the launch stream, median of five repeats of K steps
    repeats_ms = []
    for _ in range(5):
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for i in range(args.steps):
            s.sample_batch(ring[i % ring_len], out=out)
        ev1.record()
        torch.cuda.synchronize()
        repeats_ms.append(ev0.elapsed_time(ev1) / args.steps)
    kernel_ms = statistics.median(repeats_ms)
    achieved = step_bytes / (kernel_ms * 1e-3) / 1e9
    traffic, traffic_source = measured_traffic(w.name)

    line = {
        "metric": f"sampled rows/sec at vocab {w.vocab}, B={w.batch}, {W.DTYPE_NAMES[w.dtype]}, "
                  f"T={w.temperature}, top-p {w.topp}",
        "value": w.batch * args.steps / wall,
        "unit": "rows/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"{w.name}: vocab {w.vocab}, batch {w.batch}, {W.DTYPE_NAMES[w.dtype]} logits ({w.kind}), "
                               f"temperature {w.temperature}, top-p {w.topp}, per-row xorshift64* coins; "
                               f"ring of {ring_len} distinct matrices ({ring_len * step_bytes >> 20} MiB)"},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": step_kernels_text(w),
                     "kernel_ms": kernel_ms, "kernel_ms_repeats": repeats_ms, "algorithmic_bytes_per_launch": step_bytes},
    }
    if not args.no_extras:
        line["graph"] = bench_graph(w, s, ring, out, torch, dev)
        line["floors"] = bench_floors(w, ring, torch, dev)
        line["logit_chain"] = bench_logit_chain(w, ring[0], torch, dev, s, out)
        line["host_buffers"] = bench_host_buffers(w, s, ring[0], out, torch)
        line["gumbel_max"] = bench_gumbel(w, s, ring, out, torch)
        line["greedy"] = bench_greedy(w, ring, out, torch)
        line["per_row_configs"] = bench_configs(w, s, ring, out, args.steps, torch)
        line["draw_modes"] = bench_draw_modes(w, ring[0], out, torch)
        if w.dtype == W.DTYPE_BFLOAT16 and w.kind == "peaked":
            line["batch_sweep"] = bench_batch_sweep(w, torch, dev)
        del ring
        torch.cuda.empty_cache()
        line["configs"] = bench_all_configs(torch, dev, with_cpu=not args.no_cpu_baseline)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(w, got)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
