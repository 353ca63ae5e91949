#!/usr/bin/env python3
"""Benchmark of the optimizer-step hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2|cfg3|cfg4|cfg5|pipeline|accumulate|resident7b|multi] [--no-cpu-baseline]

A "step" is one fused AdamW update over one synthetic partition that is already resident in HBM.
Default workload: the Llama-7B decoder-layer partition (202,383,360 elements, bf16 gradients,
AdamW at t=100, bf16 copy-out). Prints ONE JSON line: whole-job elements/s, the roofline of the
update kernel (algorithmic bytes / measured kernel time against 8 TB/s) and the reference CPU
Adam timed on this machine's host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published

N_7B_LAYER = 4 * 4096 ** 2 + 3 * 4096 * 11008 + 2 * 4096                    # 202,383,360
N_70B_LAYER = 2 * 8192 ** 2 + 2 * 8192 * 1024 + 3 * 8192 * 28672 + 2 * 8192  # 855,654,400

# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (see the summaries under
# profiles/); None until measured for a workload.
MEASURED_TRAFFIC_BYTES = {"cfg2": 5_666_668_000, "cfg3": 5_666_667_000, "cfg4": 23_958_234_000, "accumulate": 2_453_896_000,
                          "multi": 5_666_709_000}
# The summary each literal is copied from; it carries the line "roofline.traffic = <bytes> B"
# (tests/test_bench_contract.py checks that the two agree).
TRAFFIC_SOURCE = {
    "cfg2": "profiles/adam_tile_kernel_cfg2_llama7b_layer.md",
    "cfg3": "profiles/grad_stats_and_adam_cfg3_overflow_path.md",
    "cfg4": "profiles/adam_tile_kernel_cfg4_llama70b_layer.md",
    "accumulate": "profiles/grad_accumulate_kernel_llama7b_layer.md",
    "multi": "profiles/adam_multi_kernel_cfg2_partition_16_ragged_contexts.md",
}

HP = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, bias_correction=True)


def percentile_mean(samples, lo=0.2, hi=0.8):
    """Mean of the 20th..80th percentile band, the reference's own statistic
    (flextrain/auto_config.py:48-55)."""
    s = sorted(samples)
    a, b = int(len(s) * lo), max(int(len(s) * hi), int(len(s) * lo) + 1)
    band = s[a:b]
    return sum(band) / len(band)


def make_inputs(torch, n, g_dtype, g_std, device, scale=1.0):
    """p, g, m, v and the 16-bit copy of one partition, in the library's own layout for the arrays
    of an update (one allocation, staggered starts), filled in place by the seeded generator
    (seed 0, one substream per array: the same values on any machine, on the GPU and on the host)."""
    from flextrain_amd import synth
    from flextrain_amd.memory import allocate_device_arrays
    p, m, v, g, h = allocate_device_arrays(
        [(n, torch.float32)] * 3 + [(n, g_dtype), (n, torch.bfloat16)], device)
    synth.fill_(p, 0, 0, scale=0.02)
    synth.fill_(m, 0, 1, scale=1e-4)
    synth.fill_(v, 0, 2, kind=synth.UNIFORM, scale=1e-6)
    synth.fill_(g, 0, 3, scale=g_std * scale)
    return p, g, m, v, h


def _host_description():
    """CPU model, logical CPUs and NUMA nodes of the machine the CPU baseline runs on."""
    import glob
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"cpu_model": model, "logical_cpus": os.cpu_count(), "numa_nodes": len(glob.glob("/sys/devices/system/node/node[0-9]*")) or 1}


def _host_memory_limits():
    """What bounds pinned host memory on this machine: installed and available memory, the
    locked-memory limit of the process, and the memory limit of its control group (if any)."""
    import resource
    out = {}
    try:
        with open("/proc/meminfo") as f:
            for line in f:
                key, _, rest = line.partition(":")
                if key in ("MemTotal", "MemAvailable"):
                    out["mem_total_gb" if key == "MemTotal" else "mem_available_gb"] = round(int(rest.split()[0]) * 1024 / 1e9, 1)
    except OSError:
        pass
    soft, hard = resource.getrlimit(resource.RLIMIT_MEMLOCK)
    out["rlimit_memlock"] = {"soft": "unlimited" if soft == resource.RLIM_INFINITY else soft,
                             "hard": "unlimited" if hard == resource.RLIM_INFINITY else hard}
    for path in ("/sys/fs/cgroup/memory.max", "/sys/fs/cgroup/memory/memory.limit_in_bytes"):
        try:
            with open(path) as f:
                text = f.read().strip()
            out["cgroup_memory_limit_gb"] = text if not text.isdigit() else round(int(text) / 1e9, 1)
            break
        except OSError:
            continue
    return out


def _device_description(torch, dev):
    """What the runtime says about the GPU the figures were measured on (the roofline's peak is the
    published 8 TB/s; the memory clock and bus width the driver reports are listed beside it)."""
    props = torch.cuda.get_device_properties(dev)
    out = {"name": props.name, "compute_units": props.multi_processor_count, "memory_gb": round(props.total_memory / 1e9, 1)}
    for key in ("gcnArchName", "memory_clock_rate", "memory_bus_width", "L2_cache_size"):
        value = getattr(props, key, None)
        if value is not None:
            out[key] = value
    return out


CPU_WARMUPS = 3


def _time_cpu_adam(n, budget_s):
    """Warm-up calls until the time per call has settled, then timed calls until the budget is used (at least 3, at most 20)
    of the reference CPU Adam with fp32 gradients and an fp16 copy-out on n elements in PINNED host
    memory (where the reference keeps its optimizer state, flextrain/memory/__init__.py:255-277),
    filled by the seeded generator. Returns (seconds per call as a 20-80 percentile mean, number of
    timed calls, kind, flavour)."""
    import numpy as np
    import torch

    import oracle
    from flextrain_amd import synth
    from flextrain_amd.memory import pinned_empty
    ref = oracle.reference_module()
    tp, tg, tm, tv = (pinned_empty(n, torch.float32) for _ in range(4))
    th = pinned_empty(n, torch.float16)
    scratch = torch.empty(n, dtype=torch.float32, device="cuda")  # the generator's GPU side is the fast one
    tp.copy_(synth.fill_(scratch, 0, 0, scale=0.02))
    tg.copy_(synth.fill_(scratch, 0, 3, scale=1e-3))
    del scratch
    tm.zero_()
    tv.zero_()
    th.zero_()
    if ref is not None:
        kind, oid = "reference", 4242
        ref.create_adam(oid, HP["lr"], *HP["betas"], HP["eps"], HP["weight_decay"], True, False)

        def call(t):
            ref.adam_update_copy(oid, t, HP["lr"], *HP["betas"], HP["eps"], HP["weight_decay"], True, tp, tg, tm, tv, th)
    else:
        kind = "port"
        pn, gn, mn, vn = tp.numpy(), tg.numpy(), tm.numpy(), tv.numpy()
        hn = th.numpy().view(np.uint16)

        def call(t):
            oracle.adam_step(pn, gn, mn, vn, step=t, lr=HP["lr"], betas=HP["betas"], eps=HP["eps"],
                             weight_decay=HP["weight_decay"], half_out=hn, half_dtype=oracle.F16)
    # Warm-up: at least CPU_WARMUPS calls, and on until three calls in a row agree within 5 % (the
    # first second or so of a process's OpenMP work ran up to 40 % slower on the measured hosts:
    # thread start-up, clock ramp, first use of the pinned pages), for 8 s at most.
    warm, t_begin = [], time.perf_counter()
    while len(warm) < CPU_WARMUPS or (min(warm[-3:]) < 0.95 * max(warm[-3:]) and time.perf_counter() - t_begin < 8.0) \
            or time.perf_counter() - t_begin < 1.5:
        t0 = time.perf_counter()
        call(len(warm) + 1)
        warm.append(time.perf_counter() - t0)
    times, t_begin = [], time.perf_counter()
    while len(times) < 20 and (len(times) < 3 or time.perf_counter() - t_begin < budget_s):
        t0 = time.perf_counter()
        call(len(times) + len(warm) + 1)
        times.append(time.perf_counter() - t0)
    if ref is not None:
        ref.destroy_adam(oid)
    flavour = getattr(ref, "flavour", f"libftoracle isa={oracle.best_isa()}")
    return percentile_mean(times), len(times), kind, flavour, len(warm)


def cpu_baseline(n, budget_s=14.0):
    """Times the reference CPU Adam (its own C++ compiled into oracle/_ref when present, else this
    repository's restatement) on host buffers of the workload's size: fp32 gradients and an fp16
    copy-out, the only form the reference supports; 20-80 percentile mean of the timed calls, as
    flextrain/auto_config.py:281-317 does for its own optimizer probe. The same is then timed on
    the block size that probe itself uses (2**28 elements) and reported beside it."""
    import oracle
    threads = oracle.max_threads()
    sec, calls, kind, flavour, warmups = _time_cpu_adam(n, budget_s)
    out = {
        "value": n / sec, "unit": "elements/s", "cores": threads, "kind": kind,
        "sample": f"{calls} timed calls ({warmups} warm-ups) of the CPU Adam with fp16 copy-out on {n} fp32 elements "
                  f"in pinned host memory, {threads} OpenMP threads, 20-80 percentile mean",
        "ms_per_call": sec * 1e3, "host_gbps": n * 30 / sec / 1e9, "flavour": flavour,
        "host": _host_description(),
    }
    block = 1 << 28
    bsec, bcalls, _, _, _ = _time_cpu_adam(block, budget_s * 0.4)
    out["reference_probe_block"] = {"elements": block, "value": block / bsec, "unit": "elements/s",
                                    "ms_per_call": bsec * 1e3, "timed_calls": bcalls}
    return out


def link_probe(torch):
    """What the host link carries: the library's probe (two transfers in flight per direction; the
    runtime's copies and a copy kernel; each direction alone and both at once) and the ceilings
    derived from it. The unidirectional ceiling is the best figure any method reached in either
    direction; two directions at once cannot carry more than twice that, so fractions of
    ``full_duplex_ceiling_gbps`` cannot exceed 1."""
    import ctypes

    from flextrain_amd import _C
    r = _C.LinkProbe()
    _C.check("ft_link_probe", _C.lib().ft_link_probe(1 << 30, 10, ctypes.byref(r)))
    out = {name: getattr(r, name) for name, _ in _C.LinkProbe._fields_}
    out["unidirectional_ceiling_gbps"] = max(r.h2d_copy, r.d2h_copy, r.h2d_kernel, r.d2h_kernel)
    pairings = {"copies both ways": r.both_copy, "copy kernels both ways": r.both_kernel,
                "copies in, copy kernel out": r.both_copy_in_kernel_out, "copy kernel in, copies out": r.both_kernel_in_copy_out}
    out["bidirectional_sum_measured_gbps"] = max(pairings.values())
    out["best_bidirectional_pairing"] = max(pairings, key=pairings.get)
    out["full_duplex_ceiling_gbps"] = 2 * out["unidirectional_ceiling_gbps"]
    # What the platform carries when both directions run at once, whichever way they are driven
    # (copies both ways, copy kernels both ways, either mix): the limit an offloaded step lives under.
    out["platform_full_duplex_each_way_gbps"] = out["bidirectional_sum_measured_gbps"] / 2
    return out


def measure_offload(args, torch, dev, layers, steps, warmup):
    """cfg5: the Llama-7B optimizer with fp32 master/m/v in pinned host DRAM, streamed through the
    GPU in chunks (H2D -> fused AdamW -> D2H on three streams); bf16 gradients and the bf16
    parameter copy stay on the GPU. One step = one pass over all elements, timed end to end.
    Returns (record, ok): the measurements and whether the streamed result equals the resident one."""
    import gc

    from flextrain_amd import FlexTrainCPUAdam, _C, synth
    from flextrain_amd.memory import pinned_empty

    n_full = 32 * N_7B_LAYER + 2 * 4096 * 32000
    chunk = args.chunk_elems
    # The whole state must be pinned (3 x 4 bytes per element). A machine that cannot pin that much
    # runs the largest whole-layer prefix that fits, and the record says which fraction that is.
    p = None
    pin_attempts = []  # what hipHostMalloc granted and refused on the way: shows that the size is the machine's
    while p is None:
        n = layers * N_7B_LAYER + 2 * 4096 * 32000
        t0 = time.perf_counter()
        try:
            p, m, v = (pinned_empty(n, torch.float32) for _ in range(3))
            spare = pinned_empty(3 << 30, torch.uint8)  # room for the link probe's own pinned buffers
            del spare
            pin_attempts.append({"layers": layers, "pinned_gb": round(3 * n * 4 / 1e9, 1), "granted": True})
        except _C.FtError as exc:
            pin_attempts.append({"layers": layers, "pinned_gb": round(3 * n * 4 / 1e9, 1), "granted": False,
                                 "error": str(exc)[:120]})
            p = m = v = None
            gc.collect()
            layers -= 1
            if layers < 1:
                raise RuntimeError("cannot pin even one layer of optimizer state")
    t_alloc = time.perf_counter() - t0
    g = torch.empty(n, dtype=torch.bfloat16, device=dev)
    h = torch.empty(n, dtype=torch.bfloat16, device=dev)
    t0 = time.perf_counter()
    scratch = torch.empty(chunk, dtype=torch.float32, device=dev)
    for lo in range(0, n, chunk):  # seeded state is generated on the GPU and copied down chunk by chunk
        hi = min(n, lo + chunk)
        k = hi - lo
        p[lo:hi].copy_(synth.fill_(scratch[:k], 0, 0, scale=0.02, first_index=lo))
        m[lo:hi].copy_(synth.fill_(scratch[:k], 0, 1, scale=1e-4, first_index=lo))
        v[lo:hi].copy_(synth.fill_(scratch[:k], 0, 2, kind=synth.UNIFORM, scale=1e-6, first_index=lo))
    synth.fill_(g, 0, 3, scale=1e-3)
    torch.cuda.synchronize()
    del scratch
    t_init = time.perf_counter() - t0

    link = link_probe(torch)

    eng = FlexTrainCPUAdam(offload_chunk_elems=chunk, offload_slots=args.slots, **HP)
    # keep copies of three chunks to check the streamed result against the resident kernel afterwards
    probes = sorted({0, (n // chunk // 2) * chunk, ((n - 1) // chunk) * chunk})
    before = {lo: tuple(t[lo:min(n, lo + chunk)].to(dev) for t in (p, m, v)) for lo in probes}
    group = {"step": 100}
    for _ in range(warmup):
        eng._step(group, h, p, g, m, v)
    walls, devs = [], []
    for _ in range(steps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng._step(group, h, p, g, m, v)  # blocks until the host arrays hold the new values
        torch.cuda.synchronize()
        walls.append(time.perf_counter() - t0)
        devs.append(eng.last_offload_ms() * 1e-3)
    # correctness probe: replay the same number of steps on the saved chunks with the resident kernel
    ok = True
    res = FlexTrainCPUAdam(**HP)
    for lo, (bp, bm, bv) in before.items():
        hi = min(n, lo + chunk)
        bh = torch.empty(hi - lo, dtype=torch.bfloat16, device=dev)
        for _ in range(warmup + steps):
            res._step(group, bh, bp, g[lo:hi], bm, bv)
        torch.cuda.synchronize()
        ok = ok and torch.equal(bp.cpu(), p[lo:hi]) and torch.equal(bm.cpu(), m[lo:hi]) and torch.equal(bv.cpu(), v[lo:hi]) \
            and torch.equal(bh, h[lo:hi])
    # the reference's statistic for its own probes: mean of the 20th..80th percentile band
    sec = percentile_mean(walls)
    one_way = n * 12 / sec / 1e9
    record = {
        "workload": f"cfg5: offloaded Llama-7B optimizer ({layers} of 32 layers + embedding + lm_head), "
                    "fp32 p/m/v in pinned host DRAM streamed in chunks, bf16 grads and copy on GPU",
        "elements": n, "fraction_of_full_7b": n / n_full, "chunk_elems": chunk, "slots": args.slots, "chunks": -(-n // chunk),
        "steps": steps, "warmup": warmup, "ms_per_step": sec * 1e3, "ms_per_step_statistic": "20-80 percentile mean",
        "step_ms": [round(w * 1e3, 2) for w in walls], "ms_per_step_mean": sum(walls) / len(walls) * 1e3,
        "elements_per_s": n / sec,
        "bytes_each_way": n * 12, "achieved_each_way_gbps": one_way, "achieved_total_gbps": 2 * one_way,
        "device_time_ms": sum(devs) / len(devs) * 1e3,
        "link": link,
        "frac_of_unidirectional": one_way / link["unidirectional_ceiling_gbps"],
        # two measurements of the same limit (the probe's both-directions run and this step): a
        # ratio, not a fraction of a ceiling; it sits at 1.00 and may exceed it by a per cent
        "ratio_to_bidirectional_probe": 2 * one_way / link["bidirectional_sum_measured_gbps"],
        # The step moves both directions at once, so what bounds it is what the link carries both
        # ways at once: no pairing of copy methods in the probe carries more than
        # bidirectional_sum_measured_gbps, which is below twice the unidirectional ceiling.
        "ceiling_basis": "both-ways probe",
        "ceiling_each_way_gbps": link["platform_full_duplex_each_way_gbps"],
        "setup": {"pinned_alloc_s": t_alloc, "init_s": t_init, "pinned_gb": 3 * n * 4 / 1e9},
        "host": dict(_host_memory_limits(), pin_attempts=pin_attempts,
                     largest_pinned_total_granted_gb=round((3 * n * 4 + (3 << 30)) / 1e9, 1)),
        "streamed_equals_resident_on_probe_chunks": bool(ok),
    }
    del p, m, v, g, h, before
    gc.collect()
    torch.cuda.empty_cache()
    return record, ok


def bench_offload(args, torch, dev) -> int:
    rec, ok = measure_offload(args, torch, dev, args.layers, args.steps, args.warmup)
    link = rec["link"]
    out_json = {
        "metric": "Adam step elements/s + achieved HBM GB/s (% peak) on 7B-layer partition",
        "value": rec["elements_per_s"], "unit": "elements/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": rec["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {k: rec[k] for k in ("workload", "elements", "fraction_of_full_7b", "chunk_elems", "slots", "chunks")},
        "offload": rec,
        # Both directions at the unidirectional ceiling is the most a full-duplex link can carry: a
        # fraction of it cannot exceed 1 (what both directions reach when probed together is lower
        # and is listed beside it).
        "roofline": {"bound": "host-link", "kernel": "hipMemcpyAsync H2D/D2H + adam_tile_kernel per chunk",
                     "achieved": rec["achieved_total_gbps"], "peak": link["full_duplex_ceiling_gbps"], "unit": "GB/s",
                     "frac": rec["achieved_total_gbps"] / link["full_duplex_ceiling_gbps"], "traffic": None},
    }
    print(json.dumps(out_json), flush=True)
    return 0 if ok else 3


def bench_ceilings() -> int:
    """The library's kernels beside bare kernels of the same memory traffic: runs
    flextrain_amd/ft_ceiling (a HIP program of its own, started before this process touches the
    GPU) and prints what it measured as one JSON line."""
    import subprocess

    from flextrain_amd.build import CEILING_PATH, build_ceiling
    if not os.path.exists(CEILING_PATH):  # nothing built in this tree yet
        build_ceiling()
    run = subprocess.run([CEILING_PATH], capture_output=True, text=True, timeout=300)
    if run.returncode != 0:
        print(run.stdout + run.stderr, file=sys.stderr)
        return run.returncode or 1
    cases = [json.loads(line) for line in run.stdout.splitlines() if line.startswith("{")]
    print(json.dumps({"metric": "kernel time against a bare kernel of the same traffic, 7B-layer partition", "unit": "us",
                      "data": "synthetic", "n_gpus": 1, "cases": cases}), flush=True)
    return 0


def measure_accumulate(torch, dev, steps, warmup, calibration_copy=False):
    """Gradient hand-off before the step: fp32 accumulator += bf16 micro-batch gradient over the
    7B-layer partition, clearing the source and gathering the overflow/norm statistics of the
    result in the same pass. Algorithmic bytes: read 4 + 2, write 4 + 2 = 12 B/element. Returns
    {variant: {ms_avg, achieved_gbps, bytes_per_element, wall_ms_per_step}}."""
    from flextrain_amd import synth
    from flextrain_amd.loss_scaler import GradientGuard
    from flextrain_amd.memory import allocate_device_arrays
    n = N_7B_LAYER
    guard = GradientGuard(dev)
    acc, g = allocate_device_arrays([(n, torch.float32), (n, torch.bfloat16)], dev)
    synth.fill_(g, 0, 3, scale=1e-3)
    if calibration_copy:  # a plain copy of known size, to scale the profiler's byte counters by
        scratch = torch.empty_like(acc)
        for _ in range(3):
            scratch.copy_(acc)
        torch.cuda.synchronize()
        del scratch
    variants = {
        "accumulate": dict(zero_grads=False, with_stats=False, bytes=10),
        "accumulate+clear": dict(zero_grads=True, with_stats=False, bytes=12),
        "accumulate+clear+stats": dict(zero_grads=True, with_stats=True, bytes=12),
    }
    results = {}
    for name, kw in variants.items():
        nbytes = kw.pop("bytes")
        for _ in range(warmup):
            guard.begin()
            guard.accumulate(acc, g, **kw)
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for a, b in ev:
            a.record()
            guard.begin()
            guard.accumulate(acc, g, **kw)
            b.record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        ms = sum(a.elapsed_time(b) for a, b in ev) / len(ev)
        results[name] = {"ms_avg": ms, "achieved_gbps": n * nbytes / (ms * 1e-3) / 1e9, "bytes_per_element": nbytes,
                         "wall_ms_per_step": wall * 1e3 / steps}
    del acc, g
    torch.cuda.empty_cache()
    return results


def bench_accumulate(args, torch, dev) -> int:
    n = N_7B_LAYER
    results = measure_accumulate(torch, dev, args.steps, args.warmup, args.calibration_copy)
    main = results["accumulate+clear+stats"]
    print(json.dumps({
        "metric": "Adam step elements/s + achieved HBM GB/s (% peak) on 7B-layer partition",
        "value": n / (main["wall_ms_per_step"] * 1e-3), "unit": "elements/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": main["wall_ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "accumulate: fp32 accumulator += bf16 gradient on the 7B-layer partition, source cleared, "
                               "statistics of the result in the same pass", "elements": n},
        "roofline": {"bound": "hbm", "kernel": "grad_accumulate_kernel", "achieved": main["achieved_gbps"],
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": main["achieved_gbps"] / HBM_PEAK_GBPS,
                     "traffic": MEASURED_TRAFFIC_BYTES["accumulate"], "traffic_source": TRAFFIC_SOURCE["accumulate"],
                     "algorithmic_bytes_per_launch": n * 12, "kernel_ms_avg": main["ms_avg"]},
        "variants": results,
    }), flush=True)
    return 0


def bench_pipeline(args, torch, dev) -> int:
    """The per-unit schedule of the optimizer coordinator on Llama-7B layers: while unit u is in
    backward (here: its synthetic bf16 gradient is copied into the receive buffer, one share per
    micro-batch), unit u+1 is stepped share by share with its fp32 state streamed from pinned host
    memory. One step = one pass over all units. No model runs; what is timed is the optimizer side."""
    import ctypes
    import gc

    from flextrain_amd import FlexTrainAdam, _C
    from flextrain_amd.coordinator import FlexTrainOptsCoordinator

    class Unit:
        def __init__(self, paras):
            self.paras = paras

    lib = _C.lib()
    n, mb = N_7B_LAYER, args.micro_batches
    if args.resident:
        return bench_pipeline_resident(args, torch, dev, Unit)
    units = min(args.layers, 24 + args.resident_units)  # 24 streamed layers = 58 GB of pinned state, inside what the box pins
    coord = None
    while coord is None:
        flat = [(torch.randn(n, device=dev) * 0.02).to(torch.bfloat16) for _ in range(units)]
        params = [torch.nn.Parameter(f) for f in flat]
        opt = FlexTrainAdam([{"params": params}], unit_parameter_map={u: Unit([params[u]]) for u in range(units)},
                            aligned_unit_numel=n, offload=True, **{k: HP[k] for k in ("lr", "betas", "eps", "weight_decay")})
        opt.cpu_optimizer._offload_chunk = args.chunk_elems
        opt.cpu_optimizer._offload_slots = args.slots
        opt.cpu_optimizer._offload_window_piece = args.window_piece_mi << 20
        try:
            coord = FlexTrainOptsCoordinator()
            coord.initialize(opt, flat, mb, offload=True,
                             unit_windows={"auto": None, "off": False}.get(args.windows, True),
                             window_write_through=args.windows == "write_through",
                             resident_units=args.resident_units, alpha=args.alpha)
        except _C.FtError:
            coord = None
            del opt, flat, params
            gc.collect()
            units -= 2
            if units < 2:
                print("cannot pin two layers of optimizer state", file=sys.stderr)
                return 1
    grads = (torch.randn(n, device=dev) * 1e-3).to(torch.bfloat16)
    share = n // mb
    link = link_probe(torch)

    phase_s = {"forward": [], "backward": []}

    def iteration(timed=False):
        # the reference's order (flextrain/engine.py:353-399): forward pass (steps the forward shares
        # of the previous iteration), update_states, backward pass (steps the backward shares)
        t0 = time.perf_counter()
        coord.warmup_forward_pipeline()
        for u in range(units):
            coord.pre_unit_forward(u)
            for k in range(mb):
                coord.post_micro_batch_forward(u, k)
        if timed:
            coord.synchronize()
            torch.cuda.synchronize()
            phase_s["forward"].append(time.perf_counter() - t0)
        t1 = time.perf_counter()
        opt.update_states()
        for u in reversed(range(units)):
            buf = coord.pre_unit_backward(u)
            for k in range(mb):
                buf[k * share:(k + 1) * share].copy_(grads[k * share:(k + 1) * share])
                coord.post_micro_batch_backward(u, k)
        coord.clear_backward_pipeline()
        if timed:
            torch.cuda.synchronize()
            phase_s["backward"].append(time.perf_counter() - t1)

    for _ in range(args.warmup):
        iteration()
    walls = []
    for _ in range(args.steps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        iteration(timed=True)
        torch.cuda.synchronize()
        walls.append(time.perf_counter() - t0)
    sec = sum(walls) / len(walls)
    total = units * n
    streamed_units = units - min(args.resident_units, units)
    streamed = streamed_units * n
    one_way = streamed * 12 / sec / 1e9
    # how the link's work falls into the two passes: each pass moves its share of every streamed unit
    fwd_numel = coord._mb_fwd_numel * mb
    phases = {}
    for name, numel in (("forward", fwd_numel), ("backward", n - fwd_numel)):
        t = sum(phase_s[name]) / len(phase_s[name])
        phases[name] = {"ms": t * 1e3, "elements_per_unit": numel, "bytes_each_way": streamed_units * numel * 12,
                        "each_way_gbps": streamed_units * numel * 12 / t / 1e9 if numel else 0.0}
    print(json.dumps({
        "metric": "Adam step elements/s + achieved HBM GB/s (% peak) on 7B-layer partition",
        "value": total / sec, "unit": "elements/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"pipeline: coordinator schedule over {units} Llama-7B layers, {mb} shares per unit, "
                               "fp32 state in pinned host DRAM, bf16 grads and parameters on GPU",
                   "elements": total, "units": units, "micro_batches": mb, "chunk_elems": args.chunk_elems,
                   "slots": args.slots, "unit_windows": args.windows, "window_piece_mi": args.window_piece_mi,
                   "resident_units": min(args.resident_units, units),
                   "streamed_elements": streamed, "alpha": args.alpha},
        "iteration_ms": [w * 1e3 for w in walls],
        "phases": phases,
        "link": dict(link, achieved_each_way_gbps=one_way, achieved_total_gbps=2 * one_way,
                     frac_of_unidirectional=one_way / link["unidirectional_ceiling_gbps"],
                     ratio_to_bidirectional_probe=2 * one_way / link["bidirectional_sum_measured_gbps"]),
        "roofline": {"bound": "host-link", "kernel": "hipMemcpyAsync H2D/D2H + adam_tile_kernel per share",
                     "achieved": 2 * one_way, "peak": link["full_duplex_ceiling_gbps"], "unit": "GB/s",
                     "frac": 2 * one_way / link["full_duplex_ceiling_gbps"], "traffic": None},
    }), flush=True)
    return 0


def bench_pipeline_resident(args, torch, dev, Unit) -> int:
    """The same schedule with every unit's fp32 state resident in HBM (32 layers: 78 GB): what the
    caller-shaped path costs beyond its kernels. Bytes per element and iteration: the update 28, the
    stand-in for backward (copying the unit's bf16 gradient into the receive buffer) 4, clearing the
    receive buffer 2."""
    from flextrain_amd import FlexTrainAdam
    from flextrain_amd.coordinator import FlexTrainOptsCoordinator
    n, mb, units = N_7B_LAYER, args.micro_batches, args.layers
    flat = [(torch.randn(n, device=dev) * 0.02).to(torch.bfloat16) for _ in range(units)]
    hp = {k: HP[k] for k in ("lr", "betas", "eps", "weight_decay")}
    if args.layer_groups:
        # A decoder layer as its own tensors in module order (input norm, q, k, v, o, post-attention
        # norm, gate, up, down), matrices in a weight-decay group and the two norms in a group without:
        # the group boundaries cut some shares into several step contexts.
        h, f = 4096, 11008
        sizes = [h, h * h, h * h, h * h, h * h, h, h * f, h * f, h * f]
        decay, plain, unit_params = [], [], []
        for fl in flat:
            pieces = [torch.nn.Parameter(t) for t in fl.split(sizes)]
            unit_params.append(pieces)
            for t, size in zip(pieces, sizes):
                (plain if size == h else decay).append(t)
        groups = [{"params": decay}, {"params": plain, "weight_decay": 0.0}]
    else:
        unit_params = [[torch.nn.Parameter(fl)] for fl in flat]
        groups = [{"params": [u[0] for u in unit_params]}]
    opt = FlexTrainAdam(groups, unit_parameter_map={u: Unit(unit_params[u]) for u in range(units)},
                        aligned_unit_numel=n, offload=False, **hp)
    coord = FlexTrainOptsCoordinator()
    coord.initialize(opt, flat, mb, offload=False, resident_shares=args.resident_shares or None,
                     step_stream={"auto": None, "on": True, "off": False}[args.step_stream])
    grads = (torch.randn(n, device=dev) * 1e-3).to(torch.bfloat16)
    share = n // mb

    # Optional stand-in for the arithmetic of a backward pass: per micro-batch, for each of the layer's
    # seven matrices (a x b), one (T x a)(a x b) and one (a x T)(T x b) product in bf16 = 4 T a b flops,
    # 4 x parameters x T in all, which is what the backward of a decoder layer over T tokens costs.
    tokens = args.backward_tokens
    if tokens:
        shapes = [(4096, 4096)] * 4 + [(4096, 11008)] * 3
        wide = {b: torch.randn(tokens, b, device=dev, dtype=torch.bfloat16) for b in (4096, 11008)}
        x_t = torch.randn(4096, tokens, device=dev, dtype=torch.bfloat16)
        x = torch.randn(tokens, 4096, device=dev, dtype=torch.bfloat16)
        weights = {b: torch.randn(4096, b, device=dev, dtype=torch.bfloat16) for b in (4096, 11008)}
        out_tb = {b: torch.empty(tokens, b, device=dev, dtype=torch.bfloat16) for b in (4096, 11008)}
        out_ab = {b: torch.empty(4096, b, device=dev, dtype=torch.bfloat16) for b in (4096, 11008)}

    def backward_arithmetic():
        if tokens:
            for _, b in shapes:
                torch.mm(x, weights[b], out=out_tb[b])
                torch.mm(x_t, wide[b], out=out_ab[b])

    def iteration(with_optimizer=True):
        if not with_optimizer:
            for _ in range(units * mb):
                backward_arithmetic()
            return
        opt.update_states()
        for u in reversed(range(units)):
            buf = coord.pre_unit_backward(u)
            for k in range(mb):
                backward_arithmetic()
                buf[k * share:(k + 1) * share].copy_(grads[k * share:(k + 1) * share])
                coord.post_micro_batch_backward(u, k)
        coord.clear_backward_pipeline()

    for _ in range(args.warmup):
        iteration()
    arithmetic_ms = None
    if tokens:
        iteration(with_optimizer=False)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            iteration(with_optimizer=False)
        torch.cuda.synchronize()
        arithmetic_ms = (time.perf_counter() - t0) / args.steps * 1e3
    walls, host = [], []
    for _ in range(args.steps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        iteration()
        t1 = time.perf_counter()
        torch.cuda.synchronize()
        walls.append(time.perf_counter() - t0)
        host.append(t1 - t0)
    sec = sum(walls) / len(walls)
    total = units * n
    achieved = total * 34 / sec / 1e9
    print(json.dumps({
        "metric": "Adam step elements/s + achieved HBM GB/s (% peak) on 7B-layer partition",
        "value": total / sec, "unit": "elements/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"pipeline, resident: coordinator schedule over {units} Llama-7B layers, {mb} shares per unit, "
                               "fp32 state, bf16 grads and parameters all in HBM",
                   "elements": total, "units": units, "micro_batches": mb, "bytes_per_element": 34,
                   "shares_per_unit": len(coord.unit_step_contexts(0)),
                   "contexts_per_unit": sum(len(part) for part in coord.unit_step_contexts(0)),
                   "step_stream": coord._step_stream is not None, "backward_tokens": tokens},
        "host_ms_per_iteration": sum(host) / len(host) * 1e3,
        **({"backward_arithmetic_ms": arithmetic_ms, "exposed_optimizer_ms": sec * 1e3 - arithmetic_ms} if tokens else {}),
        "roofline": {"bound": "hbm", "kernel": "adam_tile_kernel per share + gradient copy + clear", "achieved": achieved,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS, "traffic": None},
    }), flush=True)
    return 0


def measure_multi(torch, dev, segments, steps, warmup, calibration_copy=False, variants=("one_launch", "per_context")):
    """The 7B-layer partition of cfg2 cut into `segments` ragged contexts of two parameter groups
    (different weight decay and step count), the way a unit's share reaches the step engine when
    groups and buffer pieces cut it (flextrain/param_group.py:365-477): all contexts in one launch
    (ft_adam_step_multi) against one call per context (the reference's loop, flextrain/optimizer.py:44-69).
    Returns (results by variant, the contexts' lengths)."""
    import random

    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.param_group import StepContext
    n, k = N_7B_LAYER, max(1, segments)
    eng = FlexTrainCPUAdam(**HP)
    p, g, m, v, h = make_inputs(torch, n, torch.bfloat16, 1e-3, dev)
    if calibration_copy:  # a plain copy of known size, to scale the profiler's byte counters by
        scratch = torch.empty_like(p)
        for _ in range(3):
            scratch.copy_(p)
        torch.cuda.synchronize()
        del scratch
    rng = random.Random(0)
    cuts = sorted({0, n} | {rng.randrange(1, n) for _ in range(k - 1)})
    groups = [dict(HP, step=100), dict(HP, step=37, weight_decay=0.0)]
    ctxs = [StepContext(groups[i % 2], h[lo:hi], p[lo:hi], g[lo:hi], [m[lo:hi], v[lo:hi]])
            for i, (lo, hi) in enumerate(zip(cuts[:-1], cuts[1:]))]

    def one_launch():
        eng._step_many(ctxs)

    def per_context():
        for c in ctxs:
            eng._step(c.param_group, c.half_parameter, c.full_parameter, c.gradient, *c.optimizer_states)

    results = {}
    for name, fn in (("one_launch", one_launch), ("per_context", per_context)):
        if name not in variants:
            continue
        for _ in range(warmup):
            fn()
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        host = 0.0
        for a, b in ev:
            a.record()
            h0 = time.perf_counter()
            fn()
            host += time.perf_counter() - h0
            b.record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        ms = sum(a.elapsed_time(b) for a, b in ev) / len(ev)
        results[name] = {"ms_avg": ms, "achieved_gbps": n * 28 / (ms * 1e-3) / 1e9, "frac": n * 28 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                         "wall_ms_per_step": wall * 1e3 / steps, "host_us_per_step": host * 1e6 / steps}
    lengths = [c.full_parameter.numel() for c in ctxs]
    del ctxs, p, g, m, v, h
    torch.cuda.empty_cache()
    return results, lengths


def bench_multi(args, torch, dev) -> int:
    n = N_7B_LAYER
    results, lengths = measure_multi(torch, dev, args.segments, args.steps, args.warmup, args.calibration_copy)
    main = results["one_launch"]
    print(json.dumps({
        "metric": "Adam step elements/s + achieved HBM GB/s (% peak) on 7B-layer partition",
        "value": n / (main["wall_ms_per_step"] * 1e-3), "unit": "elements/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": main["wall_ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"multi: the cfg2 partition cut into {len(lengths)} ragged contexts of two parameter groups, "
                               "stepped by one launch (against one call per context)", "elements": n, "segments": len(lengths),
                   "shortest": min(lengths), "longest": max(lengths)},
        "roofline": {"bound": "hbm", "kernel": "adam_multi_kernel", "achieved": main["achieved_gbps"], "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": main["frac"],
                     "traffic": MEASURED_TRAFFIC_BYTES["multi"] if len(lengths) == 16 else None,
                     "traffic_source": TRAFFIC_SOURCE["multi"] if len(lengths) == 16 else None,
                     "algorithmic_bytes_per_launch": n * 28,
                     "kernel_ms_avg": main["ms_avg"]},
        "variants": results,
    }), flush=True)
    return 0


def bench_resident7b(args, torch, dev) -> int:
    """What 288 GB of HBM allow: the whole 7B optimizer of cfg5 (81 GB of fp32 state + 27 GB of bf16
    gradients and parameters) resident. One allocation per unit (32 decoder layers + embedding and
    lm_head), as the coordinator lays resident state out, and one launch per unit: the arrays of a
    launch then lie within a few GB of each other, which the kernel rewards (the same kernel over
    five 27 GB arrays in one launch runs at 82.6 % of peak instead of 85 %)."""
    from flextrain_amd import FlexTrainCPUAdam, synth
    from flextrain_amd.memory import allocate_device_arrays
    eng = FlexTrainCPUAdam(**HP)
    sizes = [N_7B_LAYER] * 32 + [2 * 4096 * 32000]
    units, first = [], 0
    for n in sizes:  # the units are consecutive element ranges of the four substreams
        p, m, v, g, h = allocate_device_arrays([(n, torch.float32)] * 3 + [(n, torch.bfloat16)] * 2, dev)
        synth.fill_(p, 0, 0, scale=0.02, first_index=first)
        synth.fill_(m, 0, 1, scale=1e-4, first_index=first)
        synth.fill_(v, 0, 2, kind=synth.UNIFORM, scale=1e-6, first_index=first)
        synth.fill_(g, 0, 3, scale=1e-3, first_index=first)
        units.append((h, p, g, m, v))
        first += n
    total = sum(sizes)
    group = {"step": 100}

    def one_step():
        for unit in units:
            eng._step(group, *unit)

    for _ in range(args.warmup):
        one_step()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for a, b in ev:
        a.record()
        one_step()
        b.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    dev_ms = [a.elapsed_time(b) for a, b in ev]
    avg = sum(dev_ms) / len(dev_ms)
    ms_per_step = wall * 1e3 / args.steps
    achieved = total * 28 / (avg * 1e-3) / 1e9
    out = {
        "metric": "Adam step elements/s + achieved HBM GB/s (% peak) on 7B-layer partition",
        "value": total / (ms_per_step * 1e-3), "unit": "elements/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "resident7b: the whole Llama-7B optimizer of cfg5 (6.74e9 elements, 108 GB) resident in HBM, "
                               "one allocation and one launch per unit (32 layers + embedding/lm_head)",
                   "elements": total, "launches_per_step": len(units), "bytes_per_element": 28},
        "roofline": {"bound": "hbm", "kernel": "adam_tile_kernel", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": None, "algorithmic_bytes_per_step": total * 28,
                     "step_ms_avg": avg, "step_ms_min": min(dev_ms)},
    }
    print(json.dumps(out))
    return 0


def measure_resident(torch, dev, workload, steps, warmup, calibration_copy=False):
    """cfg2 / cfg3 / cfg4 with everything resident in HBM: `warmup` untimed steps, then `steps` timed
    ones with HIP events on the stream the kernels run on (torch's current stream), recorded inside
    the timed region: one in front of every step and one behind it. A workload with a statistics pass
    then runs the same steps once more with a third event between the pass and the update, for the
    two parts, and the pass `steps` times by itself."""
    from flextrain_amd import FlexTrainCPUAdam
    from flextrain_amd.loss_scaler import GradientGuard
    eng = FlexTrainCPUAdam(**HP)
    if workload == "cfg2":
        n, g_dtype, t_step, scale, max_norm = N_7B_LAYER, torch.bfloat16, 100, 1.0, None
        p, g, m, v, h = make_inputs(torch, n, g_dtype, 1e-3, dev)
        name = "cfg2: Llama-7B decoder-layer partition resident in HBM, bf16 grads, AdamW t=100, bf16 copy-out"
        stats_pass = False
    elif workload == "cfg3":
        n, g_dtype, t_step, scale, max_norm = N_7B_LAYER, torch.float16, 100, 65536.0, None
        p, g, m, v, h = make_inputs(torch, n, g_dtype, 1e-3, dev, scale=scale)
        name = "cfg3: 7B-layer partition, fp16 grads x65536, fused overflow check + unscale + AdamW (no overflow)"
        stats_pass = True
    else:
        n, g_dtype, t_step, scale, max_norm = N_70B_LAYER, torch.bfloat16, 1000, 1.0, 1.0
        p, g, m, v, h = make_inputs(torch, n, g_dtype, 5e-3, dev)
        name = "cfg4: Llama-70B-shaped layer partition, bf16 grads, global-norm clip to 1.0 + AdamW t=1000"
        stats_pass = True
    guard = GradientGuard(dev) if stats_pass else None
    group = {"step": t_step}

    def one_step():
        if guard is not None:
            guard.begin()
            ctl = guard.add_and_decide(g, loss_scale=scale, max_grad_norm=max_norm)
            eng._step(group, h, p, g, m, v, control=ctl)
        else:
            eng._step(group, h, p, g, m, v)

    if calibration_copy:
        scratch = torch.empty_like(p)
        for _ in range(3):
            scratch.copy_(p)
        torch.cuda.synchronize()
        del scratch

    for _ in range(warmup):
        one_step()
    torch.cuda.synchronize()

    # The timed region: `steps` steps, one event in front of each and one behind it.
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
          for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        ev[i][0].record()
        one_step()
        ev[i][2].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    whole_ms = [e[0].elapsed_time(e[2]) for e in ev]
    if guard is not None:
        # The two parts of a guarded step, from a second run of the same steps with a third event
        # between the statistics pass and the update (an event between two kernels is a bubble of its
        # own, about 10 us: it stays out of the timed region above).
        for i in range(steps):
            ev[i][0].record()
            guard.begin()
            ctl = guard.add_and_decide(g, loss_scale=scale, max_grad_norm=max_norm)
            ev[i][1].record()
            eng._step(group, h, p, g, m, v, control=ctl)
            ev[i][2].record()
        torch.cuda.synchronize()
        upd_ms = [e[1].elapsed_time(e[2]) for e in ev]
        pre_ms = [e[0].elapsed_time(e[1]) for e in ev]
    else:
        upd_ms, pre_ms = whole_ms, [0.0]
    # The statistics pass by itself: `steps` launches back to back between ONE pair of events. (Inside
    # a step the event between the two kernels and the update that has just finished writing 2.8 GB
    # cost the short pass 5-10 us that are not the kernel's.)
    pre_alone = 0.0
    if guard is not None:
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        first.record()
        for _ in range(steps):
            guard.begin()
            guard.add_and_decide(g, loss_scale=scale, max_grad_norm=max_norm)
        last.record()
        torch.cuda.synchronize()
        pre_alone = first.elapsed_time(last) / steps
    del p, g, m, v, h
    torch.cuda.empty_cache()
    return {"n": n, "name": name, "grad_dtype": str(g_dtype).replace("torch.", ""), "bytes_per_elem": 28,
            "stats_pass": stats_pass, "ms_per_step": wall * 1e3 / steps, "steps": steps, "warmup": warmup,
            "upd_ms": upd_ms, "upd_avg": sum(upd_ms) / len(upd_ms), "pre_avg": sum(pre_ms) / len(pre_ms),
            "pre_alone": pre_alone, "whole_avg": sum(whole_ms) / len(whole_ms)}


def guarded_step_record(r):
    """Compact record of a step with a statistics pass in front (cfg3, cfg4): the whole step between
    one HIP event in front of it and one behind it, its two parts (from a second run with an event
    between them, which costs a bubble of its own: the parts add up to more than the step), and the
    fraction of the HBM peak at the step's 30 algorithmic bytes per element (2 for the statistics
    read, 28 for the update)."""
    n = r["n"]
    whole = r["whole_avg"]
    return {"workload": r["name"], "elements": n, "steps": r["steps"], "warmup": r["warmup"],
            "ms_per_step": whole, "wall_ms_per_step": r["ms_per_step"],
            "update_ms": r["upd_avg"], "update_frac": n * 28 / (r["upd_avg"] * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "stats_ms": r["pre_avg"], "stats_frac": n * 2 / (r["pre_avg"] * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            # the same pass launched back to back, one event pair around all launches
            "stats_alone_ms": r["pre_alone"], "stats_alone_frac": n * 2 / (r["pre_alone"] * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "bytes_per_element": 30, "frac": n * 30 / (whole * 1e-3) / 1e9 / HBM_PEAK_GBPS}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg2", choices=["cfg2", "cfg3", "cfg4", "cfg5", "pipeline", "accumulate", "resident7b", "multi", "ceilings"])
    ap.add_argument("--segments", type=int, default=16, help="multi: ragged contexts the partition is cut into")
    ap.add_argument("--micro-batches", type=int, default=4, help="pipeline: shares per unit")
    ap.add_argument("--windows", default="auto", choices=["auto", "off", "write_through", "copy_back"],
                    help="pipeline: keep a whole unit's state on the GPU while it is stepped (prefetched one unit ahead)")
    ap.add_argument("--chunk-elems", type=int, default=64 * 1024 * 1024, help="cfg5: elements per streamed chunk")
    ap.add_argument("--slots", type=int, default=3, help="cfg5: device buffer sets of the pipeline")
    ap.add_argument("--layers", type=int, default=32, help="cfg5: decoder layers (32 = the full 7B optimizer)")
    ap.add_argument("--alpha", type=float, default=0.0,
                    help="pipeline: share of every unit's step that runs during the next forward pass instead of during "
                         "backward (the reference's split_ratio.alpha)")
    ap.add_argument("--resident-units", type=int, default=0,
                    help="pipeline: units whose fp32 state stays in HBM although the others are streamed from host memory")
    ap.add_argument("--layer-groups", action="store_true",
                    help="pipeline --resident: each layer as its nine tensors in two parameter groups (matrices with weight "
                         "decay, norms without), so that group boundaries cut shares into several step contexts")
    ap.add_argument("--window-piece-mi", type=int, default=0,
                    help="pipeline: elements (in Mi) per piece of a unit window's copies (0 = the library's default)")
    ap.add_argument("--resident-shares", type=int, default=0,
                    help="pipeline --resident: launches a resident unit's update is cut into (0 = the coordinator's default)")
    ap.add_argument("--step-stream", default="auto", choices=["auto", "on", "off"],
                    help="pipeline --resident: updates on the coordinator's own stream beside the caller's kernels")
    ap.add_argument("--backward-tokens", type=int, default=0,
                    help="pipeline --resident: also run, per micro-batch, bf16 matrix products costing a decoder layer's "
                         "backward pass over this many tokens (0 = only the gradient copy)")
    ap.add_argument("--resident", action="store_true",
                    help="pipeline: keep the fp32 state of every unit in HBM instead of pinned host memory")
    ap.add_argument("--stats-keep-mib", type=int, default=None,
                    help="cfg3/cfg4: MiB at the end of the statistics pass read with caching loads (default: the library's 256)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-side-records", action="store_true",
                    help="cfg2: leave out the short side measurements (cfg3_step, cfg4_step, accumulate, multi16; about 5 s)")
    ap.add_argument("--no-offload-record", action="store_true",
                    help="cfg2: leave out the offloaded-streaming sub-record (cfg5 on the largest pinnable prefix, about 12 s)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="before the timed region, run 3 plain device copies of one fp32 array of the workload "
                         "(known size: 4 bytes/element read + 4 written) so that a rocprofv3 --pmc run of this "
                         "command holds a reference dispatch to scale FETCH_SIZE / WRITE_SIZE with")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures the optimizer step of ONE GPU's partition; --gpus must be 1 "
              "(the path shards by giving each GPU its own slice; no multi-GPU figure exists).", file=sys.stderr)
        return 2

    if args.workload == "ceilings":
        return bench_ceilings()

    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 1
    from flextrain_amd import _C
    if not os.path.exists(_C.LIB_PATH):  # nothing built in this tree yet
        from flextrain_amd.build import build_library
        build_library()

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    if args.stats_keep_mib is not None:
        _C.check("ft_set_cache_tuning", _C.lib().ft_set_cache_tuning(args.stats_keep_mib << 20))
    if args.workload == "cfg5":
        return bench_offload(args, torch, dev)
    if args.workload == "pipeline":
        return bench_pipeline(args, torch, dev)
    if args.workload == "accumulate":
        return bench_accumulate(args, torch, dev)
    if args.workload == "resident7b":
        return bench_resident7b(args, torch, dev)
    if args.workload == "multi":
        return bench_multi(args, torch, dev)
    r = measure_resident(torch, dev, args.workload, args.steps, args.warmup, args.calibration_copy)
    n, upd_ms, upd_avg = r["n"], r["upd_ms"], r["upd_avg"]
    alg_bytes = n * r["bytes_per_elem"]
    achieved = alg_bytes / (upd_avg * 1e-3) / 1e9
    out = {
        "metric": "Adam step elements/s + achieved HBM GB/s (% peak) on 7B-layer partition",
        "value": n / (r["ms_per_step"] * 1e-3),
        "unit": "elements/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": r["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": r["name"], "elements": n, "grad_dtype": r["grad_dtype"],
                   "copy_dtype": "bfloat16", "bytes_per_element": r["bytes_per_elem"]},
        "hbm_gbps": achieved,
        "hbm_frac_of_peak": achieved / HBM_PEAK_GBPS,
        "device": _device_description(torch, dev),
        "roofline": {
            "bound": "hbm", "kernel": "adam_tile_kernel", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS, "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
            "traffic_source": TRAFFIC_SOURCE.get(args.workload),
            "algorithmic_bytes_per_launch": alg_bytes, "kernel_ms_avg": upd_avg, "kernel_ms_min": min(upd_ms),
            "kernel_ms_p20_80": percentile_mean(upd_ms),
        },
    }
    if r["stats_pass"]:
        out["stats_pass"] = {"kernel": "grad_stats_kernel", "ms_avg": r["pre_avg"], "bytes": n * 2,
                             "achieved_gbps": n * 2 / (r["pre_avg"] * 1e-3) / 1e9,
                             "alone_ms_avg": r["pre_alone"], "alone_achieved_gbps": n * 2 / (r["pre_alone"] * 1e-3) / 1e9}
        out["guarded_step"] = guarded_step_record(r)
    if args.workload == "cfg2" and not args.no_side_records:
        # Every figure the documents quote, in front of whoever runs this file: the guarded steps of
        # cfg3 and cfg4 (statistics pass + decision + update), the fused accumulation pass and the
        # 16-context launch, each a short run of its own with the same harness as its --workload.
        side_steps, side_warmup = min(args.steps, 20), min(args.warmup, 3)
        for key, workload in (("cfg3_step", "cfg3"), ("cfg4_step", "cfg4")):
            out[key] = guarded_step_record(measure_resident(torch, dev, workload, side_steps, side_warmup))
        acc = measure_accumulate(torch, dev, side_steps, side_warmup)
        out["accumulate"] = {
            "workload": "fp32 accumulator += bf16 gradient on the 7B-layer partition",
            **{key: {"ms": acc[name]["ms_avg"], "bytes_per_element": acc[name]["bytes_per_element"],
                     "frac": acc[name]["achieved_gbps"] / HBM_PEAK_GBPS}
               for key, name in (("plain", "accumulate"), ("with_clear", "accumulate+clear"),
                                 ("with_clear_and_statistics", "accumulate+clear+stats"))}}
        multi, lengths = measure_multi(torch, dev, 16, side_steps, side_warmup)
        out["multi16"] = {"workload": "the cfg2 partition as 16 ragged contexts of two parameter groups",
                          "one_launch_ms": multi["one_launch"]["ms_avg"], "frac": multi["one_launch"]["frac"],
                          "one_call_per_context_ms": multi["per_context"]["ms_avg"], "bytes_per_element": 28,
                          "shortest": min(lengths), "longest": max(lengths)}
    if args.workload == "cfg2" and not args.no_offload_record:
        # The path's second target rides along: the offloaded optimizer streamed over the host link
        # (cfg5 at the largest size this machine pins), 2 warm-ups + 5 steps, beside the link probe.
        try:
            out["offload"], ok = measure_offload(args, torch, dev, args.layers, steps=5, warmup=2)
            if not ok:
                out["offload"]["error"] = "streamed and resident results differ on the probe chunks"
        except Exception as exc:  # the headline figure must not depend on how much this machine can pin
            out["offload"] = {"error": f"{type(exc).__name__}: {exc}"}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(min(n, N_7B_LAYER))
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
