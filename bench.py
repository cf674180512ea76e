#!/usr/bin/env python3
"""Benchmark of the ring KV-cache path on one MI355X.

One step = one chunk through every layer's (RoPE-on-write append + sink/window
attention), inputs already resident in HBM, steady state (cache full, ring
rotating).  Prints ONE JSON line: whole-job tokens/s, per-chunk latency, the
roofline of the dominant kernel (timed live with HIP events on the launch
stream) and the CPU oracle timed on the host cores of the same box.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload 2]
"""
from __future__ import annotations

import argparse
import gc
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E


# HBM bytes per launch, read with rocprofv3's FETCH_SIZE and WRITE_SIZE counters
# (KiB per dispatch) on this same script and scaled by what those counters read
# for the library's plain copy kernel: profiles/hbm_traffic.json, written by
# `bench.py --record-traffic DIR` from the counter runs' CSV files.  A record is
# only used for the kernels it was taken on: same key-range split count, same
# kernel sources (hash below); otherwise `traffic` is null and stderr says why.
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "hbm_traffic.json")
KERNEL_SOURCES = ("swa_attn_fwd.hip", "kv_append_rope.hip", "rope_device.h", "sdv2kv_internal.h")


def kernel_source_hash() -> str:
    import hashlib

    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "streamdiffusionv2_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload_name: str, splits: int):
    """The committed counter record for this workload, or None (with the reason on stderr)."""
    try:
        with open(TRAFFIC_JSON) as f:
            rec = json.load(f)["workloads"].get(workload_name)
    except (OSError, ValueError, KeyError) as e:
        print(f"bench: no usable {TRAFFIC_JSON} ({e}): roofline.traffic is null", file=sys.stderr)
        return None
    if rec is None:
        print(f"bench: {TRAFFIC_JSON} has no record for {workload_name}: roofline.traffic is null", file=sys.stderr)
        return None
    if rec["splits"] != splits or rec["kernel_sources"] != kernel_source_hash():
        print(f"bench: the traffic record for {workload_name} was taken with {rec['splits']} key ranges on kernel "
              f"sources {rec['kernel_sources']}, this run uses {splits} on {kernel_source_hash()}: counters must be "
              "collected again (bench.py --record-traffic); roofline.traffic is null", file=sys.stderr)
        return None
    return rec


def record_traffic(args, w):
    """Turn the CSV files of four rocprofv3 counter runs under DIR (fetch/,
    write/: this script on the workload; cfetch/, cwrite/: --calibrate-copy
    256) into the workload's record in profiles/hbm_traffic.json."""
    import collections
    import csv
    import glob

    def per_kernel(sub):
        files = glob.glob(os.path.join(args.record_traffic, sub, "**", "*counter_collection.csv"), recursive=True)
        if not files:
            raise SystemExit(f"no counter_collection.csv under {args.record_traffic}/{sub}")
        total, count = collections.defaultdict(float), collections.Counter()
        for row in csv.DictReader(open(files[0])):
            for short in ("swa_attn_fwd_kernel", "kv_append_rope_kernel", "copy16_kernel"):
                if short in row["Kernel_Name"]:
                    total[short] += float(row["Counter_Value"])
                    count[short] += 1
        return {k: total[k] / count[k] for k in total}

    fetch, write = per_kernel("fetch"), per_kernel("write")
    cfetch, cwrite = per_kernel("cfetch"), per_kernel("cwrite")
    copy_kib = 256 * 1024
    f_scale, w_scale = copy_kib / cfetch["copy16_kernel"], copy_kib / cwrite["copy16_kernel"]
    from streamdiffusionv2_amd import _capi

    rec = {
        "splits": args.num_splits or _capi.lib().sdv2_swa_attn_default_splits(w.rows, w.chunk_tokens, w.heads, w.cache_tokens),
        "kernel_sources": kernel_source_hash(),
        "fetch_scale": f_scale, "write_scale": w_scale,
        "attn": (fetch["swa_attn_fwd_kernel"] * f_scale + write["swa_attn_fwd_kernel"] * w_scale) * 1024,
        "append": (fetch["kv_append_rope_kernel"] * f_scale + write["kv_append_rope_kernel"] * w_scale) * 1024,
        "attn_fetch_kib": fetch["swa_attn_fwd_kernel"], "attn_write_kib": write["swa_attn_fwd_kernel"],
        "append_fetch_kib": fetch["kv_append_rope_kernel"], "append_write_kib": write["kv_append_rope_kernel"],
    }
    try:
        with open(TRAFFIC_JSON) as f:
            doc = json.load(f)
    except (OSError, ValueError):
        doc = {"unit": "bytes per launch (HBM reads + writes)", "workloads": {}}
    doc["workloads"][w.name] = rec
    with open(TRAFFIC_JSON, "w") as f:
        json.dump(doc, f, indent=1, sort_keys=True)
        f.write("\n")
    print(json.dumps({w.name: rec}))


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", type=int, default=2, help="index into BASELINE.json configs (1-based)")
    ap.add_argument("--num-splits", type=int, default=0)
    ap.add_argument("--skip-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU time budget for the oracle sample")
    ap.add_argument("--cpu-layers", type=int, default=2)
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                    help="only run the library's plain copy kernel on MIB mebibytes (counter calibration)")
    ap.add_argument("--record-traffic", metavar="DIR", default=None,
                    help="no GPU work: read the counter CSVs of rocprofv3 runs under DIR (fetch/, write/, cfetch/, cwrite/) "
                         "and write this workload's record into profiles/hbm_traffic.json")
    ap.add_argument("--fill-phase", action="store_true",
                    help="also time every chunk of a fresh stream while its ring fills (reported apart)")
    ap.add_argument("--qk-norm", action="store_true",
                    help="also time the append with the q/k RMSNorm folded in against torch norms + plain append")
    ap.add_argument("--zero-inputs", action="store_true",
                    help="all-zero q/k/v and caches: nothing toggles, the chip holds its top clock (a diagnostic of "
                         "how much of the distance to the roofline is power, never a result)")
    ap.add_argument("--torch-reference", action="store_true",
                    help="also time the reference's op sequence in stock PyTorch on this GPU (its path without flash_attn)")
    ap.add_argument("--adaptive-sink", action="store_true",
                    help="also time the stream with the adaptive sink refresh on (one-frame chunks, one row)")
    ap.add_argument("--handoff", action="store_true",
                    help="also time the owner change of a layer's cache block (export to / import from the wire layout)")
    ap.add_argument("--launch-floor", action="store_true",
                    help="also time the library's plain copy kernel on 16 bytes (what any launch costs) and on the "
                         "append's byte count (what a pure stream of that size costs): the floor under the append kernel")
    ap.add_argument("--softmax-range", action="store_true",
                    help="also time the attention launch with the queries scaled up until rows leave the range the fast "
                         "softmax covers and waves redo their block with the running-maximum recurrence")
    ap.add_argument("--skip-module-path", action="store_true",
                    help="do not time the path as a module call drives it (fused q / k norm; shipped sink settings)")
    ap.add_argument("--skip-mfma-ceiling", action="store_true",
                    help="do not run the library's own MFMA / LDS / softmax instruction streams (what this box sustains "
                         "on the attention kernel's instruction mix)")
    ap.add_argument("--skip-mfma-reference", action="store_true",
                    help="do not time the vendor bf16 GEMM that shows what this box sustains on MFMA")
    return ap.parse_args()


def build_freqs():
    """The model's RoPE table, built on the CPU in float64 as the reference
    model does at construction (causal_model.py:631-638)."""
    from streamdiffusionv2_amd.rope import build_freqs as _bf

    return _bf()


def gpu_bench(args, w):
    from streamdiffusionv2_amd import _capi, ops, ring, workloads
    from streamdiffusionv2_amd.attention import RingKVPath

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    freqs = build_freqs()
    S, H, B = w.chunk_tokens, w.heads, w.rows
    grid_sizes = torch.tensor([list(w.grid)] * B, dtype=torch.long)
    caches = ring.new_kv_cache(w.layers, 1, w.cache_tokens, H, total_steps=1, dtype=w.dtype, device=dev)
    if B > 1:
        ring.replicate_for_stream_batch(caches, B)
    paths = [RingKVPath(sink_size=w.sink_size, adapt_sink_thr=-1) for _ in range(w.layers)]
    for path in paths:
        path.num_splits = args.num_splits or 0
    # per-layer inputs, resident in HBM before the clock starts
    qkv = []
    for layer in range(w.layers):
        q, k, v = workloads.make_qkv(w, 0, layer)
        qkv.append(tuple(torch.zeros_like(t, device=dev) if args.zero_inputs else t.to(dev) for t in (q, k, v)))
    max_chunk = (1024 - w.grid[0]) // w.grid[0]     # keep the frame index inside the RoPE table
    state = {"call": 0}

    def step(timers=None):
        call = state["call"]
        starts = [min(c, max_chunk) * S for c in workloads.row_chunks(w, call)]
        for layer in range(w.layers):
            q, k, v = qkv[layer]
            if timers is None:
                paths[layer].attend(q, k, v, grid_sizes, freqs, caches[layer], starts)
            else:
                timed_layer(paths[layer], q, k, v, caches[layer], starts, timers)
        state["call"] += 1

    table = ops.device_freqs(freqs, dev)

    def timed_layer(path, q, k, v, cache, starts, timers):
        """Same launches as attend(), each kernel with its own timing events
        (recorded in the kernel's dispatch: the kernel's duration itself)."""
        frame_tokens = w.frame_tokens
        plan = ring.plan_append(cache, path.evict_idx, starts, S, frame_tokens, path.sink_size)
        launcher = path._layer_launcher(q, k, v, cache, table, w.grid)
        launcher.patch(q, k, v, [c // frame_tokens for c in starts], plan, None)
        t = (ops.KernelTimer(), ops.KernelTimer())
        launcher.set_timers(*t)
        launcher.run_append()
        launcher.run_attention()
        launcher.set_timers()
        timers.append(t)

    # Fast-forward to the steady state without launching anything: the host
    # planner walks through the fill phase (so the eviction queues and indices
    # are exactly those of a stream that got here chunk by chunk), the index
    # tensors are set accordingly and the caches are filled with synthetic data.
    # Every launch of the run then has the steady-state shape, which keeps the
    # per-kernel averages of a profiler comparable with the ones timed here.
    fill_calls = w.cache_tokens // S + B
    gen = torch.Generator(device=dev).manual_seed(1)
    for layer in range(w.layers):
        path, cache = paths[layer], caches[layer]
        path.evict_idx = [[] for _ in range(B)]
        for call in range(fill_calls):
            starts = [min(c, max_chunk) * S for c in workloads.row_chunks(w, call)]
            plan = ring.plan_append(cache, path.evict_idx, starts, S, w.frame_tokens, path.sink_size)
            # stand in for the kernel's index stores (keeps the host mirror valid)
            cache["global_end_index"].data.copy_(torch.tensor(plan.new_global_end))
            cache["local_end_index"].data.copy_(torch.tensor(plan.new_local_end))
        for name in ("k", "v"):
            phys = cache[name].permute(0, 2, 1, 3)          # the head-major buffer itself
            if not args.zero_inputs:
                phys.copy_(torch.randn(phys.shape, generator=gen, device=dev, dtype=torch.float32) * w.input_scale)
    state["call"] = fill_calls

    # The timed pass: exactly args.steps steps between two synchronisations.  A pass that an outside stall
    # hit (another process sampling the GPU, an allocator refill: its mean then lies far above the median of
    # its own steps) says nothing about the path; it is reported as discarded and the pass is taken again,
    # at most twice.
    discarded = []
    for attempt in range(3):
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
        # The interpreter's garbage collection stays out of the pass (a collection in the middle of 60 ms
        # would be such a stall) and is run before the warm-up, not after it: the GPU must not sit idle
        # for tens of milliseconds right before the clock starts, or the first steps run at idle clocks.
        gc.collect()
        gc.disable()
        try:
            for _ in range(args.warmup):
                step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(args.steps):
                marks[i].record()
                step()
            marks[args.steps].record()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
        finally:
            gc.enable()
        ms_per_step = (t1 - t0) * 1e3 / args.steps
        per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
        ms_median = per_step[len(per_step) // 2]
        if ms_per_step <= 1.25 * ms_median or args.steps < 4:
            break
        discarded.append({"ms_per_step": ms_per_step, "ms_per_step_median": ms_median, "slowest_step_ms": per_step[-1]})

    # instrumented pass over the same steps: per-kernel durations
    timers = []
    for _ in range(args.steps):
        step(timers)
    torch.cuda.synchronize()
    t_append = sum(t[0].elapsed_ms() for t in timers) / len(timers)
    t_attn = sum(t[1].elapsed_ms() for t in timers) / len(timers)
    for t in timers:
        for x in t:
            if x:
                x.close()
    splits = args.num_splits or _capi.lib().sdv2_swa_attn_default_splits(B, S, H, w.cache_tokens)
    fill_ms = None
    if args.fill_phase:
        # a second, fresh stream from chunk 0: latency of every chunk while the ring fills
        f_caches = ring.new_kv_cache(w.layers, 1, w.cache_tokens, H, total_steps=1, dtype=w.dtype, device=dev)
        f_paths = [RingKVPath(sink_size=w.sink_size, adapt_sink_thr=-1) for _ in range(w.layers)]
        fill_ms = []
        for call in range(fill_calls):
            if call == 1 and B > 1:
                ring.replicate_for_stream_batch(f_caches, B)
            rows = 1 if (call == 0 and B > 1) else B
            starts = [min(c, max_chunk) * S for c in workloads.row_chunks(w, call)][:rows]
            torch.cuda.synchronize()
            c0 = time.perf_counter()
            for layer in range(w.layers):
                q, k, v = qkv[layer]
                f_paths[layer].attend(q[:rows], k[:rows], v[:rows], grid_sizes[:rows], freqs, f_caches[layer], starts)
            torch.cuda.synchronize()
            fill_ms.append((time.perf_counter() - c0) * 1e3)
    return {
        "ms_per_step": ms_per_step,
        "ms_median": ms_median,
        "ms_slowest": per_step[-1],
        "discarded": discarded,
        "fill_ms": fill_ms,
        "append_ms": t_append,
        "attn_ms": t_attn,
        "splits": splits,
    }


def mfma_reference(n=8192, iters=20):
    """What the box sustains on dense bf16 MFMA work: the vendor GEMM behind
    torch.matmul (hipBLASLt / rocBLAS) on n^3 problems, with random operands
    (the realistic case: the chip's clock under MFMA load depends on how much
    the data toggles) and with all-zero operands (the quietest case).  Context
    for the attention kernel's roofline fraction, not part of the timed path."""
    dev = torch.device("cuda:0")
    out = {"n": n, "unit": "TFLOP/s", "source": "torch.matmul bf16 (vendor GEMM)"}
    for kind in ("random", "zeros"):
        if kind == "random":
            a = torch.randn(n, n, device=dev).bfloat16()
            b = torch.randn(n, n, device=dev).bfloat16()
        else:
            a = torch.zeros(n, n, device=dev, dtype=torch.bfloat16)
            b = torch.zeros(n, n, device=dev, dtype=torch.bfloat16)
        for _ in range(3):
            a @ b
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            a @ b
        e1.record()
        torch.cuda.synchronize()
        out[kind] = 2 * n ** 3 / (e0.elapsed_time(e1) / iters) / 1e9
    return out


def mfma_ceiling_section(achieved_tflops):
    """What this box sustains on the attention kernel's own instruction streams
    (the library's sdv2_profile_mfma_stream, random operands, one workgroup per
    CU): the matrix instructions alone; with the LDS fragment reads of the
    kernel's 32-rows-per-wave blocking; with those of a 64-rows-per-wave
    blocking; and with the softmax instructions, tile transfers and per-tile
    barrier of the attention loop.  Context for roofline.frac: the published
    2.5 PFLOP/s is not what a power-limited chip holds on toggling operands."""
    import ctypes as C

    from streamdiffusionv2_amd import _capi

    lib = _capi.lib()
    dev = torch.device("cuda:0")
    nbytes = lib.sdv2_profile_mfma_stream_bytes()
    out = {"unit": "TFLOP/s", "operands": "random bf16, N(0, 0.3)", "workgroups": 256}
    stream = torch.cuda.current_stream(dev).cuda_stream
    flops = C.c_double()
    names = (("mfma_only_registers", _capi.STREAM_REGISTERS), ("lds_reads_32_rows_per_wave", _capi.STREAM_LDS_32_ROWS),
             ("lds_reads_64_rows_per_wave", _capi.STREAM_LDS_64_ROWS), ("attention_loop_mix", _capi.STREAM_ATTENTION_MIX),
             ("attention_loop_mix_64_rows_per_wave", _capi.STREAM_ATTENTION_MIX_64_ROWS))
    for kind in ("random", "zeros"):
        if kind == "random":
            buf = (torch.randn(nbytes // 2, device=dev) * 0.3).bfloat16()
        else:
            buf = torch.zeros(nbytes // 2, device=dev, dtype=torch.bfloat16)
        for name, mode in names:
            if kind == "zeros" and mode not in (_capi.STREAM_REGISTERS, _capi.STREAM_ATTENTION_MIX,
                                                _capi.STREAM_ATTENTION_MIX_64_ROWS):
                continue

            def launch():
                _capi.check(lib.sdv2_profile_mfma_stream(mode, buf.data_ptr(), nbytes, 150, stream, C.byref(flops)),
                            "sdv2_profile_mfma_stream")

            for _ in range(40):             # long enough for the clock to settle under the load
                launch()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(80):
                launch()
            e1.record()
            torch.cuda.synchronize()
            rate = flops.value * 80 / (e0.elapsed_time(e1) * 1e-3) / 1e12
            out[name if kind == "random" else name + "_zeros"] = rate
        del buf
    out["attention_kernel_vs_attention_loop_mix"] = achieved_tflops / out["attention_loop_mix"]
    out["frac_of_peak_attention_loop_mix"] = out["attention_loop_mix"] / PEAK_BF16_TFLOPS
    return out


def module_path_section(args, w, headline_ms):
    """What a model call executes, beside the headline (which times the path on
    q / k that are already normalised, with the sink check off):

    * ``fused_norm``: the path as CausalWanSelfAttention.forward drives it by
      default - raw q / k projections in, their RMSNorm folded into the append
      (causal_model.py:212-218), the query normalised and rotated inside the
      attention kernel;
    * ``shipped_config``: the same with the shipped v2v settings, sink 3 and
      adaptive threshold 0.2 (configs/wan_causal_dmd_v2v.yaml:53-56).  The
      inputs carry a scene direction that changes every eighth chunk, so the
      refresh check keeps the sink frames most of the time and replaces them,
      one per chunk, after a cut;
    * ``module_forward``: whole forward() calls, with the projection GEMMs
      (vendor library; q, k and v as one launch, and as three for comparison)
      around the path.
    Steady state, one chunk per step through every layer."""
    from streamdiffusionv2_amd import ring, workloads
    from streamdiffusionv2_amd.attention import CausalWanSelfAttention, RingKVPath

    dev = torch.device("cuda:0")
    freqs = build_freqs()
    S, H, B = w.chunk_tokens, w.heads, w.rows
    grid = torch.tensor([list(w.grid)] * B, dtype=torch.long)
    max_chunk = (1024 - w.grid[0]) // w.grid[0]
    eps = 1e-6
    gen = torch.Generator(device=dev).manual_seed(9)
    # raw projection outputs: a few times the unit scale, as before a norm
    qkv = [tuple((t.float() * 3.0).to(w.dtype).to(dev) for t in workloads.make_qkv(w, 0, layer)) for layer in range(w.layers)]
    wq = [(torch.rand(H * 128, device=dev, generator=gen) + 0.5).to(w.dtype) for _ in range(w.layers)]
    wk = [(torch.rand(H * 128, device=dev, generator=gen) + 0.5).to(w.dtype) for _ in range(w.layers)]
    fill = w.cache_tokens // S + B + 1
    out = {}

    def run(paths, caches, inputs_for, steps, per_step=None):
        state = {"call": 0}

        def step():
            call = state["call"]
            starts = [min(c, max_chunk) * S for c in workloads.row_chunks(w, call)]
            for layer in range(w.layers):
                q, k, v = inputs_for(call, layer)
                paths[layer].attend(q, k, v, grid, freqs, caches[layer], starts, qk_norm=(wq[layer], wk[layer], eps))
            state["call"] += 1

        for _ in range(fill + args.warmup):
            step()
        torch.cuda.synchronize()
        waits = RingKVPath.decision_waits
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        state["waits"] = RingKVPath.decision_waits - waits
        if per_step is not None:
            # the same stream a little further, every step timed and looked at on its own
            for _ in range(steps):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                step()
                e1.record()
                torch.cuda.synchronize()
                refreshed = sum(1 for p in paths if p.last_refresh and p.last_refresh[0] >= 0)
                per_step.append((e0.elapsed_time(e1), refreshed))
        return ms, state["waits"]

    def fresh(sink, thr):
        caches = ring.new_kv_cache(w.layers, 1, w.cache_tokens, H, total_steps=1, dtype=w.dtype, device=dev)
        if B > 1:
            ring.replicate_for_stream_batch(caches, B)
        return [RingKVPath(sink_size=sink, adapt_sink_thr=thr) for _ in range(w.layers)], caches

    paths, caches = fresh(w.sink_size, -1)
    ms, _ = run(paths, caches, lambda call, layer: qkv[layer], args.steps)
    out["fused_norm"] = {"ms_per_step": ms, "vs_headline": ms / headline_ms,
                         "what": "attend() on raw q / k with the q / k RMSNorm inside the kernels, sink check off"}
    # the two kernels' own durations on this path (timing events in each dispatch), a few more steps of the same stream
    from streamdiffusionv2_amd import ops
    table = ops.device_freqs(freqs, dev)
    timers = []
    call = fill + args.warmup + args.steps
    for _ in range(max(2, args.steps // 4)):
        starts = [min(c, max_chunk) * S for c in workloads.row_chunks(w, call)]
        for layer in range(w.layers):
            q, k, v = qkv[layer]
            norm = (wq[layer], wk[layer], eps)
            plan = ring.plan_append(caches[layer], paths[layer].evict_idx, starts, S, w.frame_tokens, paths[layer].sink_size)
            launcher = paths[layer]._layer_launcher(q, k, v, caches[layer], table, w.grid, norm)
            launcher.patch(q, k, v, [c // w.frame_tokens for c in starts], plan, None)
            t = (ops.KernelTimer(), ops.KernelTimer())
            launcher.set_timers(*t)
            launcher.run_append()
            launcher.run_attention()
            launcher.set_timers()
            timers.append(t)
        call += 1
    torch.cuda.synchronize()
    out["fused_norm"]["kernel_ms_per_layer"] = {
        "append_with_norm": sum(t[0].elapsed_ms() for t in timers) / len(timers),
        "attention_with_q_norm": sum(t[1].elapsed_ms() for t in timers) / len(timers)}
    out["fused_norm"]["append_bytes"] = w.append_bytes(with_q=True) * 5 // 6      # read q, k, v; write k', v
    out["fused_norm"]["append_GBps"] = out["fused_norm"]["append_bytes"] / (
        out["fused_norm"]["kernel_ms_per_layer"]["append_with_norm"] * 1e-3) / 1e9
    for t in timers:
        for x in t:
            x.close()
    del paths, caches

    if S == w.frame_tokens and B == 1:
        # two scenes: a direction common to all tokens of a chunk, added to k and v
        scenes = []
        for s_ in range(2):
            per_layer = []
            for layer in range(w.layers):
                q, k, v = qkv[layer]
                dk = torch.randn(1, 1, H, 128, device=dev, generator=gen) * 3.0 * w.input_scale
                dv = torch.randn(1, 1, H, 128, device=dev, generator=gen) * 3.0 * w.input_scale
                per_layer.append((q, (k.float() + dk).to(w.dtype), (v.float() + dv).to(w.dtype)))
            scenes.append(per_layer)
        period = 8
        paths, caches = fresh(3, 0.2)
        per_step = []
        ms, waits = run(paths, caches, lambda call, layer: scenes[(call // period) % 2][layer], max(args.steps, 2 * period),
                        per_step)
        quiet = [t for t, r in per_step if r == 0]
        busy = [t for t, r in per_step if r > 0]
        out["shipped_config"] = {
            "sink_size": 3, "adapt_sink_thr": 0.2, "ms_per_step": ms, "vs_headline": ms / headline_ms,
            "steps_timed": max(args.steps, 2 * period), "scene_cut_every_chunks": period,
            "steps_with_a_refresh": len(busy), "steps_without": len(quiet),
            "layers_refreshing_in_such_a_step": (sum(r for _, r in per_step if r > 0) / len(busy)) if busy else 0,
            "ms_per_step_refreshing": (sum(busy) / len(busy)) if busy else None,
            "ms_per_step_not_refreshing": (sum(quiet) / len(quiet)) if quiet else None,
            # times the host found a decision not yet written and had to wait for the stream (timed pass)
            "host_waits_for_a_decision": waits,
            "what": "fused norm + adaptive sink refresh (one more launch per layer), scene cut every 8th chunk"}
        del paths, caches, scenes

    # whole module calls: q / k / v / o projections around the path
    dim = H * 128
    layers = min(w.layers, 8)
    mods = [CausalWanSelfAttention(dim, H).to(dev).to(w.dtype) for _ in range(layers)]
    for m in mods:
        m.sink_size = w.sink_size
    caches = ring.new_kv_cache(layers, 1, w.cache_tokens, H, total_steps=1, dtype=w.dtype, device=dev)
    if B > 1:
        ring.replicate_for_stream_batch(caches, B)
    x = (torch.randn(B, S, dim, device=dev, generator=gen)).to(w.dtype)
    state = {"call": 0}

    def module_step():
        starts = torch.tensor([min(c, max_chunk) * S for c in workloads.row_chunks(w, state["call"])])
        for layer in range(layers):
            mods[layer](x, None, grid, freqs, None, kv_cache=caches[layer], current_start=starts)
        state["call"] += 1

    def timed():
        with torch.no_grad():
            for _ in range(fill + args.warmup):
                module_step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                module_step()
            torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / (args.steps * layers)

    per_layer = timed()
    for m in mods:
        m.fuse_qkv_projection = False          # the reference's three launches, for comparison
    per_layer_apart = timed()
    del mods, caches
    # the text cross-attention of the same block (wan_base/modules/model.py:160-196): q projection and its
    # norm, attention against the prompt's cached 512 keys, o projection
    from streamdiffusionv2_amd.attention import WanT2VCrossAttention
    cross = [WanT2VCrossAttention(dim, H).to(dev).to(w.dtype) for _ in range(layers)]
    context = torch.randn(B, 512, dim, device=dev, generator=gen).to(w.dtype)
    text_caches = [{"is_init": False, "k": None, "v": None} for _ in range(layers)]

    def cross_step():
        for layer in range(layers):
            cross[layer](x, context, None, text_caches[layer])

    with torch.no_grad():
        for _ in range(args.warmup + 2):
            cross_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            cross_step()
        torch.cuda.synchronize()
    cross_per_layer = (time.perf_counter() - t0) * 1e3 / (args.steps * layers)
    out["cross_attention_forward"] = {
        "ms_per_layer_call": cross_per_layer, "ms_per_step": cross_per_layer * w.layers, "layers_timed": layers,
        "context_tokens": 512,
        "what": "WanT2VCrossAttention.forward on the cached prompt: q projection (vendor GEMM), q RMSNorm (one launch "
                "of the library), attention, o projection; scaled to the layer count"}
    out["module_forward"] = {"ms_per_layer_call": per_layer, "ms_per_step": per_layer * w.layers, "layers_timed": layers,
                             "ms_per_step_with_three_projection_launches": per_layer_apart * w.layers,
                             "what": "CausalWanSelfAttention.forward with its defaults: q / k / v as one vendor GEMM "
                                     "on the packed weights, the path, the o projection; scaled to the layer count"}
    return out


def qk_norm_section(args, w):
    """Append with the q / k RMSNorm folded in (one kernel) against the same
    work done as the reference does it (two WanRMSNorm modules in torch, then
    the plain append kernel).  Times are per layer call, HIP events around a
    run of calls that rotates over all layers' tensors."""
    from streamdiffusionv2_amd import _capi, ops, ring, workloads
    from streamdiffusionv2_amd.attention import WanRMSNorm

    dev = torch.device("cuda:0")
    S, H, B = w.chunk_tokens, w.heads, w.rows
    layers = min(w.layers, 12)
    caches = ring.new_kv_cache(layers, 1, w.cache_tokens, H, 1, dtype=w.dtype, device=dev)
    if B > 1:
        ring.replicate_for_stream_batch(caches, B)
    table = ops.device_freqs(build_freqs(), dev)
    qkv = [tuple(t.to(dev) for t in workloads.make_qkv(w, 0, layer)) for layer in range(layers)]
    norm_q, norm_k = WanRMSNorm(H * 128, eps=1e-6).to(dev).to(w.dtype), WanRMSNorm(H * 128, eps=1e-6).to(dev).to(w.dtype)
    weights = (norm_q.weight.detach(), norm_k.weight.detach(), 1e-6)
    q_out = torch.empty_like(qkv[0][0])
    starts, dst = [3] * B, [S] * B

    def fused(i):
        q, k, v = qkv[i % layers]
        c = caches[i % layers]
        ops.kv_append_rope(q, k, v, c["k"], c["v"], table, w.grid, starts, dst, q_out=q_out, qk_norm=weights)

    def torch_norm(x, weight):
        # WanRMSNorm.forward as the reference writes it (wan_base/modules/model.py:77-86), in stock torch
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + 1e-6)).type_as(x) * weight

    def unfused(i):
        q, k, v = qkv[i % layers]
        c = caches[i % layers]
        with torch.no_grad():
            qn = torch_norm(q.flatten(2), weights[0]).view_as(q)
            kn = torch_norm(k.flatten(2), weights[1]).view_as(k)
        ops.kv_append_rope(qn, kn, v, c["k"], c["v"], table, w.grid, starts, dst, q_out=q_out)

    def library_norms(i):
        # the norms as modules of their own, each one launch of the library's kernel
        q, k, v = qkv[i % layers]
        c = caches[i % layers]
        with torch.no_grad():
            qn = norm_q(q.flatten(2)).view_as(q)
            kn = norm_k(k.flatten(2)).view_as(k)
        ops.kv_append_rope(qn, kn, v, c["k"], c["v"], table, w.grid, starts, dst, q_out=q_out)

    out = {}
    n = 4 * layers
    for name, fn in (("fused_ms", fused), ("torch_norms_plus_append_ms", unfused),
                     ("library_norm_launches_plus_append_ms", library_norms)):
        for i in range(layers):
            fn(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(n):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        out[name] = e0.elapsed_time(e1) / n
    out["bytes_per_launch"] = w.append_bytes(with_q=True)
    # the fused kernel's own duration (timing events in its dispatch): as the operator returns the rotated
    # query (read q, k, v; write q', k', v), and as the module path runs it (q is only read, for its sum of
    # squares; the attention kernel normalises and rotates the raw q itself)
    inv_rms = torch.empty(B, S, dtype=torch.float32, device=dev)

    def fused_no_q_out(i):
        q, k, v = qkv[i % layers]
        c = caches[i % layers]
        ops.kv_append_rope(q, k, v, c["k"], c["v"], table, w.grid, starts, dst, qk_norm=weights, q_inv_rms=inv_rms)

    timer = ops.KernelTimer()
    for name, fn, moved in (("fused_kernel", fused, w.append_bytes(with_q=True)),
                            ("fused_kernel_no_q_out", fused_no_q_out, w.append_bytes(with_q=True) * 5 // 6)):
        kernel_ms = []
        for i in range(n):
            timer.arm(_capi.KERNEL_APPEND)
            fn(i)
            kernel_ms.append(timer.elapsed_ms())
        out[name + "_ms"] = sum(kernel_ms) / len(kernel_ms)
        out[name + "_bytes"] = moved
        out[name + "_GBps"] = moved / (out[name + "_ms"] * 1e-3) / 1e9
    # the norm as a launch of its own (sdv2_rms_norm): read and write B * S * H * 128 elements
    flat = qkv[0][0].flatten(2)
    norm_bytes = 2 * flat.numel() * flat.element_size()
    kernel_ms = []
    for i in range(n):
        timer.arm(_capi.KERNEL_NORM)
        ops.rms_norm(qkv[i % layers][0].flatten(2), weights[0], 1e-6)
        kernel_ms.append(timer.elapsed_ms())
    out["rms_norm_kernel_ms"] = sum(kernel_ms) / len(kernel_ms)
    out["rms_norm_kernel_bytes"] = norm_bytes
    out["rms_norm_kernel_GBps"] = norm_bytes / (out["rms_norm_kernel_ms"] * 1e-3) / 1e9
    timer.close()
    out["note"] = ("fused_ms / torch_norms_plus_append_ms / library_norm_launches_plus_append_ms are host-inclusive "
                   "per-call times (the torch path launches about a dozen kernels per call); *_kernel_ms are kernels alone")
    # The consumer side (causal_model.py:387-389): the o projection reads the attention output in place.
    # Per layer: attention alone, the vendor GEMM alone, and the two back to back on one stream.
    dim = H * 128
    w_o = (torch.randn(dim, dim, device=dev) * dim ** -0.5).to(w.dtype)
    kc = [c["k"] for c in caches]
    vc = [c["v"] for c in caches]
    for c in caches:
        c["k"].normal_()
        c["v"].normal_()
    attn_out = torch.empty_like(qkv[0][0])

    def attention(i):
        ops.swa_attention(qkv[i % layers][0], kc[i % layers], vc[i % layers], None, out=attn_out)

    def o_proj(i):
        torch.nn.functional.linear(attn_out.flatten(2), w_o)

    def both(i):
        attention(i)
        o_proj(i)

    for name, fn in (("attention_ms", attention), ("o_proj_gemm_ms", o_proj), ("attention_then_o_proj_ms", both)):
        for i in range(layers):
            fn(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(n):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        out[name] = e0.elapsed_time(e1) / n
    return out


def torch_reference_section(args, w, ours_ms_per_step):
    """The reference's op sequence for this path in stock PyTorch on the same
    GPU - what models/wan/causal_model.py executes on a box without flash_attn:
    RoPE of q and k as a complex128 multiply (:94-108), the two slice writes
    into the token-major cache (:321-322), the index fills (:339-342) and
    F.scaled_dot_product_attention on the cache view (:111-137).  Restated here
    with every benefit of the doubt: expanded RoPE factors prepared once (its
    rope cache), no ``.item()`` read-backs, steady-state slot rotation on host
    integers.  A few layers are timed and scaled to the layer count."""
    import torch.nn.functional as F

    dev = torch.device("cuda:0")
    from streamdiffusionv2_amd import workloads

    B, S, H, L = w.rows, w.chunk_tokens, w.heads, w.cache_tokens
    layers = min(w.layers, 4)
    f, h, ww = w.grid
    freqs = build_freqs()
    c = freqs.shape[1]
    parts = freqs.split([c - 2 * (c // 3), c // 3, c // 3], dim=1)
    factors = torch.cat([parts[0][5:5 + f].view(f, 1, 1, -1).expand(f, h, ww, -1),
                         parts[1][:h].view(1, h, 1, -1).expand(f, h, ww, -1),
                         parts[2][:ww].view(1, 1, ww, -1).expand(f, h, ww, -1)], dim=-1).reshape(S, 1, -1).to(dev)
    caches = [{"k": torch.randn(B, L, H, 128, device=dev).bfloat16() * w.input_scale,
               "v": torch.randn(B, L, H, 128, device=dev).bfloat16() * w.input_scale,
               "global_end_index": torch.zeros(B, dtype=torch.long, device=dev),
               "local_end_index": torch.zeros(B, dtype=torch.long, device=dev)} for _ in range(layers)]
    qkv = [tuple(t.to(dev) for t in workloads.make_qkv(w, 0, layer)) for layer in range(layers)]
    slots = (L - S) // S                       # rotating slots behind the first chunk

    def rope(x):
        out = x.clone()
        for i in range(B):
            xi = torch.view_as_complex(x[i].to(torch.float64).reshape(S, H, -1, 2))
            out[i] = torch.view_as_real(xi * factors).flatten(2).type_as(x)
        return out

    def layer_call(layer, call):
        q, k, v = qkv[layer]
        cache = caches[layer]
        rq, rk = rope(q), rope(k)
        end = S + (call % slots + 1) * S
        for i in range(B):
            cache["k"][i, end - S:end] = rk[i]
            cache["v"][i, end - S:end] = v[i]
            cache["global_end_index"][i].fill_(call * S)
            cache["local_end_index"][i].fill_(L)
        x = F.scaled_dot_product_attention(rq.transpose(1, 2), cache["k"].transpose(1, 2), cache["v"].transpose(1, 2),
                                           attn_mask=None, dropout_p=0.0, is_causal=False)
        return x.transpose(1, 2).contiguous()

    for call in range(2):
        for layer in range(layers):
            layer_call(layer, call)
    torch.cuda.synchronize()
    steps = 3
    t0 = time.perf_counter()
    for call in range(2, 2 + steps):
        for layer in range(layers):
            layer_call(layer, call)
    torch.cuda.synchronize()
    per_layer_ms = (time.perf_counter() - t0) * 1e3 / (steps * layers)
    ms_per_step = per_layer_ms * w.layers
    # its attention operator alone, on the same views
    rq = rope(qkv[0][0]).transpose(1, 2)
    kt, vt = caches[0]["k"].transpose(1, 2), caches[0]["v"].transpose(1, 2)
    for _ in range(2):
        F.scaled_dot_product_attention(rq, kt, vt)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        F.scaled_dot_product_attention(rq, kt, vt)
    e1.record()
    torch.cuda.synchronize()
    sdpa_ms = e0.elapsed_time(e1) / 5
    return {"ms_per_step": ms_per_step, "sdpa_ms_per_layer": sdpa_ms,
            "sdpa_TFLOPs": w.attn_flops() / (sdpa_ms * 1e-3) / 1e12, "tokens_per_s": B * S / (ms_per_step * 1e-3), "layers_timed": layers,
            "speedup_of_this_library": ms_per_step / ours_ms_per_step,
            "what": "reference op sequence in stock PyTorch on this GPU (complex128 RoPE, slice writes, SDPA); "
                    f"torch {torch.__version__}"}


def adaptive_sink_section(args, w):
    """Steady-state chunks with the adaptive sink refresh on (sink 3, threshold
    0.2: configs/wan_causal_dmd_v2v.yaml:55-56) against the same stream with it
    off; applies to one-frame chunks only.  Wall-clock per chunk through the
    public attend(), all layers."""
    from streamdiffusionv2_amd import ring, workloads
    from streamdiffusionv2_amd.attention import RingKVPath

    if w.chunk_tokens != w.frame_tokens or w.rows != 1:
        return {"skipped": "the refresh check only runs on one-frame chunks"}
    dev = torch.device("cuda:0")
    freqs = build_freqs()
    S = w.chunk_tokens
    grid = torch.tensor([list(w.grid)], dtype=torch.long)
    qkv = [tuple(t.to(dev) for t in workloads.make_qkv(w, 0, layer)) for layer in range(w.layers)]
    out = {"sink_size": 3}
    fill = w.cache_tokens // S + 2
    for name, thr in (("off_ms_per_step", -1.0), ("on_ms_per_step", 0.2)):
        caches = ring.new_kv_cache(w.layers, 1, w.cache_tokens, w.heads, 1, dtype=w.dtype, device=dev)
        paths = [RingKVPath(sink_size=3, adapt_sink_thr=thr) for _ in range(w.layers)]

        def step(c):
            for layer in range(w.layers):
                q, k, v = qkv[layer]
                paths[layer].attend(q, k, v, grid, freqs, caches[layer], [c * S])

        for c in range(fill):
            step(c)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for c in range(fill, fill + args.steps):
            step(c)
        torch.cuda.synchronize()
        out[name] = (time.perf_counter() - t0) * 1e3 / args.steps
        if thr > -1:
            out["refreshes_in_last_step"] = sum(1 for p in paths if p.last_refresh and p.last_refresh[0] >= 0)
    out["threshold"] = 0.2
    return out


def handoff_section(args, w):
    """Owner change of every layer's block: export (cache -> token-major wire)
    and import (wire -> cache, indices shifted), one launch per tensor with the
    library's timing events in each dispatch.  Bytes per launch = the tensor
    read once and written once."""
    from streamdiffusionv2_amd import handoff, ops, ring

    dev = torch.device("cuda:0")
    layers = min(w.layers, 4)
    caches = ring.new_kv_cache(layers, 1, w.cache_tokens, w.heads, 1, dtype=w.dtype, device=dev)
    if w.rows > 1:
        ring.replicate_for_stream_batch(caches, w.rows)
    for c in caches:
        c["k"].normal_()
        c["v"].normal_()
    wires = [handoff.new_wire_like(c) for c in caches]
    timer = ops.KernelTimer()
    by = 2 * caches[0]["k"].numel() * caches[0]["k"].element_size()
    out = {"bytes_per_launch": by, "layers_sampled": layers}
    for name, pairs in (("export", [(wires[i].k, caches[i]["k"]) for i in range(layers)]),
                        ("import", [(caches[i]["k"], wires[i].k) for i in range(layers)])):
        for d, s_ in pairs:
            ops.cache_relayout(d, s_)
        ms = []
        for _ in range(5):
            for d, s_ in pairs:
                ops.cache_relayout(d, s_, timer=timer)
                ms.append(timer.elapsed_ms())
        avg = sum(ms) / len(ms)
        out[name + "_ms"] = avg
        out[name + "_GBps"] = by / (avg * 1e-3) / 1e9
    out["frac_of_hbm_peak"] = min(out["export_GBps"], out["import_GBps"]) / PEAK_HBM_GBS
    timer.close()
    return out


def launch_floor_section(args, w):
    """Kernel durations (timing events in the dispatch) of the library's plain
    16-byte-vector copy kernel: on 16 bytes - a launch that does nothing - and
    on as many bytes as the append kernel moves for this workload.  The append
    cannot be faster than the first and has no reason to be faster than the
    second; both are quoted beside it."""
    from streamdiffusionv2_amd import _capi, ops

    dev = torch.device("cuda:0")
    out = {}
    timer = ops.KernelTimer()
    lib = _capi.lib()
    moved = w.append_bytes(with_q=False)
    for name, nbytes in (("empty_launch_us", 16), ("copy_of_append_bytes_us", moved // 2 // 16 * 16)):
        src = torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        times = []
        for i in range(60):
            _capi.check(lib.sdv2_profile_time_next(_capi.KERNEL_COPY, timer.start, timer.stop), "time_next")
            ops.copy_bytes(dst, src)
            if i >= 10:
                times.append(timer.elapsed_ms() * 1e3)
        times.sort()
        out[name] = times[len(times) // 2]
    out["append_bytes"] = moved
    out["copy_GBps"] = moved / (out["copy_of_append_bytes_us"] * 1e-6) / 1e9
    timer.close()
    return out


def softmax_range_section(args, w):
    """What leaving the fast softmax's range costs.  The kernel takes exp2 of
    every scaled score against a fixed per-row reference (the largest score
    among the first 32 keys of the workgroup's range); a row whose later scores
    exceed that reference by about 100 in log2 units overflows, and the wave
    that holds it redoes its 32-row block with the running-maximum recurrence
    while the other waves of the workgroup keep the tiles coming.  Here the
    queries are scaled by growing factors (scores of standard deviation
    factor * chunk scale^2 * sqrt(128) in natural units), and then ONE query row
    alone is made extreme."""
    from streamdiffusionv2_amd import ops

    dev = torch.device("cuda:0")
    B, S, H, L = w.rows, w.chunk_tokens, w.heads, w.cache_tokens
    gen = torch.Generator(device=dev).manual_seed(3)
    q = torch.randn(B, S, H, 128, device=dev, generator=gen)
    k = torch.randn(B, H, L, 128, device=dev, generator=gen).bfloat16().permute(0, 2, 1, 3)
    v = torch.randn(B, H, L, 128, device=dev, generator=gen).bfloat16().permute(0, 2, 1, 3)
    out = torch.empty(B, S, H, 128, device=dev, dtype=torch.bfloat16)

    def timed(qq, iters=20):
        qq = qq.bfloat16()
        for _ in range(3):
            ops.swa_attention(qq, k, v, None, out=out)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            ops.swa_attention(qq, k, v, None, out=out)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters

    res = {"score_std_nat_at_factor_1": float((128 ** 0.5) / (128 ** 0.5)), "factors": {}}
    plain = timed(q)
    res["plain_ms"] = plain
    for factor in (4, 16, 32, 64, 128, 256):
        ms = timed(q * factor)
        res["factors"][str(factor)] = {"ms": ms, "ratio_to_plain": ms / plain, "finite": bool(torch.isfinite(out.float()).all())}
    one = q.clone()
    one[0, S // 2, :, :] *= 300.0
    ms = timed(one)
    res["one_extreme_row_of_%d" % S] = {"ms": ms, "ratio_to_plain": ms / plain, "finite": bool(torch.isfinite(out.float()).all())}
    return res


def cpu_baseline(args, w):
    """The CPU oracle (a PyTorch restatement of the reference's op sequence)
    on this box's host cores: a bounded sample of steady-state chunks on a few
    layers, scaled to the full layer count."""
    from oracle import sdv2_oracle as oracle
    from streamdiffusionv2_amd import workloads

    # The reference's CPU path runs on torch's intra-op pool.  A one-GPU box of this pool gives a
    # job a share of 16 host cores whatever os.cpu_count() shows (OMP_NUM_THREADS says so there):
    # the thread count follows that share, and both numbers are reported.
    host_cpus = os.cpu_count() or 1
    share = int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or 16
    threads = max(1, min(host_cpus, share))
    torch.set_num_threads(threads)
    freqs = oracle.build_freqs()
    S, B = w.chunk_tokens, w.rows
    n_layers = min(args.cpu_layers, w.layers)
    caches = oracle.new_kv_cache(n_layers, 1, w.cache_tokens, w.heads, 1, dtype=w.dtype)
    if B > 1:
        oracle.replicate_for_stream_batch(caches, B)
    layers = [oracle.RingAttentionOracle(sink_size=w.sink_size, adapt_sink_thr=-1) for _ in range(n_layers)]
    grids = [list(w.grid)] * B
    qkv = [workloads.make_qkv(w, 0, layer) for layer in range(n_layers)]
    fill_calls = w.cache_tokens // S + B
    call = 0
    for _ in range(fill_calls):
        starts = workloads.row_starts(w, call)
        for layer in range(n_layers):
            q, k, v = qkv[layer]
            layers[layer].step(q, k, v, grids, freqs, caches[layer], starts, with_attention=False)
        call += 1
    t0 = time.perf_counter()
    n_chunks = 0
    while n_chunks < 3 or (time.perf_counter() - t0 < args.cpu_seconds and n_chunks < 400):
        starts = workloads.row_starts(w, call)
        for layer in range(n_layers):
            q, k, v = qkv[layer]
            layers[layer].step(q, k, v, grids, freqs, caches[layer], starts)
        call += 1
        n_chunks += 1
    dt = time.perf_counter() - t0
    per_layer_chunk = dt / (n_chunks * n_layers)
    per_chunk = per_layer_chunk * w.layers
    return {
        "value": B * S / per_chunk,
        "unit": "tokens/s",
        "cores": threads,
        "host_cpu_count": host_cpus,
        "kind": "port",
        "sample": (f"{n_chunks} steady-state chunks x {n_layers} layer(s) of {w.name} "
                   f"({dt:.1f} s), scaled to {w.layers} layers; torch {torch.__version__}"),
        "ms_per_step": per_chunk * 1e3,
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the ring KV-cache path is not sharded across GPUs in this "
              "build (no collectives); run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    from streamdiffusionv2_amd import workloads

    w = workloads.WORKLOADS[args.workload]
    if w.dtype != torch.bfloat16:
        print("workload 1 is the reference's CPU-runnable parity case (fp32 tensors, checked by the GPU tests), "
              "not a bench line; the measured workloads are 2-5", file=sys.stderr)
        sys.exit(2)
    if args.record_traffic:
        record_traffic(args, w)
        return
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the KV-cache path has no CPU fallback)", file=sys.stderr)
        sys.exit(2)
    from streamdiffusionv2_amd import build_ext

    build_ext.ensure_built()       # the library normally comes with the tree; compile only when it is absent
    if args.calibrate_copy:
        from streamdiffusionv2_amd import ops

        n = args.calibrate_copy << 20
        src = torch.empty(n, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(4):
            ops.copy_bytes(dst, src)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_bytes": n, "launches": 4}))
        return

    g = gpu_bench(args, w)
    tokens = w.rows * w.chunk_tokens
    attn_s = g["attn_ms"] * 1e-3
    achieved_tflops = w.attn_flops() / attn_s / 1e12
    # the query is rotated inside the attention kernel: the append moves K and V only
    append_gbs = w.append_bytes(with_q=False) / (g["append_ms"] * 1e-3) / 1e9
    hbm = measured_traffic(w.name, g["splits"])
    result = {
        "metric": "kv_append_attn_tokens_per_s",
        "value": tokens / (g["ms_per_step"] * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": g["ms_per_step"],
        "ms_per_step_median": g["ms_median"],
        "ms_slowest_step": g["ms_slowest"],
        # timed passes thrown away because an outside stall hit them (mean above 1.25 x the pass's own median
        # step); empty in a normal run
        "timed_passes_discarded": g["discarded"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic, all zeros (clock diagnostic, not a result)" if args.zero_inputs else "synthetic",
        "config": {
            "workload": w.name,
            "layers": w.layers, "rows": w.rows, "heads": w.heads, "head_dim": 128,
            "chunk_tokens": w.chunk_tokens, "cache_tokens": w.cache_tokens,
            "grid": list(w.grid), "kv_splits": g["splits"] & 255,
            # of each XCD's share of the (row, head) pairs, how many take one key range more
            "kv_splits_one_more_on_pairs_per_xcd": g["splits"] >> 8,
        },
        "roofline": {
            "kernel": "swa_attn_fwd_kernel",
            "bound": "mfma",
            "achieved": achieved_tflops,
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved_tflops / PEAK_BF16_TFLOPS,
            "traffic": hbm["attn"] if hbm else None,
            "flops_per_launch": w.attn_flops(),
            "avg_launch_ms": g["attn_ms"],
        },
        "roofline_append": {
            "kernel": "kv_append_rope_kernel",
            "bound": "hbm",
            "achieved": append_gbs,
            "peak": PEAK_HBM_GBS,
            "unit": "GB/s",
            "frac": append_gbs / PEAK_HBM_GBS,
            "traffic": hbm["append"] if hbm else None,
            "bytes_per_launch": w.append_bytes(with_q=False),
            "avg_launch_ms": g["append_ms"],
        },
        "kernel_ms_per_layer": {
            "append": g["append_ms"], "attn": g["attn_ms"],
            "note": "from a second pass over the same steps in which every launch carries its own timing events "
                    "(such dispatches run about 1 % longer): their sum can exceed ms_per_step / layers slightly"},
    }
    if g["fill_ms"] is not None:
        result["fill_phase_ms_per_chunk"] = [round(x, 4) for x in g["fill_ms"]]
    if args.qk_norm:
        result["fused_qk_norm"] = qk_norm_section(args, w)
    if args.handoff:
        result["handoff"] = handoff_section(args, w)
    if args.adaptive_sink:
        result["adaptive_sink"] = adaptive_sink_section(args, w)
    if args.launch_floor:
        result["launch_floor"] = launch_floor_section(args, w)
    if args.softmax_range:
        result["softmax_range"] = softmax_range_section(args, w)
    if args.torch_reference:
        result["torch_gpu_reference"] = torch_reference_section(args, w, g["ms_per_step"])
    if not args.skip_module_path and not args.zero_inputs:
        result["module_path"] = module_path_section(args, w, g["ms_per_step"])
    if not args.skip_mfma_ceiling:
        result["mfma_ceiling"] = mfma_ceiling_section(achieved_tflops)
    if not args.skip_mfma_reference:
        ref = mfma_reference()
        ref["attention_vs_random"] = achieved_tflops / ref["random"]
        result["mfma_reference"] = ref
    if not args.skip_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args, w)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
