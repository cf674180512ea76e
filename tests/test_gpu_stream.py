"""Whole-stream GPU parity against the CPU oracle on the five benchmark
shapes: after EVERY chunk the slot written, the end indices and the eviction
queue must be identical (cache contents bit for bit), and the attention output
must stay within max-abs 2e-2 / mean-abs 2e-3 of the fp32 oracle.

Small shapes are compared in full.  At the full benchmark sizes the oracle's
attention is evaluated on a seeded sample of query rows (rows of an attention
are independent, so the sample is exact for those rows) and the cache is
compared in full at the first call, when the ring first wraps and at the end.
"""
import dataclasses

import pytest
import torch

from oracle import sdv2_oracle as oracle
from streamdiffusionv2_amd import workloads

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 2e-2, 2e-3


def _bits(t):
    return t.contiguous().view(torch.int16 if t.dtype == torch.bfloat16 else torch.int32)


def _run(w, gpu_device, layers, calls, sample_rows=None, full_compare_at=None, pool=None, first_layer=0,
         attention_every=1, max_abs=MAX_ABS, mean_abs=MEAN_ABS):
    """`pool` (workloads.InputPool) replaces the per-call random draw for long
    streams; `first_layer` offsets the layer number that selects the inputs;
    with `attention_every` = n the attention output is checked on every n-th
    call and on the last one (the cache state is checked on every call)."""
    from streamdiffusionv2_amd import ring, rope
    from streamdiffusionv2_amd.attention import RingKVPath

    print(f"stream parity: {w.name} layers={first_layer}..{first_layer + layers - 1} calls={calls} "
          f"sample={sample_rows}", flush=True)
    freqs = rope.build_freqs()
    B, S = w.rows, w.chunk_tokens
    g_caches = ring.new_kv_cache(layers, 1, w.cache_tokens, w.heads, 1, dtype=w.dtype, device=gpu_device)
    o_caches = oracle.new_kv_cache(layers, 1, w.cache_tokens, w.heads, 1, dtype=w.dtype)
    g_paths = [RingKVPath(sink_size=w.sink_size) for _ in range(layers)]
    o_paths = [oracle.RingAttentionOracle(sink_size=w.sink_size) for _ in range(layers)]
    grids = [list(w.grid)] * B
    gen = torch.Generator().manual_seed(17)
    worst_max, worst_mean = 0.0, 0.0
    for call in range(calls):
        if call == 1 and B > 1:
            ring.replicate_for_stream_batch(g_caches, B)
            oracle.replicate_for_stream_batch(o_caches, B)
        rows = 1 if (call == 0 and B > 1) else B
        starts = workloads.row_starts(w, call)[:rows]
        for layer in range(layers):
            if pool is None:
                q, k, v = workloads.make_qkv(w, call, first_layer + layer, rows=rows)
            else:
                q, k, v = pool.qkv(call, first_layer + layer, rows=rows)
            got, got_q = g_paths[layer].attend(
                q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), torch.tensor(grids[:rows]), freqs,
                g_caches[layer], starts, return_roped_query=True)
            _, want_q, seq = o_paths[layer].step(q, k, v, grids[:rows], freqs, o_caches[layer], starts,
                                                 with_attention=False)
            torch.cuda.synchronize()
            # integer state
            assert g_paths[layer].evict_idx == o_paths[layer].evict_idx
            assert g_paths[layer].last_plan.new_local_end == seq
            for name in ("global_end_index", "local_end_index"):
                assert g_caches[layer][name].cpu().tolist() == o_caches[layer][name].tolist(), (call, name)
            # roped query and the written slot, bit for bit
            assert torch.equal(_bits(got_q.cpu()), _bits(want_q)), f"roped q differs at call {call}"
            for r, (a, b) in enumerate(o_paths[layer].last_writes):
                for name in ("k", "v"):
                    assert torch.equal(_bits(g_caches[layer][name][r, a:b].cpu()),
                                       _bits(o_caches[layer][name][r, a:b])), (call, layer, r, name)
            if full_compare_at is None or call in full_compare_at:
                for name in ("k", "v"):
                    assert torch.equal(g_caches[layer][name], o_caches[layer][name].to(gpu_device)), (call, name)
            # attention
            if call % attention_every and call != calls - 1:
                continue
            if sample_rows is None:
                idx = torch.arange(S)
            else:
                idx = torch.randperm(S, generator=gen)[:sample_rows].sort().values
            want = oracle.attention_fp32_reference(
                want_q[:, idx], o_caches[layer]["k"], o_caches[layer]["v"], seq)
            err = (got[:, idx.to(gpu_device)].float().cpu() - want).abs()
            assert torch.isfinite(err).all()
            worst_max = max(worst_max, err.max().item())
            worst_mean = max(worst_mean, err.mean().item())
            assert err.max().item() <= max_abs, (call, layer, err.max().item())
            assert err.mean().item() <= mean_abs, (call, layer, err.mean().item())
    print(f"  worst max-abs {worst_max:.3e}, worst mean-abs {worst_mean:.3e}", flush=True)


def _small(w, **kw):
    return dataclasses.replace(w, **kw)


def test_c1_fp32_plumbing(gpu_device):
    # fp32 storage: append and ring state are bit-exact in fp32, and the attention is
    # computed in fp32 throughout, so it is held to fp32 agreement with the fp32 oracle
    _run(workloads.WORKLOADS[1], gpu_device, layers=1, calls=10, max_abs=5e-6, mean_abs=5e-7)


@pytest.mark.parametrize("cfg,grid,layers,calls", [
    (2, (1, 6, 10), 2, 14),
    (3, (3, 4, 6), 2, 12),
    (4, (1, 4, 10), 1, 10),
    (5, (3, 5, 8), 2, 12),
])
def test_scaled_down_streams_full_compare(gpu_device, cfg, grid, layers, calls):
    w = _small(workloads.WORKLOADS[cfg], grid=grid)
    _run(w, gpu_device, layers=layers, calls=calls)


def test_c2_full_size(gpu_device):
    w = workloads.WORKLOADS[2]
    _run(w, gpu_device, layers=2, calls=14, sample_rows=96, full_compare_at={0, 5, 6, 13})


def test_c4_full_size(gpu_device):
    w = workloads.WORKLOADS[4]
    _run(w, gpu_device, layers=1, calls=9, sample_rows=48, full_compare_at={0, 6, 8})


def test_c3_full_size(gpu_device):
    w = workloads.WORKLOADS[3]
    _run(w, gpu_device, layers=1, calls=8, sample_rows=32, full_compare_at={0, 4, 7})


def test_c5_full_size_with_outliers(gpu_device):
    w = workloads.WORKLOADS[5]
    _run(w, gpu_device, layers=1, calls=9, sample_rows=24, full_compare_at={0, 7, 8})


def _wrap_calls(w, calls):
    """Calls at which the ring starts a new round over its rotating slots."""
    slots = w.cache_tokens // w.chunk_tokens
    return {c for c in range(slots, calls + w.rows) if (c - slots) % (slots - 1) == 0}


@pytest.mark.parametrize("first_layer", [0, 10, 20])
def test_c2_stated_length(gpu_device, first_layer):
    """Config 2 as stated: 30 layers (ten per case) x 50 chunks, so the ring
    of five rotating slots goes round nine times.  Cache compared in full at the
    first call, at every wrap and at the end."""
    w = workloads.WORKLOADS[2]
    assert w.layers == 30 and w.chunks == 50
    _run(w, gpu_device, layers=10, calls=w.chunks, sample_rows=8, first_layer=first_layer,
         full_compare_at={0, w.chunks - 1} | _wrap_calls(w, w.chunks), pool=workloads.InputPool(w, seed=first_layer))


@pytest.mark.parametrize("cfg,first_layer", [(4, 0), (4, 1), (3, 0), (3, 1), (5, 0), (5, 1)])
def test_c3_c4_c5_stated_chunk_counts(gpu_device, cfg, first_layer):
    """Configs 3, 4 and 5 over their stated 40 / 30 / 25 chunks, two layers
    each (one per case)."""
    w = workloads.WORKLOADS[cfg]
    _run(w, gpu_device, layers=1, calls=w.chunks, sample_rows=16 if cfg == 4 else 8, first_layer=first_layer,
         full_compare_at={0, w.chunks - 1} | _wrap_calls(w, w.chunks), pool=workloads.InputPool(w, seed=cfg),
         attention_every=1 if cfg == 4 else 5)


def test_kernel_timers_measure_each_kernel(gpu_device):
    """Timing events armed for a kernel are recorded with that kernel alone:
    two positive, plausible durations for the append and the attention of one
    layer call, and the call's result is unchanged by them."""
    from streamdiffusionv2_amd import ops, ring, rope
    from streamdiffusionv2_amd.attention import RingKVPath

    torch.manual_seed(0)
    heads, grid, S, cap = 2, (1, 8, 16), 128, 1024
    freqs = rope.build_freqs()
    table = ops.device_freqs(freqs, gpu_device)
    cache = ring.new_kv_cache(1, 1, cap, heads, 1, device=gpu_device)[0]
    cache["k"].normal_()
    cache["v"].normal_()
    path = RingKVPath(sink_size=1)
    path.num_splits = 2
    q, k, v = (torch.randn(1, S, heads, 128, device=gpu_device).bfloat16() for _ in range(3))
    ref = path.attend(q, k, v, torch.tensor([grid]), freqs, cache, [0]).clone()      # builds the launcher
    path.evict_idx = None
    cache["global_end_index"].zero_()
    cache["local_end_index"].zero_()
    plan = ring.plan_append(cache, [[]], [0], S, 128, 1)
    launcher = path._layer_launcher(q, k, v, cache, table, grid)
    out = launcher.patch(q, k, v, [0], plan, None)
    timers = [ops.KernelTimer() for _ in range(2)]
    launcher.set_timers(*timers)
    launcher.run_append()
    launcher.run_attention()
    launcher.set_timers()
    torch.cuda.synchronize()
    times = [t.elapsed_ms() for t in timers]
    assert all(0.0 < t < 5.0 for t in times), times
    assert torch.equal(out, ref)
    for t in timers:
        t.close()


def test_layer_call_replays_from_a_hip_graph(gpu_device):
    """The library neither allocates nor synchronises, so a layer call (append,
    split attention, merge) can be captured into a HIP graph.  A captured call
    always writes the slot it was planned for, so it is replayed here for that
    slot with fresh inputs in the same static buffers; every replay, with eager
    work and synchronisations in between, must equal the eager result."""
    from streamdiffusionv2_amd import ops, ring, rope

    torch.manual_seed(1)
    heads, grid, S, cap = 2, (1, 8, 16), 128, 1024
    table = ops.device_freqs(rope.build_freqs(), gpu_device)
    cache = ring.new_kv_cache(1, 1, cap, heads, 1, device=gpu_device)[0]
    cache["k"].normal_()
    cache["v"].normal_()
    cache["local_end_index"].fill_(cap)
    cache["global_end_index"].fill_(10 * S)
    base_k, base_v = cache["k"].clone(), cache["v"].clone()
    q, k, v = (torch.zeros(1, S, heads, 128, device=gpu_device, dtype=torch.bfloat16) for _ in range(3))
    plan = ring.AppendPlan([3 * S], [11 * S], [cap])
    launcher = ops.LayerLauncher(cache["k"], cache["v"], cache["global_end_index"], cache["local_end_index"],
                                 table, grid, q)
    launcher.forced_splits = 2
    ops._workspace(gpu_device, 1 << 22)            # grown before the capture, not inside it

    def call():
        return launcher.launch(q, k, v, [10], plan, None)

    call()                                         # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static = call()
    for trial in range(4):
        fresh = [torch.randn(1, S, heads, 128, device=gpu_device).bfloat16() for _ in range(3)]
        for dst, src in zip((q, k, v), fresh):
            dst.copy_(src)
        cache["k"].copy_(base_k)
        cache["v"].copy_(base_v)
        graph.replay()
        torch.cuda.synchronize()
        got, got_k = out_static.clone(), cache["k"].clone()
        # the same call eagerly, from the same starting cache
        cache["k"].copy_(base_k)
        cache["v"].copy_(base_v)
        want = call().clone()
        torch.cuda.synchronize()
        assert torch.equal(got, want), trial
        assert torch.equal(got_k, cache["k"]), trial
        assert cache["global_end_index"].tolist() == [11 * S]
