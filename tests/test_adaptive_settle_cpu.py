"""Host side of the adaptive sink refresh when the decision is made on the
device: ``RingKVPath.attend`` plans a call as if no row refreshed, the
decision kernel moves the write of an evicting row by itself, and the host
corrects its queue when the state is next needed.

Checked here on the CPU, with the three GPU entry points of ``attend``
replaced by stand-ins that follow a scripted list of decisions: after every
call the slot the device would write and, whenever the test looks, the
eviction queues must equal those of the reference order of operations - insert
(frame + 1) * frame_tokens at the head of the queue FIRST, then place the chunk
(causal_model.py:297-299 before :302-337) - run on a second cache dict with the
same ``ring.plan_append``.  Covers the fill phase (a refresh there stays at the
head of the queue until the first eviction), steady state, several rows, and
the pass counter of the sequential mode (several calls per chunk on a one-row
cache).
"""
import random

import pytest
import torch

from streamdiffusionv2_amd import attention, ring

FT = 6            # tokens per frame
GRID = (1, 2, 3)


class _Stream:
    def synchronize(self):
        pass


class _Launcher:
    """Stands in for ops.LayerLauncher: records where the append would write."""

    def __init__(self):
        self.writes = []
        self.roped_q = torch.zeros(1)

    def launch(self, q, k, v, start_frames, plan, seq, mask_tokens, override):
        dst = list(plan.dst_start)
        if override is not None:
            for i, o in enumerate(override.tolist()[:len(dst)]):
                if o >= 0:
                    dst[i] = o
        self.writes.append(dst)
        return torch.zeros_like(q)


def _cpu_cache(rows, cap_frames, total_steps):
    return {"k": torch.zeros(rows, cap_frames * FT, 1, 128), "v": torch.zeros(rows, cap_frames * FT, 1, 128),
            "global_end_index": torch.zeros(rows, dtype=torch.long),
            "local_end_index": torch.zeros(rows, dtype=torch.long),
            "total_steps": total_steps, "current_step": total_steps}


def _patched_path(monkeypatch, script, sink):
    """A RingKVPath whose device calls are stand-ins; script[n][i] is the
    decision for row i in the n-th call that runs the check."""
    path = attention.RingKVPath(sink_size=sink, adapt_sink_thr=0.2)
    launcher = _Launcher()
    calls = {"n": 0}

    def fake_similarity(k, v, k_cache, v_cache, table, grid_hw, start_frames, sink_frames, threshold,
                        dst_start_override=None, override_rows=(), refresh_out=None, **kept):
        decisions = script[calls["n"]]
        calls["n"] += 1
        rows = k.shape[0]
        refresh = refresh_out if refresh_out is not None else torch.empty(rows, dtype=torch.int32)
        for i in range(rows):
            refresh[i] = decisions[i]
            if dst_start_override is not None:      # what the deciding workgroup of sink_similarity_kernel stores
                dst_start_override[i] = decisions[i] * k.shape[1] if decisions[i] >= 0 and override_rows[i] else -1
        return None, refresh

    monkeypatch.setattr(attention.ops, "device_freqs", lambda freqs, dev: None)
    monkeypatch.setattr(attention.ops, "sink_similarity", fake_similarity)
    monkeypatch.setattr(path, "_layer_launcher", lambda *a, **kw: launcher)
    monkeypatch.setattr(attention.torch.cuda, "current_stream", lambda dev=None: _Stream())
    monkeypatch.setattr(path, "_kept_sink_sums", lambda kv_cache, rows, heads: None)
    monkeypatch.setattr(path, "_decision_buffers",
                        lambda rows, dev: (torch.full((rows,), -1, dtype=torch.int64),
                                           torch.empty(rows, dtype=torch.int32)))
    return path, launcher


def _reference_order(cache, queues, decisions, starts, sink):
    """Insert first, then place: the order the reference works in."""
    for i, frame in enumerate(decisions):
        if frame >= 0:
            queues[i].insert(0, (frame + 1) * FT)
    return ring.plan_append(cache, queues, starts, FT, FT, sink)


@pytest.mark.parametrize("look_every_call", [True, False])
@pytest.mark.parametrize("seed", range(6))
def test_lazy_settle_matches_the_reference_order(monkeypatch, seed, look_every_call):
    rng = random.Random(seed)
    rows = rng.choice([1, 1, 2, 3])
    sink = rng.choice([1, 2, 3])
    cap_frames = sink + rng.choice([2, 3, 4])
    passes = rng.choice([1, 2, 3]) if rows == 1 else 1          # the pass counter only acts on one-row caches
    chunks = cap_frames + 7
    script = [[rng.choice([-1, -1, rng.randrange(sink)]) for _ in range(rows)] for _ in range(chunks * passes)]

    path, launcher = _patched_path(monkeypatch, script, sink)
    cache = _cpu_cache(rows, cap_frames, passes)
    want_cache = _cpu_cache(rows, cap_frames, passes)
    want_queues = [[] for _ in range(rows)]
    x = torch.zeros(rows, FT, 1, 128, dtype=torch.bfloat16)
    n = 0
    for chunk in range(chunks):
        starts = [max(chunk - r, 0) * FT for r in range(rows)]
        for _ in range(passes):
            want = _reference_order(want_cache, want_queues, script[n], starts, sink)
            path.attend(x, x, x, torch.tensor([GRID] * rows), None, cache, starts)
            n += 1
            assert launcher.writes[-1] == want.dst_start, (chunk, script[n - 1])
            if look_every_call or rng.random() < 0.15:
                assert path.last_refresh == script[n - 1]
                assert path.evict_idx == want_queues
                assert path.last_plan.dst_start == want.dst_start
                assert path.last_plan.new_local_end == want.new_local_end
            assert cache["current_step"] == want_cache["current_step"]
    assert path.evict_idx == want_queues
    assert any(f >= 0 for row in script for f in row)


def test_full_cache_with_an_empty_queue_decides_at_once(monkeypatch):
    """Every frame of the cache is sink: an eviction is only possible through a
    refresh, so the decision is needed before the call can be planned; without
    one the reference's IndexError surfaces (causal_model.py:306)."""
    script = [[-1], [-1], [1], [-1]]
    path, launcher = _patched_path(monkeypatch, script, sink=2)
    cache = _cpu_cache(1, 2, 1)
    x = torch.zeros(1, FT, 1, 128, dtype=torch.bfloat16)
    grid = torch.tensor([GRID])
    path.attend(x, x, x, grid, None, cache, [0])
    path.attend(x, x, x, grid, None, cache, [FT])
    assert path.evict_idx == [[]]
    path.attend(x, x, x, grid, None, cache, [2 * FT])          # refreshes sink frame 1
    assert launcher.writes[-1] == [FT] and path.last_refresh == [1] and path.evict_idx == [[]]
    with pytest.raises(IndexError):
        path.attend(x, x, x, grid, None, cache, [3 * FT])


def test_settle_is_public_and_idempotent(monkeypatch):
    script = [[-1]] * 3 + [[0]] + [[-1]] * 3
    path, launcher = _patched_path(monkeypatch, script, sink=1)
    cache = _cpu_cache(1, 3, 1)
    x = torch.zeros(1, FT, 1, 128, dtype=torch.bfloat16)
    for c in range(4):
        path.attend(x, x, x, torch.tensor([GRID]), None, cache, [c * FT])
    assert path._pending is not None
    path.settle()
    assert path._pending is None
    queue = [list(q) for q in path.evict_idx]
    path.settle()
    assert path.evict_idx == queue
    # the refreshed sink frame took the write; the rotation slot stays at the head for the next call
    assert launcher.writes[-1] == [0] and queue == [[2 * FT, 3 * FT]]
