"""Pins for the ring placement state machine: hand traces (tests/golden),
the closed-form slot schedule on a sweep of cache sizes, structural
invariants, the multi-pass (no-batch) overwrite and the error path; then the
host planner of the shipped package is held to the oracle on random streams.
"""
import json
import os
import random

import pytest
import torch

from oracle import sdv2_oracle as oracle
from streamdiffusionv2_amd import ring

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "ring_traces.json")
FT = 6          # tokens per latent frame in these tests: grid (f, 2, 3)
H = 1


def _tiny_inputs(rows, n_tok, tag):
    # V rows carry (tag, token) so cache contents identify the chunk
    v = torch.zeros(rows, n_tok, H, 128)
    for r in range(rows):
        v[r, :, 0, 0] = tag[r]
        v[r, :, 0, 1] = torch.arange(n_tok)
    k = torch.randn(rows, n_tok, H, 128)
    q = torch.randn(rows, n_tok, H, 128)
    return q, k, v


def _run_oracle_stream(cache_frames, sink, frames_seq, total_steps=1, passes=1):
    """Feed chunks of frames_seq[i] frames; returns per-call records."""
    freqs = oracle.build_freqs()
    cache = oracle.new_kv_cache(1, 1, cache_frames * FT, H, total_steps, dtype=torch.float32)[0]
    layer = oracle.RingAttentionOracle(sink_size=sink, adapt_sink_thr=-1)
    rec, start = [], 0
    for c, fr in enumerate(frames_seq):
        q, k, v = _tiny_inputs(1, fr * FT, [c])
        for _ in range(passes):
            layer.step(q, k, v, [(fr, 2, 3)], freqs, cache, [start], with_attention=False)
            rec.append({
                "chunk": c,
                "write": layer.last_writes[0],
                "evict_idx": list(layer.evict_idx[0]),
                "local_end": int(cache["local_end_index"][0]),
                "global_end": int(cache["global_end_index"][0]),
                "owner": cache["v"][0, :, 0, 0].clone(),
                "current_step": cache["current_step"],
            })
        start += fr * FT
    return rec


@pytest.mark.parametrize("trace", json.load(open(GOLDEN))["traces"], ids=lambda t: t["name"])
def test_hand_traces(trace):
    n = len(trace["steps"])
    frames = [trace["first_chunk_frames"]] + [trace["chunk_frames"]] * (n - 1)
    rec = _run_oracle_stream(trace["cache_frames"], trace["sink_size"], frames)
    for got, want in zip(rec, trace["steps"]):
        assert [x // FT for x in got["write"]] == want["write"]
        assert [x // FT for x in got["evict_idx"]] == want["evict_idx"]
        assert got["local_end"] // FT == want["local_end"]


@pytest.mark.parametrize("cache_frames", range(2, 9))
@pytest.mark.parametrize("sink", range(0, 4))
@pytest.mark.parametrize("chunk_frames", [1, 2])
def test_closed_form_slot_schedule(cache_frames, sink, chunk_frames):
    if cache_frames % chunk_frames:
        pytest.skip("chunk must divide the cache for the closed form")
    n_slots = cache_frames // chunk_frames
    permanent = max(1, sink // chunk_frames)
    n_chunks = 3 * n_slots + 2
    if permanent >= n_slots:
        # nothing is evictable: the reference hits an empty queue once the cache is full
        with pytest.raises(IndexError):
            _run_oracle_stream(cache_frames, sink, [chunk_frames] * n_chunks)
        return
    rec = _run_oracle_stream(cache_frames, sink, [chunk_frames] * n_chunks)
    S = chunk_frames * FT
    cap = cache_frames * FT
    resident = {}
    for c, r in enumerate(rec):
        slot = ring.closed_form_slot(c, n_slots, permanent)
        assert r["write"] == (slot * S, (slot + 1) * S)
        resident[slot] = c
        # invariants
        assert r["global_end"] == (c + 1) * S
        assert r["local_end"] == min((c + 1) * S, cap)
        assert r["local_end"] <= cap
        # cache contents: every slot holds exactly the chunk last written there
        for s, owner in resident.items():
            assert torch.all(r["owner"][s * S:(s + 1) * S] == owner)
        # slot 0 (the first chunk) is never overwritten
        assert torch.all(r["owner"][:S] == 0)
    # the eviction queue is always a rotation of the fill-phase list
    fill = rec[n_slots - 1]["evict_idx"]
    for r in rec[n_slots:]:
        e = r["evict_idx"]
        assert sorted(e) == sorted(fill)
        i = fill.index(e[0])
        assert e == fill[i:] + fill[:i]


def test_v_is_stored_verbatim_and_k_is_rotated():
    freqs = oracle.build_freqs()
    cache = oracle.new_kv_cache(1, 1, 4 * FT, H, 1, dtype=torch.bfloat16)[0]
    layer = oracle.RingAttentionOracle(sink_size=1)
    q, k, v = (t.bfloat16() for t in _tiny_inputs(1, FT, [3]))
    v = torch.randn_like(v.float()).bfloat16()
    layer.step(q, k, v, [(1, 2, 3)], freqs, cache, [0], with_attention=False)
    assert torch.equal(cache["v"][0, :FT].view(torch.int16), v[0].view(torch.int16))
    want_k = oracle.causal_rope_apply(k, [(1, 2, 3)], freqs, [0])
    assert torch.equal(cache["k"][0, :FT].view(torch.int16), want_k[0].view(torch.int16))
    assert not cache["k"][0, FT:].any() and not cache["v"][0, FT:].any()


def test_resubmission_is_idempotent_while_filling():
    # prepare() runs the first chunk num_steps times with the same current_start
    rec = _run_oracle_stream(4, 1, [1, 1], total_steps=3, passes=3)
    assert [r["write"] for r in rec[:3]] == [(0, FT)] * 3
    assert [r["evict_idx"] for r in rec[:3]] == [[2 * FT]] * 3
    assert [r["local_end"] for r in rec[3:]] == [2 * FT] * 3


def test_multi_pass_overwrite_rotates_once_per_chunk():
    # batch-1 cache, 3 denoising passes per chunk (inference_wo_batch): the
    # python counter current_step lets one pass per chunk rotate the queue
    # (causal_model.py:310-316)
    rec = _run_oracle_stream(3, 1, [1] * 6, total_steps=3, passes=3)
    full = [r for r in rec if r["local_end"] == 3 * FT]
    rotations = sum(1 for a, b in zip(full, full[1:]) if a["evict_idx"] != b["evict_idx"])
    chunks_after_full = len({r["chunk"] for r in full})
    assert rotations in (chunks_after_full - 1, chunks_after_full)
    for r in full:
        assert 1 <= r["current_step"] <= 3
        assert sorted(r["evict_idx"]) == [2 * FT, 3 * FT]


def test_empty_queue_raises_index_error():
    # cache of one slot: full after the first chunk, nothing evictable
    with pytest.raises(IndexError):
        _run_oracle_stream(1, 0, [1, 1])


def test_new_kv_cache_contract():
    cache = oracle.new_kv_cache(2, 1, 24, 3, 4)
    assert len(cache) == 2
    for c in cache:
        assert set(c) == {"k", "v", "global_end_index", "local_end_index", "total_steps", "current_step"}
        assert c["k"].shape == (1, 24, 3, 128) and c["k"].dtype == torch.bfloat16
        assert c["global_end_index"].dtype == torch.long and c["global_end_index"].tolist() == [0]
        assert c["total_steps"] == 4 and c["current_step"] == 4
    oracle.replicate_for_stream_batch(cache, 3)
    assert cache[0]["k"].shape[0] == 3 and cache[0]["local_end_index"].shape == (3,)


# ---------------------------------------------------------------------------
# host planner of the package == oracle state machine
# ---------------------------------------------------------------------------

def _cpu_cache_for_planner(rows, cap, total_steps):
    c = ring.new_kv_cache(1, 1, cap, H, total_steps, dtype=torch.float32, device="cpu")[0]
    if rows > 1:
        lst = [c]
        ring.replicate_for_stream_batch(lst, rows)
    return c


@pytest.mark.parametrize("seed", range(6))
def test_host_planner_matches_oracle_on_random_streams(seed):
    rng = random.Random(seed)
    rows = rng.choice([1, 1, 2, 4])
    chunk_frames = rng.choice([1, 1, 2, 3])
    slots = rng.choice([2, 3, 4, 6])
    cap = slots * chunk_frames * FT
    sink = rng.choice([0, 1, chunk_frames, chunk_frames + 1])
    total_steps = rng.choice([1, 3]) if rows == 1 else 1
    S = chunk_frames * FT
    if max(1, sink // chunk_frames) >= slots:
        sink = 0
    freqs = oracle.build_freqs()

    o_cache = oracle.new_kv_cache(1, 1, cap, H, total_steps, dtype=torch.float32)[0]
    if rows > 1:
        lst = [o_cache]
        oracle.replicate_for_stream_batch(lst, rows)
    o_layer = oracle.RingAttentionOracle(sink_size=sink)
    h_cache = _cpu_cache_for_planner(rows, cap, total_steps)
    evict = [[] for _ in range(rows)]

    for call in range(4 * slots):
        chunks = [0] * rows if call == 0 else [max(call - j, 1) for j in range(rows)]
        starts = [c * S for c in chunks]
        for _ in range(total_steps):
            q, k, v = _tiny_inputs(rows, S, chunks)
            _, _, seq = o_layer.step(q, k, v, [(chunk_frames, 2, 3)] * rows, freqs, o_cache, starts,
                                     with_attention=False)
            plan = ring.plan_append(h_cache, evict, starts, S, FT, sink)
            # the kernel would store these; emulate it without touching _version
            h_cache["global_end_index"].data.copy_(torch.tensor(plan.new_global_end))
            h_cache["local_end_index"].data.copy_(torch.tensor(plan.new_local_end))
            assert plan.dst_start == [w[0] for w in o_layer.last_writes]
            assert plan.new_local_end == seq
            assert plan.new_global_end == o_cache["global_end_index"].tolist()
            assert evict == o_layer.evict_idx
            assert h_cache["current_step"] == o_cache["current_step"]


def test_host_planner_resyncs_when_indices_are_touched_from_outside():
    cache = _cpu_cache_for_planner(1, 4 * FT, 1)
    evict = [[]]
    plan = ring.plan_append(cache, evict, [0], FT, FT, 1)
    assert plan.dst_start == [0] and plan.new_local_end == [FT]
    # an external owner rewrites the device indices in place (e.g. after moving
    # the cache between pipeline stages): the mirror must notice
    cache["global_end_index"].fill_(3 * FT)
    cache["local_end_index"].fill_(3 * FT)
    plan = ring.plan_append(cache, evict, [3 * FT], FT, FT, 1)
    assert plan.dst_start == [3 * FT] and plan.new_local_end == [4 * FT]
    # replacing the tensors (slicing the batch) also invalidates the mirror
    cache["local_end_index"] = cache["local_end_index"][:1]
    cache["global_end_index"] = torch.tensor([0])
    cache["local_end_index"] = torch.tensor([0])
    plan = ring.plan_append(cache, [[]], [0], FT, FT, 1)
    assert plan.dst_start == [0]


def test_host_planner_error_paths():
    cache = _cpu_cache_for_planner(1, FT, 1)
    evict = [[]]
    ring.plan_append(cache, evict, [0], FT, FT, 0)
    cache["global_end_index"].data.fill_(FT)
    cache["local_end_index"].data.fill_(FT)
    with pytest.raises(IndexError):
        ring.plan_append(cache, evict, [FT], FT, FT, 0)
    with pytest.raises(ValueError):
        ring.plan_append(_cpu_cache_for_planner(1, 2 * FT, 1), [[]], [0, 0], FT, FT, 0)
