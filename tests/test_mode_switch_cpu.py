"""The stream driver's switch between stream-batch and sequential denoising
(demo/vid2vid.py:113-198) with the CPU oracle plugged into the generator
stand-in, against a hand trace.

Shape: 4-frame cache, 1 sink frame, two denoising passes (so a 2-row stream
batch and total_steps = 2), one-frame chunks of f = 24 tokens.  Expectations
(units of f) follow the reference statements: both prepare passes write frame
0 (the re-submitted start makes the fill arithmetic idempotent); in sequential
mode the first pass of a chunk reads the queue head without popping
(causal_model.py:310-311) and the second pops and re-appends it (:313-316);
return_to_batch copies row 0 over the batch, copies its queue to every row
and rewinds the pass counter."""
import torch

from flow_helpers import OraclePath
from oracle import sdv2_oracle as oracle
from streamdiffusionv2_amd import stream

H, W, F = 64, 96, 24


def _build():
    gen = stream.SyntheticGenerator(1, 2, "cpu", seed=13, path_factory=OraclePath, sink_size=1, adapt_sink_thr=-1)

    def cache_factory(n, b, cap, h, steps, dtype, device):
        return oracle.new_kv_cache(n, b, cap, h, steps, dtype=dtype, device="cpu")

    pipe = stream.KVStreamPipeline(gen, height=H, width=W, num_kv_cache=4, num_sink_tokens=1,
                                   denoising_step_list=(700, 500, 0), cache_factory=cache_factory)
    pipe._replicate = oracle.replicate_for_stream_batch
    return gen, pipe


def _frames(trace):
    return [([s // F for s in starts], [a // F for a, _ in writes], [n // F for n in lens])
            for starts, writes, lens in trace]


def test_hand_trace_through_both_switches():
    gen, pipe = _build()
    path = gen.paths[0]
    g = torch.Generator().manual_seed(1)
    noise = lambda: torch.randn(1, 1, 16, H // 8, W // 8, generator=g).bfloat16()   # noqa: E731

    pipe.prepare(noise(), 0, F)
    pos = F
    for _ in range(3):
        pipe.inference_stream(noise(), pos, pos + F)
        pos += F
    assert _frames(path.trace) == [
        ([0], [0], [1]), ([0], [0], [1]),                 # prepare: two passes, same slot
        ([1, 1], [1, 1], [2, 2]),                         # registers start at the first chunk's end
        ([2, 1], [2, 1], [3, 2]),
        ([3, 2], [3, 2], [4, 3]),
    ]
    assert [[x // F for x in q] for q in path.evict_idx] == [[2, 3, 4], [2, 3, 4]]

    pipe.enter_wo_batch()
    entry = pipe.kv_cache1[0]
    assert entry["k"].shape[0] == 1 and entry["local_end_index"].tolist() == [4 * F]
    saved_k = pipe._batch_state_refs["kv_cache1"][0]["k"]
    assert entry["k"].data_ptr() == saved_k.data_ptr()    # a view, nothing copied
    del path.trace[:]
    for _ in range(4):
        pipe.inference_wo_batch(noise(), pos, pos + F)
        pos += F
    assert _frames(path.trace) == [
        ([4], [1], [4]), ([4], [1], [4]),                 # pass 1 peeks, pass 2 pops: same slot
        ([5], [2], [4]), ([5], [2], [4]),
        ([6], [3], [4]), ([6], [3], [4]),
        ([7], [1], [4]), ([7], [1], [4]),
    ]
    assert [x // F for x in path.evict_idx[0]] == [3, 4, 2]
    assert entry["current_step"] == 2

    entry["current_step"] = 1                             # as if interrupted between two passes
    pipe.return_to_batch(pos, pos + F)
    entry = pipe.kv_cache1[0]
    assert entry["k"] is saved_k and entry["k"].shape[0] == 2
    assert torch.equal(entry["k"][1], entry["k"][0]) and torch.equal(entry["v"][1], entry["v"][0])
    assert entry["local_end_index"].tolist() == [4 * F] * 2 and entry["global_end_index"].tolist() == [8 * F] * 2
    assert entry["current_step"] == entry["total_steps"] == 2
    assert [[x // F for x in q] for q in path.evict_idx] == [[3, 4, 2], [3, 4, 2]]
    # independent copies per row, as the reference's own test demands (demo/test_online_inference.py:390-404)
    assert path.evict_idx[0] is not path.evict_idx[1]
    assert pipe.kv_cache_starts == [8 * F] * 2 and pipe.kv_cache_ends == [9 * F] * 2
    assert not pipe.hidden_states.any()

    del path.trace[:]
    pipe.inference_stream(noise(), pos, pos + F)
    pipe.inference_stream(noise(), pos + F, pos + 2 * F)
    assert _frames(path.trace) == [
        ([8, 8], [2, 2], [4, 4]),
        ([9, 8], [3, 3], [4, 4]),                         # row 1 re-submits 8 but its queue moved on, as in the reference
    ]
    assert [[x // F for x in q] for q in path.evict_idx] == [[2, 3, 4], [2, 3, 4]]


def test_switches_are_idempotent_and_guarded():
    gen, pipe = _build()
    g = torch.Generator().manual_seed(2)
    pipe.prepare(torch.randn(1, 1, 16, H // 8, W // 8, generator=g).bfloat16(), 0, F)
    pipe.return_to_batch(F, 2 * F)                       # already in batch mode: nothing happens
    assert pipe.active_mode == "batch"
    pipe.enter_wo_batch()
    refs = pipe._batch_state_refs
    pipe.enter_wo_batch()                                 # second call keeps the first snapshot
    assert pipe._batch_state_refs is refs
    pipe._batch_state_refs = None
    try:
        pipe.return_to_batch(F, 2 * F)
    except RuntimeError as e:
        assert "before batch state has been captured" in str(e)
    else:
        raise AssertionError("expected RuntimeError")
