"""Pins for the adaptive sink refresh of the oracle (causal_model.py:284-299):
a hand trace of queue and writes with similarities that have closed forms, the
similarity against a float64 numpy restatement of the definition, and the
one-frame-chunk precondition."""
import numpy as np
import torch

from oracle import sdv2_oracle as oracle

GRID = (1, 2, 2)
FT = 4                      # tokens per frame
H = 1


def _chunk(direction):
    """K = 0 (so its cosine is exactly 0 after any rotation), V = `direction`
    on every token: the averaged similarity is cos(V_sink, V_new) / 2."""
    v = torch.zeros(1, FT, H, 128)
    v[0, :, 0, :len(direction)] = torch.tensor(direction, dtype=torch.float32)
    z = torch.zeros(1, FT, H, 128)
    return z.clone(), z.clone(), v


def test_hand_trace_of_refresh_decisions():
    """cap 5 frames, sink 2, threshold 0.2, one-frame chunks.  Derived by hand
    from the reference statements: the check runs first and may put
    (argmin + 1) * frame at the HEAD of the queue (:297-299); the fill branch
    appends next_end only when it lies beyond the sink (:329-332); an eviction
    takes the head and drops it when it is not beyond the sink (:312-315).
    Units below are frames."""
    e0, e1, e2 = [1, 0, 0], [0, 1, 0], [0, 0, 1]
    r = 2 ** -0.5
    # (V direction, expected sims or None, write slot, queue after the call)
    script = [
        (e0,      [0.0, 0.0],     0, [1]),                          # empty sinks: cos = 0 -> refresh frame 0
        (e1,      [0.0, 0.0],     1, [1, 1, 3]),
        (e0,      [0.5, 0.0],     2, [2, 1, 1, 3, 4]),              # frame 1 (e1) is the dissimilar one
        ([r, r],  [r / 2, r / 2], 3, [2, 1, 1, 3, 4, 5]),           # 0.354 >= 0.2: no refresh
        (e1,      [0.0, 0.5],     4, [1, 2, 1, 1, 3, 4, 5]),
        (e2,      [0.0, 0.0],     0, [1, 2, 1, 1, 3, 4, 5]),        # full: head (1) taken -> sink frame 0 rewritten, entry dropped
        (e2,      [0.5, 0.0],     1, [1, 2, 1, 1, 3, 4, 5]),        # frame 0 now holds e2; frame 1 rewritten
        (e2,      [0.5, 0.5],     0, [2, 1, 1, 3, 4, 5]),           # no refresh; head (1) still queued from the fill phase
    ]
    freqs = oracle.build_freqs()
    cache = oracle.new_kv_cache(1, 1, 5 * FT, H, 1, dtype=torch.float32)[0]
    layer = oracle.RingAttentionOracle(sink_size=2, adapt_sink_thr=0.2)
    for c, (direction, sims, slot, queue) in enumerate(script):
        q, k, v = _chunk(direction)
        layer.step(q, k, v, [GRID], freqs, cache, [c * FT], with_attention=False)
        assert torch.allclose(layer.last_sims[0], torch.tensor(sims, dtype=torch.float32), atol=1e-6), c
        assert layer.last_writes[0] == (slot * FT, (slot + 1) * FT), c
        assert [x // FT for x in layer.evict_idx[0]] == queue, c
        assert torch.equal(cache["v"][0, slot * FT:(slot + 1) * FT], v[0]), c


def test_similarity_matches_float64_definition():
    torch.manual_seed(5)
    sink, heads = 3, 2
    freqs = oracle.build_freqs()
    cache = oracle.new_kv_cache(1, 1, 6 * FT, heads, 1, dtype=torch.float32)[0]
    cache["k"].normal_()
    cache["v"].normal_()
    k_before, v_before = cache["k"].clone(), cache["v"].clone()
    q, k, v = (torch.randn(1, FT, heads, 128) for _ in range(3))
    layer = oracle.RingAttentionOracle(sink_size=sink, adapt_sink_thr=2.0)
    layer.step(q, k, v, [GRID], freqs, cache, [7 * FT], with_attention=False)
    roped = oracle.causal_rope_apply(k, [GRID], freqs, [7]).double().numpy()

    def cos(a, b):
        return float(a @ b / (np.linalg.norm(a) * np.linalg.norm(b)))

    want = []
    for j in range(sink):
        ks = k_before[0, j * FT:(j + 1) * FT].double().numpy().reshape(FT, -1).mean(0)
        vs = v_before[0, j * FT:(j + 1) * FT].double().numpy().reshape(FT, -1).mean(0)
        kn = roped[0].reshape(FT, -1).mean(0)
        vn = v[0].double().numpy().reshape(FT, -1).mean(0)
        want.append((cos(ks, kn) + cos(vs, vn)) / 2)
    assert np.allclose(layer.last_sims[0].numpy(), want, atol=1e-5)
    # threshold 2.0 always refreshes the least similar frame; the chunk lies
    # beyond the cache, so the eviction of this same call consumes the entry
    worst = int(np.argmin(want))
    assert layer.last_writes[0] == (worst * FT, (worst + 1) * FT)
    assert layer.evict_idx[0] == []


def test_check_is_skipped_for_multi_frame_chunks_and_when_off():
    freqs = oracle.build_freqs()
    for thr, frames in ((-1, 1), (0.2, 2)):
        cache = oracle.new_kv_cache(1, 1, 6 * FT, H, 1, dtype=torch.float32)[0]
        layer = oracle.RingAttentionOracle(sink_size=2, adapt_sink_thr=thr)
        x = torch.randn(1, frames * FT, H, 128)
        layer.step(x, x, x, [(frames, 2, 2)], freqs, cache, [0], with_attention=False)
        assert layer.last_sims == []
