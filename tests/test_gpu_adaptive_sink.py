"""GPU parity of the adaptive sink refresh (causal_model.py:284-299) against
the CPU oracle: the similarity operator on its own (both dtypes, both cache
layouts) and whole streams with the refresh switched on, where every decision,
every slot and the cache contents must be identical.

The decision compares an averaged cosine similarity with a threshold.  Means
are fp32 sums in a different order on the two sides and are then rounded to
bf16, so similarities agree to about one bf16 step (tolerance 1e-2 for bf16,
1e-5 for fp32).  The streams use inputs with a strong per-chunk direction so
that every decision of the oracle has a margin of at least 0.03 to the
threshold and to the runner-up frame (asserted), which makes the decisions
comparable exactly.
"""
import pytest
import torch

from oracle import sdv2_oracle as oracle

GRID = (1, 6, 8)
FT = 48
THR = 0.2
MARGIN = 0.03


def directed_chunk(gen, rows, heads, dtype, basis, scene=None, scale=0.25, ft=FT):
    """q, k, v [rows, ft, heads, 128]: noise plus a chunk-wide direction from
    the span of `basis` (the same on every token, so it survives the frame
    mean; RoPE averages part of k's away).  With `scene` (coefficients [3]) the
    direction stays near that scene's, so consecutive chunks look alike until
    the scene changes."""
    shape = (rows, ft, heads, 128)
    q = torch.randn(shape, generator=gen) * scale
    k = torch.randn(shape, generator=gen) * scale
    v = torch.randn(shape, generator=gen) * scale
    for r in range(rows):
        cv = torch.randn(basis.shape[0], generator=gen)
        ck = torch.randn(basis.shape[0], generator=gen)
        if scene is not None:
            cv, ck = 2 * scene + 0.3 * cv, 2 * scene + 0.3 * ck
        v[r] += (cv @ basis).reshape(1, heads, 128)
        k[r] += (ck @ basis).reshape(1, heads, 128)
    return q.to(dtype), k.to(dtype), v.to(dtype)


def oracle_margins_ok(sims):
    """Every decision is clear of the threshold and has a clear minimum.
    Frames never written give exactly 0 on both sides, so a tie at 0 is exact
    and resolves to the first such frame everywhere."""
    for s in sims:
        s = s.float().sort().values
        if abs(s[0].item() - THR) < MARGIN:
            return False
        tie_at_zero = s[0].item() == 0.0 and s[1].item() == 0.0
        if s[0].item() < THR and not tie_at_zero and (s[1] - s[0]).item() < MARGIN:
            return False
    return True


def test_stream_recipe_has_clear_margins_on_the_oracle():
    """CPU check of the test data itself: the seeds used below give the oracle
    clear decisions of both kinds (refresh and keep)."""
    for dtype, seed, rows in ((torch.bfloat16, 10, 1), (torch.bfloat16, 36, 2)):
        sims, refreshed = _oracle_stream(dtype, seed, rows, calls=12)[1:]
        assert oracle_margins_ok(sims), [s.tolist() for s in sims]
        assert 0 < refreshed < len(sims)


def _oracle_stream(dtype, seed, rows, calls, heads=2, sink=3, cache_frames=6, grid=GRID, with_attention=True):
    ft = grid[1] * grid[2]
    gen = torch.Generator().manual_seed(seed)
    basis = torch.randn(3, heads * 128, generator=gen)
    freqs = oracle.build_freqs()
    cache = oracle.new_kv_cache(1, 1, cache_frames * ft, heads, 1, dtype=dtype)[0]
    layer = oracle.RingAttentionOracle(sink_size=sink, adapt_sink_thr=THR)
    record, sims, refreshed = [], [], 0
    for call in range(calls):
        if call == 1 and rows > 1:
            oracle.replicate_for_stream_batch([cache], rows)
        n = 1 if call == 0 else rows
        starts = [max(call - r, 0) * ft for r in range(n)]
        if call % 4 == 0:
            scene = torch.randn(3, generator=gen)       # a scene cut every fourth chunk
        q, k, v = directed_chunk(gen, n, heads, dtype, basis, scene, ft=ft)
        out, roped_q, seq = layer.step(q, k, v, [grid] * n, freqs, cache, starts, with_attention=with_attention)
        sims.extend(layer.last_sims)
        refreshed += sum(1 for s in layer.last_sims if s.min().item() < THR)
        record.append(dict(q=q, k=k, v=v, starts=starts, out=out, roped_q=roped_q, seq=seq,
                           writes=list(layer.last_writes), queue=[list(x) for x in layer.evict_idx],
                           sims=[s.clone() for s in layer.last_sims],
                           cache_k=cache["k"].clone(), cache_v=cache["v"].clone()))
    return record, sims, refreshed


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 1e-2), (torch.float32, 1e-5)])
@pytest.mark.parametrize("head_major", [True, False])
def test_similarity_operator(gpu_device, dtype, tol, head_major):
    from streamdiffusionv2_amd import ops, rope

    print(f"sink similarity operator: {dtype} head_major={head_major}", flush=True)
    rows, heads, sink, cap = 2, 3, 3, 5 * FT
    gen = torch.Generator().manual_seed(11)
    basis = torch.randn(3, heads * 128, generator=gen)
    freqs = rope.build_freqs()
    _, k, v = directed_chunk(gen, rows, heads, dtype, basis)
    ck = torch.cat([directed_chunk(gen, rows, heads, dtype, basis)[1] for _ in range(5)], dim=1)
    cv = torch.cat([directed_chunk(gen, rows, heads, dtype, basis)[2] for _ in range(5)], dim=1)
    start_frames = [7, 2]

    roped = oracle.causal_rope_apply(k, [GRID] * rows, oracle.build_freqs(), start_frames).type_as(v)
    want = []
    for r in range(rows):
        def means(t, frames):
            return t.reshape(frames, FT, -1).mean(1)
        sk = torch.cosine_similarity(means(ck[r:r + 1, :sink * FT], sink), means(roped[r:r + 1], 1), dim=-1)
        sv = torch.cosine_similarity(means(cv[r:r + 1, :sink * FT], sink), means(v[r:r + 1], 1), dim=-1)
        want.append(((sk + sv) / 2).float())
    want = torch.stack(want)

    def on_gpu(t):
        if head_major:
            return t.permute(0, 2, 1, 3).contiguous().to(gpu_device).permute(0, 2, 1, 3)
        return t.to(gpu_device)

    table = ops.device_freqs(freqs, gpu_device)
    sim, refresh = ops.sink_similarity(k.to(gpu_device), v.to(gpu_device), on_gpu(ck), on_gpu(cv), table,
                                       GRID[1:], start_frames, sink, THR)
    torch.cuda.synchronize()
    assert (sim.cpu() - want).abs().max().item() <= tol, (sim.cpu(), want)
    for r in range(rows):
        lo = want[r].min().item()
        if abs(lo - THR) > MARGIN:
            expect = int(want[r].argmin()) if lo < THR else -1
            assert refresh[r].item() == expect
    # an impossible threshold never refreshes, a generous one picks the minimum
    _, never = ops.sink_similarity(k.to(gpu_device), v.to(gpu_device), on_gpu(ck), on_gpu(cv), table,
                                   GRID[1:], start_frames, sink, -0.999)
    assert never.cpu().tolist() == [-1] * rows
    sim2, always = ops.sink_similarity(k.to(gpu_device), v.to(gpu_device), on_gpu(ck), on_gpu(cv), table,
                                       GRID[1:], start_frames, sink, 1.5)
    assert always.cpu().tolist() == sim2.argmin(dim=1).cpu().tolist()


@pytest.mark.gpu
@pytest.mark.parametrize("heads,sink", [(40, 3), (17, 16), (64, 2), (1, 1)])
def test_similarity_operator_wide_and_deep(gpu_device, heads, sink):
    """The kernel has builds for up to 16, 40 and 64 heads (8, 20 and 32 columns
    per thread of the deciding workgroup, which takes the sink frames four,
    two or one at a time) and room for 16 sink frames; the slot hand-over is
    checked on the way (rows 0 and 2 flagged as evicting)."""
    from streamdiffusionv2_amd import ops, rope

    print(f"sink similarity operator: heads={heads} sink={sink}", flush=True)
    rows, cap = 3, (sink + 2) * FT
    gen = torch.Generator().manual_seed(heads * 100 + sink)
    basis = torch.randn(3, heads * 128, generator=gen)
    _, k, v = directed_chunk(gen, rows, heads, torch.bfloat16, basis)
    ck = torch.cat([directed_chunk(gen, rows, heads, torch.bfloat16, basis)[1] for _ in range(sink + 2)], dim=1)
    cv = torch.cat([directed_chunk(gen, rows, heads, torch.bfloat16, basis)[2] for _ in range(sink + 2)], dim=1)
    start_frames = [5, 0, 11]
    roped = oracle.causal_rope_apply(k, [GRID] * rows, oracle.build_freqs(), start_frames).type_as(v)
    want = []
    for r in range(rows):
        def means(t, frames):
            return t.reshape(frames, FT, -1).mean(1)
        sk = torch.cosine_similarity(means(ck[r:r + 1, :sink * FT], sink), means(roped[r:r + 1], 1), dim=-1)
        sv = torch.cosine_similarity(means(cv[r:r + 1, :sink * FT], sink), means(v[r:r + 1], 1), dim=-1)
        want.append(((sk + sv) / 2).float())
    want = torch.stack(want)
    table = ops.device_freqs(rope.build_freqs(), gpu_device)
    override = torch.full((rows,), 12345, dtype=torch.int64, device=gpu_device)
    sim, refresh = ops.sink_similarity(k.to(gpu_device), v.to(gpu_device), ck.to(gpu_device), cv.to(gpu_device), table,
                                       GRID[1:], start_frames, sink, 1.5, dst_start_override=override,
                                       override_rows=[True, False, True])
    torch.cuda.synchronize()
    assert (sim.cpu() - want).abs().max().item() <= 1e-2, (sim.cpu(), want)
    got = refresh.cpu().tolist()
    assert got == sim.argmin(dim=1).cpu().tolist()            # threshold 1.5: always the minimum
    assert override.cpu().tolist() == [got[0] * FT, -1, got[2] * FT]
    for r in range(rows):
        s = want[r].sort().values
        if sink == 1 or (s[1] - s[0]).item() > MARGIN:
            assert got[r] == int(want[r].argmin())


@pytest.mark.gpu
def test_similarity_operator_rejects_bad_calls(gpu_device):
    from streamdiffusionv2_amd import ops, rope

    table = ops.device_freqs(rope.build_freqs(), gpu_device)
    x = torch.zeros(1, FT, 2, 128, dtype=torch.bfloat16, device=gpu_device)
    cache = torch.zeros(1, 4 * FT, 2, 128, dtype=torch.bfloat16, device=gpu_device)
    two_frames = torch.zeros(1, 2 * FT, 2, 128, dtype=torch.bfloat16, device=gpu_device)
    with pytest.raises(RuntimeError):       # more than one frame
        ops.sink_similarity(two_frames, two_frames, cache, cache, table, GRID[1:], [0], 2, THR)
    with pytest.raises(RuntimeError):       # sink larger than the cache
        ops.sink_similarity(x, x, cache, cache, table, GRID[1:], [0], 5, THR)
    with pytest.raises(RuntimeError):       # frame beyond the RoPE table
        ops.sink_similarity(x, x, cache, cache, table, GRID[1:], [1024], 2, THR)
    with pytest.raises(RuntimeError):       # CPU tensors: no fallback
        ops.sink_similarity(x.cpu(), x.cpu(), cache.cpu(), cache.cpu(), table, GRID[1:], [0], 2, THR)
    with pytest.raises(RuntimeError):       # slot hand-over without the per-row flags
        ops.sink_similarity(x, x, cache, cache, table, GRID[1:], [0], 2, THR,
                            dst_start_override=torch.zeros(1, dtype=torch.int64, device=gpu_device))
    with pytest.raises(RuntimeError):       # decision into unpinned host memory
        ops.sink_similarity(x, x, cache, cache, table, GRID[1:], [0], 2, THR, refresh_out=torch.zeros(1, dtype=torch.int32))
    wide = torch.zeros(1, FT, 65, 128, dtype=torch.bfloat16, device=gpu_device)
    wide_cache = torch.zeros(1, 4 * FT, 65, 128, dtype=torch.bfloat16, device=gpu_device)
    with pytest.raises(RuntimeError):       # more heads than the decision kernel is built for
        ops.sink_similarity(wide, wide, wide_cache, wide_cache, table, GRID[1:], [0], 2, THR)


@pytest.mark.gpu
@pytest.mark.parametrize("look_every_call", [True, False])
@pytest.mark.parametrize("seed,rows", [(10, 1), (36, 2)])
def test_stream_with_refresh(gpu_device, seed, rows, look_every_call):
    """The decision of a call is acted on by the device at once and picked up
    by the host when the path's state is next needed.  With look_every_call
    the test reads that state after every call (the host catches up at once);
    without, nothing touches it between calls, so every decision is settled
    by the following call, as in a running stream - the cache contents, which
    the device alone determines, are compared after every call either way."""
    from streamdiffusionv2_amd import ring, rope
    from streamdiffusionv2_amd.attention import RingKVPath

    print(f"adaptive sink stream: seed={seed} rows={rows} look_every_call={look_every_call}", flush=True)
    heads, sink, cache_frames, calls = 2, 3, 6, 12
    record, sims, refreshed = _oracle_stream(torch.bfloat16, seed, rows, calls)
    assert oracle_margins_ok(sims) and 0 < refreshed < len(sims)

    freqs = rope.build_freqs()
    cache = ring.new_kv_cache(1, 1, cache_frames * FT, heads, 1, device=gpu_device)[0]
    path = RingKVPath(sink_size=sink, adapt_sink_thr=THR)
    for call, rec in enumerate(record):
        if call == 1 and rows > 1:
            ring.replicate_for_stream_batch([cache], rows)
        n = len(rec["starts"])
        got, got_q = path.attend(rec["q"].to(gpu_device), rec["k"].to(gpu_device), rec["v"].to(gpu_device),
                                 torch.tensor([GRID] * n), freqs, cache, rec["starts"], return_roped_query=True)
        torch.cuda.synchronize()
        want_refresh = [int(s.argmin()) if s.min().item() < THR else -1 for s in rec["sims"]]
        if look_every_call or call == len(record) - 1:
            assert path.last_refresh == want_refresh, call
            assert path.evict_idx == rec["queue"], call
            assert path.last_plan.new_local_end == rec["seq"], call
            assert [(a, a + FT) for a in path.last_plan.dst_start] == rec["writes"], call
        assert cache["global_end_index"].tolist()[:n] == [start + FT for start in rec["starts"]], call
        assert cache["local_end_index"].tolist()[:n] == rec["seq"], call
        assert torch.equal(got_q.cpu().view(torch.int16), rec["roped_q"].view(torch.int16)), call
        for name in ("k", "v"):
            assert torch.equal(cache[name].cpu().view(torch.int16), rec["cache_" + name].view(torch.int16)), (call, name)
        # the directed values reach several units, so the unit-scale bounds
        # (max-abs 2e-2, mean-abs 2e-3) are taken relative to the largest output
        want = oracle.attention_fp32_reference(rec["roped_q"], rec["cache_k"], rec["cache_v"], rec["seq"])
        unit = max(1.0, want.abs().max().item())
        err = (got.float().cpu() - want).abs()
        assert err.max().item() <= 2e-2 * unit and err.mean().item() <= 2e-3 * unit, call


def _oracle_sessions(seed, sessions, calls, heads=2, sink=3, cache_frames=6):
    """One oracle layer run through several streams, each on a cache of its own
    that starts out all zero; the layer (and its eviction queue, which the
    reference does not reset either) lives on."""
    gen = torch.Generator().manual_seed(seed)
    basis = torch.randn(3, heads * 128, generator=gen)
    freqs = oracle.build_freqs()
    layer = oracle.RingAttentionOracle(sink_size=sink, adapt_sink_thr=THR)
    out, sims = [], []
    for _ in range(sessions):
        cache = oracle.new_kv_cache(1, 1, cache_frames * FT, heads, 1, dtype=torch.bfloat16)[0]
        record = []
        for call in range(calls):
            if call % 4 == 0:
                scene = torch.randn(3, generator=gen)
            q, k, v = directed_chunk(gen, 1, heads, torch.bfloat16, basis, scene)
            starts = [call * FT]
            _, roped_q, seq = layer.step(q, k, v, [GRID], freqs, cache, starts, with_attention=False)
            sims.extend(layer.last_sims)
            record.append(dict(q=q, k=k, v=v, starts=starts, seq=seq, writes=list(layer.last_writes),
                               queue=[list(x) for x in layer.evict_idx], sims=[x.clone() for x in layer.last_sims],
                               cache_k=cache["k"].clone(), cache_v=cache["v"].clone()))
        out.append(record)
    return out, sims


def test_two_session_recipe_has_clear_margins_on_the_oracle():
    sessions, sims = _oracle_sessions(10, 2, 9)
    assert oracle_margins_ok(sims), [x.tolist() for x in sims]
    # the second stream starts on zeros: its first checks see cosine 0 and refresh, whatever the first stream held
    assert all(x.min().item() == 0.0 for x in sessions[1][0]["sims"])


@pytest.mark.gpu
def test_a_fresh_cache_at_the_old_address_is_summed_afresh(gpu_device):
    """The kept means of the sink frames belong to one cache dict.  A stream
    that is reset and started again (streamv2v/inference.py:161-171, then
    causal_stream_inference.py:87-107) gets a new all-zero cache, usually in
    the very memory the old one had, while the path object lives on: the first
    checks of the new stream must compare against zeros, as the reference
    does, not against what the old stream's sink frames held."""
    from streamdiffusionv2_amd import ring, rope
    from streamdiffusionv2_amd.attention import RingKVPath

    heads, sink, cache_frames = 2, 3, 6
    sessions, sims = _oracle_sessions(10, 2, 9)
    assert oracle_margins_ok(sims)
    freqs = rope.build_freqs()
    path = RingKVPath(sink_size=sink, adapt_sink_thr=THR)
    old_address = None
    for number, record in enumerate(sessions):
        cache = ring.new_kv_cache(1, 1, cache_frames * FT, heads, 1, device=gpu_device)[0]
        print(f"session {number}: cache at {cache['k'].data_ptr():#x} (the last one at {old_address})", flush=True)
        for call, rec in enumerate(record):
            path.attend(rec["q"].to(gpu_device), rec["k"].to(gpu_device), rec["v"].to(gpu_device),
                        torch.tensor([GRID]), freqs, cache, rec["starts"])
            torch.cuda.synchronize()
            want_refresh = [int(x.argmin()) if x.min().item() < THR else -1 for x in rec["sims"]]
            assert path.last_refresh == want_refresh, (number, call)
            assert path.evict_idx == rec["queue"], (number, call)
            assert [(a, a + FT) for a in path.last_plan.dst_start] == rec["writes"], (number, call)
            assert cache["local_end_index"].tolist() == rec["seq"], (number, call)
            for name in ("k", "v"):
                assert torch.equal(cache[name].cpu().view(torch.int16), rec["cache_" + name].view(torch.int16)), \
                    (number, call, name)
        old_address = hex(cache["k"].data_ptr())
        del cache


# --------------------------------------------------------------------------
# The shipped shape: 480p latent frames of 30 x 52 = 1560 tokens, sink 3,
# threshold 0.2 (configs/wan_causal_dmd_v2v.yaml:53-56), 12 heads (Wan 1.3B)
# and 40 heads (Wan 14B).  At this frame size every workgroup runs its
# four-tokens-in-flight main loop (195 tokens per workgroup) and 40 heads take
# the middle build of the kernel (20 columns per deciding thread).
# --------------------------------------------------------------------------
PROD_GRID = (1, 30, 52)
PROD_FT = 1560
PROD_STREAMS = [(12, 23, 12), (40, 23, 10)]          # heads, seed, calls


def test_production_stream_recipe_has_clear_margins_on_the_oracle():
    for heads, seed, calls in PROD_STREAMS:
        sims, refreshed = _oracle_stream(torch.bfloat16, seed, 1, calls, heads=heads, grid=PROD_GRID,
                                         with_attention=False)[1:]
        assert oracle_margins_ok(sims), [s.tolist() for s in sims]
        assert 0 < refreshed < len(sims)


@pytest.mark.gpu
@pytest.mark.parametrize("heads", [12, 40])
@pytest.mark.parametrize("head_major", [True, False])
def test_similarity_operator_production_shape(gpu_device, heads, head_major):
    from streamdiffusionv2_amd import ops, rope

    print(f"sink similarity operator at 1560-token frames: heads={heads} head_major={head_major}", flush=True)
    rows, sink, frames = 2, 3, 6
    gen = torch.Generator().manual_seed(300 + heads)
    basis = torch.randn(3, heads * 128, generator=gen)
    _, k, v = directed_chunk(gen, rows, heads, torch.bfloat16, basis, ft=PROD_FT)
    ck = torch.cat([directed_chunk(gen, rows, heads, torch.bfloat16, basis, ft=PROD_FT)[1] for _ in range(frames)], dim=1)
    cv = torch.cat([directed_chunk(gen, rows, heads, torch.bfloat16, basis, ft=PROD_FT)[2] for _ in range(frames)], dim=1)
    start_frames = [17, 3]
    roped = oracle.causal_rope_apply(k, [PROD_GRID] * rows, oracle.build_freqs(), start_frames).type_as(v)
    want = []
    for r in range(rows):
        def means(t, n):
            return t.reshape(n, PROD_FT, -1).mean(1)
        sk = torch.cosine_similarity(means(ck[r:r + 1, :sink * PROD_FT], sink), means(roped[r:r + 1], 1), dim=-1)
        sv = torch.cosine_similarity(means(cv[r:r + 1, :sink * PROD_FT], sink), means(v[r:r + 1], 1), dim=-1)
        want.append(((sk + sv) / 2).float())
    want = torch.stack(want)

    def on_gpu(t):
        if head_major:
            return t.permute(0, 2, 1, 3).contiguous().to(gpu_device).permute(0, 2, 1, 3)
        return t.to(gpu_device)

    table = ops.device_freqs(rope.build_freqs(), gpu_device)
    override = torch.full((rows,), 777, dtype=torch.int64, device=gpu_device)
    sim, refresh = ops.sink_similarity(k.to(gpu_device), v.to(gpu_device), on_gpu(ck), on_gpu(cv), table,
                                       PROD_GRID[1:], start_frames, sink, 1.5, dst_start_override=override,
                                       override_rows=[True, True])
    torch.cuda.synchronize()
    assert (sim.cpu() - want).abs().max().item() <= 1e-2, (sim.cpu(), want)
    got = refresh.cpu().tolist()
    assert got == sim.argmin(dim=1).cpu().tolist()            # threshold 1.5: always the minimum
    assert override.cpu().tolist() == [g * PROD_FT for g in got]
    for r in range(rows):
        s = want[r].sort().values
        if (s[1] - s[0]).item() > MARGIN:
            assert got[r] == int(want[r].argmin())
    # the shipped threshold
    _, shipped = ops.sink_similarity(k.to(gpu_device), v.to(gpu_device), on_gpu(ck), on_gpu(cv), table,
                                     PROD_GRID[1:], start_frames, sink, THR)
    for r in range(rows):
        lo = want[r].min().item()
        s = want[r].sort().values
        if abs(lo - THR) > MARGIN and (lo >= THR or (s[1] - s[0]).item() > MARGIN):
            assert shipped[r].item() == (int(want[r].argmin()) if lo < THR else -1)


@pytest.mark.gpu
@pytest.mark.parametrize("heads,seed,calls", PROD_STREAMS)
def test_stream_with_refresh_production_shape(gpu_device, heads, seed, calls):
    """The shipped configuration as a stream: 1560-token frames, cache of six
    frames of which three are sink frames, threshold 0.2.  The ring fills
    (calls 0-5) and then evicts; scene cuts every fourth chunk make the check
    refresh a sink frame on some calls and keep all three on others.  Decision,
    queue, slot, indices and the cache bits are compared after every call; the
    attention on a seeded sample of query rows."""
    from streamdiffusionv2_amd import ring, rope
    from streamdiffusionv2_amd.attention import RingKVPath

    print(f"adaptive sink stream at 1560-token frames: heads={heads} calls={calls}", flush=True)
    sink, cache_frames = 3, 6
    record, sims, refreshed = _oracle_stream(torch.bfloat16, seed, 1, calls, heads=heads, grid=PROD_GRID,
                                             with_attention=False)
    assert oracle_margins_ok(sims) and 0 < refreshed < len(sims)
    assert any(a < sink * PROD_FT for rec in record[cache_frames:] for a, _ in rec["writes"])   # a sink frame is rewritten

    freqs = rope.build_freqs()
    cache = ring.new_kv_cache(1, 1, cache_frames * PROD_FT, heads, 1, device=gpu_device)[0]
    path = RingKVPath(sink_size=sink, adapt_sink_thr=THR)
    gen = torch.Generator().manual_seed(5)
    for call, rec in enumerate(record):
        got, got_q = path.attend(rec["q"].to(gpu_device), rec["k"].to(gpu_device), rec["v"].to(gpu_device),
                                 torch.tensor([PROD_GRID]), freqs, cache, rec["starts"], return_roped_query=True)
        torch.cuda.synchronize()
        want_refresh = [int(s.argmin()) if s.min().item() < THR else -1 for s in rec["sims"]]
        if call % 2 == 0 or call == len(record) - 1:          # every other call settles lazily, as in a running stream
            assert path.last_refresh == want_refresh, call
            assert path.evict_idx == rec["queue"], call
            assert [(a, a + PROD_FT) for a in path.last_plan.dst_start] == rec["writes"], call
        assert cache["global_end_index"].tolist() == [rec["starts"][0] + PROD_FT], call
        assert cache["local_end_index"].tolist() == rec["seq"], call
        assert torch.equal(got_q.cpu().view(torch.int16), rec["roped_q"].view(torch.int16)), call
        for name in ("k", "v"):
            assert torch.equal(cache[name].cpu().view(torch.int16), rec["cache_" + name].view(torch.int16)), (call, name)
        idx = torch.randperm(PROD_FT, generator=gen)[:32].sort().values
        want = oracle.attention_fp32_reference(rec["roped_q"][:, idx], rec["cache_k"], rec["cache_v"], rec["seq"])
        # the recipe scales frames up to force clear decisions and the outputs
        # grow with them: the unit-scale bounds (2e-2 / 2e-3) are taken relative
        # to the largest output, as in the small-shape stream above
        unit = max(1.0, want.abs().max().item())
        err = (got[:, idx.to(gpu_device)].float().cpu() - want).abs()
        assert err.max().item() <= 2e-2 * unit and err.mean().item() <= 2e-3 * unit, call


@pytest.mark.gpu
@pytest.mark.parametrize("heads,ft_grid", [(3, GRID), (12, PROD_GRID)])
def test_kept_frame_sums_give_the_same_bits(gpu_device, heads, ft_grid):
    """With the sink frames' token sums kept between calls the operator reads
    the new chunk only; similarities and decisions must be bit for bit those of
    the call that sums every frame from the cache - through a sequence in which
    frames go stale, a filling row lands in a sink frame and an evicting row
    refreshes one."""
    from streamdiffusionv2_amd import ops, rope

    ft = ft_grid[1] * ft_grid[2]
    rows, sink, frames = 2, 3, 5
    gen = torch.Generator().manual_seed(77 + heads)
    basis = torch.randn(3, heads * 128, generator=gen)
    ck = torch.cat([directed_chunk(gen, rows, heads, torch.bfloat16, basis, ft=ft)[1] for _ in range(frames)], dim=1)
    cv = torch.cat([directed_chunk(gen, rows, heads, torch.bfloat16, basis, ft=ft)[2] for _ in range(frames)], dim=1)
    ck, cv = ck.to(gpu_device), cv.to(gpu_device)
    table = ops.device_freqs(rope.build_freqs(), gpu_device)
    kept = ops.new_sink_frame_sums(rows, heads, sink, gpu_device)
    kept.fill_(float("nan"))                       # whatever it holds is stale
    stale = [0b111, 0b111]

    def both(k, v, starts, thr, planned, evicting):
        override_a = torch.full((rows,), -5, dtype=torch.int64, device=gpu_device)
        override_b = torch.full((rows,), -5, dtype=torch.int64, device=gpu_device)
        sim_a, ref_a = ops.sink_similarity(k, v, ck, cv, table, ft_grid[1:], starts, sink, thr,
                                           dst_start_override=override_a, override_rows=evicting)
        sim_b, ref_b = ops.sink_similarity(k, v, ck, cv, table, ft_grid[1:], starts, sink, thr,
                                           dst_start_override=override_b, override_rows=evicting,
                                           frame_sums=kept, stale_frames=stale, planned_frames=planned)
        torch.cuda.synchronize()
        assert torch.equal(sim_a.view(torch.int32), sim_b.view(torch.int32))
        assert ref_a.tolist() == ref_b.tolist() and override_a.tolist() == override_b.tolist()
        return ref_b.tolist()

    def chunk():
        _, k, v = directed_chunk(gen, rows, heads, torch.bfloat16, basis, ft=ft)
        return k.to(gpu_device), v.to(gpu_device)

    # 1. everything stale, nothing lands in the sink
    k, v = chunk()
    both(k, v, [4, 9], THR, [-1, -1], [False, False])
    stale = [0, 0]
    # 2. nothing stale: only the new chunk is read (the cache rows of frame 1 of row 0 are scribbled over
    #    behind the operator's back to show it: the kept sums still describe the old contents)
    saved = ck[0, ft:2 * ft].clone()
    ck[0, ft:2 * ft] = 0
    k, v = chunk()
    sim_kept, _ = ops.sink_similarity(k, v, ck, cv, table, ft_grid[1:], [5, 10], sink, THR, frame_sums=kept,
                                      stale_frames=stale, planned_frames=[-1, -1])
    ck[0, ft:2 * ft] = saved
    sim_full, _ = ops.sink_similarity(k, v, ck, cv, table, ft_grid[1:], [5, 10], sink, THR)
    torch.cuda.synchronize()
    assert torch.equal(sim_kept.view(torch.int32), sim_full.view(torch.int32))
    # 3. a filling row (row 1) lands in sink frame 2: the append is played by hand, the kept sums follow by themselves
    k, v = chunk()
    both(k, v, [6, 2], THR, [-1, 2], [False, False])
    roped = ops.causal_rope_apply(k, [ft_grid] * rows, table, torch.tensor([6, 2]))
    ck[1, 2 * ft:3 * ft] = roped[1]
    cv[1, 2 * ft:3 * ft] = v[1]
    k, v = chunk()
    both(k, v, [7, 3], THR, [-1, -1], [False, False])
    # 4. an evicting row (row 0) refreshes: threshold 1.5 always picks the minimum; the append follows the override
    k, v = chunk()
    chosen = both(k, v, [8, 4], 1.5, [-1, -1], [True, False])
    assert chosen[0] >= 0
    roped = ops.causal_rope_apply(k, [ft_grid] * rows, table, torch.tensor([8, 4]))
    ck[0, chosen[0] * ft:(chosen[0] + 1) * ft] = roped[0]
    cv[0, chosen[0] * ft:(chosen[0] + 1) * ft] = v[0]
    k, v = chunk()
    both(k, v, [9, 5], THR, [-1, -1], [False, False])
    # 5. a frame written behind the operator's back and declared stale is summed again
    ck[1, 0:ft] = ck[1, 3 * ft:4 * ft]
    stale = [0, 0b001]
    k, v = chunk()
    both(k, v, [10, 6], THR, [-1, -1], [False, False])


@pytest.mark.gpu
@pytest.mark.parametrize("heads", [12, 40, 5])
def test_similarity_with_the_key_norm_folded_in(gpu_device, heads):
    """k handed over raw with its RMSNorm weight must give the bits of k
    normalised beforehand by the oracle's WanRMSNorm."""
    from streamdiffusionv2_amd import ops, rope

    rows, sink, frames, eps = 2, 3, 4, 1e-6
    gen = torch.Generator().manual_seed(500 + heads)
    basis = torch.randn(3, heads * 128, generator=gen)
    _, k_raw, v = directed_chunk(gen, rows, heads, torch.bfloat16, basis, scale=1.3)
    weight = (torch.rand(heads * 128, generator=gen) + 0.5).bfloat16()
    k_normed = oracle.wan_rms_norm(k_raw.flatten(2), weight, eps).view_as(k_raw)
    ck = torch.cat([directed_chunk(gen, rows, heads, torch.bfloat16, basis)[1] for _ in range(frames)], dim=1)
    cv = torch.cat([directed_chunk(gen, rows, heads, torch.bfloat16, basis)[2] for _ in range(frames)], dim=1)
    table = ops.device_freqs(rope.build_freqs(), gpu_device)
    args = (ck.to(gpu_device), cv.to(gpu_device), table, GRID[1:], [3, 8], sink, THR)
    want, want_refresh = ops.sink_similarity(k_normed.to(gpu_device), v.to(gpu_device), *args)
    got, got_refresh = ops.sink_similarity(k_raw.to(gpu_device), v.to(gpu_device), *args,
                                           k_norm=(weight.to(gpu_device), eps))
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    assert got_refresh.tolist() == want_refresh.tolist()


@pytest.mark.gpu
def test_module_with_fused_norm_and_adaptive_sink(gpu_device):
    """The shipped combination: q / k norm inside the append AND the adaptive
    sink check (which then normalises the new keys itself).  The stream must
    leave the cache that the unfused module leaves (norms applied by torch on
    the GPU add in another order: at most one ulp apart) and take the same
    decisions."""
    from streamdiffusionv2_amd import ring, rope
    from streamdiffusionv2_amd.attention import CausalWanSelfAttention

    torch.manual_seed(9)
    dim, heads = 384, 3
    mod = CausalWanSelfAttention(dim, heads).to(gpu_device).bfloat16()
    with torch.no_grad():
        mod.norm_q.weight.uniform_(0.5, 1.5)
        mod.norm_k.weight.uniform_(0.5, 1.5)
    mod.sink_size, mod.adapt_sink_thr = 2, 0.2
    freqs = rope.build_freqs()
    calls = 10
    scenes = [torch.randn(1, 1, dim) * 2 for _ in range(3)]
    xs = [(torch.randn(1, FT, dim) * 0.3 + scenes[c // 4]).bfloat16().to(gpu_device) for c in range(calls)]
    runs = []
    for fuse in (True, False):
        mod.fuse_qk_norm = fuse
        mod.evict_idx = None
        cache = ring.new_kv_cache(1, 1, 5 * FT, heads, 1, device=gpu_device)[0]
        decisions, outs = [], []
        with torch.no_grad():
            for c in range(calls):
                outs.append(mod(xs[c], None, torch.tensor([GRID]), freqs, None, kv_cache=cache, current_start=c * FT))
                decisions.append(mod.last_refresh)
        runs.append((decisions, [list(q) for q in mod.evict_idx], cache["k"].clone(), cache["v"].clone(), torch.stack(outs)))
    torch.cuda.synchronize()
    (d1, q1, k1, v1, y1), (d0, q0, k0, v0, y0) = runs
    assert d1 == d0 and q1 == q0
    assert any(d is not None and d[0] >= 0 for d in d1)            # at least one refresh happened
    assert torch.equal(v1, v0)
    ik1, ik0 = k1.cpu().view(torch.int16).int(), k0.cpu().view(torch.int16).int()
    assert (ik1 - ik0).abs().max().item() <= 1
    assert (y1.float() - y0.float()).abs().max().item() <= 3e-2
