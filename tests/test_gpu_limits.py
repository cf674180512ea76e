"""Edges of the C ABI's per-call limits: SDV2_MAX_ROWS rows per append launch
(more rows are dealt out over several launches by the wrapper), the attention
kernel's row bound, and the stream path on either side of the row limit."""
import pytest
import torch

from oracle import sdv2_oracle as oracle

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.contiguous().view(torch.int16)


@pytest.mark.parametrize("rows", [16, 17, 33])
def test_append_and_attention_many_rows(gpu_device, rows):
    from streamdiffusionv2_amd import ops, rope

    print(f"many rows: {rows}", flush=True)
    torch.manual_seed(rows)
    grid, heads = (1, 3, 4), 2
    S, cap = 12, 36
    q, k, v = (torch.randn(rows, S, heads, 128).bfloat16() for _ in range(3))
    start_frames = [(7 * r) % 1000 for r in range(rows)]
    dst = [(r % 3) * S for r in range(rows)]
    kc = torch.zeros(rows, heads, cap, 128, dtype=torch.bfloat16, device=gpu_device).permute(0, 2, 1, 3)
    vc = torch.zeros(rows, heads, cap, 128, dtype=torch.bfloat16, device=gpu_device).permute(0, 2, 1, 3)
    g_idx = torch.zeros(rows, dtype=torch.long, device=gpu_device)
    l_idx = torch.zeros(rows, dtype=torch.long, device=gpu_device)
    table = ops.device_freqs(rope.build_freqs(), gpu_device)
    got_q = ops.kv_append_rope(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), kc, vc, table, grid, start_frames,
                               dst, global_end_index=g_idx, local_end_index=l_idx,
                               new_global_end=[100 + r for r in range(rows)], new_local_end=[d + S for d in dst])
    want_q = oracle.causal_rope_apply(q, [grid] * rows, oracle.build_freqs(), start_frames).type_as(v)
    want_k = oracle.causal_rope_apply(k, [grid] * rows, oracle.build_freqs(), start_frames).type_as(v)
    torch.cuda.synchronize()
    assert torch.equal(_bits(got_q.cpu()), _bits(want_q))
    ck, cv = torch.zeros(rows, cap, heads, 128).bfloat16(), torch.zeros(rows, cap, heads, 128).bfloat16()
    for r in range(rows):
        ck[r, dst[r]:dst[r] + S], cv[r, dst[r]:dst[r] + S] = want_k[r], v[r]
    assert torch.equal(_bits(kc.cpu()), _bits(ck)) and torch.equal(_bits(vc.cpu()), _bits(cv))
    assert g_idx.tolist() == [100 + r for r in range(rows)] and l_idx.tolist() == [d + S for d in dst]
    lens = [d + S for d in dst]
    out = ops.swa_attention(got_q, kc, vc, torch.tensor(lens, dtype=torch.int32, device=gpu_device))
    want = oracle.attention_fp32_reference(want_q, ck, cv, lens)
    err = (out.float().cpu() - want).abs()
    assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3


@pytest.mark.parametrize("rows", [16, 17])
def test_stream_path_on_either_side_of_the_row_limit(gpu_device, rows):
    """16 rows go through the prebuilt launch descriptors, 17 through the
    general wrappers; both must follow the oracle."""
    from streamdiffusionv2_amd import ring, rope
    from streamdiffusionv2_amd.attention import RingKVPath

    print(f"stream path with {rows} rows", flush=True)
    heads, grid = 1, (1, 2, 4)
    S, cap = 8, 32
    freqs = rope.build_freqs()
    caches, o_caches = ring.new_kv_cache(1, 1, cap, heads, 1, device=gpu_device), oracle.new_kv_cache(1, 1, cap, heads, 1)
    ring.replicate_for_stream_batch(caches, rows)
    oracle.replicate_for_stream_batch(o_caches, rows)
    cache, o_cache = caches[0], o_caches[0]
    path, o_path = RingKVPath(sink_size=1), oracle.RingAttentionOracle(sink_size=1)
    gen = torch.Generator().manual_seed(rows)
    for call in range(7):
        starts = [call * S] * rows
        q, k, v = (torch.randn(rows, S, heads, 128, generator=gen).bfloat16() for _ in range(3))
        got = path.attend(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), torch.tensor([grid] * rows), freqs,
                          cache, starts)
        _, want_q, seq = o_path.step(q, k, v, [list(grid)] * rows, freqs, o_cache, starts, with_attention=False)
        torch.cuda.synchronize()
        assert path.evict_idx == o_path.evict_idx
        for name in ("k", "v"):
            assert torch.equal(_bits(cache[name].cpu()), _bits(o_cache[name])), (call, name)
        for name in ("global_end_index", "local_end_index"):
            assert cache[name].tolist() == o_cache[name].tolist()
        want = oracle.attention_fp32_reference(want_q, o_cache["k"], o_cache["v"], seq)
        err = (got.float().cpu() - want).abs()
        assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3


@pytest.mark.gpu
def test_a_failed_call_leaves_the_ring_state_where_it_was(gpu_device):
    """Planning advances the host's ring state before the launch is validated;
    a call the library refuses (here: a frame beyond the 1024 rows of the RoPE
    table) must not leave queue, pass counter or index mirror advanced while
    the device indices stayed put - the stream continues as if it had not been made."""
    import copy

    from streamdiffusionv2_amd import ring, rope
    from streamdiffusionv2_amd.attention import RingKVPath

    torch.manual_seed(0)
    heads, grid, S = 2, (1, 4, 6), 24
    freqs = rope.build_freqs()
    cache = ring.new_kv_cache(1, 1, 4 * S, heads, 1, device=gpu_device)[0]
    twin = ring.new_kv_cache(1, 1, 4 * S, heads, 1, device=gpu_device)[0]
    path, twin_path = RingKVPath(sink_size=1), RingKVPath(sink_size=1)
    chunks = [tuple(torch.randn(1, S, heads, 128, device=gpu_device).bfloat16() for _ in range(3)) for _ in range(7)]
    for c in range(5):
        path.attend(*chunks[c], torch.tensor([grid]), freqs, cache, [c * S])
        twin_path.attend(*chunks[c], torch.tensor([grid]), freqs, twin, [c * S])
    before = (copy.deepcopy(path.evict_idx), cache["current_step"], cache["global_end_index"].tolist(),
              cache["local_end_index"].tolist(), cache["k"].clone())
    with pytest.raises(RuntimeError):
        path.attend(*chunks[5], torch.tensor([grid]), freqs, cache, [2000 * S])      # frame 2000: beyond the table
    torch.cuda.synchronize()
    assert path.evict_idx == before[0] and cache["current_step"] == before[1]
    assert cache["global_end_index"].tolist() == before[2] and cache["local_end_index"].tolist() == before[3]
    assert torch.equal(cache["k"], before[4])
    for c in (5, 6):
        a = path.attend(*chunks[c], torch.tensor([grid]), freqs, cache, [c * S])
        b = twin_path.attend(*chunks[c], torch.tensor([grid]), freqs, twin, [c * S])
        assert torch.equal(a, b)
    assert path.evict_idx == twin_path.evict_idx
    assert torch.equal(cache["k"], twin["k"]) and torch.equal(cache["v"], twin["v"])


def test_a_split_call_after_a_refused_one_is_still_right(gpu_device):
    """A call the library refuses (status < 0) launches nothing and leaves the
    ticket words of the workspace at zero; the wrapper zeroes them again after
    any failed layer call.  Either way the next split call combines its key
    ranges as if nothing had happened."""
    from streamdiffusionv2_amd import ops

    torch.manual_seed(3)
    rows, S, H, L, sp = 1, 300, 3, 2500, 4
    q = torch.randn(rows, S, H, 128).bfloat16()
    k = torch.randn(rows, L, H, 128).bfloat16()
    v = torch.randn(rows, L, H, 128).bfloat16()
    qd, kd, vd = q.to(gpu_device), k.to(gpu_device), v.to(gpu_device)
    want = oracle.attention_fp32_reference(q, k, v, [L] * rows)
    first = ops.swa_attention(qd, kd, vd, None, num_splits=sp)
    with pytest.raises(RuntimeError):                    # refused: misaligned output pointer
        ops.swa_attention(qd, kd, vd, None, num_splits=sp, out=torch.empty(rows, S, H, 129, dtype=torch.bfloat16,
                                                                           device=gpu_device)[..., 1:])
    with pytest.raises(RuntimeError):                    # refused: more key ranges than the library takes
        ops.swa_attention(qd, kd, vd, None, num_splits=65)
    again = ops.swa_attention(qd, kd, vd, None, num_splits=sp)
    ops.reset_workspace_tickets(gpu_device)              # what a failed layer call does on its way out
    third = ops.swa_attention(qd, kd, vd, None, num_splits=sp)
    torch.cuda.synchronize()
    for got in (first, again, third):
        assert torch.equal(got, first)
        err = (got.float().cpu() - want).abs()
        assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3


def test_only_zero_filled_workspaces_are_accepted(gpu_device):
    """A caller-owned workspace must come from ops.new_workspace: a ticket word
    that does not start at zero would make a split call combine early or never,
    with no error to show for it."""
    from streamdiffusionv2_amd import _capi, ops

    q = torch.zeros(1, 64, 1, 128, dtype=torch.bfloat16, device=gpu_device)
    kv = torch.zeros(1, 2048, 1, 128, dtype=torch.bfloat16, device=gpu_device)
    need = _capi.lib().sdv2_swa_attn_workspace_bytes(1, 64, 1, 2048, 2)
    with pytest.raises(RuntimeError):
        ops.swa_attention(q, kv, kv, None, num_splits=2, workspace=torch.empty(need, dtype=torch.uint8, device=gpu_device))
    ops.swa_attention(q, kv, kv, None, num_splits=2, workspace=ops.new_workspace(gpu_device, need))
    torch.cuda.synchronize()
