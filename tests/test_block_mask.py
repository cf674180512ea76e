"""Optional block-causal mask inside the chunk.

The reference's KV-cache path applies no mask inside a chunk; its cache-less
path uses kv_idx < ends[q_idx] | q_idx == kv_idx with ends = end of the query's
block (causal_model.py:670-686).  CPU: the oracle's cache-position form of that
rule against the formula itself on logical positions (brute force, tiny sizes,
with the chunk at the start, in the middle and at the end of the ring).
GPU: the kernel against the oracle on ragged shapes, splits, both layouts, the
exact fallback, and a whole stream with 3-frame chunks masked per frame."""
import pytest
import torch

from oracle import sdv2_oracle as oracle

MAX_ABS, MEAN_ABS = 2e-2, 2e-3


def _reference_formula_mask(n_frames_before, chunk_frames, frame_tokens, frames_per_block):
    """The reference formula on logical positions: all cached tokens come
    first (in time order), then the chunk; rows = the chunk's queries."""
    total = (n_frames_before + chunk_frames) * frame_tokens
    block = frame_tokens * frames_per_block
    ends = [0] * total
    # blocks are aligned to the start of the chunk (the reference aligns them to
    # the start of the sequence; the cached prefix is then a whole number of blocks)
    for q in range(total):
        ends[q] = (q // block + 1) * block
    first = n_frames_before * frame_tokens
    return [[(kv < ends[q]) or (q == kv) for kv in range(total)] for q in range(first, total)]


@pytest.mark.parametrize("slot", [0, 2, 4])
@pytest.mark.parametrize("frames_per_block", [1, 2])
def test_cache_position_mask_equals_reference_formula(slot, frames_per_block):
    ft, chunk_frames, cache_frames = 3, 4, 8          # prefix of 4 frames = whole blocks for 1 and 2
    S, L = chunk_frames * ft, cache_frames * ft
    want_logical = _reference_formula_mask(cache_frames - chunk_frames, chunk_frames, ft, frames_per_block)
    got = oracle.chunk_block_mask(S, L, slot * ft, frames_per_block * ft)
    # physical position -> logical position: the chunk occupies [slot, slot + chunk) frames of
    # the ring, everything else holds older frames (their order does not matter to the rule)
    older = [p for p in range(L) if not (slot * ft <= p < slot * ft + S)]
    logical_of = {p: i for i, p in enumerate(older)}
    for t in range(S):
        logical_of[slot * ft + t] = len(older) + t
    for t in range(S):
        for p in range(L):
            assert bool(got[t, p]) == want_logical[t][logical_of[p]], (t, p)
    # nothing outside the chunk is ever hidden; the own block is always visible
    assert got[:, [p for p in range(L) if p in older]].all()
    for t in range(S):
        b = t // (frames_per_block * ft)
        assert got[t, slot * ft + b * frames_per_block * ft: slot * ft + (b + 1) * frames_per_block * ft].all()


def test_oracle_attention_with_mask_matches_explicit_softmax():
    torch.manual_seed(1)
    S, L, H, start, bt = 6, 16, 2, 5, 2
    q, k, v = torch.randn(1, S, H, 128), torch.randn(1, L, H, 128), torch.randn(1, L, H, 128)
    got = oracle.attention_with_kvcache(q, k, v, torch.tensor([L], dtype=torch.int32), [start], bt)
    for t in range(S):
        visible = [p for p in range(L) if not (start + (t // bt + 1) * bt <= p < start + S)]
        for h in range(H):
            s = (k[0, visible, h] @ q[0, t, h]) / 128 ** 0.5
            want = torch.softmax(s.double(), 0).float() @ v[0, visible, h]
            assert torch.allclose(got[0, t, h], want, atol=2e-5)
    # a block as long as the chunk hides nothing
    plain = oracle.attention_with_kvcache(q, k, v, torch.tensor([L], dtype=torch.int32))
    whole = oracle.attention_with_kvcache(q, k, v, torch.tensor([L], dtype=torch.int32), [start], S)
    assert torch.allclose(plain, whole, atol=1e-6)


def _close(got, want):
    err = (got.float().cpu() - want).abs()
    assert torch.isfinite(got.float()).all()
    assert err.max().item() <= MAX_ABS and err.mean().item() <= MEAN_ABS, (err.max().item(), err.mean().item())


@pytest.mark.gpu
@pytest.mark.parametrize("S,L,bt,starts,splits,head_major", [
    (300, 1000, 100, [450], 1, True),          # chunk in the middle, blocks not tile aligned
    (300, 1000, 100, [0], 2, False),           # chunk first
    (300, 1000, 100, [700], 3, True),          # chunk last, split
    (520, 1300, 130, [100, 777], 1, True),     # two rows, two query tiles per row
    (96, 96, 32, [0], 1, True),                # nothing but the chunk: later blocks fully hidden
    (384, 576, 192, [192], 3, True),           # the third key range is entirely hidden from the first block
])
def test_kernel_block_mask(gpu_device, S, L, bt, starts, splits, head_major):
    from streamdiffusionv2_amd import ops

    print(f"block mask: S={S} L={L} bt={bt} starts={starts} splits={splits}", flush=True)
    torch.manual_seed(3)
    rows, H = len(starts), 2
    q = torch.randn(rows, S, H, 128).bfloat16()
    k = torch.randn(rows, L, H, 128).bfloat16()
    v = torch.randn(rows, L, H, 128).bfloat16()
    want = oracle.attention_fp32_reference(q, k, v, [L] * rows, starts, bt)
    unmasked = oracle.attention_fp32_reference(q, k, v, [L] * rows)
    assert (want - unmasked).abs().max() > 0.05           # the mask matters on this input

    def dev(t):
        return t.permute(0, 2, 1, 3).contiguous().to(gpu_device).permute(0, 2, 1, 3) if head_major else t.to(gpu_device)

    got = ops.swa_attention(q.to(gpu_device), dev(k), dev(v), None, num_splits=splits,
                            chunk_key_start=starts, mask_block_tokens=bt)
    torch.cuda.synchronize()
    _close(got, want)
    # a block as long as the chunk: same as no mask
    got = ops.swa_attention(q.to(gpu_device), dev(k), dev(v), None, num_splits=splits,
                            chunk_key_start=starts, mask_block_tokens=S)
    _close(got, unmasked)


@pytest.mark.gpu
def test_block_mask_with_exact_fallback_and_lengths(gpu_device):
    """Extreme scores force the running-maximum pass, where a query's first
    tiles can be hidden entirely; per-row lengths stay honoured."""
    from streamdiffusionv2_amd import ops

    torch.manual_seed(4)
    rows, S, L, H, bt = 2, 192, 640, 2, 64
    q = (torch.randn(rows, S, H, 128) * 14).bfloat16()
    k = (torch.randn(rows, L, H, 128) * 14).bfloat16()
    v = torch.randn(rows, L, H, 128).bfloat16()
    starts, lens = [0, 300], [500, 640]
    want = oracle.attention_fp32_reference(q, k, v, lens, starts, bt)
    got = ops.swa_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device),
                            torch.tensor(lens, dtype=torch.int32, device=gpu_device),
                            chunk_key_start=starts, mask_block_tokens=bt)
    torch.cuda.synchronize()
    _close(got, want)


@pytest.mark.gpu
def test_bad_mask_arguments(gpu_device):
    from streamdiffusionv2_amd import ops

    x = torch.zeros(1, 64, 1, 128, dtype=torch.bfloat16, device=gpu_device)
    kv = torch.zeros(1, 128, 1, 128, dtype=torch.bfloat16, device=gpu_device)
    with pytest.raises(RuntimeError):
        ops.swa_attention(x, kv, kv, None, mask_block_tokens=32)                       # no chunk position
    with pytest.raises(RuntimeError):
        ops.swa_attention(x, kv, kv, None, chunk_key_start=[100], mask_block_tokens=32)   # chunk leaves the view
    with pytest.raises(RuntimeError):
        ops.swa_attention(x, kv, kv, None, chunk_key_start=[0], mask_block_tokens=-1)


@pytest.mark.gpu
def test_stream_with_frame_blocks(gpu_device):
    """3-frame chunks with a per-frame mask through the ring path: slots,
    indices and cache bit-exact, attention within tolerance of the oracle
    running the same option."""
    from streamdiffusionv2_amd import ring, rope
    from streamdiffusionv2_amd.attention import RingKVPath

    grid, ft, heads, cache_frames = (3, 4, 8), 32, 2, 12
    S = 3 * ft
    freqs = rope.build_freqs()
    g_cache = ring.new_kv_cache(1, 1, cache_frames * ft, heads, 1, device=gpu_device)[0]
    o_cache = oracle.new_kv_cache(1, 1, cache_frames * ft, heads, 1)[0]
    g_path, o_path = RingKVPath(sink_size=1), oracle.RingAttentionOracle(sink_size=1)
    g_path.block_frames = o_path.block_frames = 1
    gen = torch.Generator().manual_seed(8)
    for call in range(7):                                   # fills after 4 chunks, then evicts
        q, k, v = (torch.randn(1, S, heads, 128, generator=gen).bfloat16() for _ in range(3))
        got = g_path.attend(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), torch.tensor([grid]), freqs,
                            g_cache, [call * S])
        _, roped_q, seq = o_path.step(q, k, v, [grid], freqs, o_cache, [call * S], with_attention=False)
        torch.cuda.synchronize()
        assert g_path.evict_idx == o_path.evict_idx
        for name in ("k", "v"):
            assert torch.equal(g_cache[name].cpu().view(torch.int16), o_cache[name].view(torch.int16)), (call, name)
        start = o_path.last_writes[0][0]
        want = oracle.attention_fp32_reference(roped_q, o_cache["k"], o_cache["v"], seq, [start], ft)
        plain = oracle.attention_fp32_reference(roped_q, o_cache["k"], o_cache["v"], seq)
        assert (want - plain).abs().max() > 0.05
        _close(got, want)
