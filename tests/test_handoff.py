"""Hand-off of a cache block between owners
(streamv2v/communication/kv_cache_manager.py:48-148).

CPU: the oracle's restatement of the ownership logic against the cases the
reference's own tests hold (streamv2v/communication/test_communication.py:303-337:
three ranks x ten blocks; statistics; a gap in the intervals is inconsistent)
and hand-worked ones, then the package's host logic against the oracle.

GPU: the wire format is the reference's token-major contiguous tensor, so the
export must equal ``.contiguous()`` of the logical cache bit for bit, the
import must restore it bit for bit in either physical layout, the indices must
arrive with the rank shift, and a stream continued on the receiving cache must
go on exactly like the oracle's uninterrupted stream.
"""
import pytest
import torch

from oracle import sdv2_oracle as oracle
from streamdiffusionv2_amd import handoff


class _Pipe:
    """What KVCacheManager reads from a pipeline (kv_cache_manager.py:32-35)."""

    def __init__(self, kv_cache1, frame_seq_length=16, steps=(700, 500, 0)):
        self.kv_cache1 = kv_cache1
        self.frame_seq_length = frame_seq_length
        self.denoising_step_list = list(steps)


def _reference_fixture_cache(n=30):
    g = torch.Generator().manual_seed(0)
    return [{"k": torch.randn(1, 8, 16, 64, generator=g), "v": torch.randn(1, 8, 16, 64, generator=g),
             "global_end_index": torch.tensor([16]), "local_end_index": torch.tensor([16])} for _ in range(n)]


# ---------------------------------------------------------------- oracle pins
def test_oracle_owners_reference_case():
    # test_communication.py:303-311
    owners = oracle.compute_block_owners(torch.tensor([[0, 10], [10, 20], [20, 30]]), 30)
    assert owners.shape == (30,)
    assert owners.tolist() == [0] * 10 + [1] * 10 + [2] * 10


def test_oracle_owners_hand_cases():
    # a gap stays -1, an empty or inverted interval owns nothing, a later rank wins an overlap
    assert oracle.compute_block_owners(torch.tensor([[0, 2], [3, 5]]), 6).tolist() == [0, 0, -1, 1, 1, -1]
    assert oracle.compute_block_owners(torch.tensor([[0, 4], [2, 2], [3, 1]]), 4).tolist() == [0, 0, 0, 0]
    assert oracle.compute_block_owners(torch.tensor([[0, 3], [2, 5]]), 5).tolist() == [0, 0, 1, 1, 1]
    # an interval reaching past the end is cut by the slice
    assert oracle.compute_block_owners(torch.tensor([[0, 2], [2, 9]]), 4).tolist() == [0, 0, 1, 1]


def test_oracle_moved_blocks_hand_case():
    old = torch.tensor([[0, 10], [10, 20], [20, 30]])
    new = torch.tensor([[0, 8], [8, 22], [22, 30]])
    # blocks 8, 9 leave rank 0; blocks 20, 21 leave rank 2; nothing leaves rank 1
    assert oracle.moved_blocks_by_donor(old, new, 30) == {0: [8, 9], 2: [20, 21]}
    assert oracle.moved_blocks_by_donor(old, old, 30) == {}
    # a block nobody owned before is not moved
    assert oracle.moved_blocks_by_donor(torch.tensor([[0, 2], [3, 4]]), torch.tensor([[0, 3], [3, 4]]), 4) == {}


def test_oracle_receive_block_hand_case():
    donor = {"k": torch.arange(24.).view(1, 3, 2, 4), "v": -torch.arange(24.).view(1, 3, 2, 4),
             "global_end_index": torch.tensor([4680]), "local_end_index": torch.tensor([3120])}
    for rank, want_global in ((0, 4680 + 1560 * 2 * 4), (1, 4680 + 1560 * 1 * 4), (2, 4680), (3, 4680)):
        mine = {"k": torch.zeros(1, 3, 2, 4), "v": torch.zeros(1, 3, 2, 4),
                "global_end_index": torch.tensor([7]), "local_end_index": torch.tensor([9])}
        k_before = mine["k"]
        oracle.receive_kv_block(mine, donor, donor_rank=2, rank=rank, frame_seq_length=1560, time_step_length=4)
        assert mine["k"] is k_before and torch.equal(mine["k"], donor["k"]) and torch.equal(mine["v"], donor["v"])
        assert mine["global_end_index"].tolist() == [want_global]
        assert mine["local_end_index"].tolist() == [3120]
    assert donor["global_end_index"].tolist() == [4680]


# ------------------------------------------------------- host logic vs oracle
def test_package_owner_logic_matches_oracle():
    g = torch.Generator().manual_seed(5)
    for _ in range(200):
        world = int(torch.randint(1, 6, (1,), generator=g))
        total = int(torch.randint(1, 40, (1,), generator=g))
        iv = torch.randint(0, total + 3, (world, 2), generator=g)
        iv2 = torch.randint(0, total + 3, (world, 2), generator=g)
        assert handoff.compute_block_owners(iv, total) == oracle.compute_block_owners(iv, total).tolist()
        assert handoff.compute_block_owners(iv.tolist(), total) == oracle.compute_block_owners(iv, total).tolist()
        assert handoff.moved_blocks_by_donor(iv, iv2, total) == oracle.moved_blocks_by_donor(iv, iv2, total)


def test_global_end_shift():
    assert handoff.global_end_shift(2, 0, 1560, 4) == 12480
    assert handoff.global_end_shift(2, 1, 1560, 4) == 6240
    assert handoff.global_end_shift(2, 2, 1560, 4) == 0
    assert handoff.global_end_shift(1, 3, 1560, 4) == 0


def test_manager_reference_cases():
    # test_communication.py:281-337
    mgr = handoff.KVCacheManager(_Pipe(_reference_fixture_cache()), torch.device("cpu"))
    assert mgr.frame_seq_length == 16 and mgr.time_step_length == 3
    iv = torch.tensor([[0, 10], [10, 20], [20, 30]])
    owners = mgr.compute_block_owners(iv, 30)
    assert owners.shape == (30,)
    assert torch.all(owners[:10] == 0) and torch.all(owners[10:20] == 1) and torch.all(owners[20:30] == 2)
    stats = mgr.get_kv_cache_statistics(iv, 30)
    assert stats["total_blocks"] == 30
    assert stats["block_counts"] == {0: 10, 1: 10, 2: 10}
    assert stats["memory_per_block_bytes"] == 2 * 8 * 16 * 64 * 4
    assert stats["memory_usage_bytes"][1] == 10 * stats["memory_per_block_bytes"]
    assert stats["frame_seq_length"] == 16
    assert mgr.validate_kv_cache_consistency(iv, 30)
    assert not mgr.validate_kv_cache_consistency(torch.tensor([[0, 10], [10, 20], [20, 25]]), 30)
    assert not mgr.validate_kv_cache_consistency(torch.tensor([[0, 10], [10, 10], [10, 30]]), 30)


def test_manager_cleanup_zeroes_foreign_blocks():
    cache = _reference_fixture_cache(6)
    mgr = handoff.KVCacheManager(_Pipe(cache), torch.device("cpu"), rank=1)
    assert mgr.cleanup_kv_cache(torch.tensor([[0, 2], [2, 4], [4, 6]]), 6) == 4
    for bi in range(6):
        empty = not cache[bi]["k"].any() and not cache[bi]["v"].any()
        assert empty == (bi not in (2, 3))


# ------------------------------------------------------------------------ GPU
def _bits(t):
    return t.contiguous().view(torch.int16 if t.dtype == torch.bfloat16 else torch.int32)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 37, 5), (3, 260, 12), (2, 64, 40)])
def test_relayout_round_trip(gpu_device, dtype, shape):
    from streamdiffusionv2_amd import ops, ring

    rows, cap, heads = shape
    print(f"relayout: rows={rows} cap={cap} heads={heads} {dtype}", flush=True)
    torch.manual_seed(rows * 1000 + cap)
    logical = torch.randn(rows, cap, heads, 128).to(dtype)
    entry = ring.new_kv_cache(1, rows, cap, heads, 1, dtype=dtype, device=gpu_device)[0]
    assert entry["k"].stride(2) > entry["k"].stride(1)          # head-major in memory
    entry["k"].copy_(logical.to(gpu_device))
    wire = torch.full((rows, cap, heads, 128), 7.0, dtype=dtype, device=gpu_device)
    ops.cache_relayout(wire, entry["k"])
    torch.cuda.synchronize()
    assert wire.is_contiguous() and torch.equal(_bits(wire.cpu()), _bits(logical))
    # back into head-major, into token-major, and into a cache with room to spare (larger row stride)
    for target in (ring.new_kv_cache(1, rows, cap, heads, 1, dtype=dtype, device=gpu_device)[0]["k"],
                   torch.zeros(rows, cap, heads, 128, dtype=dtype, device=gpu_device),
                   torch.zeros(rows, heads, cap + 9, 128, dtype=dtype, device=gpu_device).permute(0, 2, 1, 3)[:, :cap]):
        ops.cache_relayout(target, wire)
        torch.cuda.synchronize()
        assert torch.equal(_bits(target.cpu()), _bits(logical))
    spare = torch.zeros(rows, heads, cap + 9, 128, dtype=dtype, device=gpu_device)
    ops.cache_relayout(spare.permute(0, 2, 1, 3)[:, :cap], wire)
    torch.cuda.synchronize()
    assert not spare[:, :, cap:].any()                         # nothing written past the block


@pytest.mark.gpu
def test_relayout_indices_and_errors(gpu_device):
    from streamdiffusionv2_amd import ops

    src = torch.randn(2, 8, 3, 128, device=gpu_device).bfloat16()
    dst = torch.zeros_like(src)
    sg, sl = torch.tensor([100, 200], device=gpu_device), torch.tensor([30, 40], device=gpu_device)
    dg, dl = torch.zeros(2, dtype=torch.int64, device=gpu_device), torch.zeros(2, dtype=torch.int64, device=gpu_device)
    ops.cache_relayout(dst, src, (dg, dl), (sg, sl), global_end_shift=12480)
    torch.cuda.synchronize()
    assert torch.equal(dst, src)
    assert dg.tolist() == [12580, 12680] and dl.tolist() == [30, 40]
    assert sg.tolist() == [100, 200]
    # indices only
    empty = src[:, :0]
    dg.zero_()
    ops.cache_relayout(torch.zeros_like(empty), empty, (dg, dl), (sg, sl), global_end_shift=-1)
    torch.cuda.synchronize()
    assert dg.tolist() == [99, 199]
    with pytest.raises(RuntimeError):            # shapes differ
        ops.cache_relayout(dst[:, :4], src)
    with pytest.raises(RuntimeError):            # dtype differs
        ops.cache_relayout(dst.float(), src)
    with pytest.raises(RuntimeError):            # one index pair only
        ops.cache_relayout(dst, src, (dg, dl), None)
    with pytest.raises(RuntimeError):            # destination rows alias each other
        ops.cache_relayout(dst[:1].expand(2, -1, -1, -1), src)
    with pytest.raises(RuntimeError):            # no CPU path
        ops.cache_relayout(dst.cpu(), src.cpu())


@pytest.mark.gpu
@pytest.mark.parametrize("receiver_head_major", [True, False])
@pytest.mark.parametrize("donor_rank,rank", [(0, 1), (2, 0)])
def test_stream_continues_on_the_receiver(gpu_device, receiver_head_major, donor_rank, rank):
    """Five chunks on the donor (the ring wraps at the fourth), hand-off of
    every layer's block, then four more chunks on the receiver; the oracle runs
    the nine chunks on one cache, with receive_kv_block applied to its indices
    at the same point."""
    from streamdiffusionv2_amd import ring, rope
    from streamdiffusionv2_amd.attention import RingKVPath

    print(f"hand-off stream: donor {donor_rank} -> rank {rank}, head-major receiver {receiver_head_major}", flush=True)
    layers, heads, grid, cap_frames, steps = 2, 3, (1, 4, 6), 3, 2
    S = grid[1] * grid[2]
    cap = cap_frames * S
    freqs = rope.build_freqs()
    donor = ring.new_kv_cache(layers, 1, cap, heads, 1, device=gpu_device)
    recv = ring.new_kv_cache(layers, 1, cap, heads, 1, device=gpu_device, head_major=receiver_head_major)
    o_cache = oracle.new_kv_cache(layers, 1, cap, heads, 1)
    paths = [RingKVPath(sink_size=1) for _ in range(layers)]
    o_paths = [oracle.RingAttentionOracle(sink_size=1) for _ in range(layers)]
    pipe_d, pipe_r = _Pipe(donor, S, range(steps)), _Pipe(recv, S, range(steps))
    wires = {}
    mgr_d = handoff.KVCacheManager(pipe_d, gpu_device, rank=donor_rank,
                                   exchange=lambda w, bi, src: wires.setdefault(bi, w))
    mgr_r = handoff.KVCacheManager(pipe_r, gpu_device, rank=rank, exchange=lambda w, bi, src: wires[bi])
    gen = torch.Generator().manual_seed(11)
    shift = handoff.global_end_shift(donor_rank, rank, S, steps)
    start = 0
    for call in range(9):
        if call == 5:
            old = [[0, layers] if r == donor_rank else [0, 0] for r in range(3)]
            new = [[0, layers] if r == rank else [0, 0] for r in range(3)]
            moved = handoff.moved_blocks_by_donor(old, new, layers)
            assert moved == {donor_rank: list(range(layers))}
            mgr_d.broadcast_kv_blocks(moved[donor_rank], donor_rank)
            mgr_r.broadcast_kv_blocks(moved[donor_rank], donor_rank)
            torch.cuda.synchronize()
            for layer in range(layers):
                w = wires[layer]
                assert w.k.is_contiguous() and w.v.is_contiguous()
                assert torch.equal(_bits(w.k.cpu()), _bits(o_cache[layer]["k"]))
                assert torch.equal(_bits(w.v.cpu()), _bits(o_cache[layer]["v"]))
                before = {n: o_cache[layer][n].clone() for n in ("k", "v", "global_end_index", "local_end_index")}
                oracle.receive_kv_block(o_cache[layer], before, donor_rank, rank, S, steps)
                for n in ("k", "v"):
                    assert torch.equal(_bits(recv[layer][n].cpu()), _bits(o_cache[layer][n])), (layer, n)
                    assert torch.equal(donor[layer][n], before[n].to(gpu_device))      # the donor keeps its block
                for n in ("global_end_index", "local_end_index"):
                    assert recv[layer][n].tolist() == o_cache[layer][n].tolist()
                assert recv[layer]["global_end_index"].tolist() == [before["global_end_index"].item() + shift]
            start += shift          # the receiving stage is that much further on in the stream
        cache = donor if call < 5 else recv
        for layer in range(layers):
            q, k, v = (torch.randn(1, S, heads, 128, generator=gen).bfloat16() for _ in range(3))
            got = paths[layer].attend(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), torch.tensor([grid]), freqs,
                                      cache[layer], [start])
            _, want_q, seq = o_paths[layer].step(q, k, v, [list(grid)], freqs, o_cache[layer], [start],
                                                 with_attention=False)
            torch.cuda.synchronize()
            assert paths[layer].evict_idx == o_paths[layer].evict_idx
            for n in ("global_end_index", "local_end_index"):
                assert cache[layer][n].tolist() == o_cache[layer][n].tolist(), (call, n)
            for n in ("k", "v"):
                assert torch.equal(_bits(cache[layer][n].cpu()), _bits(o_cache[layer][n])), (call, layer, n)
            ref = oracle.attention_fp32_reference(want_q, o_cache[layer]["k"], o_cache[layer]["v"], seq)
            err = (got.float().cpu() - ref).abs()
            assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3
        start += S
