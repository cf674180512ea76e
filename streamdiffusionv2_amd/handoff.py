"""Hand-off of a layer's KV-cache block between owners.

Mirror of ``KVCacheManager`` (streamv2v/communication/kv_cache_manager.py):
who owns which block (``compute_block_owners`` :86-108), which blocks move
when the intervals change (``rebalance_kv_cache_by_diff`` :110-148) and what a
move does to the receiver's dict (``broadcast_kv_blocks`` :48-84): k, v and the
two index tensors are replaced by the donor's, and a receiver of lower rank
adds ``frame_seq_length * (donor - rank) * num_steps`` to ``global_end_index``.

What is built here is everything on ONE device: the wire format and the two
copies at its ends.  The reference broadcasts its token-major
[B, cap, H, 128] tensors as they are; this package keeps a cache head-major in
HBM, so a block is brought into the reference's wire layout by
``export_block`` (one launch per tensor, ``sdv2_cache_relayout``) and absorbed
by ``import_block`` (the same kernel the other way, with the index hand-over
and the rank shift folded into the launch).  The transport between the two is
the caller's: ``KVCacheManager`` takes it as the ``exchange`` callable, which on
several GPUs would broadcast the four wire tensors from the donor and here
defaults to handing the donor's wire straight back.

The eviction queues (``evict_idx``) are module state in the reference and are
not part of its broadcast; they are not moved here either.  With the adaptive
sink refresh on, read a layer's ``evict_idx`` (or call its ``settle()``) before
its block changes owner, so that no decision is still on its way to the host.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence

import torch

from . import ops, ring


@dataclass
class BlockWire:
    """One block as it travels: the reference's tensors, token-major and
    contiguous (kv_cache_manager.py:70-78)."""
    k: torch.Tensor                    # [B, cap, H, 128]
    v: torch.Tensor
    global_end_index: torch.Tensor     # int64 [B]
    local_end_index: torch.Tensor

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.k, self.v, self.global_end_index, self.local_end_index))


def _intervals(block_intervals) -> List[List[int]]:
    if isinstance(block_intervals, torch.Tensor):
        return [[int(a), int(b)] for a, b in block_intervals.tolist()]
    return [[int(a), int(b)] for a, b in block_intervals]


def compute_block_owners(block_intervals, total_blocks: int) -> List[int]:
    """Owner rank of every block for [start, end) intervals per rank, -1 where
    no interval covers it; later ranks win overlaps
    (kv_cache_manager.py:98-106)."""
    owners = [-1] * total_blocks
    for r, (s, e) in enumerate(_intervals(block_intervals)):
        if e > s:
            # python slice semantics of owners[s:e] = r
            for i in range(*slice(s, e).indices(total_blocks)):
                owners[i] = r
    return owners


def moved_blocks_by_donor(old_block_intervals, new_block_intervals, total_blocks: int) -> Dict[int, List[int]]:
    """Blocks whose owner changes, grouped by previous owner, in the order the
    reference visits them (kv_cache_manager.py:128-136); blocks nobody owned
    before are not moved."""
    old = compute_block_owners(old_block_intervals, total_blocks)
    new = compute_block_owners(new_block_intervals, total_blocks)
    moved: Dict[int, List[int]] = {}
    for i in range(total_blocks):
        if old[i] != new[i] and old[i] >= 0:
            moved.setdefault(old[i], []).append(i)
    return moved


def global_end_shift(donor_rank: int, rank: int, frame_seq_length: int, time_step_length: int) -> int:
    """What a receiver adds to ``global_end_index`` (kv_cache_manager.py:81-82):
    a lower-ranked stage is ``donor - rank`` pipeline slots ahead in the
    stream, each slot worth ``num_steps`` frames of tokens."""
    return frame_seq_length * (donor_rank - rank) * time_step_length if donor_rank > rank else 0


def new_wire_like(entry: dict) -> BlockWire:
    k = entry["k"]
    return BlockWire(
        k=torch.empty(tuple(k.shape), dtype=k.dtype, device=k.device),
        v=torch.empty(tuple(k.shape), dtype=k.dtype, device=k.device),
        global_end_index=torch.empty_like(entry["global_end_index"]),
        local_end_index=torch.empty_like(entry["local_end_index"]),
    )


def export_block(entry: dict, wire: Optional[BlockWire] = None) -> BlockWire:
    """The donor's side: the dict's tensors in the reference's layout."""
    if wire is None:
        wire = new_wire_like(entry)
    src_idx = (entry["global_end_index"], entry["local_end_index"])
    ops.cache_relayout(wire.k, entry["k"], (wire.global_end_index, wire.local_end_index), src_idx, 0)
    ops.cache_relayout(wire.v, entry["v"])
    return wire


def import_block(entry: dict, wire: BlockWire, donor_rank: int, rank: int, frame_seq_length: int,
                 time_step_length: int) -> None:
    """The receiver's side: the dict's tensors are overwritten in place (they
    keep their layout and identity) and ``global_end_index`` is shifted."""
    shift = global_end_shift(donor_rank, rank, frame_seq_length, time_step_length)
    dst_idx = (entry["global_end_index"], entry["local_end_index"])
    ops.cache_relayout(entry["k"], wire.k, dst_idx, (wire.global_end_index, wire.local_end_index), shift)
    ops.cache_relayout(entry["v"], wire.v)
    ring.forget_index_mirror(entry)      # the host copy of the indices is stale now


class KVCacheManager:
    """Same surface as the reference class; ``rank`` is given instead of read
    from a process group, and the transport is the ``exchange`` callable
    ``(wire, block_index, donor_rank) -> wire`` (default: loop back)."""

    def __init__(self, pipeline, device, rank: int = 0,
                 exchange: Optional[Callable[[BlockWire, int, int], BlockWire]] = None):
        self.pipeline = pipeline
        self.device = torch.device(device)
        self.rank = rank
        self.frame_seq_length = pipeline.frame_seq_length
        self.time_step_length = len(pipeline.denoising_step_list)
        self.exchange = exchange if exchange is not None else (lambda wire, block_index, donor_rank: wire)

    def broadcast_kv_blocks(self, block_indices: Sequence[int], donor_rank: int) -> None:
        """kv_cache_manager.py:48-84.  The donor keeps its block untouched (a
        broadcast leaves the source as it is, and its shift is zero)."""
        for bi in block_indices:
            entry = self.pipeline.kv_cache1[bi]
            wire = export_block(entry) if self.rank == donor_rank else new_wire_like(entry)
            wire = self.exchange(wire, bi, donor_rank)
            if self.rank != donor_rank:
                import_block(entry, wire, donor_rank, self.rank, self.frame_seq_length, self.time_step_length)

    def compute_block_owners(self, block_intervals, total_blocks: int) -> torch.Tensor:
        return torch.tensor(compute_block_owners(block_intervals, total_blocks), dtype=torch.int64)

    def rebalance_kv_cache_by_diff(self, old_block_intervals, new_block_intervals, total_blocks: int) -> int:
        """kv_cache_manager.py:110-148; returns the number of donors."""
        moved = moved_blocks_by_donor(old_block_intervals, new_block_intervals, total_blocks)
        for src, blocks in moved.items():
            self.broadcast_kv_blocks(blocks, donor_rank=src)
        return len(moved)

    def get_kv_cache_statistics(self, block_intervals, total_blocks: int) -> dict:
        """kv_cache_manager.py:150-183."""
        owners = compute_block_owners(block_intervals, total_blocks)
        counts = {r: owners.count(r) for r in range(len(_intervals(block_intervals)))}
        per_block = 0
        cache = getattr(self.pipeline, "kv_cache1", None)
        if cache:
            first = cache[0]
            if "k" in first and "v" in first:
                per_block = sum(first[n].numel() * first[n].element_size() for n in ("k", "v"))
        return {
            "block_counts": counts,
            "memory_usage_bytes": {r: c * per_block for r, c in counts.items()},
            "total_blocks": total_blocks,
            "memory_per_block_bytes": per_block,
            "frame_seq_length": self.frame_seq_length,
        }

    def validate_kv_cache_consistency(self, block_intervals, total_blocks: int) -> bool:
        """kv_cache_manager.py:205-241."""
        owners = compute_block_owners(block_intervals, total_blocks)
        if any(o == -1 for o in owners):
            return False
        for r, (s, e) in enumerate(_intervals(block_intervals)):
            if s < 0 or e > total_blocks or s >= e:
                return False
            if any(owners[i] != r for i in range(s, e)):
                return False
        return True

    def cleanup_kv_cache(self, block_intervals, total_blocks: int) -> int:
        """Zero k and v of the blocks this rank does not own
        (kv_cache_manager.py:243-266); returns how many."""
        owners = compute_block_owners(block_intervals, total_blocks)
        cache = getattr(self.pipeline, "kv_cache1", None) or []
        cleaned = 0
        for bi in range(total_blocks):
            if owners[bi] != self.rank and bi < len(cache):
                for n in ("k", "v"):
                    if n in cache[bi]:
                        cache[bi][n].zero_()
                cleaned += 1
        return cleaned
