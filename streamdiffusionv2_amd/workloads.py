"""Synthetic stream workloads for the KV-cache path (benchmark + parity tests).

Five shapes, from the CPU-plumbing case to a 720p long-window stress; each is
a stream of equal chunks through ``layers`` independent ring caches.  Inputs
are seeded N(0,1) per (chunk, layer) so the GPU path and the CPU oracle see the
same numbers.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Tuple

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    dtype: torch.dtype
    layers: int
    rows: int                   # stream batch B (one cache per denoising stage)
    heads: int
    grid: Tuple[int, int, int]  # (f, h, w) of one chunk
    cache_frames: int
    chunks: int
    input_scale: float = 1.0
    outlier_fraction: float = 0.0   # share of K token rows scaled x8
    sink_size: int = 1

    @property
    def frame_tokens(self) -> int:
        return self.grid[1] * self.grid[2]

    @property
    def chunk_tokens(self) -> int:
        return self.grid[0] * self.frame_tokens

    @property
    def cache_tokens(self) -> int:
        return self.cache_frames * self.frame_tokens

    # algorithmic traffic / work of one layer call in steady state (cache full)
    def append_bytes(self, with_q: bool = True) -> int:
        e = 2 if self.dtype == torch.bfloat16 else 4
        n = self.rows * self.chunk_tokens * self.heads * 128 * e
        return (6 if with_q else 4) * n

    def attn_flops(self) -> int:
        return 4 * self.rows * self.heads * self.chunk_tokens * self.cache_tokens * 128

    def attn_bytes(self) -> int:
        e = 2
        return 2 * self.rows * self.heads * 128 * e * (self.cache_tokens + self.chunk_tokens)


WORKLOADS = {
    1: Workload("c1_cpu_fp32_plumbing", torch.float32, 1, 1, 12, (1, 30, 52), 4, 10),
    2: Workload("c2_wan1.3b_1560tok_6frames", torch.bfloat16, 30, 1, 12, (1, 30, 52), 6, 50,
                input_scale=128 ** -0.5),
    3: Workload("c3_wan1.3b_b4_4680tok_12frames", torch.bfloat16, 30, 4, 12, (3, 30, 52), 12, 40),
    4: Workload("c4_wan14b_1560tok_6frames", torch.bfloat16, 40, 1, 40, (1, 30, 52), 6, 30),
    5: Workload("c5_720p_b2_10800tok_21frames", torch.bfloat16, 30, 2, 12, (3, 45, 80), 21, 25,
                outlier_fraction=0.01),
}


def make_qkv(w: Workload, chunk: int, layer: int, seed: int = 0, rows: int = None):
    """Seeded q, k, v [rows, S, H, 128] on the CPU in the workload's dtype."""
    rows = w.rows if rows is None else rows
    gen = torch.Generator().manual_seed(seed + 1000 * chunk + layer)
    shape = (rows, w.chunk_tokens, w.heads, 128)
    q = torch.randn(shape, generator=gen) * w.input_scale
    k = torch.randn(shape, generator=gen) * w.input_scale
    v = torch.randn(shape, generator=gen) * w.input_scale
    if w.outlier_fraction > 0:
        hot = torch.rand((rows, w.chunk_tokens, 1, 1), generator=gen) < w.outlier_fraction
        k = torch.where(hot, k * 8.0, k)
    return q.to(w.dtype), k.to(w.dtype), v.to(w.dtype)


class InputPool:
    """Inputs for long streams without a random-number pass per call: one
    seeded N(0,1) pool in the workload's dtype, of which q, k and v of every
    (chunk, layer) are windows at distinct offsets (so no two calls see the same
    tensors, and the GPU path and the CPU oracle see the same numbers).  The
    outlier rows of a workload are drawn per call from its own seed."""

    def __init__(self, w: Workload, seed: int = 0, offsets: int = 1 << 16):
        self.w = w
        self.n = w.rows * w.chunk_tokens * w.heads * 128
        self.span = 8 * offsets
        gen = torch.Generator().manual_seed(seed)
        self.pool = (torch.randn(3 * (self.n + self.span), generator=gen) * w.input_scale).to(w.dtype)
        self.seed = seed

    def qkv(self, chunk: int, layer: int, rows: int = None):
        w = self.w
        rows = w.rows if rows is None else rows
        n = rows * w.chunk_tokens * w.heads * 128
        off = 8 * ((chunk * 7919 + layer * 104729 + 13) % (self.span // 8))
        shape = (rows, w.chunk_tokens, w.heads, 128)
        q, k, v = (self.pool[off + j * (self.n + self.span):][:n].view(shape) for j in range(3))
        if w.outlier_fraction > 0:
            gen = torch.Generator().manual_seed(self.seed + 1000 * chunk + layer)
            hot = torch.rand((rows, w.chunk_tokens), generator=gen) < w.outlier_fraction
            k = k.clone()
            k[hot] = k[hot] * 8.0
        return q, k, v


def row_chunks(w: Workload, call: int) -> List[int]:
    """Chunk number each row works on at call ``call`` of a staggered stream
    batch.  Call 0 is the first chunk on every row (the reference runs it once
    and replicates the cache); afterwards row j trails row 0 by j chunks and
    rows that have not started yet resubmit chunk 1, as the shift register of
    the stream driver does (causal_stream_inference.py:248-249, 265-272)."""
    if call == 0:
        return [0] * w.rows
    return [max(call - j, 1) for j in range(w.rows)]


def row_starts(w: Workload, call: int) -> List[int]:
    """current_start per row: absolute token offset of the row's chunk."""
    return [c * w.chunk_tokens for c in row_chunks(w, call)]
