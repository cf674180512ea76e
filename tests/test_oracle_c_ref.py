"""The PyTorch oracle pinned from another side: oracle/rope_ring_ref.c restates
the two bit-exact pieces of the path (causal_rope_apply with its table
expansion, causal_model.py:57-108; the placement state machine, :279-342) in
plain C, compiled with gcc and -ffp-contract=off.  The two restatements share
no code, so a slip in either (a wrong pair order, a fused multiply-add, a
rounding in the wrong place, an off-by-one in the queue) shows up as a
difference.  The C side is first checked on its own against the hand traces
and an identity case."""
import ctypes as C
import json
import os
import random

import numpy as np
import pytest
import torch

from oracle import build_c_ref
from oracle import sdv2_oracle as oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ring_traces.json")


@pytest.fixture(scope="module")
def cref():
    lib = C.CDLL(str(build_c_ref.build()))
    lib.sdv2_ref_rope.restype = C.c_int
    lib.sdv2_ref_rope.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_long]
    lib.sdv2_ref_ring_step.restype = C.c_long
    lib.sdv2_ref_ring_step.argtypes = [C.POINTER(C.c_long), C.POINTER(C.c_int), C.c_int, C.POINTER(C.c_long),
                                       C.POINTER(C.c_long), C.POINTER(C.c_int), C.c_int, C.c_int, C.c_long, C.c_long,
                                       C.c_long, C.c_long, C.c_int]
    return lib


def _c_rope(lib, x, grid, start_frame, table):
    """x [S, H, 128] bf16 -> roped bf16, through the C restatement."""
    src = np.ascontiguousarray(x.contiguous().view(torch.int16).numpy())
    dst = np.zeros_like(src)
    rc = lib.sdv2_ref_rope(src.ctypes.data, dst.ctypes.data, x.shape[1], table.ctypes.data, table.shape[0],
                           grid[0], grid[1], grid[2], start_frame)
    assert rc == 0
    return torch.from_numpy(dst).view(torch.bfloat16)


class _CRing:
    """One cache row driven through sdv2_ref_ring_step."""

    def __init__(self, lib, cap, frame_tokens, sink, total_steps=1, cache_rows=1):
        self.lib, self.cap, self.ft, self.sink, self.total, self.rows = lib, cap, frame_tokens, sink, total_steps, cache_rows
        self.queue = (C.c_long * 64)()
        self.n = C.c_int(0)
        self.g, self.l = C.c_long(0), C.c_long(0)
        self.step_ctr = C.c_int(total_steps)

    def step(self, start, tokens):
        return self.lib.sdv2_ref_ring_step(self.queue, C.byref(self.n), 64, C.byref(self.g), C.byref(self.l),
                                           C.byref(self.step_ctr), self.total, self.rows, self.cap, start, tokens,
                                           self.ft, self.sink)

    @property
    def q(self):
        return [self.queue[i] for i in range(self.n.value)]


def test_c_rope_identity_and_quarter_turn(cref):
    """Position (0, 0, 0) multiplies by 1 + 0i; a table of i everywhere maps
    (a, b) to (-b, a) - fixed by the definition, not by either restatement."""
    table = torch.view_as_real(oracle.build_freqs()).contiguous().numpy()
    x = torch.randn(1, 3, 128).bfloat16()
    assert torch.equal(_c_rope(cref, x, (1, 1, 1), 0, table).view(torch.int16), x.view(torch.int16))
    quarter = np.zeros((4, 64, 2))
    quarter[..., 1] = 1.0
    y = _c_rope(cref, x, (1, 1, 1), 2, quarter).float()
    xf = x.float()
    assert torch.equal(y[..., 0::2], -xf[..., 1::2]) and torch.equal(y[..., 1::2], xf[..., 0::2])
    assert cref.sdv2_ref_rope(0, 0, 1, table.ctypes.data, 1024, 2, 1, 1, 1023) == -1     # frame 1024 is off the table


@pytest.mark.parametrize("trace", json.load(open(GOLDEN))["traces"], ids=lambda t: t["name"])
def test_c_ring_hand_traces(cref, trace):
    ft = 6
    ring_c = _CRing(cref, trace["cache_frames"] * ft, ft, trace["sink_size"])
    start = 0
    for i, want in enumerate(trace["steps"]):
        frames = trace["first_chunk_frames"] if i == 0 else trace["chunk_frames"]
        dst = ring_c.step(start, frames * ft)
        assert [dst // ft, (dst + frames * ft) // ft] == want["write"]
        assert [x // ft for x in ring_c.q] == want["evict_idx"]
        assert ring_c.l.value // ft == want["local_end"]
        start += frames * ft


@pytest.mark.parametrize("seed", range(8))
def test_torch_oracle_rope_equals_c(cref, seed):
    rng = random.Random(seed)
    grid = (rng.randint(1, 3), rng.randint(1, 7), rng.randint(1, 9))
    heads = rng.randint(1, 5)
    S = grid[0] * grid[1] * grid[2]
    start = rng.randint(0, 1024 - grid[0])
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(1, S, heads, 128, generator=g) * rng.choice([0.1, 1.0, 30.0])).bfloat16()
    freqs = oracle.build_freqs()
    want = oracle.causal_rope_apply(x, [grid], freqs, [start]).type_as(x)
    got = _c_rope(cref, x[0], grid, start, torch.view_as_real(freqs).contiguous().numpy())
    assert torch.equal(got.view(torch.int16), want[0].view(torch.int16))


@pytest.mark.parametrize("seed", range(12))
def test_torch_oracle_ring_equals_c(cref, seed):
    """Random streams: ragged first chunk, resubmitted starts, several passes
    per chunk on a one-row cache; slot, queue, both indices and the pass
    counter after every call, including the call on which the reference
    raises IndexError."""
    rng = random.Random(100 + seed)
    ft = 4
    cap_frames, sink = rng.randint(2, 7), rng.randint(0, 3)
    chunk_frames = rng.choice([1, 1, 2])
    passes = rng.choice([1, 1, 2, 3])
    cap = cap_frames * ft
    cache = oracle.new_kv_cache(1, 1, cap, 1, passes, dtype=torch.float32)[0]
    layer = oracle.RingAttentionOracle(sink_size=sink, adapt_sink_thr=-1)
    ring_c = _CRing(cref, cap, ft, sink, total_steps=passes)
    freqs = oracle.build_freqs()
    start = 0
    for call in range(cap_frames + 6):
        frames = rng.randint(1, 2) if call == 0 else chunk_frames
        tokens = frames * ft
        x = torch.zeros(1, tokens, 1, 128)
        for _ in range(passes):
            try:
                layer.step(x, x, x, [(frames, 2, 2)], freqs, cache, [start], with_attention=False)
                raised = False
            except (IndexError, ValueError, RuntimeError):
                raised = True
            dst = ring_c.step(start, tokens)
            if raised:
                assert dst < 0 or dst + tokens > cap
                return
            assert (dst, dst + tokens) == tuple(layer.last_writes[0])
            assert ring_c.q == list(layer.evict_idx[0])
            assert ring_c.g.value == int(cache["global_end_index"][0]) and ring_c.l.value == int(cache["local_end_index"][0])
            assert ring_c.step_ctr.value == cache["current_step"]
        if rng.random() < 0.85:
            start += tokens          # otherwise the same start is submitted again
