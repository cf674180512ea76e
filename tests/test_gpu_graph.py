"""A layer call recorded into a HIP graph replays exactly.

The library's entry points only enqueue kernels on the caller's stream: no
allocation, no synchronisation, no memory-set node.  A caller with a fixed
schedule can therefore capture them (append, attention with its merge, and the
adaptive sink decision that hands its slot to the append on the device) and
replay the graph on new inputs.  Every replay is compared bit for bit with the
same calls made eagerly on the same data, with eager work and a synchronisation
between replays.
"""
import pytest
import torch

from oracle import sdv2_oracle as oracle

pytestmark = pytest.mark.gpu

MAX_ABS = 2e-2
MEAN_ABS = 2e-3


def _bits(t):
    return t.contiguous().view(torch.int16)


class _Layer:
    """Static tensors of one layer call: two rows, head-major caches that are
    full (every key valid), a 120-token chunk (ragged query and key tiles)."""

    def __init__(self, dev, seed):
        from streamdiffusionv2_amd import ops

        self.grid, self.heads, self.rows = (1, 10, 12), 3, 2
        self.tokens, self.cap = 120, 600
        gen = torch.Generator().manual_seed(seed)
        shape = (self.rows, self.tokens, self.heads, 128)
        self.q = torch.zeros(shape, dtype=torch.bfloat16, device=dev)
        self.k = torch.zeros_like(self.q)
        self.v = torch.zeros_like(self.q)
        self.q_out = torch.zeros_like(self.q)
        self.out = torch.zeros_like(self.q)
        cache_shape = (self.rows, self.heads, self.cap, 128)
        self.kc = (torch.randn(cache_shape, generator=gen) * 0.5).bfloat16().to(dev).permute(0, 2, 1, 3)
        self.vc = (torch.randn(cache_shape, generator=gen) * 0.5).bfloat16().to(dev).permute(0, 2, 1, 3)
        self.g_idx = torch.zeros(self.rows, dtype=torch.long, device=dev)
        self.l_idx = torch.zeros(self.rows, dtype=torch.long, device=dev)
        self.seq_lens = torch.full((self.rows,), self.cap, dtype=torch.int32, device=dev)
        self.table = ops.device_freqs(oracle.build_freqs(), dev)
        self.override = torch.full((self.rows,), -1, dtype=torch.long, device=dev)
        self.refresh = torch.full((self.rows,), -7, dtype=torch.int32, device=dev)
        need = ops._capi.lib().sdv2_swa_attn_workspace_bytes(self.rows, self.tokens, self.heads, self.cap, 3)
        self.workspace = ops.new_workspace(dev, need)

    def load(self, gen):
        shape = tuple(self.q.shape)
        for t in (self.q, self.k, self.v):
            t.copy_((torch.randn(shape, generator=gen) * 0.5).bfloat16())

    def call(self, adaptive):
        from streamdiffusionv2_amd import ops

        starts, dst = [9, 4], [360, 240]
        override = None
        if adaptive:
            # sink of two frames, both rows about to evict: the slot comes from the device
            ops.sink_similarity(self.k, self.v, self.kc, self.vc, self.table, self.grid[1:], starts, 2, 0.5,
                                dst_start_override=self.override, override_rows=[True, True],
                                refresh_out=self.refresh)
            override = self.override
        ops.kv_append_rope(self.q, self.k, self.v, self.kc, self.vc, self.table, self.grid, starts, dst,
                           q_out=self.q_out, global_end_index=self.g_idx, local_end_index=self.l_idx,
                           new_global_end=[1200, 600], new_local_end=[600, 600], dst_start_override=override)
        ops.swa_attention(self.q_out, self.kc, self.vc, self.seq_lens, out=self.out, num_splits=3,
                          workspace=self.workspace)

    def state(self):
        return [t.clone() for t in (self.q_out, self.out, self.kc, self.vc, self.g_idx, self.l_idx, self.override,
                                    self.refresh)]


@pytest.mark.parametrize("adaptive", [False, True])
def test_layer_call_replays_from_a_hip_graph(gpu_device, adaptive):
    dev = gpu_device
    eager, graphed = _Layer(dev, seed=5), _Layer(dev, seed=5)
    warm = torch.Generator().manual_seed(1)
    for layer in (eager, graphed):           # first calls set up per-device state outside the capture
        layer.load(warm)
        layer.call(adaptive)
    torch.cuda.synchronize()
    graphed.kc.copy_(eager.kc)
    graphed.vc.copy_(eager.vc)

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):            # records on a side stream of default priority
        graphed.call(adaptive)
    torch.cuda.synchronize()
    # what the capture itself did or did not execute must not matter
    graphed.kc.copy_(eager.kc)
    graphed.vc.copy_(eager.vc)

    refreshed = set()
    for replay in range(4):
        data = torch.Generator().manual_seed(100 + replay)
        eager.load(data)
        data = torch.Generator().manual_seed(100 + replay)
        graphed.load(data)
        for layer in (eager, graphed):
            layer.g_idx.zero_()
            layer.override.fill_(-1)
            layer.refresh.fill_(-7)
        eager.call(adaptive)
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("q_out", "out", "k cache", "v cache", "global end", "local end", "override", "refresh"),
                              eager.state(), graphed.state()):
            same = torch.equal(_bits(a), _bits(b)) if a.dtype == torch.bfloat16 else torch.equal(a, b)
            assert same, f"replay {replay}: {name} differs from the eager call"
        assert graphed.g_idx.tolist() == [1200, 600]
        if adaptive:
            refreshed.update(graphed.refresh.tolist())
            for r, frame in enumerate(graphed.refresh.tolist()):
                assert graphed.override[r].item() == (frame * graphed.tokens if frame >= 0 else -1)
        # the eager side against the fp32 oracle, once: the comparison above is not two wrong results
        if replay == 0:
            want = oracle.attention_fp32_reference(eager.q_out.cpu(), eager.kc.cpu(), eager.vc.cpu(),
                                                   [eager.cap] * eager.rows)
            err = (graphed.out.cpu().float() - want.float()).abs()
            assert err.max().item() <= MAX_ABS and err.mean().item() <= MEAN_ABS
    if adaptive:
        assert refreshed - {-7}, "the decision kernel never ran in a replay"
