"""Adapters that put the CPU oracle layer, or the GPU path with a call trace,
behind the attend() call the generator stand-in of the stream drivers makes."""
from oracle import sdv2_oracle as oracle


class OraclePath:
    """Adapter: the oracle layer behind the attend() call of the package."""

    def __init__(self):
        self.inner = oracle.RingAttentionOracle()
        self.trace = []

    sink_size = property(lambda s: s.inner.sink_size, lambda s, v: setattr(s.inner, "sink_size", v))
    adapt_sink_thr = property(lambda s: s.inner.adapt_sink_thr, lambda s, v: setattr(s.inner, "adapt_sink_thr", v))
    evict_idx = property(lambda s: s.inner.evict_idx, lambda s, v: setattr(s.inner, "evict_idx", v))

    def attend(self, q, k, v, grid_sizes, freqs, kv_cache, current_start):
        out, _, seq = self.inner.step(q, k, v, grid_sizes.tolist(), freqs, kv_cache, current_start)
        self.trace.append((list(current_start), list(self.inner.last_writes), seq))
        return out


class TracedGpuPath:
    def __init__(self):
        from streamdiffusionv2_amd.attention import RingKVPath

        self.inner = RingKVPath()
        self.trace = []

    sink_size = property(lambda s: s.inner.sink_size, lambda s, v: setattr(s.inner, "sink_size", v))
    adapt_sink_thr = property(lambda s: s.inner.adapt_sink_thr, lambda s, v: setattr(s.inner, "adapt_sink_thr", v))
    evict_idx = property(lambda s: s.inner.evict_idx, lambda s, v: setattr(s.inner, "evict_idx", v))

    def attend(self, q, k, v, grid_sizes, freqs, kv_cache, current_start):
        out = self.inner.attend(q, k, v, grid_sizes, freqs, kv_cache, current_start)
        plan = self.inner.last_plan
        S = q.shape[1]
        self.trace.append((list(current_start), [(d, d + S) for d in plan.dst_start], list(plan.new_local_end)))
        return out
