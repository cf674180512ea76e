"""The staged stream flow (prepare / chunk_video / encode_chunk /
denoise_chunk) on the GPU path against the same flow with the CPU oracle
plugged into the generator stand-in: identical integer state after every chunk
(positions per row, slot written, eviction queues, indices, warm-up Nones) and
close outputs."""
import pytest
import torch

from oracle import sdv2_oracle as oracle

pytestmark = pytest.mark.gpu


class OraclePath:
    """Adapter: the oracle layer behind the attend() call of the package."""

    def __init__(self):
        self.inner = oracle.RingAttentionOracle()
        self.trace = []

    sink_size = property(lambda s: s.inner.sink_size, lambda s, v: setattr(s.inner, "sink_size", v))
    adapt_sink_thr = property(lambda s: s.inner.adapt_sink_thr, lambda s, v: setattr(s.inner, "adapt_sink_thr", v))
    evict_idx = property(lambda s: s.inner.evict_idx)

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
    evict_idx = property(lambda s: s.inner.evict_idx)

    def attend(self, q, k, v, grid_sizes, freqs, kv_cache, current_start):
        out = self.inner.attend(q, k, v, grid_sizes, freqs, kv_cache, current_start)
        plan = self.inner.last_plan
        S = q.shape[1]
        self.trace.append((list(current_start), [(d, d + S) for d in plan.dst_start], list(plan.new_local_end)))
        return out


@pytest.mark.parametrize("mode", ["single", "single-wo"])
def test_staged_flow_matches_oracle_flow(gpu_device, mode):
    from streamdiffusionv2_amd import stream

    H, W = 64, 96              # latent 8 x 12 -> 4 x 6 = 24 tokens per frame
    layers, heads = 2, 2
    video = torch.randn(1, 3, 1 + 4 * 9, H, W, generator=torch.Generator().manual_seed(3))

    def build(device, factory, cache_factory=None):
        gen = stream.SyntheticGenerator(layers, heads, device, seed=11, path_factory=factory,
                                        sink_size=1, adapt_sink_thr=-1)
        pipe = stream.KVStreamPipeline(gen, height=H, width=W, num_kv_cache=4, num_sink_tokens=1,
                                       denoising_step_list=(700, 500, 0), cache_factory=cache_factory)
        staged = stream.StagedStreamPipeline(pipe, mode=mode, height=H, width=W, seed=5)
        staged.t_refresh = 6    # exercise the position clamp inside a short video
        return gen, pipe, staged

    def cpu_cache_factory(n, b, cap, h, steps, dtype, device):
        return oracle.new_kv_cache(n, b, cap, h, steps, dtype=dtype, device="cpu")

    g_gen, g_pipe, g_staged = build(gpu_device, TracedGpuPath)
    o_gen, o_pipe, o_staged = build("cpu", OraclePath, cpu_cache_factory)
    o_pipe._replicate = oracle.replicate_for_stream_batch

    outs = []
    for staged in (g_staged, o_staged):
        staged.prepare("a prompt")
        res = []
        noise_scale = staged.noise_scale
        for chunk in staged.chunk_video(video):
            enc = staged.encode_chunk(video, chunk, previous_noise_scale=noise_scale,
                                      initial_noise_scale=staged.noise_scale)
            noise_scale = enc.noise_scale
            res.append((enc.current_start, enc.current_end, enc.current_step, staged.denoise_chunk(enc)))
        outs.append(res)
    torch.cuda.synchronize()

    assert len(outs[0]) == len(outs[1]) == 9
    for (gs, ge, gstep, gd), (os_, oe, ostep, od) in zip(*outs):
        assert (gs, ge, gstep) == (os_, oe, ostep)
        assert (gd is None) == (od is None)
        if gd is not None:
            assert gd.last_frame_only == od.last_frame_only
            assert gd.denoised_pred.shape == od.denoised_pred.shape
            diff = (gd.denoised_pred.float().cpu() - od.denoised_pred.float()).abs()
            assert diff.max().item() < 0.15 and diff.mean().item() < 0.02
    # warm-up of the stream batch: in 'single' mode the first num_steps-1 stream calls return None
    nones = [d is None for *_, d in outs[0]]
    assert nones == ([False, True] + [False] * 7 if mode == "single" else [False] * 9)
    # integer trace of every layer call: positions per row, slot written, lengths
    for gp, op in zip(g_gen.paths, o_gen.paths):
        assert gp.trace == op.trace
        assert gp.evict_idx == op.evict_idx
    for gc, oc in zip(g_pipe.kv_cache1, o_pipe.kv_cache1):
        assert gc["global_end_index"].cpu().tolist() == oc["global_end_index"].tolist()
        assert gc["local_end_index"].cpu().tolist() == oc["local_end_index"].tolist()
        assert gc["current_step"] == oc["current_step"]
    # the clamp was reached: last calls sit at the cache's last frame
    assert g_gen.paths[0].trace[-1][0][0] == g_pipe.kv_cache_length - g_pipe.frame_seq_length
