"""The staged stream flow (prepare / chunk_video / encode_chunk /
denoise_chunk) on the GPU path against the same flow with the CPU oracle
plugged into the generator stand-in: identical integer state after every chunk
(positions per row, slot written, eviction queues, indices, warm-up Nones) and
close outputs."""
import pytest
import torch

from oracle import sdv2_oracle as oracle

pytestmark = pytest.mark.gpu


from flow_helpers import OraclePath, TracedGpuPath  # noqa: E402


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


def test_switch_to_sequential_mode_and_back(gpu_device):
    """Stream batch -> sequential (row-0 views) -> stream batch again
    (demo/vid2vid.py:113-198) on the GPU path against the same driver with the
    oracle plugged in: identical positions, slots, lengths, queues, indices
    and pass counters after every call; close outputs."""
    from streamdiffusionv2_amd import stream

    H, W = 64, 96
    layers, heads, fsl = 2, 2, 24

    def build(device, factory, cache_factory=None):
        gen = stream.SyntheticGenerator(layers, heads, device, seed=13, path_factory=factory,
                                        sink_size=1, adapt_sink_thr=-1)
        pipe = stream.KVStreamPipeline(gen, height=H, width=W, num_kv_cache=4, num_sink_tokens=1,
                                       denoising_step_list=(700, 500, 0), cache_factory=cache_factory)
        return gen, pipe

    def cpu_cache_factory(n, b, cap, h, steps, dtype, device):
        return oracle.new_kv_cache(n, b, cap, h, steps, dtype=dtype, device="cpu")

    g_gen, g_pipe = build(gpu_device, TracedGpuPath)
    o_gen, o_pipe = build("cpu", OraclePath, cpu_cache_factory)
    o_pipe._replicate = oracle.replicate_for_stream_batch

    gen = torch.Generator().manual_seed(9)
    noises = [torch.randn(1, 1, 16, H // 8, W // 8, generator=gen).bfloat16() for _ in range(12)]
    results = []
    for pipe in (g_pipe, o_pipe):
        dev = pipe.device
        outs, pos = [], 0
        outs.append(pipe.prepare(noises[0].to(dev), 0, fsl))
        pos = fsl
        for i in range(1, 4):
            outs.append(pipe.inference_stream(noises[i].to(dev), pos, pos + fsl))
            pos += fsl
        pipe.enter_wo_batch()
        assert pipe.active_mode == "wo_batch" and pipe.kv_cache1[0]["k"].shape[0] == 1
        for i in range(4, 8):
            outs.append(pipe.inference_wo_batch(noises[i].to(dev), pos, pos + fsl))
            pos += fsl
        pipe.return_to_batch(pos, pos + fsl)
        assert pipe.active_mode == "batch" and pipe.kv_cache1[0]["k"].shape[0] == pipe.batch_size
        for entry in pipe.kv_cache1:                      # row 0 was broadcast over the batch
            for name in ("k", "v", "global_end_index", "local_end_index"):
                assert all(torch.equal(entry[name][r], entry[name][0]) for r in range(1, pipe.batch_size))
            assert entry["current_step"] == entry["total_steps"]
        for i in range(8, 12):
            outs.append(pipe.inference_stream(noises[i].to(dev), pos, pos + fsl))
            pos += fsl
        results.append(outs)
    torch.cuda.synchronize()

    for gp, op in zip(g_gen.paths, o_gen.paths):
        assert gp.trace == op.trace
        assert gp.evict_idx == op.evict_idx
    for gc, oc in zip(g_pipe.kv_cache1, o_pipe.kv_cache1):
        assert gc["global_end_index"].cpu().tolist() == oc["global_end_index"].tolist()
        assert gc["local_end_index"].cpu().tolist() == oc["local_end_index"].tolist()
        assert gc["current_step"] == oc["current_step"]
    for g, o in zip(*results):
        diff = (g.float().cpu() - o.float()).abs()
        assert diff.max().item() < 0.15 and diff.mean().item() < 0.02
