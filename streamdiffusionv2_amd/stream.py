"""Stream drivers around the KV-cache path.

``KVStreamPipeline`` owns the per-layer ``kv_cache1`` dicts and reproduces the
state handling of the reference's ``CausalStreamInferencePipeline``
(models/wan/causal_stream_inference.py): cache allocation (:87-107), the
first-chunk ``prepare`` with its ``num_steps`` passes and batch replication
(:124-255), the stream-batch shift registers of ``inference_stream``
(:257-296) and the sequential ``inference_wo_batch`` (:298-348).

``StagedStreamPipeline`` reproduces the chunk arithmetic of the staged API
``StreamDiffusionV2Pipeline`` (streamdiffusionv2/pipeline.py:228-414):
``prepare`` / ``chunk_video`` / ``encode_chunk`` / ``denoise_chunk`` with the
first-chunk length, the ``t_refresh`` position clamp, the motion-adaptive
noise scale and the warm-up of the stream batch.

Everything outside the path is a stand-in, because it is out of scope here:
the VAE encoder is replaced by average pooling to the latent grid, and the
DiT by a stack of fixed random projections that turn latent patches into
per-layer q/k/v and attention output back into latents.  The stand-ins are
deterministic, so a CPU run with the oracle plugged into the same stack gives
the reference result for the whole flow.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, List, Optional, Sequence

import torch

from . import ring, rope
from .attention import RingKVPath

BASE_CHUNK = 4          # video frames per latent frame (streamv2v/inference.py:99)
T_REFRESH = 50          # streamv2v/inference.py:100


class SyntheticGenerator:
    """Stand-in for the causal DiT: ``layers`` KV-cache attention layers fed by
    fixed random projections of the patchified latent.

    latents [B, F, 16, h8, w8] -> tokens [B, F*(h8/2)*(w8/2), 64] -> per layer
    (q, k, v) = tokens @ W_l reshaped to [B, S, H, 128]; layer outputs are
    projected back to 64 features, summed and un-patchified.
    ``path_factory()`` builds one KV path per layer; the default is the GPU
    path, tests plug the CPU oracle in.
    """

    def __init__(self, layers: int, heads: int, device, dtype=torch.bfloat16, seed: int = 0,
                 path_factory: Optional[Callable[[], object]] = None, sink_size: int = 3,
                 adapt_sink_thr: float = -1):
        self.layers, self.heads, self.device, self.dtype = layers, heads, torch.device(device), dtype
        gen = torch.Generator().manual_seed(seed)
        feat = 64
        self.w_qkv = [
            (torch.randn(feat, 3 * heads * 128, generator=gen) / feat ** 0.5).to(dtype).to(self.device)
            for _ in range(layers)
        ]
        self.w_out = [
            (torch.randn(heads * 128, feat, generator=gen) / (heads * 128) ** 0.5).to(dtype).to(self.device)
            for _ in range(layers)
        ]
        factory = path_factory or (lambda: RingKVPath())
        self.paths = [factory() for _ in range(layers)]
        for p in self.paths:
            p.sink_size, p.adapt_sink_thr = sink_size, adapt_sink_thr
        self.freqs = rope.build_freqs()

    @staticmethod
    def patchify(latents: torch.Tensor):
        b, f, c, h, w = latents.shape
        x = latents.reshape(b, f, c, h // 2, 2, w // 2, 2).permute(0, 1, 3, 5, 2, 4, 6)
        return x.reshape(b, f * (h // 2) * (w // 2), c * 4), (f, h // 2, w // 2)

    @staticmethod
    def unpatchify(tokens: torch.Tensor, grid, channels: int = 16):
        f, h, w = grid
        b = tokens.shape[0]
        x = tokens.reshape(b, f, h, w, channels, 2, 2).permute(0, 1, 4, 2, 5, 3, 6)
        return x.reshape(b, f, channels, h * 2, w * 2)

    def __call__(self, latents: torch.Tensor, kv_cache: List[dict], current_start) -> torch.Tensor:
        tokens, grid = self.patchify(latents.to(self.dtype))
        b, s, _ = tokens.shape
        grid_sizes = torch.tensor([list(grid)] * b, dtype=torch.long)
        acc = torch.zeros(b, s, 64, dtype=torch.float32, device=tokens.device)
        for layer in range(self.layers):
            qkv = (tokens @ self.w_qkv[layer]).view(b, s, 3, self.heads, 128)
            q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
            o = self.paths[layer].attend(q, k, v, grid_sizes, self.freqs, kv_cache[layer], current_start)
            acc += (o.reshape(b, s, self.heads * 128) @ self.w_out[layer]).float()
        return self.unpatchify(acc.to(self.dtype), grid)


class KVStreamPipeline:
    """State owner of the stream: ``kv_cache1``, ``hidden_states`` and the
    ``kv_cache_starts`` / ``kv_cache_ends`` shift registers."""

    def __init__(self, generator: SyntheticGenerator, height: int = 480, width: int = 832,
                 num_kv_cache: int = 6, num_sink_tokens: int = 3, adapt_sink_threshold: float = -1,
                 denoising_step_list: Sequence[int] = (700, 500, 0), num_frame_per_block: int = 1,
                 t2v: bool = False, cache_factory: Optional[Callable[..., List[dict]]] = None):
        self.generator = generator
        self.device = generator.device
        self.num_transformer_blocks = generator.layers
        self.num_heads = generator.heads
        self.frame_seq_length = (height // 16) * (width // 16)           # :47-50
        self.num_kv_cache = num_kv_cache
        self.kv_cache_length = self.frame_seq_length * num_kv_cache
        self.num_sink_tokens = num_sink_tokens
        self.adapt_sink_threshold = adapt_sink_threshold
        steps = list(denoising_step_list)
        if steps[-1] != 0:
            raise ValueError("denoising_step_list must end with 0")
        self.denoising_step_list = steps if t2v else steps[:-1]           # :77-81
        self.num_frame_per_block = num_frame_per_block
        self.kv_cache1: Optional[List[dict]] = None
        self.hidden_states: Optional[torch.Tensor] = None
        self.kv_cache_starts: Optional[List[int]] = None
        self.kv_cache_ends: Optional[List[int]] = None
        self.batch_size = 1
        self.active_mode = "batch"
        self._batch_state_refs: Optional[dict] = None
        self._cache_factory = cache_factory or ring.new_kv_cache
        self._replicate = ring.replicate_for_stream_batch

    # -- causal_stream_inference.py:87-107 ---------------------------------
    def _initialize_kv_cache(self, batch_size: int, dtype, device) -> None:
        for p in self.generator.paths:
            p.sink_size = self.num_sink_tokens
            p.adapt_sink_thr = self.adapt_sink_threshold
            if hasattr(p, "forget_sink_sums"):
                p.forget_sink_sums()      # a new cache: nothing a path summed before describes it
        self.kv_cache1 = self._cache_factory(
            self.num_transformer_blocks, batch_size, self.kv_cache_length, self.num_heads,
            len(self.denoising_step_list), dtype=dtype, device=device)

    def reset_stream_state(self) -> None:
        """streamv2v/inference.py:161-171.  The eviction queues live on the
        attention modules and are NOT reset, as in the reference."""
        self.kv_cache1 = None
        self.hidden_states = None
        for p in self.generator.paths:
            if hasattr(p, "forget_sink_sums"):
                p.forget_sink_sums()

    # -- causal_stream_inference.py:124-255 --------------------------------
    def prepare(self, noise: torch.Tensor, current_start: int = 0, current_end: Optional[int] = None,
                batch_denoise: bool = True, replicate: Optional[Callable] = None) -> torch.Tensor:
        if self.kv_cache1 is None:
            self._initialize_kv_cache(noise.shape[0], noise.dtype, self.device)
        denoised = None
        for _ in self.denoising_step_list:
            # every denoising pass re-submits the same current_start
            denoised = self.generator(noise, self.kv_cache1, [current_start])
        if not batch_denoise:
            return denoised
        self.batch_size = len(self.denoising_step_list)
        (replicate or self._replicate)(self.kv_cache1, self.batch_size)
        self.hidden_states = torch.zeros(
            (self.batch_size, self.num_frame_per_block, *noise.shape[2:]), dtype=noise.dtype, device=self.device)
        self.kv_cache_starts = [current_end] * self.batch_size
        self.kv_cache_ends = [current_end + self.frame_seq_length] * self.batch_size
        return denoised

    # -- causal_stream_inference.py:257-296 --------------------------------
    def inference_stream(self, noise: torch.Tensor, current_start: int, current_end: int,
                         current_step: Optional[int] = None) -> torch.Tensor:
        self.hidden_states[1:] = self.hidden_states[:-1].clone()
        self.hidden_states[0] = noise[0]
        self.kv_cache_starts = [current_start] + self.kv_cache_starts[:-1]
        self.kv_cache_ends = [current_end] + self.kv_cache_ends[:-1]
        self.hidden_states = self.generator(self.hidden_states, self.kv_cache1, self.kv_cache_starts)
        return self.hidden_states

    # -- causal_stream_inference.py:298-348 --------------------------------
    def inference_wo_batch(self, noise: torch.Tensor, current_start: int, current_end: int,
                           current_step: Optional[int] = None) -> torch.Tensor:
        out = noise
        for _ in self.denoising_step_list:
            out = self.generator(noise, self.kv_cache1, [current_start])
        return out


    def _settle_paths(self) -> None:
        for path in self.generator.paths:
            settle = getattr(path, "settle", None)
            if settle is not None:
                settle()

    # -- demo/vid2vid.py:113-135 -------------------------------------------
    _CACHE_TENSORS = ("k", "v", "global_end_index", "local_end_index")

    def enter_wo_batch(self) -> None:
        """Switch a running stream batch to sequential (no-batch) denoising:
        every cache dict is narrowed to views of its row 0, the batch tensors
        are kept aside untouched.  Nothing is copied."""
        if self.active_mode == "wo_batch":
            return
        self._settle_paths()               # host ring state current before the dicts are re-sliced
        self._batch_state_refs = {
            "kv_cache1": [{name: entry[name] for name in self._CACHE_TENSORS} for entry in self.kv_cache1],
            "hidden_states": self.hidden_states,
            "kv_cache_starts": self.kv_cache_starts,
            "kv_cache_ends": self.kv_cache_ends,
        }
        for entry, saved in zip(self.kv_cache1, self._batch_state_refs["kv_cache1"]):
            for name in self._CACHE_TENSORS:
                entry[name] = saved[name][:1]
        self.active_mode = "wo_batch"

    # -- demo/vid2vid.py:137-198 -------------------------------------------
    def return_to_batch(self, current_start: int, current_end: int) -> None:
        """Back to the stream batch: row 0 (the only row the sequential mode
        advanced) is copied over every other row of the batch tensors, each
        row's eviction queue becomes a copy of row 0's, the pass counter is
        rewound, the pipeline registers restart from the session position."""
        if self.active_mode == "batch":
            return
        if self._batch_state_refs is None:
            raise RuntimeError("Cannot restore batch mode before batch state has been captured")
        self._settle_paths()
        for entry, saved in zip(self.kv_cache1, self._batch_state_refs["kv_cache1"]):
            for name in self._CACHE_TENSORS:
                t = saved[name]
                if t.shape[0] > 1 and t.stride(0) != 0:
                    t[1:].copy_(t[:1].expand_as(t[1:]))
                entry[name] = t
            ring.contents_changed(entry)       # rows rewritten here: kept sums of the sink frames are stale
            if "total_steps" in entry:
                entry["current_step"] = entry["total_steps"]
        self.hidden_states = torch.zeros_like(self._batch_state_refs["hidden_states"])
        n = len(self._batch_state_refs["kv_cache_starts"])
        self.kv_cache_starts = [int(current_start)] * n
        self.kv_cache_ends = [int(current_end)] * n
        for path in self.generator.paths:
            if isinstance(path.evict_idx, list) and path.evict_idx:
                path.evict_idx = [list(path.evict_idx[0]) for _ in range(self.hidden_states.shape[0])]
        self.active_mode = "batch"
        self._batch_state_refs = None


@dataclass
class VideoChunk:
    frames: torch.Tensor
    start_idx: int
    end_idx: int
    current_start: int
    current_end: int


@dataclass
class EncodedChunk:
    noisy_latents: torch.Tensor
    current_start: int
    current_end: int
    noise_scale: float
    current_step: Optional[int]


@dataclass
class DenoisedChunk:
    denoised_pred: torch.Tensor
    last_frame_only: bool


def compute_noise_scale_and_step(video, end_idx, chunk_size, noise_scale, init_noise_scale):
    """streamv2v/inference.py:51-57."""
    cur = video[:, :, end_idx - chunk_size:end_idx]
    prev = video[:, :, end_idx - chunk_size - 1:end_idx - 1]
    motion = (torch.sqrt(((cur - prev) ** 2).mean(dim=(0, 1, 3, 4))).max() / 0.2).clamp(0, 1)
    new_scale = (init_noise_scale - 0.1 * motion.item()) * 0.9 + noise_scale * 0.1
    return new_scale, int(1000 * new_scale) - 100


class StagedStreamPipeline:
    """``prepare`` / ``chunk_video`` / ``encode_chunk`` / ``denoise_chunk`` with
    the arithmetic of ``StreamDiffusionV2Pipeline`` (pipeline.py:228-414)."""

    def __init__(self, pipeline: KVStreamPipeline, mode: str = "single", noise_scale: float = 0.8,
                 height: int = 480, width: int = 832, seed: int = 0):
        if mode not in {"single", "single-wo"}:
            raise ValueError("StagedStreamPipeline only supports 'single' and 'single-wo'")
        self.pipeline = pipeline
        self.mode = mode
        self.noise_scale = float(noise_scale)
        self.height, self.width = height, width
        self.chunk_size = BASE_CHUNK * pipeline.num_frame_per_block
        self.num_steps = len(pipeline.denoising_step_list)
        self.t_refresh = T_REFRESH
        self.prompt: Optional[str] = None
        self.processed = 0
        self._next_chunk_index = 0
        self._gen = torch.Generator().manual_seed(seed)

    def prepare(self, prompt: str) -> None:
        self.prompt = prompt
        self.pipeline.reset_stream_state()
        self.processed = 0
        self._next_chunk_index = 0

    def chunk_video(self, video: torch.Tensor) -> List[VideoChunk]:
        """video [1, C, T, H, W]; first chunk 1 + chunk_size frames (pipeline.py:235-279)."""
        total = video.shape[2]
        if total < 1 + self.chunk_size:
            raise ValueError(f"video must contain at least {1 + self.chunk_size} frames")
        fsl = self.pipeline.frame_seq_length
        per = self.chunk_size // BASE_CHUNK
        chunks, start_idx, end_idx = [], 0, 1 + self.chunk_size
        cs, ce = 0, fsl * (1 + per)
        chunks.append(VideoChunk(video[:, :, start_idx:end_idx], start_idx, end_idx, cs, ce))
        while True:
            start_idx, end_idx = end_idx, end_idx + self.chunk_size
            if end_idx > total:
                break
            cs, ce = ce, ce + per * fsl
            chunks.append(VideoChunk(video[:, :, start_idx:end_idx], start_idx, end_idx, cs, ce))
        return chunks

    def _stand_in_vae_encode(self, frames: torch.Tensor) -> torch.Tensor:
        """[1, C, T, H, W] -> latents [1, 16, T', H/8, W/8]: average pooling in
        place of the Wan VAE (out of scope).  T' = 1 + (T-1)//4 for the first
        chunk, T//4 afterwards, as the causal VAE yields."""
        t = frames.shape[2]
        first = t % BASE_CHUNK == 1
        x = frames.float()
        if first:
            head, rest = x[:, :, :1], x[:, :, 1:]
            parts = [head] + ([rest.reshape(*rest.shape[:2], -1, BASE_CHUNK, *rest.shape[3:]).mean(3)] if rest.shape[2] else [])
            x = torch.cat(parts, dim=2)
        else:
            x = x.reshape(*x.shape[:2], -1, BASE_CHUNK, *x.shape[3:]).mean(3)
        x = torch.nn.functional.avg_pool3d(x, kernel_size=(1, 8, 8))
        reps = -(-16 // x.shape[1])
        return x.repeat(1, reps, 1, 1, 1)[:, :16]

    def encode_chunk(self, video: torch.Tensor, chunk: VideoChunk, previous_noise_scale=None,
                     initial_noise_scale=None) -> EncodedChunk:
        """pipeline.py:282-320."""
        noise_scale = self.noise_scale if previous_noise_scale is None else float(previous_noise_scale)
        init = self.noise_scale if initial_noise_scale is None else float(initial_noise_scale)
        current_step = None
        if chunk.start_idx != 0:
            noise_scale, current_step = compute_noise_scale_and_step(video, chunk.end_idx, self.chunk_size, noise_scale, init)
        latents = self._stand_in_vae_encode(chunk.frames).transpose(2, 1).contiguous().to(torch.bfloat16)
        noise = torch.randn(latents.shape, generator=self._gen).to(torch.bfloat16)
        noisy = (noise * noise_scale + latents * (1 - noise_scale)).to(self.pipeline.device)
        return EncodedChunk(noisy, chunk.current_start, chunk.current_end, float(noise_scale), current_step)

    def denoise_chunk(self, chunk: EncodedChunk) -> Optional[DenoisedChunk]:
        """pipeline.py:362-414."""
        if self.prompt is None:
            raise RuntimeError("Call prepare(prompt) before denoise_chunk(...)")
        p = self.pipeline
        if self._next_chunk_index == 0:
            pred = p.prepare(chunk.noisy_latents, chunk.current_start, chunk.current_end,
                             batch_denoise=self.mode == "single")
            self._next_chunk_index += 1
            return DenoisedChunk(pred, last_frame_only=False)
        cs, ce = chunk.current_start, chunk.current_end
        if cs // p.frame_seq_length >= self.t_refresh:
            cs = p.kv_cache_length - p.frame_seq_length
            ce = cs + (self.chunk_size // BASE_CHUNK) * p.frame_seq_length
        if self.mode == "single":
            pred = p.inference_stream(chunk.noisy_latents, cs, ce, chunk.current_step)
            self.processed += 1
            self._next_chunk_index += 1
            if self.processed < self.num_steps:
                return None
            return DenoisedChunk(pred, last_frame_only=True)
        pred = p.inference_wo_batch(chunk.noisy_latents, cs, ce, chunk.current_step)
        self.processed += 1
        self._next_chunk_index += 1
        return DenoisedChunk(pred, last_frame_only=True)
