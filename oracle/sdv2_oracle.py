"""CPU oracle for the causal Wan DiT ring-buffer KV-cache path.

TEST INFRASTRUCTURE ONLY.  This module restates, in plain PyTorch on the CPU,
the algorithm of the reference's KV-cache attention path so that the HIP
kernels can be checked against it.  Nothing in the shipped package imports
it; only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg
of ``bench.py`` may.  It is never a fallback for the GPU path.

Every function names the reference lines it follows (paths are relative to
the reference tree):

=========================  ====================================================
function                   reference
=========================  ====================================================
rope_params                models/wan/wan_base/modules/model.py:29-36
build_freqs                models/wan/causal_model.py:631-638
expand_rope_freqs          models/wan/causal_model.py:57-91
causal_rope_apply          models/wan/causal_model.py:94-108
attention_with_kvcache     models/wan/causal_model.py:111-157
new_kv_cache               models/wan/causal_stream_inference.py:87-107
RingAttentionOracle.step   models/wan/causal_model.py:250-384
replicate_for_stream_batch models/wan/causal_stream_inference.py:221-225
StreamShiftRegister        models/wan/causal_stream_inference.py:248-272
chunk_schedule             streamdiffusionv2/pipeline.py:235-279, 386-391
noise_scale_and_step       streamv2v/inference.py:51-57
wan_rms_norm               models/wan/wan_base/modules/model.py:70-86
chunk_block_mask           models/wan/causal_model.py:670-686 (carried over to
                           cache positions)
cross_attention_with_cache models/wan/wan_base/modules/model.py:160-196
new_crossattn_cache        models/wan/causal_stream_inference.py:109-122
compute_block_owners       streamv2v/communication/kv_cache_manager.py:86-108
moved_blocks_by_donor      streamv2v/communication/kv_cache_manager.py:126-136
receive_kv_block           streamv2v/communication/kv_cache_manager.py:66-82
=========================  ====================================================

``oracle/rope_ring_ref.c`` restates ``causal_rope_apply`` (with the table
expansion) and the placement state machine once more, in plain C without any
shared code; ``tests/test_oracle_c_ref.py`` requires the two to agree bit for
bit and checks the C side on its own against the hand traces.

Pinning (what fixes each function independently of this file) lives in
``tests/test_oracle_*.py`` (and, for the four functions at the end of the
table, in ``tests/test_fused_qk_norm.py``, ``tests/test_block_mask.py``,
``tests/test_cross_attention_cache.py``; the three block hand-off functions in
``tests/test_handoff.py``, against the cases of the reference's own
streamv2v/communication/test_communication.py:303-337 and hand-worked ones; the adaptive sink refresh inside
``RingAttentionOracle.step`` in ``tests/test_oracle_adaptive_sink.py``): closed forms for the tables, a scalar IEEE-double
loop for the rotation and its double->float->bf16 rounding, hand traces of the
slot schedule held as JSON under ``tests/golden/``, brute-force list
simulation of the ring, and a float64 numpy softmax for the attention.  The
attention operator itself is third-party in the reference (flash_attn
2.7.4.post1 or torch SDPA) and the reference holds no test vector for it:
parity there is pinned by the mathematics only (tolerance from the task
statement: max-abs 2e-2, mean-abs 2e-3 against fp32).
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------
# RoPE tables
# --------------------------------------------------------------------------

def rope_params(max_seq_len: int, dim: int, theta: float = 10000.0) -> torch.Tensor:
    """complex128 [max_seq_len, dim/2]: exp(i * pos * theta^(-2j/dim)).

    Follows model.py:29-36: integer positions times reciprocal powers in
    float64, then ``torch.polar`` with unit magnitude.
    """
    if dim % 2:
        raise ValueError("rope dim must be even")
    exponents = torch.arange(0, dim, 2).to(torch.float64).div(dim)
    inv = 1.0 / torch.pow(theta, exponents)
    angles = torch.outer(torch.arange(max_seq_len), inv)
    return torch.polar(torch.ones_like(angles), angles)


def build_freqs(head_dim: int = 128, max_pos: int = 1024) -> torch.Tensor:
    """The model's [max_pos, head_dim/2] table: temporal | height | width
    columns (22 | 21 | 21 for head_dim 128), causal_model.py:631-638."""
    sixth = head_dim // 6
    return torch.cat(
        [
            rope_params(max_pos, head_dim - 4 * sixth),
            rope_params(max_pos, 2 * sixth),
            rope_params(max_pos, 2 * sixth),
        ],
        dim=1,
    )


def split_freqs(freqs: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Column split used by the causal path (causal_model.py:77-78)."""
    c = freqs.shape[1]
    t, h, w = freqs.split([c - 2 * (c // 3), c // 3, c // 3], dim=1)
    return t, h, w


def expand_rope_freqs(freqs: torch.Tensor, f: int, h: int, w: int, start_frame: int) -> torch.Tensor:
    """Per-token multipliers [f*h*w, 1, C/2] for a chunk whose first latent
    frame sits at absolute frame ``start_frame``; token order is (f, h, w)
    row-major (causal_model.py:64-68)."""
    tab_t, tab_h, tab_w = split_freqs(freqs)
    part_t = tab_t[start_frame:start_frame + f].repeat_interleave(h * w, dim=0)
    part_h = tab_h[:h].repeat_interleave(w, dim=0).repeat(f, 1)
    part_w = tab_w[:w].repeat(h, 1).repeat(f, 1)
    return torch.cat([part_t, part_h, part_w], dim=-1).unsqueeze(1)


def causal_rope_apply(
    x: torch.Tensor,
    grid_sizes: Sequence[Sequence[int]],
    freqs: torch.Tensor,
    start_frames: Sequence[int],
) -> torch.Tensor:
    """Rotate interleaved pairs of x [B, S, H, D] in float64 complex and cast
    back to x.dtype (causal_model.py:94-108).  ``start_frames`` has one entry
    per row."""
    out = x.clone()
    heads = x.size(2)
    for row, ((f, h, w), sf) in enumerate(zip(grid_sizes, start_frames)):
        n_tok = f * h * w
        mult = expand_rope_freqs(freqs, f, h, w, int(sf))
        as_complex = torch.view_as_complex(
            x[row, :n_tok].to(torch.float64).reshape(n_tok, heads, -1, 2)
        )
        out[row, :n_tok] = torch.view_as_real(as_complex * mult).flatten(2).type_as(x)
    return out


def wan_rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """WanRMSNorm.forward (wan_base/modules/model.py:77-86) over the last
    dimension: float32 normalisation, back to x's dtype, times the weight."""
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)).type_as(x) * weight


# --------------------------------------------------------------------------
# KV-cache attention (the operator the flash kernel replaces)
# --------------------------------------------------------------------------

def chunk_block_mask(q_tokens: int, keys: int, chunk_start: int, block_tokens: int) -> torch.Tensor:
    """Boolean [q_tokens, keys], True = visible: the block-causal rule of the
    cache-less path, kv_idx < ends[q_idx] (causal_model.py:670-686), carried
    over to cache positions.  The chunk's own keys sit at
    [chunk_start, chunk_start + q_tokens); whatever else the cache holds is
    older than the chunk and visible; inside the chunk query t sees its own
    block and the earlier ones, i.e. not [chunk_start + (t // b + 1) * b,
    chunk_start + q_tokens)."""
    t = torch.arange(q_tokens).unsqueeze(1)
    key = torch.arange(keys).unsqueeze(0)
    hidden_from = chunk_start + (t // block_tokens + 1) * block_tokens
    return ~((key >= hidden_from) & (key < chunk_start + q_tokens))


def _sdpa_rows(q, k_cache, v_cache, lens, out_dtype, widen, chunk_start, block_tokens):
    rows = []
    for b, n in enumerate(lens):
        qq, kk, vv = widen(
            q[b:b + 1].transpose(1, 2),
            k_cache[b:b + 1, :n].transpose(1, 2),
            v_cache[b:b + 1, :n].transpose(1, 2),
        )
        mask = None
        if block_tokens:
            mask = chunk_block_mask(q.shape[1], n, int(chunk_start[b]), block_tokens)
        o = F.scaled_dot_product_attention(qq, kk, vv, attn_mask=mask, dropout_p=0.0, is_causal=False)
        rows.append(o.transpose(1, 2) if out_dtype is None else o.transpose(1, 2).to(out_dtype))
    return torch.cat(rows, dim=0).contiguous()


def attention_with_kvcache(
    q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, cache_seqlens: torch.Tensor,
    chunk_start: Optional[Sequence[int]] = None, block_tokens: int = 0,
) -> torch.Tensor:
    """softmax(q k^T / sqrt(D)) v over the first cache_seqlens[b] keys of each
    row, no mask inside the chunk (causal_model.py:111-157) unless
    ``block_tokens`` asks for the block-causal one (see chunk_block_mask).
    bf16/fp16 inputs are up-cast to fp32 on the CPU exactly as the reference
    fallback does."""
    out_dtype = q.dtype

    def widen(*ts):
        if q.device.type == "cpu" and q.dtype in (torch.float16, torch.bfloat16):
            return tuple(t.float() for t in ts)
        return ts

    span = k_cache.shape[1]
    if not block_tokens and bool(torch.all(cache_seqlens == span)):
        qq, kk, vv = widen(q.transpose(1, 2), k_cache.transpose(1, 2), v_cache.transpose(1, 2))
        o = F.scaled_dot_product_attention(qq, kk, vv, attn_mask=None, dropout_p=0.0, is_causal=False)
        return o.transpose(1, 2).to(out_dtype).contiguous()
    return _sdpa_rows(q, k_cache, v_cache, cache_seqlens.tolist(), out_dtype, widen, chunk_start, block_tokens)


def attention_fp32_reference(
    q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, cache_seqlens: Sequence[int],
    chunk_start: Optional[Sequence[int]] = None, block_tokens: int = 0,
) -> torch.Tensor:
    """fp32 result (not rounded to the input dtype) — the yardstick the
    2e-2 / 2e-3 tolerances are stated against."""
    return _sdpa_rows(q, k_cache, v_cache, list(cache_seqlens), None, lambda *ts: tuple(t.float() for t in ts),
                      chunk_start, block_tokens)


# --------------------------------------------------------------------------
# kv_cache dict + ring state machine
# --------------------------------------------------------------------------

def new_kv_cache(
    num_layers: int,
    batch_size: int,
    cache_tokens: int,
    num_heads: int,
    total_steps: int,
    dtype: torch.dtype = torch.bfloat16,
    device: str = "cpu",
    head_dim: int = 128,
) -> List[dict]:
    """Per-layer dicts with the reference's keys, shapes and dtypes
    (causal_stream_inference.py:98-105)."""
    layers = []
    for _ in range(num_layers):
        layers.append(
            {
                "k": torch.zeros([batch_size, cache_tokens, num_heads, head_dim], dtype=dtype, device=device),
                "v": torch.zeros([batch_size, cache_tokens, num_heads, head_dim], dtype=dtype, device=device),
                "global_end_index": torch.tensor([0], dtype=torch.long, device=device),
                "local_end_index": torch.tensor([0], dtype=torch.long, device=device),
                "total_steps": total_steps,
                "current_step": total_steps,
            }
        )
    return layers


def replicate_for_stream_batch(kv_cache: List[dict], batch_size: int) -> None:
    """One cache per denoising stage after the first chunk
    (causal_stream_inference.py:221-225)."""
    for entry in kv_cache:
        entry["k"] = entry["k"].repeat(batch_size, 1, 1, 1)
        entry["v"] = entry["v"].repeat(batch_size, 1, 1, 1)
        entry["global_end_index"] = entry["global_end_index"].repeat(batch_size)
        entry["local_end_index"] = entry["local_end_index"].repeat(batch_size)


class RingAttentionOracle:
    """One layer's self-attention on the KV-cache path, after the q/k/v
    projections: RoPE, ring append, attention (causal_model.py:250-384).

    Module state mirrors the reference attributes ``sink_size``,
    ``adapt_sink_thr`` and ``evict_idx`` (causal_model.py:177-179).
    """

    def __init__(self, sink_size: int = 3, adapt_sink_thr: float = -1):
        self.sink_size = sink_size
        self.adapt_sink_thr = adapt_sink_thr
        self.evict_idx: Optional[List[List[int]]] = None
        # None = the chunk is one block (reference cache path); n = blocks of n frames
        self.block_frames: Optional[int] = None
        # what the last call did, for tests: per row (dst_start, dst_end)
        self.last_writes: List[Tuple[int, int]] = []
        # per row the averaged similarities of the adaptive sink check, or None
        self.last_sims: List[Optional[torch.Tensor]] = []

    def step(
        self,
        q: torch.Tensor,
        k: torch.Tensor,
        v: torch.Tensor,
        grid_sizes: Sequence[Sequence[int]],
        freqs: torch.Tensor,
        kv_cache: dict,
        current_start: Sequence[int],
        with_attention: bool = True,
    ):
        """Returns (attention output or None, roped_query, seq_lens list)."""
        frame_tokens = int(grid_sizes[0][1]) * int(grid_sizes[0][2])
        starts = [int(c) for c in current_start]
        start_frames = [c // frame_tokens for c in starts]
        roped_q = causal_rope_apply(q, grid_sizes, freqs, start_frames).type_as(v)
        roped_k = causal_rope_apply(k, grid_sizes, freqs, start_frames).type_as(v)

        cap = kv_cache["k"].shape[1]
        cache_rows = kv_cache["k"].shape[0]
        n_new = roped_q.shape[1]
        sink_tokens = self.sink_size * frame_tokens

        if self.evict_idx is None:
            self.evict_idx = [[]]
        if len(self.evict_idx) < cache_rows:
            self.evict_idx = [list(self.evict_idx[0]) for _ in range(cache_rows)]

        seq_lens: List[int] = []
        self.last_writes = []
        self.last_sims = []
        for i, c_start in enumerate(starts):
            c_end = c_start + n_new
            queue = self.evict_idx[i]

            if sink_tokens > 0 and self.adapt_sink_thr > -1 and n_new <= frame_tokens:
                # similarity of each sink frame's mean K / V to the new chunk's
                # (causal_model.py:284-299)
                def frame_means(t, frames):
                    return t.reshape(frames, frame_tokens, -1).mean(1)

                sim_k = torch.cosine_similarity(
                    frame_means(kv_cache["k"][i:i + 1, :sink_tokens], self.sink_size),
                    frame_means(roped_k[i:i + 1], 1), dim=-1)
                sim_v = torch.cosine_similarity(
                    frame_means(kv_cache["v"][i:i + 1, :sink_tokens], self.sink_size),
                    frame_means(v[i:i + 1], 1), dim=-1)
                sim = (sim_k + sim_v) / 2
                self.last_sims.append(sim.clone())
                if sim.min() < self.adapt_sink_thr:
                    queue.insert(0, (int(torch.argmin(sim).item()) + 1) * frame_tokens)

            local_prev = int(kv_cache["local_end_index"][i].item())
            global_prev = int(kv_cache["global_end_index"][i].item())
            if c_end > cap or local_prev >= cap:
                # cache full: overwrite the slot whose END offset heads the queue.
                # The indices are rewound first, so an empty queue raises
                # IndexError with them already changed, as in the reference.
                kv_cache["global_end_index"][i].fill_(c_start)
                kv_cache["local_end_index"][i].fill_(cap)
                dst_end = queue[0]
                if cache_rows == 1 and kv_cache["current_step"] > 1:
                    kv_cache["current_step"] -= 1
                else:
                    head = queue.pop(0)
                    if head > sink_tokens:
                        queue.append(head)
                    kv_cache["current_step"] = kv_cache["total_steps"]
                local_new = cap
            else:
                local_new = local_prev + c_end - global_prev
                next_end = c_end + n_new
                if sink_tokens < next_end <= cap and (not queue or queue[-1] != next_end):
                    queue.append(next_end)
                dst_end = local_new
            dst_start = dst_end - n_new
            kv_cache["k"][i:i + 1, dst_start:dst_end] = roped_k[i:i + 1]
            kv_cache["v"][i:i + 1, dst_start:dst_end] = v[i:i + 1]
            self.last_writes.append((dst_start, dst_end))
            kv_cache["global_end_index"][i].fill_(c_end)
            kv_cache["local_end_index"][i].fill_(local_new)
            seq_lens.append(local_new)

        out = None
        if with_attention:
            lens = torch.tensor(seq_lens, dtype=torch.int32)
            span = int(lens.max().item())
            block_tokens = 0
            if self.block_frames is not None and self.block_frames * frame_tokens < n_new:
                block_tokens = self.block_frames * frame_tokens
            out = attention_with_kvcache(
                roped_q, kv_cache["k"][:, :span], kv_cache["v"][:, :span], lens,
                [a for a, _ in self.last_writes], block_tokens,
            )
        return out, roped_q, seq_lens


def new_crossattn_cache(num_layers: int, batch_size: int, heads: int, dtype=torch.bfloat16,
                        text_tokens: int = 512) -> List[dict]:
    """causal_stream_inference.py:109-122."""
    return [
        {
            "k": torch.zeros(batch_size, text_tokens, heads, 128, dtype=dtype),
            "v": torch.zeros(batch_size, text_tokens, heads, 128, dtype=dtype),
            "is_init": False,
        }
        for _ in range(num_layers)
    ]


def cross_attention_with_cache(q: torch.Tensor, make_kv, context_lens, crossattn_cache: Optional[dict]):
    """The cache logic of WanT2VCrossAttention.forward
    (wan_base/modules/model.py:172-192) around the attention operator:
    ``make_kv()`` stands for the K/V projections of the text context and is
    only called when the cache is absent or not initialised; an initialised
    cache is read as it is.  Attention = softmax(q k^T / sqrt(128)) v over the
    first context_lens[i] keys of row i (all keys when None)."""
    if crossattn_cache is not None and crossattn_cache["is_init"]:
        k, v = crossattn_cache["k"], crossattn_cache["v"]
    else:
        k, v = make_kv()
        if crossattn_cache is not None:
            crossattn_cache["is_init"] = True
            crossattn_cache["k"] = k
            crossattn_cache["v"] = v
    lens = [k.shape[1]] * q.shape[0] if context_lens is None else [int(n) for n in context_lens]
    return attention_with_kvcache(q, k, v, torch.tensor(lens, dtype=torch.int32))


# --------------------------------------------------------------------------
# drivers: stream-batch shift register and chunk arithmetic
# --------------------------------------------------------------------------

class StreamShiftRegister:
    """``kv_cache_starts`` / ``kv_cache_ends`` of the stream-batch driver:
    initialised to the first chunk's end (causal_stream_inference.py:248-249),
    shifted down one row per call with the new chunk entering at row 0
    (:265-272)."""

    def __init__(self, batch_size: int, first_chunk_end: int, frame_tokens: int):
        self.starts = [first_chunk_end] * batch_size
        self.ends = [first_chunk_end + frame_tokens] * batch_size

    def push(self, current_start: int, current_end: int) -> Tuple[List[int], List[int]]:
        self.starts = [current_start] + self.starts[:-1]
        self.ends = [current_end] + self.ends[:-1]
        return list(self.starts), list(self.ends)


def chunk_schedule(
    n_chunks: int,
    frame_tokens: int,
    frames_per_block: int,
    cache_tokens: int,
    t_refresh: int = 50,
) -> List[Tuple[int, int]]:
    """(current_start, current_end) handed to the model for each chunk of a
    video-to-video stream.  The first chunk spans 1 + frames_per_block latent
    frames; later ones frames_per_block; once current_start // frame_tokens
    reaches t_refresh the position is pinned to the cache's last frame
    (pipeline.py:249-251, 263-278, 386-391; inference.py:100)."""
    out = []
    start, end = 0, frame_tokens * (1 + frames_per_block)
    for idx in range(n_chunks):
        cs, ce = start, end
        if idx > 0 and cs // frame_tokens >= t_refresh:
            cs = cache_tokens - frame_tokens
            ce = cs + frames_per_block * frame_tokens
        out.append((cs, ce))
        start, end = end, end + frames_per_block * frame_tokens
    return out


def noise_scale_and_step(
    video: torch.Tensor, end_idx: int, chunk_size: int, noise_scale: float, init_noise_scale: float
) -> Tuple[float, int]:
    """Motion-adaptive noise scale (inference.py:51-57): RMS frame difference,
    max over the chunk's frames, /0.2 clamped to [0,1]; EMA 0.9/0.1."""
    cur = video[:, :, end_idx - chunk_size:end_idx]
    prev = video[:, :, end_idx - chunk_size - 1:end_idx - 1]
    motion = (torch.sqrt(((cur - prev) ** 2).mean(dim=(0, 1, 3, 4))).max() / 0.2).clamp(0, 1)
    scale = (init_noise_scale - 0.1 * motion.item()) * 0.9 + noise_scale * 0.1
    return scale, int(1000 * scale) - 100


def mix_noise(latents: torch.Tensor, noise: torch.Tensor, noise_scale: float) -> torch.Tensor:
    """noisy = noise*sigma + z*(1-sigma) (pipeline.py:310-314)."""
    return noise * noise_scale + latents * (1 - noise_scale)


# --------------------------------------------------------------------------
# Hand-off of a cache block between pipeline stages
# --------------------------------------------------------------------------
def compute_block_owners(block_intervals: torch.Tensor, total_blocks: int) -> torch.Tensor:
    """Owner rank per block from [start, end) intervals per rank, -1 = nobody
    (kv_cache_manager.py:98-106)."""
    owners = torch.full((total_blocks,), -1, dtype=torch.int64)
    for r in range(block_intervals.shape[0]):
        s = int(block_intervals[r, 0].item())
        e = int(block_intervals[r, 1].item())
        if e > s:
            owners[s:e] = r
    return owners


def moved_blocks_by_donor(old_block_intervals: torch.Tensor, new_block_intervals: torch.Tensor,
                          total_blocks: int) -> dict:
    """Blocks whose owner changes, keyed by the previous owner
    (kv_cache_manager.py:126-136)."""
    old = compute_block_owners(old_block_intervals, total_blocks)
    new = compute_block_owners(new_block_intervals, total_blocks)
    moved = {}
    for i in range(total_blocks):
        o, n = int(old[i].item()), int(new[i].item())
        if o != n and o >= 0:
            moved.setdefault(o, []).append(i)
    return moved


def receive_kv_block(entry: dict, donor_entry: dict, donor_rank: int, rank: int, frame_seq_length: int,
                     time_step_length: int) -> None:
    """What a rank's dict holds after ``broadcast_kv_blocks`` of one block
    (kv_cache_manager.py:66-82): the donor's four tensors, copied in place, and
    on a rank below the donor ``global_end_index`` moved on by
    frame_seq_length * (donor - rank) * num_steps.  The donor itself
    (rank == donor_rank) ends up unchanged."""
    for name in ("k", "v", "global_end_index", "local_end_index"):
        entry[name].copy_(donor_entry[name])
    if donor_rank > rank:
        entry["global_end_index"] += frame_seq_length * (donor_rank - rank) * time_step_length
