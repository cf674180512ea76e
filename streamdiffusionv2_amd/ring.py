"""Host side of the ring KV cache: the per-layer ``kv_cache`` dict and the
integer state machine that decides where each chunk lands.

The dict keeps the reference's contract (models/wan/causal_stream_inference.py:98-105):
``k``/``v`` of logical shape [B, cap, H, 128], ``global_end_index`` and
``local_end_index`` as int64 [B] device tensors mutated in place, and the
python ints ``total_steps``/``current_step``.  ``k``/``v`` are permuted views of
head-major [B, H, cap, 128] buffers, so a chunk's rows for one head are one
contiguous run in HBM.

The placement policy restates models/wan/causal_model.py:268-342 on host
integers only.  The reference reads the two index tensors back with ``.item()``
for every row of every layer; here the host carries a mirror of them (they are
a pure function of the host-known ``current_start`` sequence), validated
against the tensors' identity and version counter, so the steady state issues
no device-to-host copy at all.  Tensors created under ``torch.inference_mode()``
keep no version counter: for those only the identity is checked, and code that
rewrites the two index tensors in place must call :func:`forget_index_mirror`.  The kernel stores the new index values, which
keeps the tensors authoritative for every external consumer of the dict.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import torch

HEAD_DIM = 128
_MIRROR_KEY = "_sdv2_host_index_mirror"
_GENERATION_KEY = "_sdv2_contents_generation"
_SINK_OWNER_KEY = "_sdv2_sink_sums_owner"


def tensor_version(t: torch.Tensor) -> Optional[int]:
    """The tensor's in-place edit counter, or None for a tensor created under
    ``torch.inference_mode()`` (the reference's API level runs in it,
    streamdiffusionv2/pipeline.py:281,361), which keeps none."""
    try:
        return t._version
    except RuntimeError:
        return None


def new_kv_cache(
    num_layers: int,
    batch_size: int,
    cache_tokens: int,
    num_heads: int,
    total_steps: int,
    dtype: torch.dtype = torch.bfloat16,
    device="cuda",
    head_major: bool = True,
) -> List[dict]:
    """Allocate the per-layer cache dicts of
    ``CausalStreamInferencePipeline._initialize_kv_cache``
    (causal_stream_inference.py:87-107)."""
    layers = []
    for _ in range(num_layers):
        if head_major:
            k = torch.zeros([batch_size, num_heads, cache_tokens, HEAD_DIM], dtype=dtype, device=device).permute(0, 2, 1, 3)
            v = torch.zeros([batch_size, num_heads, cache_tokens, HEAD_DIM], dtype=dtype, device=device).permute(0, 2, 1, 3)
        else:
            k = torch.zeros([batch_size, cache_tokens, num_heads, HEAD_DIM], dtype=dtype, device=device)
            v = torch.zeros([batch_size, cache_tokens, num_heads, HEAD_DIM], dtype=dtype, device=device)
        layers.append(
            {
                "k": k,
                "v": v,
                "global_end_index": torch.tensor([0], dtype=torch.long, device=device),
                "local_end_index": torch.tensor([0], dtype=torch.long, device=device),
                "total_steps": total_steps,
                "current_step": total_steps,
            }
        )
    return layers


def replicate_for_stream_batch(kv_cache: List[dict], batch_size: int) -> None:
    """One cache per denoising stage (causal_stream_inference.py:221-225).
    ``repeat`` on the underlying head-major buffer keeps the layout."""
    for entry in kv_cache:
        for name in ("k", "v"):
            t = entry[name]
            if t.stride(2) > t.stride(1):  # head-major view [B, cap, H, D]
                entry[name] = t.permute(0, 2, 1, 3).repeat(batch_size, 1, 1, 1).permute(0, 2, 1, 3)
            else:
                entry[name] = t.repeat(batch_size, 1, 1, 1)
        entry["global_end_index"] = entry["global_end_index"].repeat(batch_size)
        entry["local_end_index"] = entry["local_end_index"].repeat(batch_size)
        entry.pop(_MIRROR_KEY, None)
        entry.pop(_SINK_OWNER_KEY, None)


def new_crossattn_cache(num_layers: int, batch_size: int, heads: int, dtype=torch.bfloat16, device="cuda",
                        text_tokens: int = 512) -> List[dict]:
    """Per-layer cross-attention cache (causal_stream_inference.py:109-122):
    ``k`` / ``v`` zeros [B, 512, H, 128] and ``is_init`` False; the first
    cross-attention call of a prompt fills it (wan_base/modules/model.py:174-184)."""
    return [
        {
            "k": torch.zeros(batch_size, text_tokens, heads, 128, dtype=dtype, device=device),
            "v": torch.zeros(batch_size, text_tokens, heads, 128, dtype=dtype, device=device),
            "is_init": False,
        }
        for _ in range(num_layers)
    ]


def expand_crossattn_for_stream_batch(crossattn_cache: List[dict], batch_size: int) -> None:
    """Stream-batch expansion of the text cache (causal_stream_inference.py:227-228):
    a broadcast view, every row reads the same 512 keys (row stride 0)."""
    for entry in crossattn_cache:
        entry["k"] = entry["k"].expand(batch_size, -1, -1, -1)
        entry["v"] = entry["v"].expand(batch_size, -1, -1, -1)


@dataclass
class _IndexMirror:
    g_tensor: torch.Tensor
    l_tensor: torch.Tensor
    g_version: Optional[int]
    l_version: Optional[int]
    global_end: List[int]
    local_end: List[int]

    def valid_for(self, kv_cache: dict) -> bool:
        g, l = kv_cache["global_end_index"], kv_cache["local_end_index"]
        return (
            g is self.g_tensor and l is self.l_tensor
            and tensor_version(g) == self.g_version and tensor_version(l) == self.l_version
        )


def _mirror(kv_cache: dict) -> _IndexMirror:
    m: Optional[_IndexMirror] = kv_cache.get(_MIRROR_KEY)
    if m is None or not m.valid_for(kv_cache):
        g, l = kv_cache["global_end_index"], kv_cache["local_end_index"]
        m = _IndexMirror(g, l, tensor_version(g), tensor_version(l), [int(x) for x in g.tolist()],
                         [int(x) for x in l.tolist()])
        kv_cache[_MIRROR_KEY] = m
    return m


def rows_evicting(kv_cache: dict, current_start: Sequence[int], n_new: int) -> List[bool]:
    """Which rows the next :func:`plan_append` sends down the evict branch
    (causal_model.py:302)."""
    cap = kv_cache["k"].shape[1]
    m = _mirror(kv_cache)
    return [int(c) + n_new > cap or m.local_end[i] >= cap for i, c in enumerate(current_start)]


def forget_index_mirror(kv_cache: dict) -> None:
    """Drop what the host remembers about this cache: its copy of the two
    index tensors (the next plan reads them back once) and, through
    :func:`contents_changed`, every layer path's kept sums of the sink frames.
    Needed after the tensors of the dict were rewritten in place by anything
    but the path's own calls - the library's hand-off kernel, a copy between
    rows, a reset (a raw device store bumps no version counter, and tensors
    created under ``torch.inference_mode()`` have none)."""
    kv_cache.pop(_MIRROR_KEY, None)
    contents_changed(kv_cache)


def contents_changed(kv_cache: dict) -> None:
    """Tell the paths that read this cache that k / v rows changed behind
    their back (see :func:`forget_index_mirror`)."""
    kv_cache[_GENERATION_KEY] = kv_cache.get(_GENERATION_KEY, 0) + 1


def contents_generation(kv_cache: dict) -> int:
    return kv_cache.get(_GENERATION_KEY, 0)


def sink_sums_owner(kv_cache: dict, create: bool = False):
    """The token that ties a path's kept sink-frame sums to THIS cache dict.
    Addresses do not identify a cache: a cache allocated after another was
    dropped usually gets the same memory back, while its contents (zeros) are
    new.  A dict that never went through a check carries no token."""
    token = kv_cache.get(_SINK_OWNER_KEY)
    if token is None and create:
        token = object()
        kv_cache[_SINK_OWNER_KEY] = token
    return token


@dataclass
class AppendPlan:
    """What one layer call does, row by row."""
    dst_start: List[int]      # first cache token written
    new_global_end: List[int]
    new_local_end: List[int]  # == seq_lens of the attention that follows
    evicting: List[bool] = None   # row took the evict branch (wrote at the head of its queue)
    held: List[bool] = None       # ... without rotating the queue (a pass before the last, causal_model.py:310-311)

    @property
    def max_seq_len(self) -> int:
        return max(self.new_local_end)


def advance_queue(queue: List[int], evicting: bool, held: bool, sink_tokens: int, next_end: int, cap: int):
    """What one call does to a row's eviction queue (causal_model.py:306-316,
    330-335).  An evicting call writes the slot ending at the head of the queue
    (returned; IndexError when there is none) and, unless the pass counter
    holds it there, rotates the head to the tail - or drops it when it lies in
    the sink, as a refreshed sink frame does.  A filling call queues the slot
    after its own once that slot lies beyond the sink."""
    if evicting:
        dst_end = queue[0]
        if not held:
            head = queue.pop(0)
            if head > sink_tokens:
                queue.append(head)
        return dst_end
    if sink_tokens < next_end <= cap and (not queue or queue[-1] != next_end):
        queue.append(next_end)
    return None


def plan_append(
    kv_cache: dict,
    evict_idx: List[List[int]],
    current_start: Sequence[int],
    n_new: int,
    frame_tokens: int,
    sink_size: int,
) -> AppendPlan:
    """Advance the ring state by one call and say where the chunk of each row
    goes.  Mutates ``evict_idx`` and ``kv_cache['current_step']`` and the host
    index mirror exactly as causal_model.py:279-342 mutates its state; the
    device index tensors are written by the append kernel.

    Raises IndexError when the cache is full and the eviction queue is empty
    (causal_model.py:306) and ValueError when the slot would start before the
    cache (the reference's negative slice would fail on a shape mismatch).
    """
    cap = kv_cache["k"].shape[1]
    cache_rows = kv_cache["k"].shape[0]
    sink_tokens = sink_size * frame_tokens
    m = _mirror(kv_cache)
    if len(m.local_end) < len(current_start):
        raise ValueError(
            f"current_start has {len(current_start)} rows but the cache indices have {len(m.local_end)}"
        )

    dst_start, new_g, new_l, evicting, held = [], [], [], [], []
    for i, c_start in enumerate(current_start):
        c_start = int(c_start)
        c_end = c_start + n_new
        queue = evict_idx[i]
        evicting.append(c_end > cap or m.local_end[i] >= cap)
        held.append(evicting[-1] and cache_rows == 1 and kv_cache["current_step"] > 1)
        if evicting[-1]:
            m.global_end[i], m.local_end[i] = c_start, cap
            dst_end = advance_queue(queue, True, held[-1], sink_tokens, 0, cap)
            if held[-1]:
                kv_cache["current_step"] -= 1
            else:
                kv_cache["current_step"] = kv_cache["total_steps"]
            local_new = cap
        else:
            local_new = m.local_end[i] + c_end - m.global_end[i]
            advance_queue(queue, False, False, sink_tokens, c_end + n_new, cap)
            dst_end = local_new
        start = dst_end - n_new
        if start < 0 or dst_end > cap:
            raise ValueError(f"row {i}: chunk of {n_new} tokens would be written at [{start}, {dst_end}) of a {cap}-token cache")
        dst_start.append(start)
        new_g.append(c_end)
        new_l.append(local_new)
        m.global_end[i], m.local_end[i] = c_end, local_new
    return AppendPlan(dst_start, new_g, new_l, evicting, held)


def closed_form_slot(chunk: int, n_slots: int, n_permanent: int) -> int:
    """Slot of chunk number ``chunk`` for uniform chunks that divide the
    cache, one pass per chunk and no adaptive refresh: fill 0..n_slots-1, then
    rotate over the evictable slots.  Eviction is therefore an index update."""
    if chunk < n_slots:
        return chunk
    return n_permanent + (chunk - n_slots) % (n_slots - n_permanent)
