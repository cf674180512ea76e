"""``CausalWanSelfAttention`` with the KV-cache path on the sdv2kv kernels.

Same constructor, attributes and ``forward`` signature as the reference module
(models/wan/causal_model.py:160-200), so a block can hold it unchanged:
``sink_size``, ``adapt_sink_thr`` and ``evict_idx`` are plain attributes set
and copied from outside (causal_stream_inference.py:95-96,
demo/vid2vid.py:150-156).  The projections and RMS norms around the path are
ordinary PyTorch modules; the path itself (RoPE, ring append, attention) is
two HIP kernels and no device-to-host copy.
"""
from __future__ import annotations

import copy
import time
from typing import List, Optional

import torch
import torch.nn as nn

from . import ops, ring


class WanRMSNorm(nn.Module):
    """RMS norm over the full model dim in fp32 (wan_base/modules/model.py:70-86)."""

    def __init__(self, dim: int, eps: float = 1e-5):
        super().__init__()
        self.dim = dim
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x):
        if not torch.is_grad_enabled() and ops.rms_norm_supported(x, self.weight):
            # one launch of the library's kernel (the bits of the expression below on the CPU)
            # instead of the seven kernels the expression becomes on the device
            return ops.rms_norm(x, self.weight.detach(), self.eps)
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + self.eps)).type_as(x) * self.weight


_HOST_LIST_CACHE: dict = {}


def _host_ints(value, slot: str, rows: Optional[int] = None) -> List[int]:
    """``current_start`` / ``grid_sizes`` as python ints.  A device tensor costs
    one copy per distinct (tensor, version): the same tensor is handed to every
    layer of a forward, so all but the first layer hit the one-entry cache.  A
    tensor without a version counter (created under ``torch.inference_mode()``)
    may have been rewritten in place unnoticed - the reference shifts its
    ``kv_cache_starts`` that way (causal_stream_inference.py:268-269) - and is
    read every time."""
    if isinstance(value, torch.Tensor):
        version = ring.tensor_version(value)
        if value.device.type == "cpu" or version is None:
            out = value.reshape(-1).tolist()
        else:
            stamp = (version, value.data_ptr(), tuple(value.shape))
            hit = _HOST_LIST_CACHE.get(slot)
            if hit is not None and hit[0] is value and hit[1] == stamp:
                out = hit[2]
            else:
                out = value.reshape(-1).tolist()
                _HOST_LIST_CACHE[slot] = (value, stamp, out)
    elif isinstance(value, (list, tuple)):
        out = list(value)
    else:
        out = [value]
    out = [int(x) for x in out]
    if rows is not None and len(out) == 1 and rows > 1:
        out = out * rows
    return out


class RingKVPath:
    """The KV-cache path without the projections around it: ring state
    (``sink_size``, ``adapt_sink_thr``, ``evict_idx``; causal_model.py:177-179)
    plus :meth:`attend`.  ``CausalWanSelfAttention`` mixes it in; benchmarks and
    tests that feed q/k/v directly use it on its own."""

    def __init__(self, sink_size: int = 3, adapt_sink_thr: float = -1):
        self.sink_size = sink_size
        self.adapt_sink_thr = adapt_sink_thr
        self.evict_idx = None

    # Ring state as the outside sees it.  With the adaptive sink refresh the
    # decision of a call is made on the device and acted on there (the append
    # that follows takes its slot from the decision kernel); the host picks it
    # up when it next needs the state - normally a whole model pass later, when
    # this layer is called again - so the stream never waits for a read-back.
    # Reading any of the three attributes settles an outstanding decision first.
    _evict_idx: Optional[List[List[int]]] = None
    _last_plan = None
    _last_refresh = None
    _pending = None

    @property
    def evict_idx(self) -> Optional[List[List[int]]]:
        self._settle()
        return self._evict_idx

    @evict_idx.setter
    def evict_idx(self, value) -> None:
        self._settle()
        self._evict_idx = value

    @property
    def last_plan(self):
        """The :class:`ring.AppendPlan` of the last call."""
        self._settle()
        return self._last_plan

    @property
    def last_refresh(self) -> Optional[List[int]]:
        """Per row, the sink frame the last call's adaptive check chose to
        overwrite (-1: none); None when the check did not run."""
        self._settle()
        return self._last_refresh

    def settle(self) -> None:
        """Make the host ring state current.  Call it before the cache dict of
        this layer is re-sliced, replaced or handed to another owner."""
        self._settle()

    def _settle(self) -> None:
        """Bring the host ring state up to date with the device's decision of
        the last call.  A refresh puts (frame + 1) * frame_tokens at the head
        of the row's queue before the call's own queue step
        (causal_model.py:297-299, then :306-316 or :330-335); the end indices
        and the pass counter do not depend on the queue, so the queue (and,
        for an evicting row, the slot recorded in the plan) is all there is to
        correct."""
        pending = self._pending
        if pending is None:
            return
        self._pending = None
        refresh = self._await_decision(pending["host"], pending["stream"])
        self._last_refresh = refresh
        plan, tokens, frame_tokens = pending["plan"], pending["tokens"], pending["frame_tokens"]
        sink_tokens = pending["sink_size"] * frame_tokens
        for i, frame in enumerate(refresh):
            if frame < 0:
                continue
            queue = list(pending["queues"][i])
            queue.insert(0, (frame + 1) * frame_tokens)
            dst_end = ring.advance_queue(queue, plan.evicting[i], plan.held[i], sink_tokens,
                                         pending["starts"][i] + 2 * tokens, pending["cap"])
            self._evict_idx[i][:] = queue
            if plan.evicting[i]:
                plan.dst_start[i] = dst_end - tokens      # where the decision kernel sent the append

    # 0 lets the library choose how many key ranges an attention call is split into
    num_splits = 0
    # None: the chunk is one block, nothing is masked inside it (what the
    # reference's cache path does).  n: blocks of n latent frames, a query sees
    # the cache and its chunk's blocks up to its own (the cache-less path's
    # kv_idx < ends[q_idx], causal_model.py:670-686).
    block_frames: Optional[int] = None

    # what the pinned decision words hold from the launch until the kernel has written them
    _NOT_YET = -(2 ** 31)
    # How often (all paths of the process) a reader found the words still preset
    # and had to wait for the stream: zero in a stream whose layers are called
    # once per model pass; benchmarks print it.
    decision_waits = 0

    def _decision_buffers(self, rows: int, dev):
        """Per path: the device slot override the decision kernel writes and
        the pinned host words it writes the decision to."""
        buf = getattr(self, "_decision", None)
        if buf is None or buf[0].numel() != rows or buf[0].device != dev:
            buf = (torch.full((rows,), -1, dtype=torch.int64, device=dev),
                   torch.empty((rows,), dtype=torch.int32, pin_memory=True))
            self._decision = buf
        return buf

    def _await_decision(self, host: torch.Tensor, stream) -> List[int]:
        """The decision of the last check, once it is on the host.  Nothing is
        recorded on the stream for it (an event between the decision kernel and
        the append costs the stream 6 us per layer): the words are preset to a
        value no decision takes, the kernel stores straight into them, and only
        a reader that comes before they have arrived waits for the stream."""
        refresh = host.tolist()
        if self._NOT_YET in refresh:
            # The host runs ahead of the stream (it enqueues a layer call in a fraction of the time the GPU
            # takes for it), so the kernel that writes these words may not have run yet.  Watching the words
            # lets the host go on the moment they arrive, with the stream still full of work; waiting for the
            # whole stream would drain it first.
            RingKVPath.decision_waits += 1
            deadline = time.monotonic() + 2.0
            while self._NOT_YET in refresh and time.monotonic() < deadline:
                time.sleep(0)
                refresh = host.tolist()
        if self._NOT_YET in refresh:
            stream.synchronize()
            refresh = host.tolist()
            if self._NOT_YET in refresh:
                raise RuntimeError("the adaptive sink decision never arrived: the launch that was to write it failed")
        return refresh

    # Token sums of the cached sink frames, kept between the adaptive checks of
    # this path so that a check reads the new chunk only.  `stale` holds, per
    # cache row, the sink frames whose sums have to be taken from the cache
    # again: all of them for a new cache, and any frame written by a call that
    # did not run the check.
    _sink_sums = None

    def forget_sink_sums(self) -> None:
        """Call after the sink frames of this layer's cache were written behind
        the path's back (copied over, reset, received from another owner)."""
        self._sink_sums = None

    def _kept_sink_sums(self, kv_cache, rows: int, heads: int):
        """The kept sums for this cache, all stale when anything says they may
        not describe it: another dict (also a fresh one that got the old one's
        memory back: the dict carries the token, not the address), other
        tensors, another shape or sink size, contents changed from outside."""
        key = (kv_cache["k"].data_ptr(), kv_cache["v"].data_ptr(), tuple(kv_cache["k"].shape), self.sink_size,
               ring.contents_generation(kv_cache))
        kept = self._sink_sums
        if kept is None or kept["key"] != key or len(kept["stale"]) != rows \
                or kept["owner"] is not ring.sink_sums_owner(kv_cache):
            kept = dict(key=key, owner=ring.sink_sums_owner(kv_cache, create=True),
                        stale=[(1 << self.sink_size) - 1] * rows,
                        sums=ops.new_sink_frame_sums(rows, heads, self.sink_size, kv_cache["k"].device))
            self._sink_sums = kept
        return kept

    def _sink_frames_written(self, kv_cache, plan, tokens: int, frame_tokens: int) -> None:
        """A call that did not run the check wrote plan.dst_start: the kept sums
        of the sink frames it touched are stale."""
        kept = self._sink_sums
        if kept is None or kept["key"][0] != kv_cache["k"].data_ptr() \
                or kept["owner"] is not ring.sink_sums_owner(kv_cache):
            return
        for i, dst in enumerate(plan.dst_start[:len(kept["stale"])]):
            for frame in range(dst // frame_tokens, min(self.sink_size, (dst + tokens - 1) // frame_tokens + 1)):
                kept["stale"][i] |= 1 << frame

    def _layer_launcher(self, q, k, v, kv_cache, table, grid, qk_norm=None, keep_roped_q=False):
        """The cached launch descriptors for this layer, rebuilt when the
        cache, the shapes, the grid or the norm weights change.  keep_roped_q:
        the caller wants the normalised, rotated query back, so the append
        writes it (otherwise, with the norm folded in, no such tensor exists)."""
        launcher = getattr(self, "_launcher", None)
        in_attention = not (keep_roped_q and qk_norm is not None)
        if launcher is None or not launcher.matches(q, k, v, kv_cache, table, qk_norm) \
                or launcher.rope_in_attention != in_attention \
                or (launcher.ap.grid_f, launcher.ap.grid_h, launcher.ap.grid_w) != tuple(grid):
            launcher = ops.LayerLauncher(kv_cache["k"], kv_cache["v"], kv_cache["global_end_index"],
                                         kv_cache["local_end_index"], table, grid, q, k, v, qk_norm=qk_norm,
                                         rope_in_attention=in_attention)
            self._launcher = launcher
        if launcher.forced_splits != self.num_splits:
            launcher.forced_splits = self.num_splits
            launcher.span = -1
        return launcher

    def attend(self, q, k, v, grid_sizes, freqs, kv_cache, current_start,
               return_roped_query: bool = False, qk_norm=None):
        """RoPE + ring append + attention for q/k/v [B, S, H, 128]
        (causal_model.py:250-384).  With ``qk_norm`` = (q weight, k weight,
        eps), q and k are the raw projection outputs and their RMSNorm
        (qkv_fn, causal_model.py:212-218) runs inside the append kernel."""
        rows = q.shape[0]
        grids = _host_ints(grid_sizes, "grid")
        f, h, w = grids[0], grids[1], grids[2]
        for r in range(1, len(grids) // 3):
            if tuple(grids[3 * r:3 * r + 3]) != (f, h, w):
                raise RuntimeError("all rows of a call must share one (F, H, W) grid")
        frame_tokens = h * w
        starts = _host_ints(current_start, "start", rows)
        if len(starts) != rows:
            raise RuntimeError(f"current_start has {len(starts)} entries for {rows} rows")

        self._settle()
        cache_rows = kv_cache["k"].shape[0]
        if self._evict_idx is None:
            self._evict_idx = [[]]
        if len(self._evict_idx) < cache_rows:
            self._evict_idx = [list(self._evict_idx[0]) for _ in range(cache_rows)]

        table = ops.device_freqs(freqs, q.device)
        self._last_refresh = None
        adaptive = self.sink_size * frame_tokens > 0 and self.adapt_sink_thr > -1 and q.shape[1] <= frame_tokens
        k_norm = (qk_norm[1], qk_norm[2]) if qk_norm is not None else None
        if adaptive:
            if q.shape[1] != frame_tokens:
                raise RuntimeError(
                    f"adaptive sink refresh needs one-frame chunks ({frame_tokens} tokens), got {q.shape[1]}"
                )   # the reference's reshape(1, frame_seqlen, -1) fails the same way
            evicting = ring.rows_evicting(kv_cache, starts, q.shape[1])
            if any(e and not queue for e, queue in zip(evicting, self._evict_idx)):
                # A full cache with an empty queue can only go on if this very call
                # refreshes (otherwise causal_model.py:306 raises IndexError):
                # the decision is needed before anything can be planned.
                _, refresh = ops.sink_similarity(
                    k, v, kv_cache["k"], kv_cache["v"], table, (h, w), [c // frame_tokens for c in starts],
                    self.sink_size, self.adapt_sink_thr, k_norm=k_norm)
                self._last_refresh = refresh.tolist()
                for i, frame in enumerate(self._last_refresh):
                    if frame >= 0:
                        self._evict_idx[i].insert(0, (frame + 1) * frame_tokens)
                adaptive = False
            else:
                queues_before = [list(queue) for queue in self._evict_idx]

        # Planning advances the host's ring state (queues, pass counter, index mirror) before the launches
        # are validated: a call that fails - a frame beyond the RoPE table, say - must leave it where it was.
        undo = (copy.deepcopy(self._evict_idx), kv_cache.get("current_step"))
        try:
            # planned as if no row refreshed; _settle() corrects the host state later where one did
            plan = ring.plan_append(kv_cache, self._evict_idx, starts, q.shape[1], frame_tokens, self.sink_size)
            override = None
            if adaptive:
                # adaptive sink refresh (causal_model.py:284-299): one fused
                # reduction on the device, whose decision goes straight to the
                # append below and, written into pinned memory by the kernel, to the host
                override, host = self._decision_buffers(rows, q.device)
                assert self._pending is None, "the last decision must be settled before its words are preset again"
                host.fill_(self._NOT_YET)
                kept = self._kept_sink_sums(kv_cache, rows, q.shape[2])
                extra = {}
                if kept is not None:
                    # where the chunk lands by the plan, if that is a sink frame: a row still filling,
                    # or an evicting one whose queue is headed by a refresh decided while it was filling
                    planned = [d // frame_tokens if d < self.sink_size * frame_tokens else -1 for d in plan.dst_start]
                    extra = dict(frame_sums=kept["sums"], stale_frames=list(kept["stale"]), planned_frames=planned)
                    kept["stale"] = [0] * rows        # summed now, and kept current by the decision kernel from here on
                ops.sink_similarity(
                    k, v, kv_cache["k"], kv_cache["v"], table, (h, w), [c // frame_tokens for c in starts],
                    self.sink_size, self.adapt_sink_thr, dst_start_override=override, override_rows=plan.evicting,
                    refresh_out=host, k_norm=k_norm, **extra)
                self._pending = dict(stream=torch.cuda.current_stream(q.device), host=host, plan=plan, queues=queues_before, starts=list(starts),
                                     tokens=q.shape[1], frame_tokens=frame_tokens, sink_size=self.sink_size,
                                     cap=kv_cache["k"].shape[1])
            if not adaptive:
                self._sink_frames_written(kv_cache, plan, q.shape[1], frame_tokens)
            span = plan.max_seq_len
            seq = None
            if any(n != span for n in plan.new_local_end):
                # rows differ only while the stream batch is still filling; the
                # lengths are a handful of host ints, shipped asynchronously
                seq = torch.tensor(plan.new_local_end, dtype=torch.int32).to(q.device, non_blocking=True)
            self._last_plan = plan
            mask_tokens = 0
            if self.block_frames is not None and self.block_frames * frame_tokens < q.shape[1]:
                mask_tokens = self.block_frames * frame_tokens

            if q.dtype == torch.bfloat16 and rows <= ops._capi.MAX_ROWS:
                # steady-state fast path: launch descriptors are built once per
                # (cache, shape) and only patched per call
                launcher = self._layer_launcher(q, k, v, kv_cache, table, (f, h, w), qk_norm, return_roped_query)
                start_frames = [c // frame_tokens for c in starts]
                out = launcher.launch(q, k, v, start_frames, plan, seq, mask_tokens, override)
                if return_roped_query:
                    # the attention kernel rotates q on the fly and keeps no copy: the
                    # stand-alone rotation gives the same bits (one arithmetic for both)
                    if launcher.roped_q is not None:
                        return out, launcher.roped_q.clone()
                    return out, ops.causal_rope_apply(q, [(f, h, w)] * rows, table, torch.tensor(start_frames))
                return out

            roped_q = ops.kv_append_rope(
                q, k, v, kv_cache["k"], kv_cache["v"], table, (f, h, w),
                [c // frame_tokens for c in starts], plan.dst_start,
                global_end_index=kv_cache["global_end_index"],
                local_end_index=kv_cache["local_end_index"],
                new_global_end=plan.new_global_end,
                new_local_end=plan.new_local_end,
                qk_norm=qk_norm,
                dst_start_override=override,
            )
            mask = dict(chunk_key_start=list(plan.dst_start), mask_block_tokens=mask_tokens) if mask_tokens else {}
            # (fp32 storage, the reference's CPU-runnable configuration, is computed in
            # fp32 throughout by a plain kernel; the matrix-core kernel is the bf16 one)
            out = ops.swa_attention(roped_q, kv_cache["k"][:, :span], kv_cache["v"][:, :span], seq, **mask)
            if return_roped_query:
                return out, roped_q
            return out

        except Exception:
            if self._pending is not None:
                # a decision kernel may be on its way: let it store its (now unwanted) words
                # before a later call presets them again
                self._pending["stream"].synchronize()
            self._evict_idx, self._pending, self._sink_sums = undo[0], None, None
            # a launch that was refused started nothing; one that failed on the device may have left
            # ticket words of this stream's workspaces non-zero, which every later call would trip over
            ops.reset_workspace_tickets(q.device)
            if undo[1] is not None:
                kv_cache["current_step"] = undo[1]
            ring.forget_index_mirror(kv_cache)        # the device tensors are authoritative again
            raise

class CausalWanSelfAttention(nn.Module, RingKVPath):

    def __init__(self, dim, num_heads, window_size=(-1, -1), qk_norm=True, eps=1e-6):
        assert dim % num_heads == 0
        nn.Module.__init__(self)
        self.dim = dim
        self.num_heads = num_heads
        self.head_dim = dim // num_heads
        self.window_size = window_size
        self.qk_norm = qk_norm
        self.eps = eps

        # The q / k RMSNorm runs inside the append kernel (its sum of squares in
        # the order of torch's CPU kernel, so the cache holds the bits the
        # reference's CPU path would store); False applies the two norms as
        # separate torch modules before the path.
        self.fuse_qk_norm = True

        # The q, k and v projections (causal_model.py:212-218 calls the three
        # Linears one after the other) run as ONE vendor GEMM on the three
        # weights laid end to end: at 1560 tokens x 1536 the three launches take
        # 60 us and the one 26 us, with the same bits out (every output element
        # is the same dot product over `dim`).  q, k and v are then strided views
        # of one [B, S, 3 * dim] tensor, which the kernels of the path read as
        # they are.  The packed copy of the weights (3 * dim * dim elements per
        # layer) is rebuilt whenever a weight or bias has been replaced or
        # written.  Only plain nn.Linear layers without forward hooks are packed
        # (a wrapped layer or a hook gets the three calls it expects); False
        # keeps the three launches and no copy.
        self.fuse_qkv_projection = True
        self._packed = None

        # ring state, same defaults as causal_model.py:177-179
        self.sink_size = 3
        self.adapt_sink_thr = -1
        self.evict_idx: Optional[List[List[int]]] = None

        self.q = nn.Linear(dim, dim)
        self.k = nn.Linear(dim, dim)
        self.v = nn.Linear(dim, dim)
        self.o = nn.Linear(dim, dim)
        self.norm_q = WanRMSNorm(dim, eps=eps) if qk_norm else nn.Identity()
        self.norm_k = WanRMSNorm(dim, eps=eps) if qk_norm else nn.Identity()

    # ------------------------------------------------------------------
    def _packed_qkv(self):
        """(weight [3 * dim, dim], bias [3 * dim] or None) of the q, k and v
        Linears laid end to end, rebuilt when any of the six tensors has been
        replaced (another tensor, dtype or device) or written in place."""
        layers = (self.q, self.k, self.v)
        for layer in layers:
            # only plain Linears that nobody watches: a wrapped or replaced layer (an adapter, a quantised
            # Linear) computes something else than x W^T + b, and a hook expects its layer to be called
            if type(layer) is not nn.Linear or layer._forward_hooks or layer._forward_pre_hooks:
                return None
        tensors = [t for layer in layers for t in (layer.weight, layer.bias)]

        def edits(t):
            try:
                return t._version
            except RuntimeError:                   # a tensor made under inference_mode() counts no edits:
                return -1                          # after writing such a weight in place, set _packed = None

        key = tuple((t.data_ptr(), edits(t), t.dtype, t.device) if t is not None else None for t in tensors)
        packed = self._packed
        if packed is None or packed[0] != key:
            with torch.no_grad():
                weight = torch.cat([layer.weight.detach() for layer in layers], 0)
                biases = [layer.bias for layer in layers]
                bias = None
                if all(b is not None for b in biases):
                    bias = torch.cat([b.detach() for b in biases], 0)
                elif any(b is not None for b in biases):
                    return None                    # mixed: keep the three launches
            packed = (key, weight, bias)
            self._packed = packed
        return packed[1], packed[2]

    def project_qkv(self, x):
        """The three projections of x [B, S, dim] -> q, k, v, each [B, S, dim]
        (views of one tensor when they come out of one GEMM)."""
        import torch.nn.modules.module as _hooks
        watched = _hooks._global_forward_hooks or _hooks._global_forward_pre_hooks
        packed = self._packed_qkv() if self.fuse_qkv_projection and not torch.is_grad_enabled() and not watched else None
        if packed is None:
            return self.q(x), self.k(x), self.v(x)
        y = nn.functional.linear(x, packed[0], packed[1])
        d = self.dim
        return y[..., :d], y[..., d:2 * d], y[..., 2 * d:]

    def forward(
        self,
        x,
        seq_lens,
        grid_sizes,
        freqs,
        block_mask,
        kv_cache=None,
        current_start=0,
        current_end=0,
        causal_rope_cache=None,
    ):
        """x [B, S, dim]; grid_sizes [B, 3] = (F, H, W); freqs complex128
        [1024, head_dim/2]; ``current_end`` and ``causal_rope_cache`` are
        accepted and unused, as ``current_end`` is in the reference (:281)."""
        if kv_cache is None:
            raise NotImplementedError(
                "only the KV-cache inference path is built; the cache-less flex-attention "
                "training path (causal_model.py:220-249) is out of scope"
            )
        b, s, n, d = *x.shape[:2], self.num_heads, self.head_dim
        q, k, v = self.project_qkv(x)
        v = v.view(b, s, n, d)
        if self.qk_norm and self.fuse_qk_norm and x.dtype in (torch.bfloat16, torch.float32) \
                and self.num_heads <= 64:
            # the two RMSNorms run inside the append kernel
            q, k = q.view(b, s, n, d), k.view(b, s, n, d)
            norm = (self.norm_q.weight.detach(), self.norm_k.weight.detach(), self.eps)
            out = self.attend(q, k, v, grid_sizes, freqs, kv_cache, current_start, qk_norm=norm)
        else:
            q = self.norm_q(q).view(b, s, n, d)
            k = self.norm_k(k).view(b, s, n, d)
            out = self.attend(q, k, v, grid_sizes, freqs, kv_cache, current_start)
        return self.o(out.flatten(2))


class WanT2VCrossAttention(nn.Module):
    """Text cross-attention with the per-prompt K/V cache
    (wan_base/modules/model.py:160-196): same constructor, child module names
    and ``forward(x, context, context_lens, crossattn_cache=None)``.  The first
    call of a prompt projects the context and stores K/V in the cache dict;
    later calls read them.  The attention itself is the library's kernel on
    the 512 cached keys."""

    def __init__(self, dim, num_heads, window_size=(-1, -1), qk_norm=True, eps=1e-6):
        assert dim % num_heads == 0
        super().__init__()
        self.dim = dim
        self.num_heads = num_heads
        self.head_dim = dim // num_heads
        self.window_size = window_size
        self.qk_norm = qk_norm
        self.eps = eps
        self.q = nn.Linear(dim, dim)
        self.k = nn.Linear(dim, dim)
        self.v = nn.Linear(dim, dim)
        self.o = nn.Linear(dim, dim)
        self.norm_q = WanRMSNorm(dim, eps=eps) if qk_norm else nn.Identity()
        self.norm_k = WanRMSNorm(dim, eps=eps) if qk_norm else nn.Identity()

    def forward(self, x, context, context_lens, crossattn_cache=None):
        """x [B, L1, dim]; context [B, L2, dim]; context_lens [B] or None."""
        b, n, d = x.size(0), self.num_heads, self.head_dim
        q = self.norm_q(self.q(x)).view(b, -1, n, d)
        if crossattn_cache is not None and crossattn_cache["is_init"]:
            k, v = crossattn_cache["k"], crossattn_cache["v"]
        else:
            k = self.norm_k(self.k(context)).view(b, -1, n, d)
            v = self.v(context).view(b, -1, n, d)
            if crossattn_cache is not None:
                crossattn_cache["is_init"] = True
                crossattn_cache["k"] = k
                crossattn_cache["v"] = v
        out = ops.flash_attention(q, k, v, k_lens=context_lens)
        return self.o(out.flatten(2))
