"""Operator-level Python surface over the sdv2kv C ABI.

``flash_attn_with_kvcache`` keeps the four-argument call the reference makes
(models/wan/causal_model.py:353-358); ``kv_append_rope`` is the fused
replacement for causal_rope_apply + the per-row slice writes (:253-266,
:321-342).  PyTorch supplies device memory and the current stream only.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence, Tuple

import torch

from . import _capi

HEAD_DIM = _capi.HEAD_DIM

_DTYPES = {torch.bfloat16: _capi.DTYPE_BF16, torch.float32: _capi.DTYPE_F32}


def _require_gpu(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    for t in tensors:
        if t is None:
            continue
        if t.device.type != "cuda":
            raise RuntimeError(
                "sdv2kv operators run on the GPU only (tensor on %s); there is no CPU path" % t.device
            )
        if t.device != dev:
            raise RuntimeError(f"tensors on different devices: {t.device} vs {dev}")
    return dev


def _stride3(t: torch.Tensor, name: str) -> _capi.Stride3:
    if t.dim() != 4 or t.shape[-1] != HEAD_DIM:
        raise RuntimeError(f"{name}: expected [rows, tokens, heads, {HEAD_DIM}], got {tuple(t.shape)}")
    if t.shape[-1] > 1 and t.stride(-1) != 1:
        raise RuntimeError(f"{name}: last dimension must be contiguous (stride {t.stride(-1)})")
    return _capi.Stride3(t.stride(0), t.stride(1), t.stride(2))


def _stream_ptr(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


def _current_device_index() -> int:
    return torch.cuda.current_device()


class _NoSwitch:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on_device(dev: torch.device):
    """Context in which ``dev`` is the current device: torch's guard when it is
    another one, nothing at all (the usual case, and several microseconds less
    per call) when it already is."""
    return _NO_SWITCH if torch.cuda.current_device() == dev.index else torch.cuda.device(dev)


def _i64_array(values: Sequence[int]):
    return (C.c_int64 * len(values))(*[int(v) for v in values])


_FREQS_CACHE: dict = {}


def device_freqs(freqs: torch.Tensor, device: torch.device) -> torch.Tensor:
    """The complex128 [rows, 64] RoPE table as float64 [rows, 64, 2] on
    ``device``.  Converted once per (table, device)."""
    try:
        version = freqs._version
    except RuntimeError:            # created under torch.inference_mode(): no edit counter
        version = None
    key = (id(freqs), version, freqs.data_ptr(), str(device))
    hit = _FREQS_CACHE.get(key)
    if hit is not None and hit[0] is freqs:
        return hit[1]
    if freqs.dtype != torch.complex128 or freqs.dim() != 2 or freqs.shape[1] != HEAD_DIM // 2:
        raise RuntimeError(
            f"freqs must be complex128 [rows, {HEAD_DIM // 2}], got {freqs.dtype} {tuple(freqs.shape)}"
        )
    table = torch.view_as_real(freqs.detach().resolve_conj()).contiguous().to(device)
    if len(_FREQS_CACHE) > 8:
        _FREQS_CACHE.clear()
    _FREQS_CACHE[key] = (freqs, table)
    return table


def _check_norm(qk_norm, dtype, heads: int, dev) -> None:
    wq, wk, eps = qk_norm
    for w in (wq, wk):
        if w.dtype != dtype or w.numel() != heads * HEAD_DIM or not w.is_contiguous() or w.device != dev:
            raise RuntimeError(f"norm weights must be contiguous {dtype} tensors of {heads * HEAD_DIM} elements on {dev}")
    if not eps >= 0:
        raise RuntimeError("norm eps must be >= 0")


def _check_override(t: torch.Tensor, rows: int, dev) -> None:
    if t.dtype != torch.int64 or t.numel() < rows or not t.is_contiguous() or t.device != dev:
        raise RuntimeError(f"dst_start_override must be a contiguous int64 tensor with one entry per row on {dev}")


def kv_append_rope(
    q: Optional[torch.Tensor],
    k: torch.Tensor,
    v: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    freqs_table: torch.Tensor,
    grid: Tuple[int, int, int],
    start_frames: Sequence[int],
    dst_starts: Sequence[int],
    q_out: Optional[torch.Tensor] = None,
    global_end_index: Optional[torch.Tensor] = None,
    local_end_index: Optional[torch.Tensor] = None,
    new_global_end: Optional[Sequence[int]] = None,
    new_local_end: Optional[Sequence[int]] = None,
    qk_norm: Optional[Tuple[torch.Tensor, torch.Tensor, float]] = None,
    dst_start_override: Optional[torch.Tensor] = None,
    q_inv_rms: Optional[torch.Tensor] = None,
) -> Optional[torch.Tensor]:
    """RoPE q and k, write k' and v into the cache at ``dst_starts`` and store
    the new end indices.  Returns the roped query (``q_out`` or a new tensor).

    ``dst_start_override`` (device int64 [B], written by
    :func:`sink_similarity`) replaces ``dst_starts[i]`` where it holds a value
    >= 0.

    ``qk_norm`` = (q weight, k weight, eps) folds the WanRMSNorm of the
    projection outputs in (wan_base/modules/model.py:70-86): q and k are then
    the raw projection outputs.  With ``q_inv_rms`` (float32 [B, S] on the
    device) the kernel stores 1 / rms of every q token there and writes NO
    rotated query (returns None): :func:`swa_attention` takes the raw q with
    ``q_norm=(q weight, q_inv_rms)`` and normalises and rotates it itself.

    ``freqs_table`` is :func:`device_freqs` output.  Rows are processed in
    groups of at most 16 per launch.
    """
    dev = _require_gpu(k, v, k_cache, v_cache, freqs_table, q, q_out, global_end_index, local_end_index)
    if k.dtype not in _DTYPES:
        raise RuntimeError(f"unsupported dtype {k.dtype}")
    for t in (q, v, k_cache, v_cache, q_out):
        if t is not None and t.dtype != k.dtype:
            raise RuntimeError(f"dtype mismatch: {t.dtype} vs {k.dtype}")
    rows, tokens, heads, _ = k.shape
    if q_inv_rms is not None:
        if qk_norm is None or q is None or q_out is not None:
            raise RuntimeError("q_inv_rms goes with qk_norm and q, and replaces q_out")
        if q_inv_rms.dtype != torch.float32 or q_inv_rms.numel() != rows * tokens or not q_inv_rms.is_contiguous() \
                or q_inv_rms.device != dev:
            raise RuntimeError(f"q_inv_rms must be a contiguous float32 tensor of {rows} x {tokens} elements on {dev}")
    elif q is not None and q_out is None:
        q_out = torch.empty((rows, tokens, heads, HEAD_DIM), dtype=q.dtype, device=dev)
    for name, t in (("q", q), ("v", v), ("q_out", q_out)):
        if t is not None and tuple(t.shape) != tuple(k.shape):
            raise RuntimeError(f"{name} shape {tuple(t.shape)} differs from k {tuple(k.shape)}")
    if k_cache.shape[0] < rows or v_cache.shape != k_cache.shape or k_cache.shape[2] != heads:
        raise RuntimeError(f"cache shape {tuple(k_cache.shape)} / {tuple(v_cache.shape)} does not fit k {tuple(k.shape)}")
    if len(start_frames) != rows or len(dst_starts) != rows:
        raise RuntimeError("start_frames and dst_starts need one entry per row")
    for idx in (global_end_index, local_end_index):
        if idx is not None and (idx.dtype != torch.int64 or idx.numel() < rows or not idx.is_contiguous()):
            raise RuntimeError("end-index tensors must be contiguous int64 with one entry per row")
    if freqs_table.dtype != torch.float64 or not freqs_table.is_contiguous():
        raise RuntimeError("freqs_table must be the contiguous float64 view from device_freqs()")
    if qk_norm is not None:
        _check_norm(qk_norm, k.dtype, heads, dev)
        if q is None:
            raise RuntimeError("the fused q/k norm needs q")
    if dst_start_override is not None:
        _check_override(dst_start_override, rows, dev)

    lib = _capi.lib()
    stream = _stream_ptr(dev)
    with _on_device(dev):
        for r0 in range(0, rows, _capi.MAX_ROWS):
            r1 = min(rows, r0 + _capi.MAX_ROWS)
            p = _capi.AppendParams()
            sl = slice(r0, r1)
            if q is not None:
                p.q_in, p.q_in_stride = q[sl].data_ptr(), _stride3(q, "q")
                if q_out is not None:
                    p.q_out, p.q_out_stride = q_out[sl].data_ptr(), _stride3(q_out, "q_out")
                else:
                    p.q_inv_rms = q_inv_rms.data_ptr() + 4 * r0 * tokens
            p.k_in, p.k_in_stride = k[sl].data_ptr(), _stride3(k, "k")
            p.v_in, p.v_in_stride = v[sl].data_ptr(), _stride3(v, "v")
            p.k_cache, p.k_cache_stride = k_cache[sl].data_ptr(), _stride3(k_cache, "k_cache")
            p.v_cache, p.v_cache_stride = v_cache[sl].data_ptr(), _stride3(v_cache, "v_cache")
            p.freqs = freqs_table.data_ptr()
            p.freq_rows = freqs_table.shape[0]
            p.dtype = _DTYPES[k.dtype]
            p.rows, p.tokens, p.heads, p.head_dim = r1 - r0, tokens, heads, HEAD_DIM
            p.grid_f, p.grid_h, p.grid_w = (int(x) for x in grid)
            p.cache_tokens = k_cache.shape[1]
            sf = _i64_array(start_frames[r0:r1])
            ds = _i64_array(dst_starts[r0:r1])
            p.start_frame = C.cast(sf, C.POINTER(C.c_int64))
            p.dst_start = C.cast(ds, C.POINTER(C.c_int64))
            if global_end_index is not None or local_end_index is not None:
                if new_global_end is None or new_local_end is None:
                    raise RuntimeError("new_global_end/new_local_end are required with the index tensors")
                ng = _i64_array(new_global_end[r0:r1])
                nl = _i64_array(new_local_end[r0:r1])
                p.new_global_end = C.cast(ng, C.POINTER(C.c_int64))
                p.new_local_end = C.cast(nl, C.POINTER(C.c_int64))
                if global_end_index is not None:
                    p.global_end_index = global_end_index.data_ptr() + 8 * r0
                if local_end_index is not None:
                    p.local_end_index = local_end_index.data_ptr() + 8 * r0
            p.stream = stream
            if qk_norm is not None:
                p.q_norm_weight, p.k_norm_weight = qk_norm[0].data_ptr(), qk_norm[1].data_ptr()
                p.norm_eps = float(qk_norm[2])
            if dst_start_override is not None:
                p.dst_start_override = dst_start_override.data_ptr() + 8 * r0
            _capi.check(lib.sdv2_kv_append_rope(C.byref(p)), "sdv2_kv_append_rope")
    return q_out


def causal_rope_apply(x: torch.Tensor, grid_sizes, freqs: torch.Tensor, start_frame=0, rope_cache=None) -> torch.Tensor:
    """The reference's ``causal_rope_apply`` (causal_model.py:94-108) as one
    launch per run of rows with the same grid: row i of ``x`` [B, L, H, 128]
    is rotated over its first f*h*w tokens for ``grid_sizes[i]`` = (f, h, w)
    starting at frame ``start_frame`` (an int, or one entry per row); later
    tokens and rows without a grid are returned as they are.  Bit-identical to
    the reference's complex128 product rounded to ``x``'s dtype.

    ``freqs`` is the model's complex128 table or :func:`device_freqs` output.
    ``rope_cache`` (the reference's pre-expanded per-token factors) is accepted
    and not used: the kernel indexes the table itself.  The KV-cache path does
    not call this: its append rotates q and k while it writes the cache.
    """
    dev = _require_gpu(x)
    if x.dtype not in _DTYPES:
        raise RuntimeError(f"unsupported dtype {x.dtype}")
    rows, length, heads, _ = x.shape
    grids = grid_sizes.tolist() if isinstance(grid_sizes, torch.Tensor) else [list(g) for g in grid_sizes]
    grids = [tuple(int(n) for n in g) for g in grids][:rows]
    if isinstance(start_frame, torch.Tensor):
        starts = [int(s) for s in start_frame.reshape(-1).tolist()][:len(grids)]
        grids = grids[:len(starts)]                    # the reference zips the two
    else:
        starts = [int(start_frame)] * len(grids)
    for f, h, w in grids:
        if min(f, h, w) <= 0 or f * h * w > length:
            raise RuntimeError(f"grid {(f, h, w)} does not fit {length} tokens")
    table = freqs if freqs.dtype == torch.float64 and freqs.device == dev else device_freqs(freqs, dev)
    if table.dim() != 3 or tuple(table.shape[1:]) != (HEAD_DIM // 2, 2) or not table.is_contiguous():
        raise RuntimeError("freqs must be the complex128 table or the float64 view from device_freqs()")
    _stride3(x, "x")
    whole = len(grids) == rows and all(f * h * w == length for f, h, w in grids)
    out = torch.empty_like(x) if whole else x.clone()
    if out.stride() != x.stride():
        raise RuntimeError("x must be dense (its copy did not keep the strides)")

    lib = _capi.lib()
    with _on_device(dev):
        r0 = 0
        while r0 < len(grids):
            r1 = r0 + 1
            while r1 < len(grids) and r1 - r0 < _capi.MAX_ROWS and grids[r1] == grids[r0]:
                r1 += 1
            f, h, w = grids[r0]
            p = _capi.AppendParams()
            p.q_in, p.q_in_stride = x[r0:r1].data_ptr(), _stride3(x, "x")
            p.q_out, p.q_out_stride = out[r0:r1].data_ptr(), _stride3(out, "out")
            p.freqs, p.freq_rows = table.data_ptr(), table.shape[0]
            p.dtype = _DTYPES[x.dtype]
            p.rows, p.tokens, p.heads, p.head_dim = r1 - r0, f * h * w, heads, HEAD_DIM
            p.grid_f, p.grid_h, p.grid_w = f, h, w
            sf = _i64_array(starts[r0:r1])
            p.start_frame = C.cast(sf, C.POINTER(C.c_int64))
            p.stream = _stream_ptr(dev)
            _capi.check(lib.sdv2_kv_append_rope(C.byref(p)), "sdv2_kv_append_rope")
            r0 = r1
    return out


_WORKSPACES: dict = {}


TICKET_BYTES = 65536          # head of an attention workspace (256 bytes for a sink-similarity one)


def new_workspace(dev: torch.device, nbytes: int) -> torch.Tensor:
    """A split-KV workspace as the library wants it: zero-filled once (its
    ticket words start at zero and every call leaves them there).  Only
    buffers made here are accepted as ``workspace=``: a ticket word that does
    not start at zero makes a split call combine early or never, silently."""
    ws = torch.zeros(max(nbytes, 1), dtype=torch.uint8, device=dev)
    ws._sdv2_workspace = True
    return ws


def reset_workspace_tickets(dev: torch.device) -> None:
    """Zero the ticket words of this stream's workspaces again.  Every call
    that completes leaves them at zero; after a launch that failed on the
    device they may not be."""
    if dev.type != "cuda" or not (_WORKSPACES or _SIM_WORKSPACES):
        return
    key = (dev, _stream_ptr(dev))
    for pool in (_WORKSPACES, _SIM_WORKSPACES):
        ws = pool.get(key)
        if ws is not None:
            ws[:TICKET_BYTES].zero_()


def _workspace(dev: torch.device, nbytes: int, pool: Optional[dict] = None) -> torch.Tensor:
    """Scratch for split-KV partials, one buffer per (device, stream), grown on
    demand and reused.  Calls on one stream run one after another, so they can
    share a buffer; calls on different streams may overlap in time and must not
    (their tickets and partial results would mix), so each stream gets its own."""
    pool = _WORKSPACES if pool is None else pool
    key = (dev, _stream_ptr(dev))
    ws = pool.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = new_workspace(dev, nbytes)
        pool[key] = ws
    return ws


def chunk_starts_tensor(starts, rows: int, q_tokens: int, max_seq_len: int, dev) -> torch.Tensor:
    """Per-row cache position of the chunk's own keys as the int32 device
    tensor the attention kernel reads; host values are range-checked here."""
    if isinstance(starts, torch.Tensor):
        if starts.dtype != torch.int32 or starts.numel() != rows or starts.device != dev or not starts.is_contiguous():
            raise RuntimeError("chunk_key_start must be a contiguous int32 device tensor with one entry per row")
        return starts
    if starts is None or len(starts) != rows:
        raise RuntimeError("mask_block_tokens needs chunk_key_start with one entry per row")
    for x in starts:
        if x < 0 or x + q_tokens > max_seq_len:
            raise RuntimeError(f"chunk_key_start {x} puts the chunk outside the {max_seq_len}-key view")
    return torch.tensor([int(x) for x in starts], dtype=torch.int32).to(dev, non_blocking=True)


def swa_attention(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    seq_lens: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
    num_splits: int = 0,
    softmax_scale: Optional[float] = None,
    workspace: Optional[torch.Tensor] = None,
    chunk_key_start: Optional[torch.Tensor] = None,
    mask_block_tokens: int = 0,
    static_scratch: bool = False,
    rope: Optional[Tuple[torch.Tensor, Sequence[int], Sequence[int]]] = None,
    q_norm: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
) -> torch.Tensor:
    """out[b] = softmax(q[b] k_cache[b,:seq_lens[b]]^T * scale) v_cache[b,:seq_lens[b]].

    ``rope`` = (:func:`device_freqs` table, (grid_h, grid_w), start frame per
    row): q is the query BEFORE RoPE and is rotated inside the kernel exactly as
    :func:`kv_append_rope` would have rotated it (S must be whole frames).  A
    caller-owned ``workspace`` must come from :func:`new_workspace` (zero-filled).
    With ``q_norm`` = (q norm weight, q_inv_rms from :func:`kv_append_rope`) as
    well, q is the raw q projection and is RMS-normalised before the rotation.

    ``static_scratch`` takes the library's allocation-free entry point
    (``sdv2_swa_attn_fwd_static``): partial results of a split call go to device
    memory the library holds itself (64 MiB per GPU, shared by all calls on
    that GPU), no workspace is sized or allocated here; with ``out`` given the
    whole call then allocates nothing.

    q [B,S,H,128] bf16; k_cache/v_cache [B,L,H,128] bf16 views with any row /
    token / head strides; seq_lens int32 [B] on the device (None = L).  All
    three may be fp32 instead (the reference's CPU-runnable configuration): the
    result is then computed in fp32 throughout, by a plain kernel that walks the
    whole key range (q rotated beforehand, ``num_splits`` ignored).
    With ``mask_block_tokens`` = b in (0, S) and ``chunk_key_start`` (int32 [B]
    on the device, or host ints: where each row's own chunk sits in the cache)
    query token t does not see the chunk's later blocks
    [start + (t // b + 1) * b, start + S).
    """
    dev = _require_gpu(q, k_cache, v_cache, seq_lens, out, workspace)
    if q.dtype not in _DTYPES or k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise RuntimeError("swa_attention takes q and both caches in one dtype, bf16 or fp32; got %s/%s/%s"
                           % (q.dtype, k_cache.dtype, v_cache.dtype))
    fp32 = q.dtype == torch.float32
    if fp32 and (rope is not None or static_scratch):
        raise RuntimeError("fp32 attention takes rotated queries and one key range (no rope=, no static_scratch=)")
    rows, q_tokens, heads, _ = q.shape
    if k_cache.shape[0] != rows or k_cache.shape[2] != heads or v_cache.shape != k_cache.shape:
        raise RuntimeError(f"cache view {tuple(k_cache.shape)} / {tuple(v_cache.shape)} does not match q {tuple(q.shape)}")
    if seq_lens is not None and (seq_lens.dtype != torch.int32 or seq_lens.numel() != rows or not seq_lens.is_contiguous()):
        raise RuntimeError("seq_lens must be a contiguous int32 tensor with one entry per row")
    if out is None:
        out = torch.empty((rows, q_tokens, heads, HEAD_DIM), dtype=q.dtype, device=dev)
    elif out.dtype != q.dtype or tuple(out.shape) != tuple(q.shape):
        raise RuntimeError("out must have q's dtype and shape")

    lib = _capi.lib()
    max_seq_len = k_cache.shape[1]
    if fp32:
        num_splits = 1          # the fp32 kernel walks the whole key range
    elif num_splits <= 0:
        num_splits = lib.sdv2_swa_attn_default_splits(rows, q_tokens, heads, max_seq_len)
    need = 0 if static_scratch else lib.sdv2_swa_attn_workspace_bytes(rows, q_tokens, heads, max_seq_len, num_splits)
    if workspace is not None and not getattr(workspace, "_sdv2_workspace", False):
        raise RuntimeError("workspace= takes a buffer made by ops.new_workspace() (zero-filled ticket words)")
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = _workspace(dev, need)

    p = _capi.AttnParams()
    p.q, p.q_stride = q.data_ptr(), _stride3(q, "q")
    p.k_cache, p.k_stride = k_cache.data_ptr(), _stride3(k_cache, "k_cache")
    p.v_cache, p.v_stride = v_cache.data_ptr(), _stride3(v_cache, "v_cache")
    p.out, p.out_stride = out.data_ptr(), _stride3(out, "out")
    p.seq_lens = seq_lens.data_ptr() if seq_lens is not None else None
    p.rows, p.q_tokens, p.heads, p.head_dim = rows, q_tokens, heads, HEAD_DIM
    p.max_seq_len = max_seq_len
    p.num_splits = num_splits
    p.dtype = _DTYPES[q.dtype]
    p.softmax_scale = float(softmax_scale) if softmax_scale else 0.0
    if need:
        p.workspace = workspace.data_ptr()
        p.workspace_bytes = workspace.numel() * workspace.element_size()
    p.stream = _stream_ptr(dev)
    if mask_block_tokens:
        chunk_key_start = chunk_starts_tensor(chunk_key_start, rows, q_tokens, max_seq_len, dev)
        p.mask_block_tokens = int(mask_block_tokens)
        p.chunk_key_start = chunk_key_start.data_ptr()
    if rope is not None:
        table, grid_hw, start_frames = rope
        if table.dtype != torch.float64 or not table.is_contiguous() or table.device != dev:
            raise RuntimeError("rope table must be the contiguous float64 view from device_freqs() on q's device")
        if len(start_frames) != rows:
            raise RuntimeError("rope needs one start frame per row")
        frames = _i64_array(start_frames)
        p.rope_freqs, p.rope_freq_rows = table.data_ptr(), table.shape[0]
        p.rope_grid_h, p.rope_grid_w = int(grid_hw[0]), int(grid_hw[1])
        p.rope_start_frame = C.cast(frames, C.POINTER(C.c_int64))
    if q_norm is not None:
        weight, inv_rms = q_norm
        if rope is None:
            raise RuntimeError("q_norm needs rope=: the kernel normalises the raw query, then rotates it")
        if weight.dtype != q.dtype or weight.numel() != heads * HEAD_DIM or not weight.is_contiguous() or weight.device != dev:
            raise RuntimeError(f"the q norm weight must be a contiguous {q.dtype} tensor of {heads * HEAD_DIM} elements on {dev}")
        if inv_rms.dtype != torch.float32 or inv_rms.numel() != rows * q_tokens or not inv_rms.is_contiguous() \
                or inv_rms.device != dev:
            raise RuntimeError(f"q_inv_rms must be a contiguous float32 tensor of {rows} x {q_tokens} elements on {dev}")
        p.q_norm_weight, p.q_inv_rms = weight.data_ptr(), inv_rms.data_ptr()
    with _on_device(dev):
        if static_scratch:
            _capi.check(lib.sdv2_swa_attn_fwd_static(C.byref(p)), "sdv2_swa_attn_fwd_static")
        else:
            _capi.check(lib.sdv2_swa_attn_fwd(C.byref(p)), "sdv2_swa_attn_fwd")
    return out


_SIM_WORKSPACES: dict = {}


def sink_similarity(
    k: torch.Tensor,
    v: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    freqs_table: torch.Tensor,
    grid_hw: Sequence[int],
    start_frames: Sequence[int],
    sink_frames: int,
    threshold: float,
    dst_start_override: Optional[torch.Tensor] = None,
    override_rows: Sequence[bool] = (),
    refresh_out: Optional[torch.Tensor] = None,
    k_norm: Optional[Tuple[torch.Tensor, float]] = None,
    frame_sums: Optional[torch.Tensor] = None,
    stale_frames: Sequence[int] = (),
    planned_frames: Sequence[int] = (),
):
    """Adaptive sink refresh decision (causal_model.py:284-299) for a
    one-frame chunk, before its append.

    With ``dst_start_override`` (device int64 [B]) the decision is also handed
    to the append that follows on the stream: row i gets the start of the
    refreshed sink frame when it refreshes and ``override_rows[i]`` says the
    row is about to evict, else -1.  ``refresh_out`` (int32 [B]) receives the
    decision instead of a new device tensor; it may be PINNED host memory, which
    the kernel then writes directly (valid on the host once the stream has
    passed this call).

    ``k_norm`` = (k norm weight, eps): k is the raw k projection and its
    RMSNorm is applied inside, as :func:`kv_append_rope` with ``qk_norm`` does.

    ``frame_sums`` (from :func:`new_sink_frame_sums`) keeps the means of the
    cached sink frames between calls, so that only the new chunk is read:
    ``stale_frames[i]`` is a bit mask of the sink frames of row i whose means
    must be taken from the cache again (written behind this operator's back,
    or never summed), ``planned_frames[i]`` the sink frame the append that
    follows writes to by the host's plan, or -1.

    k is the chunk's key BEFORE RoPE, v its value, both [B,S,H,128]; the caches
    are read as they are.  Returns (similarity float32 [B, sink_frames],
    refresh int32 [B]) on the device: refresh[i] is the sink frame of row i to
    overwrite next, or -1.
    """
    dev = _require_gpu(k, v, k_cache, v_cache, freqs_table)
    if not (k.dtype == v.dtype == k_cache.dtype == v_cache.dtype):
        raise RuntimeError("k, v and the caches must share one dtype")
    rows, tokens, heads, _ = k.shape
    if tuple(v.shape) != tuple(k.shape):
        raise RuntimeError("k and v must have one shape")
    if k_cache.shape[0] < rows or v_cache.shape != k_cache.shape or k_cache.shape[2] != heads:
        raise RuntimeError(f"cache {tuple(k_cache.shape)} does not match the chunk {tuple(k.shape)}")
    lib = _capi.lib()
    need = lib.sdv2_sink_similarity_workspace_bytes(rows, tokens, heads, sink_frames)
    ws = _workspace(dev, need, _SIM_WORKSPACES)      # (zero-filled: its ticket words start at zero)
    similarity = torch.empty((rows, sink_frames), dtype=torch.float32, device=dev)
    if refresh_out is None:
        refresh = torch.empty((rows,), dtype=torch.int32, device=dev)
    else:
        refresh = refresh_out
        on_device = refresh.device == dev or (refresh.device.type == "cpu" and refresh.is_pinned())
        if refresh.dtype != torch.int32 or refresh.numel() < rows or not refresh.is_contiguous() or not on_device:
            raise RuntimeError(f"refresh_out must be a contiguous int32 tensor with one entry per row, on {dev} or pinned")

    p = _capi.SinkSimParams()
    p.k_in, p.k_in_stride = k.data_ptr(), _stride3(k, "k")
    p.v_in, p.v_in_stride = v.data_ptr(), _stride3(v, "v")
    p.k_cache, p.k_cache_stride = k_cache.data_ptr(), _stride3(k_cache, "k_cache")
    p.v_cache, p.v_cache_stride = v_cache.data_ptr(), _stride3(v_cache, "v_cache")
    p.freqs, p.freq_rows = freqs_table.data_ptr(), freqs_table.shape[0]
    if k.dtype not in _DTYPES:
        raise RuntimeError(f"unsupported dtype {k.dtype}")
    p.dtype = _DTYPES[k.dtype]
    p.rows, p.tokens, p.heads, p.head_dim = rows, tokens, heads, HEAD_DIM
    p.grid_h, p.grid_w = int(grid_hw[0]), int(grid_hw[1])
    p.sink_frames = int(sink_frames)
    p.threshold = float(threshold)
    p.cache_tokens = k_cache.shape[1]
    starts = _i64_array(start_frames)
    p.start_frame = C.cast(starts, C.POINTER(C.c_int64))
    p.similarity, p.refresh = similarity.data_ptr(), refresh.data_ptr()
    p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
    p.stream = _stream_ptr(dev)
    if dst_start_override is not None:
        _check_override(dst_start_override, rows, dev)
        if len(override_rows) != rows:
            raise RuntimeError("override_rows needs one flag per row")
        p.dst_start_override = dst_start_override.data_ptr()
        p.override_rows = sum(1 << i for i, flag in enumerate(override_rows) if flag)
    if k_norm is not None:
        weight, eps = k_norm
        if weight.dtype != k.dtype or weight.numel() != heads * HEAD_DIM or not weight.is_contiguous() \
                or weight.device != dev:
            raise RuntimeError(f"the k norm weight must be a contiguous {k.dtype} tensor of {heads * HEAD_DIM} elements on {dev}")
        p.k_norm_weight, p.norm_eps = weight.data_ptr(), float(eps)
    if frame_sums is not None:
        want = lib.sdv2_sink_frame_sums_bytes(rows, heads, sink_frames)
        if frame_sums.device != dev or not frame_sums.is_contiguous() \
                or frame_sums.numel() * frame_sums.element_size() < want:
            raise RuntimeError(f"frame_sums must be a contiguous buffer of at least {want} bytes on {dev}")
        if len(stale_frames) != rows or len(planned_frames) != rows:
            raise RuntimeError("frame_sums needs stale_frames and planned_frames with one entry per row")
        stale = (C.c_uint32 * rows)(*[int(x) & 0xffffffff for x in stale_frames])
        planned = (C.c_int32 * rows)(*[int(x) for x in planned_frames])
        p.frame_sums = frame_sums.data_ptr()
        p.stale_frames = C.cast(stale, C.POINTER(C.c_uint32))
        p.planned_frame = C.cast(planned, C.POINTER(C.c_int32))
    with _on_device(dev):
        _capi.check(lib.sdv2_sink_similarity(C.byref(p)), "sdv2_sink_similarity")
    return similarity, refresh


def new_sink_frame_sums(rows: int, heads: int, sink_frames: int, dev) -> torch.Tensor:
    """The buffer :func:`sink_similarity` keeps the sink frames' means in
    between calls (everything in it starts out stale)."""
    n = _capi.lib().sdv2_sink_frame_sums_bytes(rows, heads, sink_frames)
    return torch.empty(max(n // 4, 1), dtype=torch.float32, device=dev)


class KernelTimer:
    """A start/stop pair of the library's timing events (a measurement hook,
    include/sdv2kv_profile.h).  Armed for a kernel (:meth:`arm`, or
    ``LayerLauncher.set_timers``) it is recorded in the dispatch of this
    thread's next launch of that kernel, so :meth:`elapsed_ms` is the kernel's
    duration as a profiler reports it, without the gap separate stream events
    add."""

    def __init__(self):
        lib = _capi.lib()
        self.start, self.stop = C.c_void_p(), C.c_void_p()
        _capi.check(lib.sdv2_event_create(C.byref(self.start)), "sdv2_event_create")
        _capi.check(lib.sdv2_event_create(C.byref(self.stop)), "sdv2_event_create")

    def arm(self, kernel: int) -> None:
        """Time this thread's next launch of ``kernel`` (``_capi.KERNEL_*``)."""
        _capi.check(_capi.lib().sdv2_profile_time_next(kernel, self.start, self.stop), "sdv2_profile_time_next")

    def elapsed_ms(self) -> float:
        ms = C.c_float()
        _capi.check(_capi.lib().sdv2_event_elapsed_ms(self.start, self.stop, C.byref(ms)), "sdv2_event_elapsed_ms")
        return ms.value

    def close(self) -> None:
        lib = _capi.lib()
        for e in (self.start, self.stop):
            if e:
                lib.sdv2_event_destroy(e)
        self.start, self.stop = C.c_void_p(), C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class LayerLauncher:
    """Pre-built launch descriptors for one layer's (append, attention) pair.

    A chunk step calls the path once per transformer block, every time with the
    same cache, shapes and strides; only the slot, the RoPE frame, the index
    values and the q/k/v pointers change.  Building the two C structs from
    scratch costs more host time than the kernels take on the GPU, so they are
    built once per (cache, shape) and patched per call.
    """

    @staticmethod
    def _sig(t):
        return (tuple(t.shape), tuple(t.stride()), t.dtype)

    def __init__(self, k_cache, v_cache, global_end_index, local_end_index, freqs_table, grid, q_like, k_like=None,
                 v_like=None, qk_norm=None, rope_in_attention=True):
        k_like = q_like if k_like is None else k_like
        v_like = q_like if v_like is None else v_like
        rows, tokens, heads, _ = q_like.shape
        if tuple(k_like.shape) != tuple(q_like.shape) or tuple(v_like.shape) != tuple(q_like.shape):
            raise RuntimeError("q, k and v must have one shape")
        if rows > _capi.MAX_ROWS:
            raise RuntimeError(f"LayerLauncher handles at most {_capi.MAX_ROWS} rows")
        if q_like.dtype != torch.bfloat16:
            raise RuntimeError("LayerLauncher is the bf16 fast path")
        dev = _require_gpu(k_cache, v_cache, global_end_index, local_end_index, freqs_table, q_like)
        self.dev = dev
        self.rows, self.tokens, self.heads = rows, tokens, heads
        self.in_sig = (self._sig(q_like), self._sig(k_like), self._sig(v_like))
        self.cache_sig = (k_cache.data_ptr(), v_cache.data_ptr(), tuple(k_cache.shape), tuple(k_cache.stride()),
                          tuple(v_cache.stride()), global_end_index.data_ptr(), local_end_index.data_ptr())
        self.k_cache, self.v_cache = k_cache, v_cache
        self.lib = _capi.lib()
        # The query is rotated where it is consumed, inside the attention kernel,
        # so the append moves K and V only.  With the q / k norm folded into the
        # append the append still reads q - the norm needs the sum of squares of
        # whole tokens - but only leaves 1 / rms per token (``q_inv_rms``) for the
        # attention kernel, which normalises and rotates.  On request
        # (rope_in_attention=False) the append rotates q as well and hands the
        # attention the rotated copy in ``roped_q``.
        self.rope_in_attention = bool(rope_in_attention)
        self.roped_q = None if self.rope_in_attention else torch.empty(
            (rows, tokens, heads, HEAD_DIM), dtype=torch.bfloat16, device=dev)
        self.q_inv_rms = torch.empty((rows, tokens), dtype=torch.float32, device=dev) \
            if self.rope_in_attention and qk_norm is not None else None
        self.sf = (C.c_int64 * rows)()
        self.ds = (C.c_int64 * rows)()
        self.ng = (C.c_int64 * rows)()
        self.nl = (C.c_int64 * rows)()

        ap = _capi.AppendParams()
        ap.k_in_stride = _stride3(k_like, "k")
        ap.v_in_stride = _stride3(v_like, "v")
        if not self.rope_in_attention:
            ap.q_in_stride = _stride3(q_like, "q")
            ap.q_out, ap.q_out_stride = self.roped_q.data_ptr(), _stride3(self.roped_q, "q_out")
        elif self.q_inv_rms is not None:
            ap.q_in_stride = _stride3(q_like, "q")
            ap.q_inv_rms = self.q_inv_rms.data_ptr()
        ap.k_cache, ap.k_cache_stride = k_cache.data_ptr(), _stride3(k_cache, "k_cache")
        ap.v_cache, ap.v_cache_stride = v_cache.data_ptr(), _stride3(v_cache, "v_cache")
        ap.freqs, ap.freq_rows = freqs_table.data_ptr(), freqs_table.shape[0]
        ap.dtype = _capi.DTYPE_BF16
        ap.rows, ap.tokens, ap.heads, ap.head_dim = rows, tokens, heads, HEAD_DIM
        ap.grid_f, ap.grid_h, ap.grid_w = (int(x) for x in grid)
        ap.cache_tokens = k_cache.shape[1]
        ap.start_frame = C.cast(self.sf, C.POINTER(C.c_int64))
        ap.dst_start = C.cast(self.ds, C.POINTER(C.c_int64))
        ap.global_end_index = global_end_index.data_ptr()
        ap.local_end_index = local_end_index.data_ptr()
        ap.new_global_end = C.cast(self.ng, C.POINTER(C.c_int64))
        ap.new_local_end = C.cast(self.nl, C.POINTER(C.c_int64))
        self.qk_norm = qk_norm
        if qk_norm is not None:
            _check_norm(qk_norm, q_like.dtype, heads, dev)
            ap.q_norm_weight, ap.k_norm_weight = qk_norm[0].data_ptr(), qk_norm[1].data_ptr()
            ap.norm_eps = float(qk_norm[2])
        self.ap, self.ap_ref = ap, C.byref(ap)
        self.freqs_table = freqs_table

        at = _capi.AttnParams()
        if self.rope_in_attention:
            at.q_stride = _stride3(q_like, "q")
            at.rope_freqs, at.rope_freq_rows = freqs_table.data_ptr(), freqs_table.shape[0]
            at.rope_grid_h, at.rope_grid_w = int(grid[1]), int(grid[2])
            at.rope_start_frame = C.cast(self.sf, C.POINTER(C.c_int64))
            if self.q_inv_rms is not None:
                at.q_norm_weight, at.q_inv_rms = qk_norm[0].data_ptr(), self.q_inv_rms.data_ptr()
        else:
            at.q, at.q_stride = self.roped_q.data_ptr(), _stride3(self.roped_q, "q")
        at.k_cache, at.k_stride = k_cache.data_ptr(), _stride3(k_cache, "k_cache")
        at.v_cache, at.v_stride = v_cache.data_ptr(), _stride3(v_cache, "v_cache")
        at.rows, at.q_tokens, at.heads, at.head_dim = rows, tokens, heads, HEAD_DIM
        self.at, self.at_ref = at, C.byref(at)
        self.span = -1
        self.workspace_need = 0
        self.out_stride = None
        self.forced_splits = 0                       # 0 = the library's own choice
        self.timers = (None, None)

    def matches(self, q, k, v, kv_cache, freqs_table, qk_norm=None) -> bool:
        if (self._sig(q), self._sig(k), self._sig(v)) != self.in_sig or freqs_table is not self.freqs_table:
            return False
        if (qk_norm is None) != (self.qk_norm is None):
            return False
        if qk_norm is not None and (qk_norm[0].data_ptr() != self.qk_norm[0].data_ptr()
                                    or qk_norm[1].data_ptr() != self.qk_norm[1].data_ptr()
                                    or float(qk_norm[2]) != float(self.qk_norm[2])):
            return False
        kc, vc = kv_cache["k"], kv_cache["v"]
        return self.cache_sig == (kc.data_ptr(), vc.data_ptr(), tuple(kc.shape), tuple(kc.stride()), tuple(vc.stride()),
                                  kv_cache["global_end_index"].data_ptr(), kv_cache["local_end_index"].data_ptr())

    def patch(self, q, k, v, start_frames, plan, seq_lens: Optional[torch.Tensor] = None,
              mask_block_tokens: int = 0, dst_start_override: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Fill in what changes from call to call and allocate the output
        [rows, S, H, 128]; nothing is launched."""
        ap, at = self.ap, self.at
        if dst_start_override is not None:
            _check_override(dst_start_override, self.rows, self.dev)
        ap.dst_start_override = dst_start_override.data_ptr() if dst_start_override is not None else None
        at.mask_block_tokens = mask_block_tokens
        if mask_block_tokens:
            self.chunk_starts = chunk_starts_tensor(plan.dst_start, self.rows, self.tokens, plan.max_seq_len, self.dev)
            at.chunk_key_start = self.chunk_starts.data_ptr()
        for i in range(self.rows):
            self.sf[i] = start_frames[i]
            self.ds[i] = plan.dst_start[i]
            self.ng[i] = plan.new_global_end[i]
            self.nl[i] = plan.new_local_end[i]
        ap.k_in, ap.v_in = k.data_ptr(), v.data_ptr()
        if self.rope_in_attention:
            at.q = q.data_ptr()
            if self.q_inv_rms is not None:
                ap.q_in = q.data_ptr()
        else:
            ap.q_in = q.data_ptr()
        stream = _stream_ptr(self.dev)
        ap.stream = stream
        span = plan.max_seq_len
        if span != self.span:
            self.span = span
            at.max_seq_len = span
            at.num_splits = self.forced_splits or self.lib.sdv2_swa_attn_default_splits(
                self.rows, self.tokens, self.heads, span)
            self.workspace_need = self.lib.sdv2_swa_attn_workspace_bytes(self.rows, self.tokens, self.heads, span,
                                                                         at.num_splits)
        if self.workspace_need:
            ws = _workspace(self.dev, self.workspace_need)      # this stream's; may have been regrown by another shape
            at.workspace, at.workspace_bytes = ws.data_ptr(), ws.numel()
        out = torch.empty((self.rows, self.tokens, self.heads, HEAD_DIM), dtype=torch.bfloat16, device=self.dev)
        if self.out_stride is None:
            self.out_stride = _stride3(out, "out")
            at.out_stride = self.out_stride
        at.out = out.data_ptr()
        at.seq_lens = seq_lens.data_ptr() if seq_lens is not None else None
        at.stream = stream
        return out

    def set_timers(self, append: Optional[KernelTimer] = None, attention: Optional[KernelTimer] = None) -> None:
        """Attach (or, with None, detach) kernel timers for the next launches."""
        self.timers = (append, attention)

    def run_append(self) -> None:
        if self.timers[0] is not None:
            self.timers[0].arm(_capi.KERNEL_APPEND)
        _capi.check(self.lib.sdv2_kv_append_rope(self.ap_ref), "sdv2_kv_append_rope")

    def run_attention(self) -> None:
        if self.timers[1] is not None:
            self.timers[1].arm(_capi.KERNEL_ATTENTION)
        _capi.check(self.lib.sdv2_swa_attn_fwd(self.at_ref), "sdv2_swa_attn_fwd")

    def launch(self, q, k, v, start_frames, plan, seq_lens: Optional[torch.Tensor] = None,
               mask_block_tokens: int = 0, dst_start_override: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Append + attention for one call; returns the attention output
        [rows, S, H, 128]."""
        out = self.patch(q, k, v, start_frames, plan, seq_lens, mask_block_tokens, dst_start_override)
        if _current_device_index() != self.dev.index:
            with torch.cuda.device(self.dev):
                self.run_append()
                self.run_attention()
        else:
            self.run_append()
            self.run_attention()
        return out


def flash_attn_with_kvcache(q, k_cache, v_cache, cache_seqlens=None):
    """Same call as the reference makes on flash_attn_interface
    (causal_model.py:353-358): defaults mean causal=False and scale 1/sqrt(D)."""
    if cache_seqlens is not None and cache_seqlens.dtype != torch.int32:
        cache_seqlens = cache_seqlens.to(torch.int32)
    return swa_attention(q, k_cache, v_cache, cache_seqlens)


# the reference's own fallback operator has the same four arguments and result
# (causal_model.py:111-157); with this package both names are one kernel
attention_with_kvcache_fallback = flash_attn_with_kvcache


def flash_attention(q, k, v, q_lens=None, k_lens=None, dropout_p=0.0, softmax_scale=None, q_scale=None,
                    causal=False, window_size=(-1, -1), deterministic=False, dtype=torch.bfloat16, version=None):
    """The reference's generic attention entry (wan_base/modules/attention.py,
    ``flash_attention``) for the cases the cached inference path uses:
    cross-attention of a chunk against the cached text keys / values
    (wan_base/modules/model.py:192), i.e. no causal mask, no window, no dropout,
    every query row valid.  k / v may be ``expand``-ed views (row stride 0, as
    causal_stream_inference.py:227-228 makes them).  Inputs that are not bf16
    are computed in bf16 and the result is returned in q's dtype, as the
    reference does with its ``dtype`` argument."""
    if causal or tuple(window_size) != (-1, -1) or dropout_p or q_lens is not None:
        raise NotImplementedError("flash_attention here covers the cached inference path: "
                                  "causal=False, window_size=(-1, -1), dropout_p=0, q_lens=None")
    if dtype != torch.bfloat16:
        raise NotImplementedError("the attention kernel computes in bf16")
    out_dtype = q.dtype
    scale = None
    if q_scale is not None or softmax_scale is not None:
        scale = (q_scale if q_scale is not None else 1.0) * \
                (softmax_scale if softmax_scale is not None else HEAD_DIM ** -0.5)
    if k_lens is not None:
        k_lens = k_lens.to(device=q.device, dtype=torch.int32).contiguous()
    qb, kb, vb = (t if t.dtype == torch.bfloat16 else t.to(torch.bfloat16) for t in (q, k, v))
    if qb.stride(-1) != 1:
        qb = qb.contiguous()
    out = swa_attention(qb, kb, vb, k_lens, softmax_scale=scale)
    return out if out_dtype == torch.bfloat16 else out.to(out_dtype)


def cache_relayout(
    dst: torch.Tensor,
    src: torch.Tensor,
    dst_indices: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
    src_indices: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
    global_end_shift: int = 0,
    timer: Optional["KernelTimer"] = None,
) -> None:
    """``dst[...] = src[...]`` for two [rows, cap, heads, 128] tensors in any
    stride order, plus, with both index pairs (global_end_index,
    local_end_index) given, ``dst_global = src_global + global_end_shift`` and
    ``dst_local = src_local`` in the same launch: one side of the block
    hand-off of streamv2v/communication/kv_cache_manager.py:66-82."""
    flat = [dst, src] + list(dst_indices or ()) + list(src_indices or ())
    dev = _require_gpu(*flat)
    if src.dtype not in _DTYPES or dst.dtype != src.dtype:
        raise RuntimeError(f"unsupported dtype pair {dst.dtype} / {src.dtype}")
    if tuple(dst.shape) != tuple(src.shape):
        raise RuntimeError(f"shape mismatch: {tuple(dst.shape)} vs {tuple(src.shape)}")
    if (dst_indices is None) != (src_indices is None):
        raise RuntimeError("index tensors are handed over as two pairs or not at all")
    rows, tokens, heads, _ = src.shape
    p = _capi.RelayoutParams()
    p.src, p.src_stride = src.data_ptr(), _stride3(src, "src")
    p.dst, p.dst_stride = dst.data_ptr(), _stride3(dst, "dst")
    p.dtype = _DTYPES[src.dtype]
    p.rows, p.heads, p.head_dim, p.tokens = rows, heads, HEAD_DIM, tokens
    if dst_indices is not None:
        for idx in (*dst_indices, *src_indices):
            if idx.dtype != torch.int64 or idx.numel() < rows or not idx.is_contiguous():
                raise RuntimeError("end-index tensors must be contiguous int64 with one entry per row")
        p.dst_global_end_index, p.dst_local_end_index = (t.data_ptr() for t in dst_indices)
        p.src_global_end_index, p.src_local_end_index = (t.data_ptr() for t in src_indices)
        p.global_end_shift = int(global_end_shift)
    p.stream = _stream_ptr(dev)
    if timer is not None:
        timer.arm(_capi.KERNEL_RELAYOUT)
    with _on_device(dev):
        _capi.check(_capi.lib().sdv2_cache_relayout(C.byref(p)), "sdv2_cache_relayout")


def _norm_rows(t: torch.Tensor):
    """(rows, elements between rows) of a tensor [..., width] whose rows are
    contiguous and evenly spaced, else None."""
    width = t.shape[-1]
    if width > 1 and t.stride(-1) != 1:
        return None
    rows = t.numel() // width
    if t.dim() == 1 or rows <= 1:
        return rows, width
    step = expect = None
    for size, stride in zip(reversed(t.shape[:-1]), reversed(t.stride()[:-1])):
        if size == 1:
            continue
        if step is None:
            step = expect = stride
        elif stride != expect:
            return None
        expect *= size
    if step is None or step < width or step % 8 != 0:
        return None
    return rows, step


def rms_norm_supported(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Can :func:`rms_norm` take this input?  (A device tensor of a dtype the
    library knows; rows of a multiple of 128 up to 8192 contiguous elements, 16-byte
    aligned and evenly spaced; a contiguous weight of the same dtype.)"""
    width = x.shape[-1] if x.dim() else 0
    return (x.is_cuda and x.dtype in _DTYPES and weight.dtype == x.dtype and weight.device == x.device
            and width > 0 and width % HEAD_DIM == 0 and width // HEAD_DIM <= 64 and weight.numel() == width
            and weight.is_contiguous() and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0
            and _norm_rows(x) is not None)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """WanRMSNorm.forward (wan_base/modules/model.py:77-86) over the last
    dimension of x [..., width] in one launch: float32 normalisation, back to
    x's dtype, times the weight - the bits the torch expression gives on the
    CPU.  x may be a slice of a wider tensor (rows ``width`` contiguous
    elements, a common distance apart); ``out`` defaults to a new contiguous
    tensor and may be x itself."""
    dev = _require_gpu(x, weight)
    if not rms_norm_supported(x, weight):
        raise RuntimeError(f"rms_norm takes bf16 / fp32 rows of a multiple of 128 up to 8192 contiguous, 16-byte aligned, "
                           f"evenly spaced elements with a contiguous weight of the same dtype and width, got x "
                           f"{tuple(x.shape)} {x.dtype} strides {x.stride()}, weight {tuple(weight.shape)} {weight.dtype}")
    width = x.shape[-1]
    tokens, x_step = _norm_rows(x)
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype, device=dev)
    elif out.shape != x.shape or out.dtype != x.dtype or out.device != dev:
        raise RuntimeError("out must have x's shape, dtype and device")
    rows = _norm_rows(out)
    if rows is None or out.data_ptr() % 16:
        raise RuntimeError("out: rows must be contiguous, 16-byte aligned and evenly spaced")
    p = _capi.RmsNormParams()
    p.x, p.out, p.weight = x.data_ptr(), out.data_ptr(), weight.data_ptr()
    p.x_token_stride, p.out_token_stride = x_step, rows[1]
    p.tokens, p.width, p.dtype, p.eps = tokens, width, _DTYPES[x.dtype], float(eps)
    p.stream = _stream_ptr(dev)
    with _on_device(dev):
        _capi.check(_capi.lib().sdv2_rms_norm(C.byref(p)), "sdv2_rms_norm")
    return out


def copy_bytes(dst: torch.Tensor, src: torch.Tensor) -> None:
    """Plain 16-byte-vector copy with the library's own kernel (used to scale
    hardware counters against a transfer of known size)."""
    dev = _require_gpu(dst, src)
    n = src.numel() * src.element_size()
    if dst.numel() * dst.element_size() != n or not dst.is_contiguous() or not src.is_contiguous():
        raise RuntimeError("copy_bytes needs contiguous tensors of equal byte size")
    with _on_device(dev):
        _capi.check(_capi.lib().sdv2_copy_bytes(dst.data_ptr(), src.data_ptr(), n, _stream_ptr(dev)), "sdv2_copy_bytes")
