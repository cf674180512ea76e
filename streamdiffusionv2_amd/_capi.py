"""ctypes binding of the sdv2kv C ABI (include/sdv2kv.h; the measurement hooks of
include/sdv2kv_profile.h at the end).

The shared library is the product: there is no Python or CPU fallback.  When
it is missing, :func:`lib` raises ImportError with the build command.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path
from typing import Optional

LIB_PATH = Path(__file__).resolve().parent / "_lib" / "libsdv2kv.so"

ABI_VERSION = 12
HEAD_DIM = 128
MAX_ROWS = 16

SDV2_OK = 0
SDV2_ERR_INVALID_ARG = -1
SDV2_ERR_UNSUPPORTED = -2
SDV2_ERR_OUT_OF_RANGE = -3
SDV2_ERR_WORKSPACE = -4
SDV2_ERR_LAUNCH = -5
SDV2_ERR_SCRATCH_LIMIT = -6
STATIC_SCRATCH_BYTES = 64 << 20

DTYPE_BF16 = 0
DTYPE_F32 = 1

KERNEL_APPEND, KERNEL_ATTENTION, KERNEL_RELAYOUT, KERNEL_SINK, KERNEL_COPY, KERNEL_NORM = range(6)
STREAM_REGISTERS, STREAM_LDS_32_ROWS, STREAM_LDS_64_ROWS, STREAM_ATTENTION_MIX, STREAM_ATTENTION_MIX_64_ROWS = range(5)

# every symbol include/sdv2kv.h and include/sdv2kv_profile.h declare
EXPORTED_SYMBOLS = (
    "sdv2_abi_version",
    "sdv2_status_string",
    "sdv2_kv_append_rope",
    "sdv2_swa_attn_default_splits",
    "sdv2_swa_attn_workspace_bytes",
    "sdv2_swa_attn_fwd",
    "sdv2_swa_attn_fwd_static",
    "sdv2_sink_similarity_workspace_bytes",
    "sdv2_sink_frame_sums_bytes",
    "sdv2_sink_similarity",
    "sdv2_cache_relayout",
    "sdv2_rms_norm",
    "sdv2_event_create",
    "sdv2_event_destroy",
    "sdv2_event_elapsed_ms",
    "sdv2_profile_time_next",
    "sdv2_copy_bytes",
    "sdv2_profile_mfma_stream_bytes",
    "sdv2_profile_mfma_stream",
)


class Stride3(C.Structure):
    _fields_ = [("row", C.c_int64), ("token", C.c_int64), ("head", C.c_int64)]


class AppendParams(C.Structure):
    _fields_ = [
        ("q_in", C.c_void_p), ("k_in", C.c_void_p), ("v_in", C.c_void_p),
        ("q_out", C.c_void_p), ("k_cache", C.c_void_p), ("v_cache", C.c_void_p),
        ("q_in_stride", Stride3), ("k_in_stride", Stride3), ("v_in_stride", Stride3),
        ("q_out_stride", Stride3), ("k_cache_stride", Stride3), ("v_cache_stride", Stride3),
        ("freqs", C.c_void_p),
        ("freq_rows", C.c_int32),
        ("dtype", C.c_int32),
        ("rows", C.c_int32), ("tokens", C.c_int32), ("heads", C.c_int32), ("head_dim", C.c_int32),
        ("grid_f", C.c_int32), ("grid_h", C.c_int32), ("grid_w", C.c_int32),
        ("cache_tokens", C.c_int64),
        ("start_frame", C.POINTER(C.c_int64)),
        ("dst_start", C.POINTER(C.c_int64)),
        ("global_end_index", C.c_void_p),
        ("local_end_index", C.c_void_p),
        ("new_global_end", C.POINTER(C.c_int64)),
        ("new_local_end", C.POINTER(C.c_int64)),
        ("stream", C.c_void_p),
        ("q_norm_weight", C.c_void_p),
        ("k_norm_weight", C.c_void_p),
        ("norm_eps", C.c_float),
        ("dst_start_override", C.c_void_p),
        ("q_inv_rms", C.c_void_p),
    ]


class AttnParams(C.Structure):
    _fields_ = [
        ("q", C.c_void_p), ("k_cache", C.c_void_p), ("v_cache", C.c_void_p), ("out", C.c_void_p),
        ("seq_lens", C.c_void_p),
        ("q_stride", Stride3), ("k_stride", Stride3), ("v_stride", Stride3), ("out_stride", Stride3),
        ("rows", C.c_int32), ("q_tokens", C.c_int32), ("heads", C.c_int32), ("head_dim", C.c_int32),
        ("max_seq_len", C.c_int32),
        ("num_splits", C.c_int32),
        ("softmax_scale", C.c_float),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_size_t),
        ("stream", C.c_void_p),
        ("mask_block_tokens", C.c_int32),
        ("chunk_key_start", C.c_void_p),
        ("rope_freqs", C.c_void_p),
        ("rope_freq_rows", C.c_int32),
        ("rope_grid_h", C.c_int32), ("rope_grid_w", C.c_int32),
        ("rope_start_frame", C.POINTER(C.c_int64)),
        ("dtype", C.c_int32),
        ("q_norm_weight", C.c_void_p),
        ("q_inv_rms", C.c_void_p),
    ]


class SinkSimParams(C.Structure):
    _fields_ = [
        ("k_in", C.c_void_p), ("v_in", C.c_void_p), ("k_cache", C.c_void_p), ("v_cache", C.c_void_p),
        ("k_in_stride", Stride3), ("v_in_stride", Stride3), ("k_cache_stride", Stride3), ("v_cache_stride", Stride3),
        ("freqs", C.c_void_p),
        ("freq_rows", C.c_int32),
        ("dtype", C.c_int32),
        ("rows", C.c_int32), ("tokens", C.c_int32), ("heads", C.c_int32), ("head_dim", C.c_int32),
        ("grid_h", C.c_int32), ("grid_w", C.c_int32),
        ("sink_frames", C.c_int32),
        ("threshold", C.c_float),
        ("cache_tokens", C.c_int64),
        ("start_frame", C.POINTER(C.c_int64)),
        ("similarity", C.c_void_p),
        ("refresh", C.c_void_p),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_size_t),
        ("stream", C.c_void_p),
        ("dst_start_override", C.c_void_p),
        ("override_rows", C.c_uint32),
        ("k_norm_weight", C.c_void_p),
        ("norm_eps", C.c_float),
        ("frame_sums", C.c_void_p),
        ("stale_frames", C.POINTER(C.c_uint32)),
        ("planned_frame", C.POINTER(C.c_int32)),
    ]


class RmsNormParams(C.Structure):
    _fields_ = [
        ("x", C.c_void_p), ("out", C.c_void_p), ("weight", C.c_void_p),
        ("x_token_stride", C.c_int64), ("out_token_stride", C.c_int64),
        ("tokens", C.c_int64),
        ("width", C.c_int32),
        ("dtype", C.c_int32),
        ("eps", C.c_float),
        ("stream", C.c_void_p),
    ]


class RelayoutParams(C.Structure):
    _fields_ = [
        ("src", C.c_void_p), ("dst", C.c_void_p),
        ("src_stride", Stride3), ("dst_stride", Stride3),
        ("dtype", C.c_int32),
        ("rows", C.c_int32), ("heads", C.c_int32), ("head_dim", C.c_int32),
        ("tokens", C.c_int64),
        ("src_global_end_index", C.c_void_p), ("src_local_end_index", C.c_void_p),
        ("dst_global_end_index", C.c_void_p), ("dst_local_end_index", C.c_void_p),
        ("global_end_shift", C.c_int64),
        ("stream", C.c_void_p),
    ]


_LIB: Optional[C.CDLL] = None


def lib() -> C.CDLL:
    """Load libsdv2kv.so once and declare the prototypes."""
    global _LIB
    if _LIB is not None:
        return _LIB
    # The streams and pointers handed to the library come from PyTorch, so both
    # must sit on ONE HIP runtime: importing torch first makes the library's
    # libamdhip64 dependency resolve to the copy torch has already loaded.
    # Loaded the other way round, the process holds two runtimes and every
    # launch on a torch stream fails.
    import torch  # noqa: F401

    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: the KV-cache path has no fallback. Build it with "
            "`python -m streamdiffusionv2_amd.build_ext` (needs ROCm hipcc)."
        )
    handle = C.CDLL(str(LIB_PATH))
    handle.sdv2_abi_version.restype = C.c_int
    handle.sdv2_abi_version.argtypes = []
    handle.sdv2_status_string.restype = C.c_char_p
    handle.sdv2_status_string.argtypes = [C.c_int]
    handle.sdv2_kv_append_rope.restype = C.c_int
    handle.sdv2_kv_append_rope.argtypes = [C.POINTER(AppendParams)]
    handle.sdv2_swa_attn_default_splits.restype = C.c_int
    handle.sdv2_swa_attn_default_splits.argtypes = [C.c_int32] * 4
    handle.sdv2_swa_attn_workspace_bytes.restype = C.c_size_t
    handle.sdv2_swa_attn_workspace_bytes.argtypes = [C.c_int32] * 5
    handle.sdv2_swa_attn_fwd.restype = C.c_int
    handle.sdv2_swa_attn_fwd.argtypes = [C.POINTER(AttnParams)]
    handle.sdv2_swa_attn_fwd_static.restype = C.c_int
    handle.sdv2_swa_attn_fwd_static.argtypes = [C.POINTER(AttnParams)]
    handle.sdv2_sink_similarity_workspace_bytes.restype = C.c_size_t
    handle.sdv2_sink_similarity_workspace_bytes.argtypes = [C.c_int32] * 4
    handle.sdv2_sink_frame_sums_bytes.restype = C.c_size_t
    handle.sdv2_sink_frame_sums_bytes.argtypes = [C.c_int32] * 3
    handle.sdv2_sink_similarity.restype = C.c_int
    handle.sdv2_sink_similarity.argtypes = [C.POINTER(SinkSimParams)]
    handle.sdv2_cache_relayout.restype = C.c_int
    handle.sdv2_cache_relayout.argtypes = [C.POINTER(RelayoutParams)]
    handle.sdv2_rms_norm.restype = C.c_int
    handle.sdv2_rms_norm.argtypes = [C.POINTER(RmsNormParams)]
    handle.sdv2_event_create.restype = C.c_int
    handle.sdv2_event_create.argtypes = [C.POINTER(C.c_void_p)]
    handle.sdv2_event_destroy.restype = C.c_int
    handle.sdv2_event_destroy.argtypes = [C.c_void_p]
    handle.sdv2_event_elapsed_ms.restype = C.c_int
    handle.sdv2_event_elapsed_ms.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]
    handle.sdv2_profile_time_next.restype = C.c_int
    handle.sdv2_profile_time_next.argtypes = [C.c_int, C.c_void_p, C.c_void_p]
    handle.sdv2_copy_bytes.restype = C.c_int
    handle.sdv2_copy_bytes.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
    handle.sdv2_profile_mfma_stream_bytes.restype = C.c_size_t
    handle.sdv2_profile_mfma_stream_bytes.argtypes = []
    handle.sdv2_profile_mfma_stream.restype = C.c_int
    handle.sdv2_profile_mfma_stream.argtypes = [C.c_int, C.c_void_p, C.c_size_t, C.c_int32, C.c_void_p,
                                                C.POINTER(C.c_double)]
    if handle.sdv2_abi_version() != ABI_VERSION:
        raise ImportError(
            f"{LIB_PATH} has ABI version {handle.sdv2_abi_version()}, expected {ABI_VERSION}: rebuild it"
        )
    _LIB = handle
    return handle


def check(status: int, what: str) -> None:
    """Map a C status to the reference's error convention (RuntimeError)."""
    if status != SDV2_OK:
        msg = lib().sdv2_status_string(status).decode()
        raise RuntimeError(f"{what} failed: {msg} (status {status})")
