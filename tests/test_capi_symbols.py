"""The C-ABI library loads without a GPU, exports every function that
include/sdv2kv.h (operators) and include/sdv2kv_profile.h (measurement hooks)
declare, and rejects bad arguments before touching HIP."""
import ctypes as C
import inspect
import os
import re

import pytest
import torch

from streamdiffusionv2_amd import _capi

INCLUDE = os.path.join(os.path.dirname(os.path.dirname(__file__)), "include")
HEADER = os.path.join(INCLUDE, "sdv2kv.h")
PROFILE_HEADER = os.path.join(INCLUDE, "sdv2kv_profile.h")


def declared_functions(headers=(HEADER, PROFILE_HEADER)):
    names = set()
    for header in headers:
        text = re.sub(r"/\*.*?\*/", "", open(header).read(), flags=re.S)
        names |= set(re.findall(r"\b(sdv2_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_every_header_in_include_is_covered():
    assert sorted(os.listdir(INCLUDE)) == ["sdv2kv.h", "sdv2kv_profile.h"]


def test_operator_header_holds_no_measurement_api():
    """What a binding of the path has to mirror is sdv2kv.h alone: timing and
    counter-calibration hooks live in sdv2kv_profile.h."""
    ops_only = declared_functions((HEADER,))
    assert not [n for n in ops_only if "event" in n or "profile" in n or "copy_bytes" in n]
    text = open(HEADER).read()
    assert "timing" not in text and "stages" not in text


def test_header_functions_are_exported():
    names = declared_functions()
    assert sorted(_capi.EXPORTED_SYMBOLS) == names
    lib = _capi.lib()
    for n in names:
        assert hasattr(lib, n), n
    assert lib.sdv2_abi_version() == _capi.ABI_VERSION


def test_header_constants_match_binding():
    text = open(HEADER).read()
    assert int(re.search(r"#define SDV2_MAX_ROWS (\d+)", text).group(1)) == _capi.MAX_ROWS
    assert int(re.search(r"#define SDV2_HEAD_DIM (\d+)", text).group(1)) == _capi.HEAD_DIM
    for name in ("INVALID_ARG", "UNSUPPORTED", "OUT_OF_RANGE", "WORKSPACE", "LAUNCH", "SCRATCH_LIMIT"):
        val = int(re.search(rf"SDV2_ERR_{name} = (-\d+)", text).group(1))
        assert getattr(_capi, f"SDV2_ERR_{name}") == val
    # struct field order of the binding follows the header
    for struct, cls in (("sdv2_append_params", _capi.AppendParams), ("sdv2_attn_params", _capi.AttnParams)):
        body = re.search(rf"typedef struct {struct} \{{(.*?)\}} {struct};", text, flags=re.S).group(1)
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        fields = []
        for decl in body.split(";"):
            decl = decl.strip()
            if not decl:
                continue
            names = re.sub(r"^(const\s+)?[A-Za-z0-9_]+\s*\**", "", decl)
            fields += [n.strip().lstrip("*") for n in names.split(",")]
        assert fields == [f[0] for f in cls._fields_], struct


def test_argument_validation_without_gpu():
    lib = _capi.lib()
    assert lib.sdv2_kv_append_rope(None) == _capi.SDV2_ERR_INVALID_ARG
    assert lib.sdv2_swa_attn_fwd(None) == _capi.SDV2_ERR_INVALID_ARG
    p = _capi.AppendParams()
    p.head_dim = 64
    assert lib.sdv2_kv_append_rope(C.byref(p)) == _capi.SDV2_ERR_UNSUPPORTED
    p.head_dim, p.dtype = 128, 7
    assert lib.sdv2_kv_append_rope(C.byref(p)) == _capi.SDV2_ERR_UNSUPPORTED
    p.dtype, p.rows, p.tokens, p.heads = 0, _capi.MAX_ROWS + 1, 8, 1
    assert lib.sdv2_kv_append_rope(C.byref(p)) == _capi.SDV2_ERR_INVALID_ARG
    p.rows, p.grid_f, p.grid_h, p.grid_w = 1, 1, 2, 3      # 6 != 8 tokens
    assert lib.sdv2_kv_append_rope(C.byref(p)) == _capi.SDV2_ERR_INVALID_ARG
    # rotation of q alone: no k, v, caches - and then no index, norm or device slot either
    r = _capi.AppendParams()
    r.head_dim, r.rows, r.tokens, r.heads = 128, 1, 6, 1
    r.grid_f, r.grid_h, r.grid_w = 1, 2, 3
    r.freqs = 256
    assert lib.sdv2_kv_append_rope(C.byref(r)) == _capi.SDV2_ERR_INVALID_ARG     # nothing to rotate
    r.q_in, r.q_out = 256, 512
    r.k_in = 768                                                                # k without v and the caches
    assert lib.sdv2_kv_append_rope(C.byref(r)) == _capi.SDV2_ERR_INVALID_ARG
    r.k_in = None
    r.global_end_index = 1024
    assert lib.sdv2_kv_append_rope(C.byref(r)) == _capi.SDV2_ERR_INVALID_ARG     # an index without a cache
    r.global_end_index = None
    assert lib.sdv2_kv_append_rope(C.byref(r)) == _capi.SDV2_ERR_INVALID_ARG     # no start_frame
    a = _capi.AttnParams()
    a.head_dim = 96
    assert lib.sdv2_swa_attn_fwd(C.byref(a)) == _capi.SDV2_ERR_UNSUPPORTED
    a.head_dim, a.rows, a.q_tokens, a.heads, a.max_seq_len = 128, 1, 4, 1, 8
    assert lib.sdv2_swa_attn_fwd(C.byref(a)) == _capi.SDV2_ERR_INVALID_ARG     # null tensors
    a.dtype = 7
    assert lib.sdv2_swa_attn_fwd(C.byref(a)) == _capi.SDV2_ERR_UNSUPPORTED     # neither bf16 nor fp32
    a.dtype = _capi.DTYPE_F32
    assert lib.sdv2_swa_attn_fwd(C.byref(a)) == _capi.SDV2_ERR_INVALID_ARG     # fp32: null tensors all the same
    a.q, a.k_cache, a.v_cache, a.out = 256, 512, 768, 1024
    for st in (a.q_stride, a.k_stride, a.v_stride, a.out_stride):
        st.row, st.token, st.head = 1024, 128, 128
    a.rope_freqs = 2048
    assert lib.sdv2_swa_attn_fwd(C.byref(a)) == _capi.SDV2_ERR_UNSUPPORTED     # fp32 queries arrive rotated
    a.rope_freqs, a.q_stride.token = None, 130
    assert lib.sdv2_swa_attn_fwd(C.byref(a)) == _capi.SDV2_ERR_INVALID_ARG     # fp32 strides in multiples of 4
    assert b"workspace" in lib.sdv2_status_string(_capi.SDV2_ERR_WORKSPACE)
    with pytest.raises(RuntimeError, match="status -3"):
        _capi.check(_capi.SDV2_ERR_OUT_OF_RANGE, "x")


def test_split_heuristic_and_workspace_size():
    lib = _capi.lib()
    assert lib.sdv2_swa_attn_workspace_bytes(1, 1560, 12, 9360, 1) == 0
    s = lib.sdv2_swa_attn_default_splits(1, 1560, 12, 9360)
    assert s >= 2
    nq = 1568 * 12                     # query rows in whole 32-row blocks
    need = lib.sdv2_swa_attn_workspace_bytes(1, 1560, 12, 9360, s)
    # 64 KB of ticket words; per split and query row: 128 fp16 values, the row's scale and its log-sum-exp
    assert s * nq * (128 * 2 + 4 + 4) + 65536 <= need <= s * nq * (128 * 2 + 4 + 4) + 65536 + 2 * 256
    # the Wan 14B shape still fits the static scratch of the allocation-free entry point
    assert lib.sdv2_swa_attn_workspace_bytes(1, 1560, 40, 9360, 0) <= _capi.STATIC_SCRATCH_BYTES
    # plenty of query tiles: splitting only pays through round quantisation, never beyond a few
    assert 1 <= lib.sdv2_swa_attn_default_splits(4, 4680, 12, 18720) <= 4
    assert lib.sdv2_swa_attn_default_splits(64, 8192, 16, 512) == 1        # short cache, huge grid


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_capi, "_LIB", None)
    monkeypatch.setattr(_capi, "LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(ImportError, match="no fallback"):
        _capi.lib()


def test_cpu_tensors_are_refused():
    from streamdiffusionv2_amd import ops

    q = torch.zeros(1, 8, 1, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU only") as err:
        ops.flash_attn_with_kvcache(q=q, k_cache=q, v_cache=q, cache_seqlens=None)
    # the reference turns a RuntimeError that names "DeviceType::CUDA" into a silent
    # SDPA fallback (causal_model.py:359-372): errors of this path must never look like that
    assert "DeviceType::CUDA" not in str(err.value)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.swa_attention(q, q, q)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.causal_rope_apply(q, [(1, 2, 4)], torch.zeros(4, 64, dtype=torch.complex128))
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.attention_with_kvcache_fallback(q, q, q, None)


def test_module_signature_matches_reference():
    from streamdiffusionv2_amd.attention import CausalWanSelfAttention

    # models/wan/causal_model.py:162-167 and :189-200
    assert list(inspect.signature(CausalWanSelfAttention.__init__).parameters) == [
        "self", "dim", "num_heads", "window_size", "qk_norm", "eps"]
    assert list(inspect.signature(CausalWanSelfAttention.forward).parameters) == [
        "self", "x", "seq_lens", "grid_sizes", "freqs", "block_mask", "kv_cache",
        "current_start", "current_end", "causal_rope_cache"]
    m = CausalWanSelfAttention(256, 2)
    assert (m.sink_size, m.adapt_sink_thr, m.evict_idx) == (3, -1, None)
    assert {n for n, _ in m.named_children()} == {"q", "k", "v", "o", "norm_q", "norm_k"}
    with pytest.raises(NotImplementedError):
        m(torch.zeros(1, 4, 256), None, None, None, None, kv_cache=None)


def test_plain_c_caller(tmp_path):
    """include/sdv2kv.h compiles as C99, the library links from a C program and
    validates its arguments there (no GPU needed: every check returns before
    the first launch)."""
    import shutil
    import subprocess

    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    from streamdiffusionv2_amd import _capi

    here = os.path.dirname(os.path.abspath(__file__))
    root = os.path.dirname(here)
    exe = tmp_path / "abi_check"
    lib_dir = str(_capi.LIB_PATH.parent)
    build = subprocess.run(
        ["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(root, "include"),
         os.path.join(here, "c_abi", "abi_check.c"), "-o", str(exe), "-L", lib_dir, "-lsdv2kv",
         "-L/opt/rocm/lib", "-Wl,-rpath," + lib_dir, "-Wl,-rpath,/opt/rocm/lib", "-Wl,--allow-shlib-undefined"],
        capture_output=True, text=True)
    assert build.returncode == 0, build.stderr
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "all checks passed" in run.stdout
    assert "splits for 1x1560 tokens, 12 heads, 9360 keys: 3" in run.stdout
    # the ctypes structures must have the C compiler's layout
    import ctypes as C
    import re

    for c_name, binding, last in (("sdv2_append_params", _capi.AppendParams, "q_inv_rms"),
                                  ("sdv2_attn_params", _capi.AttnParams, "q_inv_rms"),
                                  ("sdv2_sink_sim_params", _capi.SinkSimParams, "planned_frame"),
                                  ("sdv2_rms_norm_params", _capi.RmsNormParams, "eps"),
                                  ("sdv2_relayout_params", _capi.RelayoutParams, "global_end_shift")):
        m = re.search(rf"layout {c_name} size=(\d+) stream=(\d+) {last}=(\d+)", run.stdout)
        assert m, run.stdout
        assert (C.sizeof(binding), binding.stream.offset, getattr(binding, last).offset) == tuple(map(int, m.groups())), c_name


def test_documented_ctypes_struct_matches_the_binding():
    """The integration guide shows a ctypes mirror of sdv2_attn_params for
    callers who bind the library themselves; its field list must be the one the
    package's own binding uses (a missing field shifts every later one)."""
    import re

    from streamdiffusionv2_amd import _capi

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "INTEGRATION.md")).read()
    block = text[text.index("class AttnParams(C.Structure):"):]
    block = block[:block.index("p = AttnParams(")]
    documented = re.findall(r'\("(\w+)",', block)
    assert documented == [name for name, _ in _capi.AttnParams._fields_]


def test_entry_points_build_only_when_no_library_is_there(monkeypatch, tmp_path):
    """smoke(), bench.py and the GPU test session call ``ensure_built``: a
    present library is loaded as it is, a missing one is compiled; the package
    loader itself never compiles (it raises, see above)."""
    from streamdiffusionv2_amd import build_ext

    calls = []
    monkeypatch.setattr(build_ext, "build", lambda verbose=False: calls.append(verbose) or build_ext.LIB_PATH)
    assert build_ext.ensure_built() == build_ext.LIB_PATH and calls == []
    monkeypatch.setattr(build_ext, "LIB_PATH", tmp_path / "libsdv2kv.so")
    assert build_ext.ensure_built() == tmp_path / "libsdv2kv.so" and calls == [False]
