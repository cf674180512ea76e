"""The allocation-free attention entry point, sdv2_swa_attn_fwd_static, against
sdv2_swa_attn_fwd: same kernels, partial results in the library's own static
device memory instead of a caller workspace, so the outputs must be identical
bit for bit.  Two calls in a row share the scratch (the second smaller than
the first, so stale partials of the first lie right behind its own); a call
that needs more than the static 64 MiB is refused and launches nothing."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _attn_params(q, kc, vc, out, seq_lens, splits, workspace=None):
    from streamdiffusionv2_amd import _capi, ops

    p = _capi.AttnParams()
    p.q, p.q_stride = q.data_ptr(), ops._stride3(q, "q")
    p.k_cache, p.k_stride = kc.data_ptr(), ops._stride3(kc, "k")
    p.v_cache, p.v_stride = vc.data_ptr(), ops._stride3(vc, "v")
    p.out, p.out_stride = out.data_ptr(), ops._stride3(out, "out")
    p.seq_lens = seq_lens.data_ptr() if seq_lens is not None else None
    p.rows, p.q_tokens, p.heads, p.head_dim = q.shape[0], q.shape[1], q.shape[2], 128
    p.max_seq_len = kc.shape[1]
    p.num_splits = splits
    if workspace is not None:
        p.workspace, p.workspace_bytes = workspace.data_ptr(), workspace.numel()
    p.stream = torch.cuda.current_stream(q.device).cuda_stream
    return p


def _case(dev, gen, rows, q_tokens, heads, keys, lens):
    def rnd(*shape):
        return (torch.randn(*shape, generator=gen) * 0.7).bfloat16().to(dev)
    q = rnd(rows, q_tokens, heads, 128)
    kc = rnd(rows, heads, keys, 128).permute(0, 2, 1, 3)        # head-major cache behind the logical view
    vc = rnd(rows, heads, keys, 128).permute(0, 2, 1, 3)
    seq = torch.tensor(lens, dtype=torch.int32, device=dev) if lens is not None else None
    return q, kc, vc, seq


def test_static_entry_point_matches_the_workspace_one(gpu_device):
    from oracle import sdv2_oracle as oracle
    from streamdiffusionv2_amd import _capi

    lib = _capi.lib()
    gen = torch.Generator().manual_seed(41)
    # first a large call (three key ranges, ragged tiles, per-row lengths), then a
    # smaller one on the same GPU: its partials overwrite only the head of what the first left
    cases = [(2, 700, 5, 3000, [3000, 2177], 3), (1, 200, 3, 1100, None, 2), (1, 64, 2, 640, [333], 0)]
    for rows, q_tokens, heads, keys, lens, splits in cases:
        print(f"static scratch: rows={rows} q={q_tokens} heads={heads} keys={keys} splits={splits}", flush=True)
        q, kc, vc, seq = _case(gpu_device, gen, rows, q_tokens, heads, keys, lens)
        need = lib.sdv2_swa_attn_workspace_bytes(rows, q_tokens, heads, keys, splits)
        ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=gpu_device)
        want = torch.full_like(q, float("nan"))
        got = torch.full_like(q, float("nan"))
        _capi.check(lib.sdv2_swa_attn_fwd(C.byref(_attn_params(q, kc, vc, want, seq, splits, ws))), "sdv2_swa_attn_fwd")
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated(gpu_device)
        _capi.check(lib.sdv2_swa_attn_fwd_static(C.byref(_attn_params(q, kc, vc, got, seq, splits))),
                    "sdv2_swa_attn_fwd_static")
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(gpu_device) == before
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
        # and against the oracle, to the attention bound
        n = lens if lens is not None else [keys] * rows
        ref = oracle.attention_fp32_reference(q.cpu(), kc.cpu(), vc.cpu(), n)
        err = (got.float().cpu() - ref).abs()
        assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3


def test_static_entry_point_refuses_more_than_it_holds(gpu_device):
    from streamdiffusionv2_amd import _capi

    lib = _capi.lib()
    # Wan 1.3B at batch 4, three-frame chunks: 178 MB of partials with three key ranges
    rows, q_tokens, heads, keys, splits = 4, 4680, 12, 18720, 3
    assert lib.sdv2_swa_attn_workspace_bytes(rows, q_tokens, heads, keys, splits) > _capi.STATIC_SCRATCH_BYTES
    q = torch.zeros(rows, q_tokens, heads, 128, dtype=torch.bfloat16, device=gpu_device)
    kc = torch.zeros(rows, keys, heads, 128, dtype=torch.bfloat16, device=gpu_device)
    out = torch.full_like(q, 3.0)
    status = lib.sdv2_swa_attn_fwd_static(C.byref(_attn_params(q, kc, kc, out, None, splits)))
    assert status == _capi.SDV2_ERR_SCRATCH_LIMIT
    assert "scratch" in lib.sdv2_status_string(status).decode()
    torch.cuda.synchronize()
    assert bool((out == 3.0).all())                      # nothing was launched
    # unsplit, the same shape needs no scratch and goes through
    _capi.check(lib.sdv2_swa_attn_fwd_static(C.byref(_attn_params(q, kc, kc, out, None, 1))), "static, unsplit")
    torch.cuda.synchronize()
    assert bool((out == 0.0).all())
    # more key ranges than the library ever takes: the plain entry point's answer, not a scratch complaint
    too_many = _attn_params(q, kc, kc, out, None, 65)
    assert lib.sdv2_swa_attn_fwd_static(C.byref(too_many)) == _capi.SDV2_ERR_INVALID_ARG
    ws = torch.zeros(8, dtype=torch.uint8, device=gpu_device)
    too_many.workspace, too_many.workspace_bytes = ws.data_ptr(), ws.numel()
    assert lib.sdv2_swa_attn_fwd(C.byref(too_many)) == _capi.SDV2_ERR_INVALID_ARG
    # fp32 tensors walk one key range and need no scratch, whatever the shape and num_splits say
    qf = torch.zeros(4, 4680, 12, 128, dtype=torch.float32, device=gpu_device)
    kf = torch.zeros(4, 640, 12, 128, dtype=torch.float32, device=gpu_device)
    of = torch.full_like(qf, 3.0)
    fp32 = _attn_params(qf, kf, kf, of, None, 64)
    fp32.dtype = _capi.DTYPE_F32
    assert lib.sdv2_swa_attn_workspace_bytes(4, 4680, 12, 640, 64) > _capi.STATIC_SCRATCH_BYTES   # were it bf16
    _capi.check(lib.sdv2_swa_attn_fwd_static(C.byref(fp32)), "static, fp32")
    torch.cuda.synchronize()
    assert bool((of == 0.0).all())


def test_static_entry_point_at_the_wan_shapes(gpu_device):
    """The two shapes the 64 MiB are sized for: 1560 queries against 9360 keys
    with 12 heads (three key ranges) and with 40 heads (four)."""
    from streamdiffusionv2_amd import _capi

    lib = _capi.lib()
    gen = torch.Generator().manual_seed(43)
    for heads in (40, 12):                      # the larger first
        q, kc, vc, _ = _case(gpu_device, gen, 1, 1560, heads, 9360, None)
        splits = lib.sdv2_swa_attn_default_splits(1, 1560, heads, 9360)
        need = lib.sdv2_swa_attn_workspace_bytes(1, 1560, heads, 9360, 0)
        assert splits > 1 and 0 < need <= _capi.STATIC_SCRATCH_BYTES
        ws = torch.zeros(need, dtype=torch.uint8, device=gpu_device)
        want, got = torch.empty_like(q), torch.empty_like(q)
        _capi.check(lib.sdv2_swa_attn_fwd(C.byref(_attn_params(q, kc, vc, want, None, 0, ws))), "sdv2_swa_attn_fwd")
        _capi.check(lib.sdv2_swa_attn_fwd_static(C.byref(_attn_params(q, kc, vc, got, None, 0))),
                    "sdv2_swa_attn_fwd_static")
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
