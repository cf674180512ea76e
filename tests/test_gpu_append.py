"""GPU parity of the fused RoPE-on-write append against the CPU oracle:
cache contents, roped query and indices must be bit-exact."""
import pytest
import torch

from oracle import sdv2_oracle as oracle

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.contiguous().view(torch.int16 if t.dtype == torch.bfloat16 else torch.int32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("head_major", [True, False])
@pytest.mark.parametrize("grid,heads,rows", [((1, 6, 10), 12, 1), ((3, 5, 8), 5, 3), ((2, 30, 52), 12, 2)])
def test_append_matches_oracle_bitwise(gpu_device, dtype, head_major, grid, heads, rows):
    from streamdiffusionv2_amd import ops

    torch.manual_seed(1234)
    f, h, w = grid
    S = f * h * w
    cap = 4 * S
    freqs = oracle.build_freqs()
    q = torch.randn(rows, S, heads, 128).to(dtype)
    k = torch.randn(rows, S, heads, 128).to(dtype)
    v = torch.randn(rows, S, heads, 128).to(dtype)
    start_frames = [7 + 3 * r for r in range(rows)]
    dst = [(r % 4) * S for r in range(rows)]

    want_q = oracle.causal_rope_apply(q, [grid] * rows, freqs, start_frames)
    want_k = oracle.causal_rope_apply(k, [grid] * rows, freqs, start_frames)

    if head_major:
        kc = torch.zeros(rows, heads, cap, 128, dtype=dtype, device=gpu_device).permute(0, 2, 1, 3)
        vc = torch.zeros(rows, heads, cap, 128, dtype=dtype, device=gpu_device).permute(0, 2, 1, 3)
    else:
        kc = torch.zeros(rows, cap, heads, 128, dtype=dtype, device=gpu_device)
        vc = torch.zeros(rows, cap, heads, 128, dtype=dtype, device=gpu_device)
    g_idx = torch.zeros(rows, dtype=torch.long, device=gpu_device)
    l_idx = torch.zeros(rows, dtype=torch.long, device=gpu_device)
    table = ops.device_freqs(freqs, gpu_device)
    got_q = ops.kv_append_rope(
        q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), kc, vc, table, grid, start_frames, dst,
        global_end_index=g_idx, local_end_index=l_idx,
        new_global_end=[100 + r for r in range(rows)], new_local_end=[200 + r for r in range(rows)],
    )
    torch.cuda.synchronize()
    assert torch.equal(_bits(got_q.cpu()), _bits(want_q))
    kc_cpu, vc_cpu = kc.cpu(), vc.cpu()
    for r in range(rows):
        assert torch.equal(_bits(kc_cpu[r, dst[r]:dst[r] + S]), _bits(want_k[r]))
        assert torch.equal(_bits(vc_cpu[r, dst[r]:dst[r] + S]), _bits(v[r]))
        # everything outside the written slot stays zero
        mask = torch.ones(cap, dtype=torch.bool)
        mask[dst[r]:dst[r] + S] = False
        assert not kc_cpu[r, mask].any() and not vc_cpu[r, mask].any()
    assert g_idx.tolist() == [100 + r for r in range(rows)]
    assert l_idx.tolist() == [200 + r for r in range(rows)]


def test_append_special_values(gpu_device):
    """NaN of either sign, infinities, signed zeros, bf16 subnormals, values
    near the largest bf16 and round-to-even ties in the inputs: the rotation in
    double and the rounding to bf16 must still give the CPU result bit for bit
    wherever that result is a number; where it is a NaN the GPU result is a
    NaN too (PyTorch's own paths encode a NaN result differently, so there is
    no one bit pattern to match)."""
    from streamdiffusionv2_amd import ops

    torch.manual_seed(7)
    grid, heads = (1, 4, 8), 2
    S = 32
    freqs = oracle.build_freqs()
    q = torch.randn(1, S, heads, 128)
    k = torch.randn(1, S, heads, 128)
    specials = torch.tensor([float("nan"), -float("nan"), float("inf"), -float("inf"), 0.0, -0.0,
                             1e-40, -1e-40, 3.3895e38, 1.00390625, 1.01171875])
    idx = torch.randperm(S * heads * 128)[:400]
    k.view(-1)[idx] = specials[torch.arange(400) % len(specials)]
    q.view(-1)[idx[:50]] = specials[torch.arange(50) % len(specials)]
    q, k = q.bfloat16(), k.bfloat16()
    v = torch.randn(1, S, heads, 128).bfloat16()
    want_q = oracle.causal_rope_apply(q, [grid], freqs, [5])
    want_k = oracle.causal_rope_apply(k, [grid], freqs, [5])
    kc = torch.zeros(1, S, heads, 128, dtype=torch.bfloat16, device=gpu_device)
    vc = torch.zeros_like(kc)
    got_q = ops.kv_append_rope(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), kc, vc,
                               ops.device_freqs(freqs, gpu_device), grid, [5], [0])
    torch.cuda.synchronize()
    assert torch.isnan(want_k.float()).any() and torch.isinf(want_k.float()).any()
    for got, want in ((got_q.cpu(), want_q), (kc.cpu(), want_k)):
        nan = torch.isnan(want.float())
        assert torch.equal(torch.isnan(got.float()), nan)
        assert torch.equal(_bits(got)[~nan], _bits(want)[~nan])


def test_append_random_shapes(gpu_device):
    """Seeded sweep: grids with 1-4 frames, odd heights / widths, 1-41 heads,
    1-3 rows, both dtypes, both cache layouts, with and without q, with and
    without the index stores: cache slot and roped query bit for bit."""
    from streamdiffusionv2_amd import ops

    rng = torch.Generator().manual_seed(77)

    def ri(lo, hi):
        return int(torch.randint(lo, hi + 1, (1,), generator=rng).item())

    freqs = oracle.build_freqs()
    table = ops.device_freqs(freqs, gpu_device)
    for case in range(24):
        grid = (ri(1, 4), ri(1, 9), ri(1, 11))
        S = grid[0] * grid[1] * grid[2]
        heads, rows = ri(1, 41) if case % 3 == 0 else ri(1, 6), ri(1, 3)
        dtype = torch.float32 if case % 4 == 0 else torch.bfloat16
        head_major, with_q, with_idx = bool(case % 2), case % 5 != 0, case % 3 != 1
        cap = S * ri(1, 3) + ri(0, 7)
        start_frames = [ri(0, 1024 - grid[0]) for _ in range(rows)]
        dst = [ri(0, cap - S) for _ in range(rows)]
        print(f"case {case}: grid={grid} heads={heads} rows={rows} {dtype} head_major={head_major} "
              f"with_q={with_q} with_idx={with_idx} cap={cap} frames={start_frames} dst={dst}", flush=True)
        q = torch.randn(rows, S, heads, 128, generator=rng).to(dtype)
        k = torch.randn(rows, S, heads, 128, generator=rng).to(dtype)
        v = torch.randn(rows, S, heads, 128, generator=rng).to(dtype)
        want_q = oracle.causal_rope_apply(q, [grid] * rows, freqs, start_frames)
        want_k = oracle.causal_rope_apply(k, [grid] * rows, freqs, start_frames)
        shape = (rows, heads, cap, 128) if head_major else (rows, cap, heads, 128)
        kc = torch.zeros(shape, dtype=dtype, device=gpu_device)
        vc = torch.zeros(shape, dtype=dtype, device=gpu_device)
        if head_major:
            kc, vc = kc.permute(0, 2, 1, 3), vc.permute(0, 2, 1, 3)
        g_idx = torch.full((rows,), -1, dtype=torch.long, device=gpu_device)
        l_idx = torch.full((rows,), -1, dtype=torch.long, device=gpu_device)
        idx = dict(global_end_index=g_idx, local_end_index=l_idx, new_global_end=list(range(5, 5 + rows)),
                   new_local_end=list(range(9, 9 + rows))) if with_idx else {}
        got_q = ops.kv_append_rope(q.to(gpu_device) if with_q else None, k.to(gpu_device), v.to(gpu_device), kc, vc,
                                   table, grid, start_frames, dst, **idx)
        torch.cuda.synchronize()
        if with_q:
            assert torch.equal(_bits(got_q.cpu()), _bits(want_q)), case
        else:
            assert got_q is None
        kc_cpu, vc_cpu = kc.cpu(), vc.cpu()
        for r in range(rows):
            assert torch.equal(_bits(kc_cpu[r, dst[r]:dst[r] + S]), _bits(want_k[r])), (case, r)
            assert torch.equal(_bits(vc_cpu[r, dst[r]:dst[r] + S]), _bits(v[r])), (case, r)
            outside = torch.ones(cap, dtype=torch.bool)
            outside[dst[r]:dst[r] + S] = False
            assert not kc_cpu[r, outside].any() and not vc_cpu[r, outside].any(), (case, r)
        if with_idx:
            assert g_idx.tolist() == list(range(5, 5 + rows)) and l_idx.tolist() == list(range(9, 9 + rows))
        else:
            assert g_idx.tolist() == [-1] * rows


@pytest.mark.parametrize("fused_norm", [False, True])
def test_append_slot_chosen_on_the_device(gpu_device, fused_norm):
    """dst_start_override: a value >= 0 that fits the cache replaces the host's
    slot for that row, -1 and values that would leave the cache do not (both
    append kernels)."""
    from streamdiffusionv2_amd import ops

    print(f"append with a device-chosen slot, fused norm {fused_norm}", flush=True)
    torch.manual_seed(7)
    rows, grid, heads = 4, (1, 4, 6), 3
    S = 24
    cap = 5 * S
    q, k, v = (torch.randn(rows, S, heads, 128).bfloat16() for _ in range(3))
    start_frames = [2, 3, 4, 5]
    host_dst = [S, 2 * S, 3 * S, 4 * S]
    override = torch.tensor([0, -1, cap - S + 1, 2 * S], dtype=torch.int64)   # row 2 would overrun the cache
    lands = [0, 2 * S, 3 * S, 2 * S]
    weights = None
    kn, qn = k, q
    if fused_norm:
        wq, wk = (torch.rand(heads * 128) + 0.5).bfloat16(), (torch.rand(heads * 128) + 0.5).bfloat16()
        weights = (wq.to(gpu_device), wk.to(gpu_device), 1e-6)
        qn = oracle.wan_rms_norm(q.flatten(2), wq, 1e-6).view_as(q)
        kn = oracle.wan_rms_norm(k.flatten(2), wk, 1e-6).view_as(k)
    want_k = oracle.causal_rope_apply(kn, [grid] * rows, oracle.build_freqs(), start_frames).type_as(v)
    kc = torch.zeros(rows, heads, cap, 128, dtype=torch.bfloat16, device=gpu_device).permute(0, 2, 1, 3)
    vc = torch.zeros(rows, heads, cap, 128, dtype=torch.bfloat16, device=gpu_device).permute(0, 2, 1, 3)
    from streamdiffusionv2_amd import rope
    table = ops.device_freqs(rope.build_freqs(), gpu_device)
    ops.kv_append_rope(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), kc, vc, table, grid, start_frames, host_dst,
                       qk_norm=weights, dst_start_override=override.to(gpu_device))
    torch.cuda.synchronize()
    for r in range(rows):
        got_v = vc[r].cpu()
        assert torch.equal(got_v[lands[r]:lands[r] + S], v[r]), r
        untouched = torch.ones(cap, dtype=torch.bool)
        untouched[lands[r]:lands[r] + S] = False
        assert not got_v[untouched].any() and not kc[r].cpu()[untouched].any(), r
        got_k = kc[r, lands[r]:lands[r] + S].cpu()
        if fused_norm:      # the fused sum of squares may differ from torch's in the last place
            assert (got_k.float() - want_k[r].float()).abs().max().item() <= 2 ** -6 * want_k[r].float().abs().max().item()
        else:
            assert torch.equal(_bits(got_k), _bits(want_k[r])), r
    with pytest.raises(RuntimeError):       # wrong dtype
        ops.kv_append_rope(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), kc, vc, table, grid, start_frames,
                           host_dst, dst_start_override=override.int().to(gpu_device))
    with pytest.raises(RuntimeError):       # not on the device
        ops.kv_append_rope(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), kc, vc, table, grid, start_frames,
                           host_dst, dst_start_override=override)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_stand_alone_rotation_matches_oracle_bitwise(gpu_device, dtype):
    """``causal_rope_apply`` on its own, called the way the reference calls it
    (causal_model.py:253-259): rows with different grids, a tensor of start
    frames, tokens past a row's grid and a row without a grid stay as they
    are, and no cache is involved."""
    from streamdiffusionv2_amd import ops

    torch.manual_seed(31)
    heads, length = 5, 150
    grids = [(2, 5, 12), (2, 5, 12), (3, 5, 10), (1, 6, 8)]          # 120, 120, 150, 48 tokens
    x = torch.randn(5, length, heads, 128).to(dtype)                 # the fifth row has no grid
    starts = [3, 17, 0, 1000]
    freqs = oracle.build_freqs()
    want = oracle.causal_rope_apply(x, grids, freqs, starts)

    got = ops.causal_rope_apply(x.to(gpu_device), torch.tensor(grids), freqs,
                                start_frame=torch.tensor(starts, device=gpu_device), rope_cache=[("unused",)])
    torch.cuda.synchronize()
    assert got.dtype == dtype and got.shape == x.shape
    assert torch.equal(_bits(got.cpu()), _bits(want))
    assert torch.equal(_bits(got.cpu()[4]), _bits(x[4]))

    # one start frame for all rows, the table already on the device, every row covered in full
    y = torch.randn(3, 48, heads, 128).to(dtype)
    want = oracle.causal_rope_apply(y, [(1, 6, 8)] * 3, freqs, [11] * 3)
    got = ops.causal_rope_apply(y.to(gpu_device), [(1, 6, 8)] * 3, ops.device_freqs(freqs, gpu_device), start_frame=11)
    torch.cuda.synchronize()
    assert torch.equal(_bits(got.cpu()), _bits(want))

    with pytest.raises(RuntimeError, match="does not fit"):
        ops.causal_rope_apply(y.to(gpu_device), [(2, 6, 8)] * 3, freqs)
    with pytest.raises(RuntimeError, match="status -3"):             # frame 1020 + 5 is past the 1024-row table
        ops.causal_rope_apply(x.to(gpu_device), [(5, 5, 6)], freqs, start_frame=1020)
