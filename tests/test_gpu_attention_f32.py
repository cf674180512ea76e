"""GPU parity of the fp32 attention kernel (the reference's CPU-runnable
configuration: fp32 tensors, fp32 arithmetic) against the fp32 oracle.  Both
sides compute in fp32, in different orders: agreement is held to max-abs 5e-5 /
mean-abs 5e-6 on N(0,1) inputs."""
import pytest
import torch

from oracle import sdv2_oracle as oracle

pytestmark = pytest.mark.gpu

MAX_ABS = 5e-5
MEAN_ABS = 5e-6


def _check(got, want):
    assert got.dtype == torch.float32
    err = (got - want).abs()
    assert torch.isfinite(got).all()
    assert err.max().item() <= MAX_ABS, f"max-abs {err.max().item()}"
    assert err.mean().item() <= MEAN_ABS, f"mean-abs {err.mean().item()}"


def _to_device(t, gpu_device, head_major):
    if head_major:
        return t.permute(0, 2, 1, 3).contiguous().to(gpu_device).permute(0, 2, 1, 3)
    return t.to(gpu_device)


@pytest.mark.parametrize("head_major", [True, False])
@pytest.mark.parametrize(
    "rows,S,H,L,seq",
    [
        (1, 64, 1, 32, None),
        (1, 200, 3, 1000, None),        # ragged query tile and key tile
        (2, 77, 2, 520, [520, 301]),    # per-row lengths
        (3, 5, 2, 97, [97, 1, 33]),
        (1, 1560, 2, 3120, None),
    ],
)
def test_fp32_attention_matches_fp32_oracle(gpu_device, rows, S, H, L, seq, head_major):
    from streamdiffusionv2_amd import ops

    torch.manual_seed(123)
    q = torch.randn(rows, S, H, 128)
    k = torch.randn(rows, L, H, 128)
    v = torch.randn(rows, L, H, 128)
    lens = seq if seq is not None else [L] * rows
    want = oracle.attention_fp32_reference(q, k, v, lens)
    sl = torch.tensor(lens, dtype=torch.int32, device=gpu_device) if seq is not None else None
    got = ops.swa_attention(q.to(gpu_device), _to_device(k, gpu_device, head_major), _to_device(v, gpu_device, head_major), sl)
    torch.cuda.synchronize()
    _check(got.cpu(), want)


def test_fp32_attention_random_shapes(gpu_device):
    from streamdiffusionv2_amd import ops

    gen = torch.Generator().manual_seed(2024)
    ri = lambda a, b: int(torch.randint(a, b + 1, (1,), generator=gen))
    for case in range(16):
        rows, H = ri(1, 3), ri(1, 4)
        S = ri(1, 300)
        L = max(S, ri(1, 900)) if case % 2 else ri(1, 900)
        lens = [ri(1, L) for _ in range(rows)] if case % 3 == 0 else [L] * rows
        bt, starts = 0, None
        if case % 4 == 1 and S >= 2 and L >= S:
            bt = ri(1, S - 1)
            starts = [ri(0, min(lens) - S) if min(lens) >= S else 0 for _ in range(rows)]
            if min(lens) < S:
                bt, starts = 0, None
        print(f"case {case}: rows={rows} heads={H} S={S} L={L} lens={lens} bt={bt} starts={starts}", flush=True)
        q = torch.randn(rows, S, H, 128, generator=gen)
        k = torch.randn(rows, L, H, 128, generator=gen)
        v = torch.randn(rows, L, H, 128, generator=gen)
        want = oracle.attention_fp32_reference(q, k, v, lens, starts, bt) if bt else oracle.attention_fp32_reference(q, k, v, lens)
        sl = torch.tensor(lens, dtype=torch.int32, device=gpu_device)
        kw = dict(chunk_key_start=starts, mask_block_tokens=bt) if bt else {}
        got = ops.swa_attention(q.to(gpu_device), _to_device(k, gpu_device, case % 2 == 0),
                                _to_device(v, gpu_device, case % 2 == 0), sl, **kw)
        torch.cuda.synchronize()
        _check(got.cpu(), want)


def test_fp32_attention_extreme_scores_stay_finite(gpu_device):
    """A running maximum per row: scores of several hundred either way are exact."""
    from streamdiffusionv2_amd import ops

    torch.manual_seed(5)
    q = torch.randn(1, 150, 2, 128) * 14.0
    k = torch.randn(1, 400, 2, 128) * 14.0
    v = torch.randn(1, 400, 2, 128)
    want = oracle.attention_fp32_reference(q, k, v, [400])
    got = ops.swa_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device))
    torch.cuda.synchronize()
    assert torch.isfinite(got).all()
    assert (got.cpu() - want).abs().max().item() <= 1e-3      # near one-hot rows: the winner's value, to fp32 rounding of the scores


def test_fp32_and_bf16_do_not_mix(gpu_device):
    from streamdiffusionv2_amd import ops

    q = torch.zeros(1, 4, 1, 128, device=gpu_device)
    k = torch.zeros(1, 8, 1, 128, device=gpu_device, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        ops.swa_attention(q, k, k)
    table = ops.device_freqs(__import__("streamdiffusionv2_amd.rope", fromlist=["rope"]).build_freqs(), gpu_device)
    kf = torch.zeros(1, 8, 1, 128, device=gpu_device)
    with pytest.raises(RuntimeError):
        ops.swa_attention(q, kf, kf, rope=(table, (2, 2), [0]))
