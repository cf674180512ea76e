"""Cross-attention with the per-prompt text K/V cache
(wan_base/modules/model.py:160-196; cache allocation
causal_stream_inference.py:109-122, stream-batch expansion :227-228).

CPU: the oracle's cache logic (projection only on the first call, cache read
afterwards, context_lens masking) against a float64 numpy softmax.
GPU: the library path (ops.flash_attention and the WanT2VCrossAttention
module) against the oracle, max-abs 2e-2 / mean-abs 2e-3 on unit-scale data."""
import numpy as np
import pytest
import torch

from oracle import sdv2_oracle as oracle

MAX_ABS, MEAN_ABS = 2e-2, 2e-3


def _numpy_attention(q, k, v, lens):
    q, k, v = (t.double().numpy() for t in (q, k, v))
    out = np.zeros_like(q)
    for b in range(q.shape[0]):
        for h in range(q.shape[2]):
            s = q[b, :, h] @ k[b, :lens[b], h].T / np.sqrt(q.shape[-1])
            p = np.exp(s - s.max(axis=1, keepdims=True))
            out[b, :, h] = (p / p.sum(axis=1, keepdims=True)) @ v[b, :lens[b], h]
    return out


def test_oracle_cache_logic_and_masking():
    torch.manual_seed(2)
    q = torch.randn(2, 5, 2, 128)
    k1, v1 = torch.randn(2, 16, 2, 128), torch.randn(2, 16, 2, 128)
    calls = []

    def make_kv():
        calls.append(1)
        return k1, v1

    cache = oracle.new_crossattn_cache(1, 2, 2, dtype=torch.float32, text_tokens=16)[0]
    assert cache["is_init"] is False and cache["k"].shape == (2, 16, 2, 128) and not cache["k"].any()
    lens = torch.tensor([16, 7])
    first = oracle.cross_attention_with_cache(q, make_kv, lens, cache)
    assert cache["is_init"] is True and cache["k"] is k1 and cache["v"] is v1 and len(calls) == 1

    def must_not_project():
        raise AssertionError("an initialised cache is read, not recomputed")

    second = oracle.cross_attention_with_cache(q, must_not_project, lens, cache)
    assert torch.equal(first, second)
    assert np.allclose(first.numpy(), _numpy_attention(q, k1, v1, [16, 7]), atol=2e-6)
    # no cache: projects every time; no lens: every key counts
    out = oracle.cross_attention_with_cache(q, make_kv, None, None)
    assert len(calls) == 2
    assert np.allclose(out.numpy(), _numpy_attention(q, k1, v1, [16, 16]), atol=2e-6)


def _close(got, want):
    err = (got.float().cpu() - want.float()).abs()
    assert torch.isfinite(err).all()
    assert err.max().item() <= MAX_ABS and err.mean().item() <= MEAN_ABS, (err.max().item(), err.mean().item())


@pytest.mark.gpu
@pytest.mark.parametrize("lens", [None, [512, 77], [1, 300]])
def test_flash_attention_on_text_cache(gpu_device, lens):
    from streamdiffusionv2_amd import ops

    print(f"cross attention: lens={lens}", flush=True)
    torch.manual_seed(3)
    rows, s, heads = 2, 333, 3
    q = torch.randn(rows, s, heads, 128).bfloat16()
    k = torch.randn(rows, 512, heads, 128).bfloat16()
    v = torch.randn(rows, 512, heads, 128).bfloat16()
    want = oracle.attention_fp32_reference(q, k, v, lens or [512] * rows)
    k_lens = None if lens is None else torch.tensor(lens)
    got = ops.flash_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), k_lens=k_lens)
    torch.cuda.synchronize()
    assert got.dtype == torch.bfloat16 and got.shape == q.shape
    _close(got, want)


@pytest.mark.gpu
def test_expanded_cache_and_fp32_inputs(gpu_device):
    from streamdiffusionv2_amd import ops, ring

    torch.manual_seed(4)
    rows, s, heads = 3, 130, 2
    cache = ring.new_crossattn_cache(1, 1, heads, device=gpu_device)[0]
    assert cache["k"].shape == (1, 512, heads, 128) and cache["is_init"] is False
    k = torch.randn(1, 512, heads, 128).bfloat16()
    v = torch.randn(1, 512, heads, 128).bfloat16()
    cache["k"].copy_(k)
    cache["v"].copy_(v)
    ring.expand_crossattn_for_stream_batch([cache], rows)
    assert cache["k"].shape[0] == rows and cache["k"].stride(0) == 0
    q = torch.randn(rows, s, heads, 128)
    want = oracle.attention_fp32_reference(q.bfloat16(), k.expand(rows, -1, -1, -1), v.expand(rows, -1, -1, -1),
                                           [512] * rows)
    got = ops.flash_attention(q.to(gpu_device), cache["k"], cache["v"])       # fp32 q: computed in bf16
    torch.cuda.synchronize()
    assert got.dtype == torch.float32
    _close(got, want)
    with pytest.raises(NotImplementedError):
        ops.flash_attention(q.to(gpu_device), cache["k"], cache["v"], causal=True)


@pytest.mark.gpu
def test_module_fills_then_reads_the_cache(gpu_device):
    from streamdiffusionv2_amd import ring
    from streamdiffusionv2_amd.attention import WanT2VCrossAttention

    torch.manual_seed(5)
    dim, heads, rows, s = 256, 2, 2, 96
    mod = WanT2VCrossAttention(dim, heads).to(gpu_device).bfloat16()
    assert sorted(n for n, _ in mod.named_children()) == ["k", "norm_k", "norm_q", "o", "q", "v"]
    x = torch.randn(rows, s, dim, device=gpu_device).bfloat16()
    context = torch.randn(rows, 512, dim, device=gpu_device).bfloat16()
    cache = ring.new_crossattn_cache(1, rows, heads, device=gpu_device)[0]
    with torch.no_grad():
        y1 = mod(x, context, None, cache)
        assert cache["is_init"] is True and cache["k"].shape == (rows, 512, heads, 128)
        y2 = mod(x, torch.zeros_like(context), None, cache)         # context ignored once cached
        assert torch.equal(y1, y2)
        # oracle on the same projections
        q = mod.norm_q(mod.q(x)).view(rows, s, heads, 128)
        want = oracle.cross_attention_with_cache(q.cpu(), None, None, {k_: (t.cpu() if torch.is_tensor(t) else t)
                                                                        for k_, t in cache.items()})
        want_y = mod.o(want.to(gpu_device).flatten(2))
    err = (y1.float() - want_y.float()).abs()
    assert err.max().item() <= 3e-2, err.max().item()
