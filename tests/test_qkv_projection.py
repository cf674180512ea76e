"""The module's q / k / v projections as one GEMM on the three weights laid
end to end (CausalWanSelfAttention.project_qkv): same values as the three
Linears of causal_model.py:212-218, a packed copy that follows the weights,
and on the GPU the same bits."""
import pytest
import torch

from streamdiffusionv2_amd.attention import CausalWanSelfAttention


def _separate(mod, x):
    return mod.q(x), mod.k(x), mod.v(x)


def _close(mod, x):
    with torch.no_grad():
        got, want = mod.project_qkv(x), _separate(mod, x)
    return all(torch.allclose(g, w, rtol=1e-5, atol=1e-5) for g, w in zip(got, want))


def test_one_gemm_gives_the_three_projections():
    torch.manual_seed(0)
    mod = CausalWanSelfAttention(256, 2)
    x = torch.randn(2, 7, 256)
    with torch.no_grad():
        q, k, v = mod.project_qkv(x)
    assert q.shape == k.shape == v.shape == (2, 7, 256)
    # three views of one [B, S, 3 * dim] tensor, readable per head without a copy
    assert q.stride() == (7 * 768, 768, 1) and q.untyped_storage().data_ptr() == v.untyped_storage().data_ptr()
    assert q.view(2, 7, 2, 128).stride() == (7 * 768, 768, 128, 1)
    assert _close(mod, x)
    assert sorted(mod.state_dict()) == sorted(
        ["q.weight", "q.bias", "k.weight", "k.bias", "v.weight", "v.bias", "o.weight", "o.bias",
         "norm_q.weight", "norm_k.weight"])          # the packed copy is no part of the state


def test_the_packed_copy_follows_the_weights():
    torch.manual_seed(1)
    mod = CausalWanSelfAttention(256, 2)
    x = torch.randn(1, 5, 256)
    assert _close(mod, x)
    first = mod._packed[1]
    assert _close(mod, x) and mod._packed[1] is first                    # nothing changed: nothing rebuilt
    with torch.no_grad():
        mod.k.weight.mul_(2.0)                                           # written in place
    assert _close(mod, x) and mod._packed[1] is not first
    with torch.no_grad():
        mod.v.bias.add_(1.0)
    assert _close(mod, x)
    mod.load_state_dict({name: value * 0.5 for name, value in mod.state_dict().items()})
    assert _close(mod, x)
    mod.q.weight = torch.nn.Parameter(torch.randn(256, 256))             # replaced
    assert _close(mod, x)
    mod.double()                                                         # every tensor re-made in another dtype
    assert _close(mod, x.double()) and mod._packed[1].dtype == torch.float64


def test_three_launches_when_asked_or_when_training():
    torch.manual_seed(2)
    mod = CausalWanSelfAttention(256, 2)
    x = torch.randn(1, 5, 256)
    q, _, _ = mod.project_qkv(x)                     # autograd on: the Linears themselves, graph and all
    assert q.requires_grad and q.is_contiguous() and mod._packed is None
    mod.fuse_qkv_projection = False
    with torch.no_grad():
        q, k, v = mod.project_qkv(x)
    assert q.is_contiguous() and mod._packed is None
    assert torch.equal(q, mod.q(x)) and torch.equal(v, mod.v(x))
    # a Linear without bias among the three: no packing
    mod.fuse_qkv_projection = True
    mod.k.bias = None
    with torch.no_grad():
        q, k, v = mod.project_qkv(x)
    assert k.is_contiguous() and torch.equal(k, mod.k(x))


def test_watched_or_wrapped_layers_are_called_themselves():
    """A forward hook on one of the three Linears, or a layer that is not a
    plain Linear (an adapter wrapped around it), must see its call."""
    torch.manual_seed(5)
    mod = CausalWanSelfAttention(256, 2)
    x = torch.randn(1, 5, 256)
    calls = []
    handle = mod.k.register_forward_hook(lambda m, i, o: calls.append("k"))
    with torch.no_grad():
        mod.project_qkv(x)
    assert calls == ["k"] and mod._packed is None
    handle.remove()
    with torch.no_grad():
        mod.project_qkv(x)
    assert calls == ["k"] and mod._packed is not None

    class Adapter(torch.nn.Linear):
        def forward(self, x):
            return super().forward(x) + 1.0

    wrapped = Adapter(256, 256)
    wrapped.load_state_dict(mod.v.state_dict())
    mod.v = wrapped
    with torch.no_grad():
        _, _, v = mod.project_qkv(x)
        assert torch.equal(v, wrapped(x))


def test_linears_without_bias_pack_without_one():
    torch.manual_seed(6)
    mod = CausalWanSelfAttention(256, 2)
    for layer in (mod.q, mod.k, mod.v):
        layer.bias = None
    x = torch.randn(2, 3, 256)
    assert _close(mod, x) and mod._packed is not None and mod._packed[2] is None


def test_a_module_made_under_inference_mode_packs_too():
    with torch.inference_mode():
        mod = CausalWanSelfAttention(256, 2)
        x = torch.randn(1, 3, 256)
        q, k, v = mod.project_qkv(x)
        assert torch.allclose(k, mod.k(x), rtol=1e-5, atol=1e-5)
        mod.k.weight.mul_(3.0)
        mod._packed = None                           # such tensors count no edits: the caller says so
        q, k, v = mod.project_qkv(x)
        assert torch.allclose(k, mod.k(x), rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dim,heads,tokens", [(256, 2, 24), (1536, 12, 1560), (5120, 40, 1560), (1536, 12, 4680)])
def test_same_bits_as_the_three_linears(gpu_device, dim, heads, tokens):
    """Every output element is the same dot product over `dim` whichever GEMM
    forms it; the vendor library's kernels for the two widths add it up in the
    same order at the model's shapes."""
    print(f"packed projection dim={dim} tokens={tokens}", flush=True)
    torch.manual_seed(3)
    mod = CausalWanSelfAttention(dim, heads).to(gpu_device).bfloat16()
    x = torch.randn(1, tokens, dim, device=gpu_device).bfloat16()
    with torch.inference_mode():
        got, want = mod.project_qkv(x), _separate(mod, x)
        for name, g, w in zip("qkv", got, want):
            assert torch.equal(g.contiguous().view(torch.int16), w.view(torch.int16)), name


@pytest.mark.gpu
def test_module_forward_is_the_same_with_and_without_packing(gpu_device):
    from streamdiffusionv2_amd import ring, rope
    print("module forward, packed and separate projections", flush=True)
    torch.manual_seed(4)
    dim, heads, grid, S, cap = 256, 2, (1, 4, 6), 24, 72
    mod = CausalWanSelfAttention(dim, heads).to(gpu_device).bfloat16()
    mod.sink_size = 1
    freqs = rope.build_freqs().to(gpu_device)
    grid_sizes = torch.tensor([grid], dtype=torch.long)
    xs = [torch.randn(1, S, dim, device=gpu_device).bfloat16() for _ in range(5)]
    results = []
    for packed in (True, False):
        mod.fuse_qkv_projection = packed
        mod.evict_idx = None
        cache = ring.new_kv_cache(1, 1, cap, heads, 1, dtype=torch.bfloat16, device=gpu_device)[0]
        outs = []
        with torch.inference_mode():
            for call, x in enumerate(xs):
                outs.append(mod(x, None, grid_sizes, freqs, None, kv_cache=cache, current_start=[call * S]))
        torch.cuda.synchronize()
        results.append((outs, cache))
    for a, b in zip(results[0][0], results[1][0]):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    for name in ("k", "v"):
        assert torch.equal(results[0][1][name].view(torch.int16), results[1][1][name].view(torch.int16))
