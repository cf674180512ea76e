"""The q / k RMSNorm of the projection outputs (WanRMSNorm,
wan_base/modules/model.py:70-86; applied in qkv_fn, causal_model.py:212-218)
folded into the append kernel.

CPU: the oracle's restatement against float64 numpy and the placement of the
two roundings; and the ORDER in which PyTorch's CPU kernel adds up the squares
(8-float vectors, four interleaved accumulators, blocks of 16, see
torch_order_sum), restated in numpy and required to give torch's bits.  GPU:
fused norm + RoPE + append against oracle norm -> oracle RoPE; the kernel adds
in that same order, so the cache must come out bit for bit (on a host whose
torch build uses another vector width - neither AVX2 nor AVX512 - the CPU test
of the order fails first and says so)."""
import numpy as np
import pytest
import torch

from oracle import sdv2_oracle as oracle


def test_oracle_rms_norm_against_float64():
    torch.manual_seed(0)
    x = torch.randn(2, 5, 256)
    w = torch.rand(256) + 0.5
    got = oracle.wan_rms_norm(x, w, 1e-6)
    xd = x.double().numpy()
    want = xd / np.sqrt((xd ** 2).mean(-1, keepdims=True) + 1e-6) * w.double().numpy()
    assert np.allclose(got.numpy(), want, rtol=2e-6, atol=1e-7)
    # a constant row: x / |x| * w, eps negligible
    c = torch.full((1, 1, 256), 3.0)
    assert torch.allclose(oracle.wan_rms_norm(c, w, 0.0), w.view(1, 1, -1), rtol=1e-6)
    # eps matters for a zero row: no NaN
    assert torch.equal(oracle.wan_rms_norm(torch.zeros(1, 1, 256), w, 1e-6), torch.zeros(1, 1, 256))


def test_oracle_rms_norm_rounds_before_the_weight():
    """In bf16 the normalised value is rounded to bf16 first and the product
    with the weight once more (type_as(x) * weight), not once at the end."""
    torch.manual_seed(1)
    x = torch.randn(1, 7, 256).bfloat16()
    w = (torch.rand(256) + 0.5).bfloat16()
    got = oracle.wan_rms_norm(x, w, 1e-6)
    xf = x.float()
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)
    two_roundings = ((xf * r).bfloat16().float() * w.float()).bfloat16()
    one_rounding = (xf * r * w.float()).bfloat16()
    assert torch.equal(got, two_roundings)
    assert not torch.equal(got, one_rounding)


def torch_order_sum(row, vec=8, ilp=4):
    """float32 sum of a contiguous row in the order of ATen's CPU sum kernel
    (SumKernel.cpp: cascade_sum -> vectorized_inner_sum -> row_sum ->
    multi_row_sum): element e goes to accumulator (e // vec % ilp, e % vec);
    an accumulator adds its elements in blocks of 16, every block summed in
    order from zero and the block sums added up in order (two further cascade
    levels only matter beyond 256 blocks' worth), a trailing partial block
    first; then the ilp accumulators of a vector lane in order, then the vector
    lanes in order from zero."""
    f = np.float32
    nvec = row.shape[0] // vec
    groups = nvec // ilp
    x = row[:groups * ilp * vec].reshape(groups, ilp, vec)
    level_power = max(4, int(np.ceil(np.log2(groups))) // 4) if groups > 1 else 4
    step = 1 << level_power
    acc = np.zeros((4, ilp, vec), dtype=f)
    i = 0
    while i + step <= groups:
        for _ in range(step):
            acc[0] = acc[0] + x[i]
            i += 1
        for j in range(1, 4):
            acc[j] = acc[j] + acc[j - 1]
            acc[j - 1] = 0
            if i & ((step - 1) << (j * level_power)):
                break
    while i < groups:
        acc[0] = acc[0] + x[i]
        i += 1
    for j in range(1, 4):
        acc[0] = acc[0] + acc[j]
    part = acc[0].copy()
    for v in range(groups * ilp, nvec):
        part[0] = part[0] + row[v * vec:(v + 1) * vec]
    for k in range(1, ilp):
        part[0] = part[0] + part[k]
    total = f(0)
    for e in row[nvec * vec:]:
        total = f(total + e)
    for k in range(vec):
        total = f(total + part[0][k])
    return total


@pytest.mark.parametrize("heads", [12, 40, 5, 48, 64, 1, 3])
def test_torch_cpu_sum_order_is_the_one_the_kernel_restates(heads):
    """The fused norm is bit-exact only against a definite summation order.
    This pins which one torch's CPU path uses here: the numpy restatement must
    reproduce torch's float32 sum of squares and mean of every row exactly."""
    torch.manual_seed(heads)
    width = heads * 128
    x = (torch.randn(64, width) * 3).bfloat16().float()
    sq = x.pow(2)
    want_sum = sq.sum(-1).numpy()
    got = np.array([torch_order_sum(r) for r in sq.numpy()], dtype=np.float32)
    assert np.array_equal(got.view(np.int32), want_sum.view(np.int32)), \
        f"torch's CPU sum uses another order here (capability {torch.backends.cpu.get_cpu_capability()})"
    assert np.array_equal((got / np.float32(width)).view(np.int32), sq.mean(-1).numpy().view(np.int32))


def _ulp_diff_bf16(a, b):
    ia = a.contiguous().view(torch.int16).to(torch.int32)
    ib = b.contiguous().view(torch.int16).to(torch.int32)
    # map sign-magnitude to a monotone integer line
    ia = torch.where(ia < 0, -(ia & 0x7fff), ia)
    ib = torch.where(ib < 0, -(ib & 0x7fff), ib)
    return (ia - ib).abs()


@pytest.mark.gpu
@pytest.mark.parametrize("heads", [12, 40, 5, 48, 64])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fused_norm_append(gpu_device, heads, dtype):
    from streamdiffusionv2_amd import ops, ring, rope

    print(f"fused q/k norm: heads={heads} {dtype}", flush=True)
    torch.manual_seed(2)
    rows, grid, cap = 2, (2, 5, 6), 240
    S, eps = 60, 1e-6
    freqs = rope.build_freqs()
    q = (torch.randn(rows, S, heads, 128) * 1.7).to(dtype)
    k = (torch.randn(rows, S, heads, 128) * 0.6).to(dtype)
    v = torch.randn(rows, S, heads, 128).to(dtype)
    wq = (torch.rand(heads * 128) + 0.5).to(dtype)
    wk = (torch.rand(heads * 128) + 0.5).to(dtype)
    start_frames, dst = [3, 9], [60, 120]

    qn = oracle.wan_rms_norm(q.flatten(2), wq, eps).view_as(q)
    kn = oracle.wan_rms_norm(k.flatten(2), wk, eps).view_as(k)
    want_q = oracle.causal_rope_apply(qn, [grid] * rows, oracle.build_freqs(), start_frames).type_as(v)
    want_k = oracle.causal_rope_apply(kn, [grid] * rows, oracle.build_freqs(), start_frames).type_as(v)

    caches = ring.new_kv_cache(1, 1, cap, heads, 1, dtype=dtype, device=gpu_device)
    ring.replicate_for_stream_batch(caches, rows)
    cache = caches[0]
    table = ops.device_freqs(freqs, gpu_device)
    got_q = ops.kv_append_rope(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), cache["k"], cache["v"], table,
                               grid, start_frames, dst, global_end_index=cache["global_end_index"],
                               local_end_index=cache["local_end_index"], new_global_end=[7, 8], new_local_end=[9, 10],
                               qk_norm=(wq.to(gpu_device), wk.to(gpu_device), eps))
    torch.cuda.synchronize()
    got_k = torch.stack([cache["k"][r, dst[r]:dst[r] + S] for r in range(rows)]).cpu()
    got_v = torch.stack([cache["v"][r, dst[r]:dst[r] + S] for r in range(rows)]).cpu()
    assert torch.equal(got_v, v)
    assert cache["global_end_index"].cpu().tolist() == [7, 8] and cache["local_end_index"].cpu().tolist() == [9, 10]
    for got, want in ((got_q.cpu(), want_q), (got_k, want_k)):
        bits = torch.int16 if dtype == torch.bfloat16 else torch.int32
        assert torch.equal(got.contiguous().view(bits), want.contiguous().view(bits))
    # the untouched part of the cache stays zero
    assert not cache["k"][0, :dst[0]].any() and not cache["k"][1, dst[1] + S:].any()


@pytest.mark.gpu
@pytest.mark.parametrize("heads", [12, 40, 5, 64])
def test_attention_normalises_and_rotates_the_raw_query_itself(gpu_device, heads):
    """With q_inv_rms the fused append writes no rotated query: it leaves
    1 / rms per token, and the attention kernel normalises and rotates the raw
    q projection while it loads it.  Same roundings in the same order, so cache
    bits, 1 / rms and the attention output are those of the path that goes
    through the rotated copy."""
    from streamdiffusionv2_amd import ops, ring, rope

    print(f"q norm inside the attention kernel: heads={heads}", flush=True)
    torch.manual_seed(11 + heads)
    rows, grid, cap = 2, (2, 5, 6), 240
    S, eps = 60, 1e-6
    dev = gpu_device
    q = (torch.randn(rows, S, heads, 128) * 1.7).bfloat16().to(dev)
    k = (torch.randn(rows, S, heads, 128) * 0.6).bfloat16().to(dev)
    v = torch.randn(rows, S, heads, 128).bfloat16().to(dev)
    wq = (torch.rand(heads * 128) + 0.5).bfloat16().to(dev)
    wk = (torch.rand(heads * 128) + 0.5).bfloat16().to(dev)
    start_frames, dst = [3, 9], [60, 120]
    table = ops.device_freqs(rope.build_freqs(), dev)
    results = []
    for leave_inv_rms in (False, True):
        caches = ring.new_kv_cache(1, 1, cap, heads, 1, device=dev)
        ring.replicate_for_stream_batch(caches, rows)
        cache = caches[0]
        for name in ("k", "v"):                    # older keys for the chunk to attend to
            cache[name].copy_(torch.randn(rows, cap, heads, 128, generator=torch.Generator().manual_seed(5)).bfloat16())
        inv = torch.empty(rows, S, dtype=torch.float32, device=dev) if leave_inv_rms else None
        roped = ops.kv_append_rope(q, k, v, cache["k"], cache["v"], table, grid, start_frames, dst,
                                   qk_norm=(wq, wk, eps), q_inv_rms=inv)
        if leave_inv_rms:
            assert roped is None
            out = ops.swa_attention(q, cache["k"], cache["v"], None, rope=(table, grid[1:], start_frames), q_norm=(wq, inv))
        else:
            out = ops.swa_attention(roped, cache["k"], cache["v"], None)
        torch.cuda.synchronize()
        results.append((out.cpu(), cache["k"].cpu(), cache["v"].cpu(), inv))
    (out0, k0, v0, _), (out1, k1, v1, inv) = results
    assert torch.equal(k0.view(torch.int16), k1.view(torch.int16)) and torch.equal(v0.view(torch.int16), v1.view(torch.int16))
    assert torch.equal(out0.view(torch.int16), out1.view(torch.int16))
    want_inv = torch.rsqrt(q.float().cpu().flatten(2).pow(2).mean(-1) + eps)
    assert (inv.cpu() - want_inv).abs().max().item() <= 2e-6 * want_inv.abs().max().item()


@pytest.mark.gpu
def test_q_norm_argument_errors(gpu_device):
    from streamdiffusionv2_amd import ops, rope

    table = ops.device_freqs(rope.build_freqs(), gpu_device)
    x = torch.zeros(1, 6, 2, 128, dtype=torch.bfloat16, device=gpu_device)
    cache = torch.zeros(1, 12, 2, 128, dtype=torch.bfloat16, device=gpu_device)
    w = torch.ones(256, dtype=torch.bfloat16, device=gpu_device)
    inv = torch.ones(1, 6, dtype=torch.float32, device=gpu_device)
    with pytest.raises(RuntimeError):       # 1 / rms only exists with the norm
        ops.kv_append_rope(x, x, x, cache, cache.clone(), table, (1, 2, 3), [0], [0], q_inv_rms=inv)
    with pytest.raises(RuntimeError):       # one entry per token
        ops.kv_append_rope(x, x, x, cache, cache.clone(), table, (1, 2, 3), [0], [0], qk_norm=(w, w, 1e-6), q_inv_rms=inv[:, :5])
    with pytest.raises(RuntimeError):       # the kernel normalises, then rotates: it needs the table
        ops.swa_attention(x, cache, cache, None, q_norm=(w, inv))
    with pytest.raises(RuntimeError):
        ops.swa_attention(x, cache, cache, None, rope=(table, (2, 3), [0]), q_norm=(w[:128], inv))
    ops.swa_attention(x, cache, cache, None, rope=(table, (2, 3), [0]), q_norm=(w, inv))
    torch.cuda.synchronize()


@pytest.mark.gpu
def test_module_with_and_without_fusion(gpu_device):
    from streamdiffusionv2_amd import ring, rope
    from streamdiffusionv2_amd.attention import CausalWanSelfAttention

    torch.manual_seed(3)
    dim, heads, grid = 256, 2, (1, 4, 6)
    S = 24
    mod = CausalWanSelfAttention(dim, heads).to(gpu_device).bfloat16()
    with torch.no_grad():
        mod.norm_q.weight.uniform_(0.5, 1.5)
        mod.norm_k.weight.uniform_(0.5, 1.5)
    mod.sink_size = 1
    freqs = rope.build_freqs()
    x = [torch.randn(1, S, dim, device=gpu_device).bfloat16() for _ in range(5)]
    outs = []
    for fuse in (True, False):
        mod.fuse_qk_norm = fuse
        mod.evict_idx = None
        cache = ring.new_kv_cache(1, 1, 3 * S, heads, 1, device=gpu_device)[0]
        res = []
        with torch.no_grad():
            for c in range(5):
                res.append(mod(x[c], None, torch.tensor([grid]), freqs, None, kv_cache=cache, current_start=c * S))
        outs.append((torch.stack(res), cache["k"].clone(), cache["v"].clone()))
    torch.cuda.synchronize()
    (y1, k1, v1), (y0, k0, v0) = outs
    assert torch.equal(v1, v0)
    # torch's GPU norm adds in yet another order: the unfused path may differ from the fused one by an ulp
    d = _ulp_diff_bf16(k1.cpu(), k0.cpu())
    assert d.max().item() <= 1 and (d == 0).float().mean().item() >= 0.999
    assert (y1.float() - y0.float()).abs().max().item() <= 3e-2


@pytest.mark.gpu
def test_fused_norm_argument_errors(gpu_device):
    from streamdiffusionv2_amd import ops, rope

    table = ops.device_freqs(rope.build_freqs(), gpu_device)
    x = torch.zeros(1, 6, 2, 128, dtype=torch.bfloat16, device=gpu_device)
    cache = torch.zeros(1, 12, 2, 128, dtype=torch.bfloat16, device=gpu_device)
    w = torch.ones(256, dtype=torch.bfloat16, device=gpu_device)
    with pytest.raises(RuntimeError):       # wrong length
        ops.kv_append_rope(x, x, x, cache, cache.clone(), table, (1, 2, 3), [0], [0], qk_norm=(w[:128], w, 1e-6))
    with pytest.raises(RuntimeError):       # wrong dtype
        ops.kv_append_rope(x, x, x, cache, cache.clone(), table, (1, 2, 3), [0], [0], qk_norm=(w.float(), w, 1e-6))
    with pytest.raises(RuntimeError):       # k only
        ops.kv_append_rope(None, x, x, cache, cache.clone(), table, (1, 2, 3), [0], [0], qk_norm=(w, w, 1e-6))


@pytest.mark.gpu
@pytest.mark.parametrize("fuse", [True, False])
def test_output_projection_reads_the_kernels_output_in_place(gpu_device, fuse):
    """The o projection (causal_model.py:387-389, x.flatten(2) -> self.o) must
    consume the tensor the attention kernel wrote: same storage, contiguous
    [B, S, heads * 128], nothing copied or re-laid-out in between.  And on the
    way in, with the norm folded into the append, the q / k projections' raw
    outputs reach the kernel as views of what the GEMMs wrote."""
    from streamdiffusionv2_amd import ring, rope
    from streamdiffusionv2_amd.attention import CausalWanSelfAttention

    torch.manual_seed(4)
    dim, heads, grid = 256, 2, (1, 4, 6)
    S = 24
    mod = CausalWanSelfAttention(dim, heads).to(gpu_device).bfloat16()
    mod.sink_size, mod.fuse_qk_norm = 1, fuse
    seen = {}
    inner_attend = mod.attend

    def spying_attend(q, k, v, *args, **kw):
        seen["q_in"], seen["k_in"] = q, k
        out = inner_attend(q, k, v, *args, **kw)
        seen["attn_out"] = out
        return out

    mod.attend = spying_attend
    proj_out = {}
    for name in ("q", "k"):
        getattr(mod, name).register_forward_hook(lambda m, i, o, name=name: proj_out.__setitem__(name, o))
    mod.o.register_forward_pre_hook(lambda m, inputs: seen.__setitem__("o_in", inputs[0]))
    cache = ring.new_kv_cache(1, 1, 3 * S, heads, 1, device=gpu_device)[0]
    x = torch.randn(1, S, dim, device=gpu_device).bfloat16()
    with torch.no_grad():
        y = mod(x, None, torch.tensor([grid]), rope.build_freqs(), None, kv_cache=cache, current_start=0)
    torch.cuda.synchronize()
    o_in, attn_out = seen["o_in"], seen["attn_out"]
    assert o_in.data_ptr() == attn_out.data_ptr()
    assert o_in.is_contiguous() and tuple(o_in.shape) == (1, S, dim)
    assert attn_out.is_contiguous() and tuple(attn_out.shape) == (1, S, heads, 128)
    assert tuple(y.shape) == (1, S, dim)
    if fuse:
        assert seen["q_in"].data_ptr() == proj_out["q"].data_ptr()
        assert seen["k_in"].data_ptr() == proj_out["k"].data_ptr()
