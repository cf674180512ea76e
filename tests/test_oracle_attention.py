"""Pins for the oracle's KV-cache attention (the operator that is third-party
in the reference: flash_attn 2.7.4.post1 / torch SDPA, with no test vector in
the reference tree).  The mathematics fixes it: float64 numpy softmax brute
force, closed-form special cases, masking, permutation invariance and row
independence."""
import numpy as np
import pytest
import torch

from oracle import sdv2_oracle as oracle


def numpy_attention(q, k, v, lens):
    q, k, v = (t.double().numpy() for t in (q, k, v))
    out = np.zeros_like(q)
    B, S, H, D = q.shape
    for b in range(B):
        n = lens[b]
        for h in range(H):
            s = q[b, :, h] @ k[b, :n, h].T / np.sqrt(D)
            s -= s.max(axis=1, keepdims=True)
            p = np.exp(s)
            p /= p.sum(axis=1, keepdims=True)
            out[b, :, h] = p @ v[b, :n, h]
    return torch.from_numpy(out)


@pytest.mark.parametrize("lens", [[40, 40], [40, 17]])
def test_against_float64_brute_force(lens):
    torch.manual_seed(0)
    q, k, v = torch.randn(2, 9, 3, 128), torch.randn(2, 40, 3, 128), torch.randn(2, 40, 3, 128)
    want = numpy_attention(q, k, v, lens)
    got = oracle.attention_with_kvcache(q, k, v, torch.tensor(lens, dtype=torch.int32))
    assert torch.allclose(got.double(), want, atol=2e-5)
    got32 = oracle.attention_fp32_reference(q, k, v, lens)
    assert torch.allclose(got32.double(), want, atol=2e-5)
    # bf16 storage: the fp32 up-cast path stays within bf16 rounding of the exact result
    gb = oracle.attention_with_kvcache(q.bfloat16(), k.bfloat16(), v.bfloat16(), torch.tensor(lens, dtype=torch.int32))
    wb = numpy_attention(q.bfloat16(), k.bfloat16(), v.bfloat16(), lens)
    assert gb.dtype == torch.bfloat16
    assert (gb.double() - wb).abs().max() < 2e-2


def test_special_cases():
    torch.manual_seed(1)
    q, k = torch.randn(1, 5, 2, 128), torch.randn(1, 30, 2, 128)
    # all values equal -> output is that value
    v = torch.ones(1, 30, 2, 128) * 0.75
    out = oracle.attention_with_kvcache(q, k, v, torch.tensor([30], dtype=torch.int32))
    assert torch.allclose(out, v[:, :5], atol=1e-6)
    # one key with an overwhelming logit -> its value
    v = torch.randn(1, 30, 2, 128)
    k2 = k.clone()
    k2[0, 7] = q[0, 2] * 100.0
    out = oracle.attention_with_kvcache(q, k2, v, torch.tensor([30], dtype=torch.int32))
    assert torch.allclose(out[0, 2], v[0, 7], atol=1e-4)


def test_keys_beyond_seq_len_are_ignored():
    torch.manual_seed(2)
    q, k, v = torch.randn(2, 4, 2, 128), torch.randn(2, 20, 2, 128), torch.randn(2, 20, 2, 128)
    lens = torch.tensor([20, 11], dtype=torch.int32)
    a = oracle.attention_with_kvcache(q, k, v, lens)
    k[1, 11:] = 1e4
    v[1, 11:] = -1e4
    b = oracle.attention_with_kvcache(q, k, v, lens)
    assert torch.equal(a, b)


def test_permutation_invariance_and_row_independence():
    torch.manual_seed(3)
    q, k, v = torch.randn(2, 6, 2, 128), torch.randn(2, 24, 2, 128), torch.randn(2, 24, 2, 128)
    lens = torch.tensor([24, 24], dtype=torch.int32)
    a = oracle.attention_with_kvcache(q, k, v, lens)
    perm = torch.randperm(24)
    b = oracle.attention_with_kvcache(q, k[:, perm], v[:, perm], lens)
    assert torch.allclose(a, b, atol=1e-5)         # ring order vs temporal order
    c = oracle.attention_with_kvcache(q[1:], k[1:], v[1:], lens[1:])
    assert torch.allclose(a[1:], c, atol=1e-6)


def test_no_mask_inside_the_chunk():
    # the chunk's own keys are already in the cache and every query sees all of them
    torch.manual_seed(4)
    freqs = oracle.build_freqs()
    cache = oracle.new_kv_cache(1, 1, 24, 1, 1, dtype=torch.float32)[0]
    layer = oracle.RingAttentionOracle(sink_size=1)
    q, k, v = torch.randn(1, 12, 1, 128), torch.randn(1, 12, 1, 128), torch.randn(1, 12, 1, 128)
    out, roped_q, seq = layer.step(q, k, v, [(2, 2, 3)], freqs, cache, [0])
    assert seq == [12]
    want = numpy_attention(roped_q, cache["k"][:, :12], cache["v"][:, :12], [12])
    assert torch.allclose(out.double(), want, atol=2e-5)
    # first query row attends to the LAST key of the chunk too
    k_alt = cache["k"].clone()
    k_alt[0, 11] += 5.0
    out2 = oracle.attention_with_kvcache(roped_q, k_alt[:, :12], cache["v"][:, :12], torch.tensor([12], dtype=torch.int32))
    assert not torch.allclose(out[0, 0], out2[0, 0])
