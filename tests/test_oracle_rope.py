"""Pins for the oracle's RoPE tables, expansion and rotation.

None of these re-types the oracle's formula with the same library calls: the
tables are checked against python ``math`` closed forms, the expansion against
a divmod brute force, and the rotation + rounding against a scalar loop on
python floats (IEEE double, no FMA) with explicit bit-level rounding.
"""
import math
import struct

import pytest
import torch

from oracle import sdv2_oracle as oracle


def f32_round(x: float) -> float:
    return struct.unpack("f", struct.pack("f", x))[0]


def bf16_bits_from_f32(x: float) -> int:
    u = struct.unpack("I", struct.pack("f", x))[0]
    if x != x:
        return 0x7FC0
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF


def test_table_closed_form_and_layout():
    freqs = oracle.build_freqs(128, 1024)
    assert freqs.shape == (1024, 64) and freqs.dtype == torch.complex128
    t, h, w = oracle.split_freqs(freqs)
    assert (t.shape[1], h.shape[1], w.shape[1]) == (22, 21, 21)
    # position 0 is exactly 1 + 0i; unit modulus everywhere
    assert torch.equal(torch.view_as_real(freqs[0]), torch.tensor([[1.0, 0.0]] * 64, dtype=torch.float64))
    assert torch.allclose(freqs.abs(), torch.ones(1024, 64, dtype=torch.float64), atol=1e-15)
    for tab, dim in ((t, 44), (h, 42), (w, 42)):
        for pos in (1, 2, 17, 51, 500, 1023):
            for j in (0, 1, 5, tab.shape[1] - 1):
                ang = pos * (1.0 / (10000.0 ** ((2 * j) / dim)))
                assert abs(tab[pos, j].real.item() - math.cos(ang)) < 5e-12
                assert abs(tab[pos, j].imag.item() - math.sin(ang)) < 5e-12
    # first temporal pair rotates by exactly `frame` radians
    assert abs(torch.angle(t[3, 0]).item() - 3.0) < 1e-14


def test_rope_params_rejects_odd_dim():
    with pytest.raises(ValueError):
        oracle.rope_params(8, 7)


def test_expansion_brute_force():
    freqs = oracle.build_freqs()
    f, h, w, sf = 2, 3, 4, 5
    mult = oracle.expand_rope_freqs(freqs, f, h, w, sf)
    assert mult.shape == (f * h * w, 1, 64)
    for tok in range(f * h * w):
        fi, rem = divmod(tok, h * w)
        hi, wi = divmod(rem, w)
        for p in range(64):
            pos = sf + fi if p < 22 else (hi if p < 43 else wi)
            assert mult[tok, 0, p] == freqs[pos, p]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rotation_scalar_loop_bit_exact(dtype):
    torch.manual_seed(5)
    freqs = oracle.build_freqs()
    grid, sf = (2, 2, 3), 9
    S = 12
    x = torch.randn(1, S, 2, 128).to(dtype)
    got = oracle.causal_rope_apply(x, [grid], freqs, [sf])
    xs = x.double()
    for tok in (0, 5, 11):
        fi, rem = divmod(tok, 6)
        hi, wi = divmod(rem, 3)
        for head in (0, 1):
            for p in range(64):
                pos = sf + fi if p < 22 else (hi if p < 43 else wi)
                c, d = freqs[pos, p].real.item(), freqs[pos, p].imag.item()
                a, b = xs[0, tok, head, 2 * p].item(), xs[0, tok, head, 2 * p + 1].item()
                re = a * c - b * d          # python floats: each op rounded once, no FMA
                im = a * d + b * c
                for val, idx in ((re, 2 * p), (im, 2 * p + 1)):
                    out = got[0, tok, head, idx]
                    if dtype == torch.float32:
                        assert out.item() == f32_round(val)
                    else:
                        bits = out.view(torch.int16).item() & 0xFFFF
                        assert bits == bf16_bits_from_f32(f32_round(val))


def test_rotation_invariants():
    torch.manual_seed(6)
    freqs = oracle.build_freqs()
    x = torch.randn(2, 24, 3, 128, dtype=torch.float32)
    # frame 0, h = w = 0 -> identity, bit for bit
    y0 = oracle.causal_rope_apply(x[:, :1], [(1, 1, 1)] * 2, freqs, [0, 0])
    assert torch.equal(y0, x[:, :1])
    # per-pair norm preserved; q and k share the multipliers
    y = oracle.causal_rope_apply(x, [(2, 3, 4)] * 2, freqs, [3, 40])
    n_in = x.reshape(2, 24, 3, 64, 2).double().norm(dim=-1)
    n_out = y.reshape(2, 24, 3, 64, 2).double().norm(dim=-1)
    assert torch.allclose(n_in, n_out, rtol=1e-6, atol=1e-6)
    # different start frames change only the 44 temporal dims
    y2 = oracle.causal_rope_apply(x, [(2, 3, 4)] * 2, freqs, [4, 40])
    assert torch.equal(y[0, :, :, 44:], y2[0, :, :, 44:])
    assert not torch.equal(y[0, :, :, :44], y2[0, :, :, :44])
    assert torch.equal(y[1], y2[1])


def test_double_to_bf16_goes_through_float():
    # the cast the reference applies with .type_as(): double -> float -> bf16
    v = torch.tensor([1 + 2 ** -8 + 2 ** -30], dtype=torch.float64)
    assert v.to(torch.bfloat16).item() == 1.0                 # double rounding
    assert v.float().to(torch.bfloat16).item() == 1.0
    big = torch.randn(4096, dtype=torch.float64) * 3
    assert torch.equal(big.to(torch.bfloat16), big.float().to(torch.bfloat16))
    bits = big.float().to(torch.bfloat16).view(torch.int16).tolist()
    for val, b in zip(big.tolist()[:256], bits[:256]):
        assert (b & 0xFFFF) == bf16_bits_from_f32(f32_round(val))


def test_package_table_is_the_oracle_table_bit_for_bit():
    """The package builds its table on the host with its own code; the GPU
    parity tests hand either table to the kernels, so the two must be one."""
    from streamdiffusionv2_amd import ops, rope

    for head_dim, positions in ((128, 1024), (128, 64), (96, 33)):
        mine = torch.view_as_real(rope.build_freqs(head_dim, positions))
        theirs = torch.view_as_real(oracle.build_freqs(head_dim, positions))
        assert torch.equal(mine.view(torch.int64), theirs.view(torch.int64))
    assert rope.column_split(64) == (22, 21, 21)
    # reference names (model.py:29-36, causal_model.py:111) resolve to the same code
    assert torch.equal(torch.view_as_real(rope.rope_params(50, 44)), torch.view_as_real(oracle.rope_params(50, 44)))
    with pytest.raises(ValueError):
        rope.rope_params(8, 7)
    assert ops.attention_with_kvcache_fallback is ops.flash_attn_with_kvcache
