"""Pins for the driver arithmetic around the path: stream-batch shift
register, chunk schedule with the t_refresh clamp, motion-adaptive noise."""
import math

import torch

from oracle import sdv2_oracle as oracle


def test_shift_register_brute_force():
    fsl, B = 1560, 4
    first_end = 2 * fsl
    reg = oracle.StreamShiftRegister(B, first_end, fsl)
    assert reg.starts == [first_end] * B and reg.ends == [first_end + fsl] * B
    history = []
    cs, ce = first_end, first_end + fsl
    for n in range(7):
        starts, ends = reg.push(cs, ce)
        history.append(cs)
        for j in range(B):
            want = history[n - j] if n - j >= 0 else first_end
            assert starts[j] == want
            assert ends[j] == want + fsl
        cs, ce = ce, ce + fsl


def test_chunk_schedule_closed_forms():
    fsl, nfpb, cap = 1560, 1, 6 * 1560
    sched = oracle.chunk_schedule(60, fsl, nfpb, cap, t_refresh=50)
    assert sched[0] == (0, 2 * fsl)                      # first chunk: 1 + nfpb latent frames
    for i in range(1, 49):
        assert sched[i] == ((i + 1) * fsl, (i + 2) * fsl)
        assert sched[i][0] == sched[i - 1][1]
    # chunk i starts at frame i+1; from frame 50 on the position is pinned to the cache's last frame
    assert sched[48][0] // fsl == 49
    for i in range(49, 60):
        assert sched[i] == (cap - fsl, cap)
    sched3 = oracle.chunk_schedule(5, fsl, 3, 12 * fsl)
    assert sched3[0] == (0, 4 * fsl) and sched3[1] == (4 * fsl, 7 * fsl)


def test_noise_scale_and_step():
    video = torch.zeros(1, 3, 9, 4, 4)
    video[:, :, 5:] = 0.1                                  # one frame pair differs by 0.1 everywhere
    scale, step = oracle.noise_scale_and_step(video, end_idx=9, chunk_size=4, noise_scale=0.8, init_noise_scale=0.8)
    motion = min(max(0.1 / 0.2, 0.0), 1.0)                 # RMS diff 0.1, max over frames
    want = (0.8 - 0.1 * motion) * 0.9 + 0.8 * 0.1
    assert math.isclose(scale, want, rel_tol=1e-6)
    assert step == int(1000 * scale) - 100
    still, step0 = oracle.noise_scale_and_step(torch.zeros(1, 3, 9, 4, 4), 9, 4, 0.8, 0.8)
    assert math.isclose(still, 0.8, rel_tol=1e-9) and step0 in (699, 700)
    z, n = torch.full((2, 2), 2.0), torch.full((2, 2), -1.0)
    assert torch.allclose(oracle.mix_noise(z, n, 0.25), torch.full((2, 2), 1.25))
