"""Host-side construction of the Wan 3-D RoPE table.

The model owns one complex128 table ``freqs`` [1024, head_dim/2] whose columns
are the temporal, height and width frequency pairs (22 | 21 | 21 at head_dim
128) and hands it to every attention call; the append kernel indexes it by
(frame | h | w).  The table is built once on the CPU in float64, as the
reference model does at construction (models/wan/causal_model.py:631-638 with
``rope_params`` of models/wan/wan_base/modules/model.py:29-36), so that both
sides start from bit-identical cos/sin values.
"""
from __future__ import annotations

from typing import Tuple

import torch


def axis_table(positions: int, dim: int, theta: float = 10000.0) -> torch.Tensor:
    """exp(i * pos * theta^(-2j/dim)), pos < positions, j < dim/2, complex128."""
    if dim % 2 != 0:
        raise ValueError("dim must be even")
    inv_freq = 1.0 / torch.pow(theta, torch.arange(0, dim, 2).to(torch.float64).div(dim))
    angle = torch.outer(torch.arange(positions), inv_freq)
    return torch.polar(torch.ones_like(angle), angle)


def rope_params(max_seq_len: int, dim: int, theta: float = 10000.0) -> torch.Tensor:
    """The reference's name and argument order for :func:`axis_table`
    (models/wan/wan_base/modules/model.py:29-36)."""
    return axis_table(max_seq_len, dim, theta)


def column_split(pairs: int) -> Tuple[int, int, int]:
    """How many of the ``pairs`` complex columns belong to (t, h, w)."""
    third = pairs // 3
    return pairs - 2 * third, third, third


def build_freqs(head_dim: int = 128, positions: int = 1024) -> torch.Tensor:
    sixth = head_dim // 6
    dims = (head_dim - 4 * sixth, 2 * sixth, 2 * sixth)
    return torch.cat([axis_table(positions, d) for d in dims], dim=1)
