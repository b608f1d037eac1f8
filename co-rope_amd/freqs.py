"""cos/sin tables for the half-layout rotation.

Same values and layout as the reference's ``precompute_freqs_cis``
(fused-rope/rope_attn_pytorch.py:10-49): theta_i = theta^(-2i/dim), angle[m, i] = m * theta_i in fp32, tables of
shape (seq_len, dim) whose second half repeats the first.  The kernels read only columns [0, dim/2)."""
from __future__ import annotations

import torch


def precompute_freqs_cis(dim, seq_len, theta=10000.0, device="cuda"):
    assert dim % 2 == 0, f"dim must be even, got {dim}"
    inv = 1.0 / (theta ** (torch.arange(0, dim, 2, device=device).float() / dim))
    ang = torch.outer(torch.arange(seq_len, device=device, dtype=torch.float32), inv)
    cos, sin = torch.cos(ang), torch.sin(ang)
    return torch.cat([cos, cos], dim=-1), torch.cat([sin, sin], dim=-1)
