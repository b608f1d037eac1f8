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


def rope_freqs_device(dim, seq_len, theta=10000.0, device="cuda", pos0=0, compact=False):
    """The same tables produced by the library's own kernel (no torch ops): rows are positions pos0 .. pos0+seq_len-1;
    ``compact=True`` returns (seq_len, dim/2) tables, which is all the attention kernels read."""
    from . import _lib
    lib = _lib.load()
    dev = torch.device(device)
    if dev.type != "cuda":
        raise ValueError("rope_freqs_device runs on the GPU only")
    width = dim // 2 if compact else dim
    cos = torch.empty((seq_len, width), device=dev, dtype=torch.float32)
    sin = torch.empty_like(cos)
    with torch.cuda.device(dev):
        rc = lib.corope_rope_freqs(cos.data_ptr(), sin.data_ptr(), seq_len, dim, width, cos.stride(0), int(pos0),
                                   float(theta), torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(rc, "corope_rope_freqs")
    return cos, sin
