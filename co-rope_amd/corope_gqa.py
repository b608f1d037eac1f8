"""Co-RoPE grouped-query attention forward behind the reference's call surface.

``attention(q, k, v, causal, sm_scale, theta[, warp_specialize])`` mirrors the reference's
``_attention.apply`` (corope-exp/flash_attn_co_rope_gqa_triton.py:403-456, :580), including its validation
errors (:407-425).  The forward is a hand-written gfx950 kernel reached through the C ABI.  The reference's own
"fused" operator falls back to a dense PyTorch backward (:459-577); that backward is not part of this library yet,
so differentiating through this operator raises."""
from __future__ import annotations

import torch

from . import _lib


class _CoRopeGqaAttn(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, causal, sm_scale, theta, warp_specialize=False):
        if not causal:
            raise ValueError("CoRoPE fused kernel supports causal=True only.")
        if q.ndim != 4 or k.ndim != 4 or v.ndim != 4:
            raise ValueError("Expected q, k, v to have shape (batch, heads, seqlen, dim).")
        if k.shape != v.shape:
            raise ValueError("k and v must share the same shape in GQA.")
        if q.shape[0] != k.shape[0] or q.shape[2] != k.shape[2] or q.shape[3] != k.shape[3]:
            raise ValueError("k must align with q along batch/sequence/head_dim.")
        B, Hq, N, D = q.shape
        Hkv = k.shape[1]
        if Hq % Hkv != 0:
            raise ValueError("Number of query heads must be divisible by KV heads.")
        if Hq // Hkv > 8:
            raise ValueError(f"CoRoPE backbone currently limits group_size <= 8 (got {Hq // Hkv}).")
        if not (q.is_cuda and k.is_cuda and v.is_cuda):
            raise ValueError("Co-RoPE attention runs on the GPU only: q, k, v must be on a HIP device")
        if not (q.dtype == k.dtype == v.dtype == torch.bfloat16):
            raise ValueError(f"q, k, v must be bfloat16 (got {q.dtype}, {k.dtype}, {v.dtype})")
        lib = _lib.load()
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        o = torch.empty_like(q)
        with torch.cuda.device(q.device):
            rc = lib.corope_gqa_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), B, Hq, Hkv, N, D,
                                    float(sm_scale), float(theta), torch.cuda.current_stream(q.device).cuda_stream)
        _lib.check(rc, "corope_gqa_fwd")
        ctx.group_size = Hq // Hkv
        ctx.sm_scale = sm_scale
        ctx.causal = causal
        return o

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("Co-RoPE GQA backward is not provided by the gfx950 library")


attention = _CoRopeGqaAttn.apply


def corope_attn_gqa(q, k, v, sm_scale=None, theta=10000.0, causal=True):
    """Keyword-friendly form: ``sm_scale`` defaults to 1/sqrt(D)."""
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    return attention(q, k, v, causal, sm_scale, theta)
