"""Eager-PyTorch oracle for half-layout RoPE + softmax attention (forward and backward).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke entry and by the
benchmark's cpu_baseline leg, never by the shipped package.

Restates, op for op, the reference's PyTorch path
(fused-rope/rope_attn_pytorch.py):

  precompute_freqs_cis   :10-49
  rotate_half            :52-68
  apply_rotary_emb       :71-84
  rope_attn_forward      :94-162   (_attention_pytorch.forward)
  rope_attn_backward     :165-224  (_attention_pytorch.backward)

All arithmetic runs in ``compute_dtype`` (fp32 as the reference's parity run
does, or fp64 for the pins).  The dense functions materialise (B,H,N,N)
tensors exactly like the reference; the ``*_blocked`` variants produce the
same numbers one (batch, head) slab or one query-row block at a time so that
the benchmark shapes fit in host memory.
"""
from __future__ import annotations

import math

import torch


# --------------------------------------------------------------------------- a1
def precompute_freqs_cis(dim, seq_len, theta=10000.0, device="cpu", dtype=torch.float32):
    """cos/sin tables of shape (seq_len, dim), halves duplicated.

    Reference: fused-rope/rope_attn_pytorch.py:10-49 (theta_i = theta^(-2i/dim),
    angle[m, i] = m * theta_i, table = cat([x, x], -1)).
    """
    if dim % 2:
        raise AssertionError(f"dim must be even, got {dim}")
    exponent = torch.arange(0, dim, 2, device=device).float() / dim
    inv = 1.0 / (theta ** exponent)                       # (dim/2,)
    pos = torch.arange(seq_len, device=device, dtype=torch.float32)
    ang = torch.outer(pos, inv)                           # (seq_len, dim/2) fp32 like the reference
    c, s = torch.cos(ang), torch.sin(ang)
    return (torch.cat([c, c], -1).to(dtype), torch.cat([s, s], -1).to(dtype))


# --------------------------------------------------------------------------- a2
def rotate_half(x):
    """[x1, x2] -> [-x2, x1] on the last axis (reference :52-68)."""
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def apply_rotary_emb(x, freqs_cos, freqs_sin):
    """x*cos + rotate_half(x)*sin (reference :71-84).  Inverse = pass -sin."""
    return x * freqs_cos + rotate_half(x) * freqs_sin


# --------------------------------------------------------------------------- a3
def _causal_mask(n_q, n_k, row0, device):
    """True where key index > absolute query index (strict upper triangle)."""
    rows = torch.arange(row0, row0 + n_q, device=device).unsqueeze(1)
    cols = torch.arange(n_k, device=device).unsqueeze(0)
    return cols > rows


def _softmax_rows(scores, mask):
    """Safe softmax with the reference's masking sequence (:124-151).

    Returns (weights, natural-log LSE)."""
    if mask is not None:
        scores = scores.masked_fill(mask, float("-inf"))
    row_max = scores.max(dim=-1, keepdim=True).values
    row_max = torch.where(torch.isinf(row_max), torch.zeros_like(row_max), row_max)
    e = torch.exp(scores - row_max)
    if mask is not None:
        e = e.masked_fill(mask, 0.0)
    denom = e.sum(dim=-1, keepdim=True)
    w = e / denom
    if mask is not None:
        w = w.masked_fill(mask, 0.0)
    lse = (row_max + torch.log(denom)).squeeze(-1)
    return w, lse


def rope_attn_forward(q, k, v, causal, sm_scale, freqs_cos, freqs_sin, compute_dtype=torch.float32):
    """Dense forward.  Returns (O, LSE_natural, saved) with everything in ``compute_dtype``.

    saved = (q_rot, k_rot, v, weights) is what the reference keeps for its
    backward (:158).  LSE is not produced by the reference's PyTorch path; it is
    logsumexp of the scaled, masked scores and equals ``M * ln2`` of the fused
    kernel's base-2 statistic (fused-rope/fused_rope_attn.py:316).
    """
    cd = compute_dtype
    q, k, v = q.to(cd), k.to(cd), v.to(cd)
    c, s = freqs_cos.to(cd), freqs_sin.to(cd)
    qr = apply_rotary_emb(q, c, s)
    kr = apply_rotary_emb(k, c, s)
    scores = torch.einsum("bhqd,bhkd->bhqk", qr, kr) * sm_scale
    n = q.shape[2]
    mask = _causal_mask(n, n, 0, q.device)[None, None] if causal else None
    w, lse = _softmax_rows(scores, mask)
    o = torch.einsum("bhqk,bhkd->bhqd", w, v)
    return o, lse, (qr, kr, v, w)


# --------------------------------------------------------------------------- a4
def rope_attn_backward(saved, grad_out, causal, sm_scale, freqs_cos, freqs_sin):
    """Manual backward (reference :165-224).  Returns (dq, dk, dv)."""
    qr, kr, v, w = saved
    cd = w.dtype
    g = grad_out.to(cd)
    c, s = freqs_cos.to(cd), freqs_sin.to(cd)
    dv = torch.einsum("bhqk,bhqd->bhkd", w, g)
    dw = torch.einsum("bhqd,bhkd->bhqk", g, v)
    row_dot = (dw * w).sum(dim=-1, keepdim=True)
    ds = w * (dw - row_dot)
    if causal:
        n = qr.shape[2]
        ds = ds.masked_fill(_causal_mask(n, n, 0, qr.device)[None, None], 0.0)
    dqr = torch.einsum("bhqk,bhkd->bhqd", ds, kr) * sm_scale
    dkr = torch.einsum("bhqk,bhqd->bhkd", ds, qr) * sm_scale
    dq = apply_rotary_emb(dqr, c, -s)
    dk = apply_rotary_emb(dkr, c, -s)
    return dq, dk, dv


# ------------------------------------------------------------ memory-bounded forms
def rope_attn_forward_blocked(q, k, v, causal, sm_scale, freqs_cos, freqs_sin,
                              row_block=1024, compute_dtype=torch.float32, rows=None):
    """Same numbers as ``rope_attn_forward`` without the (B,H,N,N) temporaries.

    Works one (b, h) slab and ``row_block`` query rows at a time.  ``rows``
    (1-D LongTensor of absolute query indices) restricts the computation to a
    sample of rows: attention rows are independent given K and V, so the
    returned O/LSE then have shape (B,H,len(rows),D) / (B,H,len(rows)).
    """
    cd = compute_dtype
    B, H, N, D = q.shape
    c, s = freqs_cos.to(cd), freqs_sin.to(cd)
    idx = torch.arange(N) if rows is None else rows.to(torch.long)
    o = torch.empty(B, H, idx.numel(), D, dtype=cd)
    lse = torch.empty(B, H, idx.numel(), dtype=cd)
    col = torch.arange(N).unsqueeze(0)
    for b in range(B):
        for h in range(H):
            kr = apply_rotary_emb(k[b, h].to(cd), c, s)
            vv = v[b, h].to(cd)
            for r0 in range(0, idx.numel(), row_block):
                sel = idx[r0:r0 + row_block]
                qr = apply_rotary_emb(q[b, h, sel].to(cd), c[sel], s[sel])
                sc = (qr @ kr.T) * sm_scale
                mask = (col > sel.unsqueeze(1)) if causal else None
                w, l = _softmax_rows(sc, mask)
                o[b, h, r0:r0 + row_block] = w @ vv
                lse[b, h, r0:r0 + row_block] = l
    return o, lse


def rope_attn_fwd_bwd_blocked(q, k, v, grad_out, causal, sm_scale, freqs_cos, freqs_sin,
                              compute_dtype=torch.float32):
    """Forward + manual backward one (b, h) slab at a time (dense N x N per slab).

    Returns (O, LSE, dq, dk, dv, delta) in ``compute_dtype``; delta = rowsum(O * dO)
    is the quantity the fused backward's preprocess pass produces
    (fused-rope/fused_rope_attn.py:324-337).
    """
    cd = compute_dtype
    B, H, N, D = q.shape
    o = torch.empty(B, H, N, D, dtype=cd)
    lse = torch.empty(B, H, N, dtype=cd)
    dq, dk, dv = torch.empty_like(o), torch.empty_like(o), torch.empty_like(o)
    for b in range(B):
        for h in range(H):
            sl = (slice(b, b + 1), slice(h, h + 1))
            ob, lb, saved = rope_attn_forward(q[sl], k[sl], v[sl], causal, sm_scale,
                                              freqs_cos, freqs_sin, cd)
            gq, gk, gv = rope_attn_backward(saved, grad_out[sl], causal, sm_scale,
                                            freqs_cos, freqs_sin)
            o[sl], lse[sl], dq[sl], dk[sl], dv[sl] = ob, lb, gq, gk, gv
    delta = (o * grad_out.to(cd)).sum(-1)
    return o, lse, dq, dk, dv, delta


# ------------------------------------------------------------- reference call surface
class _AttentionOracle(torch.autograd.Function):
    """Twin of the reference's ``_attention_pytorch`` (7 positional arguments)."""

    @staticmethod
    def forward(ctx, q, k, v, causal, sm_scale, freqs_cos, freqs_sin):
        cd = torch.promote_types(q.dtype, freqs_cos.dtype)   # the reference's type promotion (:108)
        if cd in (torch.float16, torch.bfloat16):
            cd = torch.float32
        o, _, saved = rope_attn_forward(q, k, v, causal, sm_scale, freqs_cos, freqs_sin, cd)
        ctx.save_for_backward(*saved, freqs_cos, freqs_sin)
        ctx.sm_scale, ctx.causal = sm_scale, causal
        return o

    @staticmethod
    def backward(ctx, grad_out):
        *saved, fc, fs = ctx.saved_tensors
        dq, dk, dv = rope_attn_backward(tuple(saved), grad_out, ctx.causal, ctx.sm_scale, fc, fs)
        return dq, dk, dv, None, None, None, None


attention_pytorch = _AttentionOracle.apply


# ------------------------------------------------------------------- FLOP model (used by bench.py)
def attention_flops(B, H, N, D, mode="fwd", causal=False):
    """The reference's FLOP model (fused-rope/bench_compare.py:61-86): two N x N x D
    matmuls, halved when causal, x2.5 for the backward; rotation FLOPs are not counted."""
    total = 2 * (2.0 * B * H * N * N * D)
    if causal:
        total *= 0.5
    if mode == "bwd":
        total *= 2.5
    return total


def lse_to_base2(lse_nat):
    """Natural-log LSE -> the fused kernel's M statistic (base 2 of the scaled scores)."""
    return lse_nat / math.log(2.0)
