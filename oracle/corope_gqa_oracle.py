"""Eager-PyTorch oracle for the Co-RoPE grouped-query attention, forward and backward.

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke entry and by the
benchmark's cpu_baseline leg, never by the shipped package.

Restates the reference's dense definition
(corope-exp/corope_attn_gqa_pytorch.py:16-134):

  inv_freq[d]   = theta^(-2d/D)                                        (:35)
  kv head       = q head // G, leader = first q head of the group      (:49-58)
  z[i, j]       = sigmoid(sm_scale * q_leader[i] . k[j])   (unmasked)  (:59)
  a[i, j]       = cumsum_j z[i, j]                                     (:60)
  delta[i, j]   = a[i, i] - a[i, j]                                    (:64)
  E_A, E_B      = q1 k1 + q2 k2,  q2 k1 - q1 k2   (per d)              (:71-72)
  score[i, j]   = sm_scale * sum_d (E_A cos(delta w_d) - E_B sin(delta w_d))   (:74-78)
  causal -inf mask, safe softmax, O = P V                              (:81-124)

``corope_gqa_forward`` is the dense form (5-D temporaries, small shapes only);
``corope_gqa_forward_rows`` produces the same numbers for a chosen set of query
rows per (batch, head) so that long sequences fit in memory.  The backward is
obtained from torch.autograd through the dense forward, which is how the
reference checks its own manual backward (:326-355); ``corope_gqa_backward_manual``
restates that manual backward in closed form and is held against autograd by the tests.
"""
from __future__ import annotations

import torch

from .rope_attn_oracle import _causal_mask, _softmax_rows


def corope_inv_freq(head_dim, theta, device="cpu", dtype=torch.float32):
    """theta^(-2d/D) for d in [0, D/2)  (reference :35)."""
    e = torch.arange(0, head_dim, 2, device=device).float() / head_dim
    return (1.0 / (theta ** e)).to(dtype)


def _check_shapes(q, k, v, causal):
    if not causal:
        raise ValueError("Co-RoPE attention supports causal=True only.")
    if q.ndim != 4 or k.ndim != 4 or v.ndim != 4:
        raise ValueError("Expected q, k, v of shape (batch, heads, seqlen, dim).")
    if k.shape != v.shape:
        raise ValueError("k and v must share the same shape.")
    if q.shape[0] != k.shape[0] or q.shape[2] != k.shape[2] or q.shape[3] != k.shape[3]:
        raise ValueError("k must align with q along batch/sequence/head_dim.")
    if q.shape[1] % k.shape[1]:
        raise ValueError(f"Number of Q heads ({q.shape[1]}) must be divisible by KV heads ({k.shape[1]}).")
    return q.shape[1] // k.shape[1]


def corope_gqa_forward(q, k, v, causal, sm_scale, theta, compute_dtype=torch.float32, return_aux=False,
                       detach_gates=False):
    """Dense Co-RoPE GQA forward; O has shape (B, Hq, N, D) in ``compute_dtype``.

    ``detach_gates`` cuts the position offsets out of the autograd graph (same output, gradients without the path
    through the leader's sigmoid gates); tests use it to show that this path is material on their inputs."""
    G = _check_shapes(q, k, v, causal)
    cd = compute_dtype
    q, k, v = q.to(cd), k.to(cd), v.to(cd)
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    w_d = corope_inv_freq(D, theta, q.device, cd)

    kx = k.repeat_interleave(G, dim=1)           # q head h reads kv head h // G
    vx = v.repeat_interleave(G, dim=1)

    lead = q[:, ::G]                             # (B, Hkv, N, D)
    z = torch.sigmoid(torch.einsum("bhqd,bhkd->bhqk", lead, k) * sm_scale)
    a = torch.cumsum(z, dim=-1).repeat_interleave(G, dim=1)          # (B, Hq, N, N)
    delta = torch.diagonal(a, dim1=-2, dim2=-1).unsqueeze(-1) - a
    if detach_gates:
        delta = delta.detach()

    h = D // 2
    q1, q2 = q[..., :h].unsqueeze(3), q[..., h:].unsqueeze(3)        # (B,Hq,N,1,h)
    k1, k2 = kx[..., :h].unsqueeze(2), kx[..., h:].unsqueeze(2)      # (B,Hq,1,N,h)
    e_a = q1 * k1 + q2 * k2
    e_b = q2 * k1 - q1 * k2
    phi = delta.unsqueeze(-1) * w_d
    scores = (e_a * torch.cos(phi) - e_b * torch.sin(phi)).sum(-1) * sm_scale

    mask = _causal_mask(N, N, 0, q.device)[None, None]
    w, lse = _softmax_rows(scores, mask)
    o = torch.einsum("bhqk,bhkd->bhqd", w, vx)
    if return_aux:
        return o, {"delta": delta, "weights": w, "lse": lse, "z": z}
    return o


def corope_gqa_forward_rows(q, k, v, causal, sm_scale, theta, rows, compute_dtype=torch.float32,
                            row_block=64):
    """Same as ``corope_gqa_forward`` for the query rows in ``rows`` only.

    Returns (B, Hq, len(rows), D).  Each row needs only its own leader logits, so
    the cost is O(len(rows) * N * D) per head instead of O(N^2 * D)."""
    G = _check_shapes(q, k, v, causal)
    cd = compute_dtype
    B, Hq, N, D = q.shape
    h = D // 2
    rows = rows.to(torch.long)
    w_d = corope_inv_freq(D, theta, q.device, cd)
    out = torch.empty(B, Hq, rows.numel(), D, dtype=cd)
    col = torch.arange(N).unsqueeze(0)
    for b in range(B):
        for hq in range(Hq):
            kv = hq // G
            kk, vv = k[b, kv].to(cd), v[b, kv].to(cd)
            k1, k2 = kk[:, :h], kk[:, h:]
            for r0 in range(0, rows.numel(), row_block):
                sel = rows[r0:r0 + row_block]
                ql = q[b, kv * G, sel].to(cd)
                z = torch.sigmoid((ql @ kk.T) * sm_scale)
                a = torch.cumsum(z, dim=-1)
                delta = a.gather(1, sel.unsqueeze(1)) - a                  # (R, N)
                qq = q[b, hq, sel].to(cd)
                q1, q2 = qq[:, None, :h], qq[:, None, h:]
                e_a = q1 * k1[None] + q2 * k2[None]
                e_b = q2 * k1[None] - q1 * k2[None]
                phi = delta.unsqueeze(-1) * w_d
                sc = (e_a * torch.cos(phi) - e_b * torch.sin(phi)).sum(-1) * sm_scale
                w, _ = _softmax_rows(sc, col > sel.unsqueeze(1))
                out[b, hq, r0:r0 + row_block] = w @ vv
    return out


def corope_gqa_backward_manual(q, k, v, grad_out, sm_scale, theta, compute_dtype=torch.float64):
    """Dense closed-form backward: (dq, dk, dv) without autograd.

    Restates the reference's manual backward (corope-exp/flash_attn_co_rope_gqa_triton.py:459-577, same as
    corope-exp/corope_attn_gqa_pytorch.py:137-300) in the decomposition the GPU kernels use, so that a test can hold it
    against autograd through ``corope_gqa_forward``:

      kt[i,j]   = key j rotated by -delta[i,j] w_d;  S = c q . kt;  dS = P (dP - rowsum(P dP))         (:519-529)
      dq        = c sum_j dS kt;   dk = c sum_{h,i} dS qt  (qt: the query rotated by +delta w_d)        (:541-547)
      g[i,j]    = dS/ddelta = c sum_d w_d (q1 kt2 - q2 kt1);  G = sum_{h in group} dS g                (:531-539, :555)
      dz[i,t]   = sum_{j<t} G[i,j]  (the reverse cumulative sum of d_a, :549-557);  W = dz z (1 - z)   (:559-560)
      dq_leader += c W k;   dk += c W^T q_leader                                                       (:561-566)
    """
    G = _check_shapes(q, k, v, True)
    cd = compute_dtype
    q, k, v, go = q.to(cd), k.to(cd), v.to(cd), grad_out.to(cd)
    B, Hq, N, D = q.shape
    Hkv, h = k.shape[1], D // 2
    w_d = corope_inv_freq(D, theta, q.device, cd)
    kx, vx = k.repeat_interleave(G, dim=1), v.repeat_interleave(G, dim=1)
    lead = q[:, ::G]
    z = torch.sigmoid(torch.einsum("bhqd,bhkd->bhqk", lead, k) * sm_scale)          # (B, Hkv, N, N)
    a = torch.cumsum(z, dim=-1)
    delta_g = torch.diagonal(a, dim1=-2, dim2=-1).unsqueeze(-1) - a
    delta = delta_g.repeat_interleave(G, dim=1)
    phi = delta.unsqueeze(-1) * w_d                                                  # (B, Hq, N, N, h)
    cs, sn = torch.cos(phi), torch.sin(phi)
    k1, k2 = kx[..., :h].unsqueeze(2), kx[..., h:].unsqueeze(2)                      # (B, Hq, 1, N, h)
    q1, q2 = q[..., :h].unsqueeze(3), q[..., h:].unsqueeze(3)                        # (B, Hq, N, 1, h)
    kt1, kt2 = k1 * cs + k2 * sn, k2 * cs - k1 * sn
    mask = _causal_mask(N, N, 0, q.device)[None, None]
    scores = (q1 * kt1 + q2 * kt2).sum(-1) * sm_scale
    p, _ = _softmax_rows(scores, mask)
    dp = torch.einsum("bhqd,bhkd->bhqk", go, vx)
    ds = p * (dp - (p * dp).sum(-1, keepdim=True))
    dv = torch.einsum("bhqk,bhqd->bhkd", p, go).view(B, Hkv, G, N, D).sum(2)
    dq = torch.cat([(ds.unsqueeze(-1) * kt1).sum(3), (ds.unsqueeze(-1) * kt2).sum(3)], dim=-1) * sm_scale
    qt1, qt2 = q1 * cs - q2 * sn, q2 * cs + q1 * sn
    dk = torch.cat([(ds.unsqueeze(-1) * qt1).sum(2), (ds.unsqueeze(-1) * qt2).sum(2)], dim=-1) * sm_scale
    dk = dk.view(B, Hkv, G, N, D).sum(2)
    g = ((q1 * kt2 - q2 * kt1) * w_d).sum(-1) * sm_scale
    big_g = (ds * g).view(B, Hkv, G, N, N).sum(2)                                    # (B, Hkv, N, N), zero above the diagonal
    dz = torch.cumsum(big_g, dim=-1) - big_g                                         # sum over j < t
    wmat = (dz * z * (1 - z)).masked_fill(mask, 0.0)
    dq = dq.clone()
    dq[:, ::G] += torch.einsum("bhqk,bhkd->bhqd", wmat, k) * sm_scale
    dk = dk + torch.einsum("bhqk,bhqd->bhkd", wmat, lead) * sm_scale
    return dq, dk, dv


class _CoRopeOracle(torch.autograd.Function):
    """Twin of the reference's Co-RoPE ``_attention_pytorch`` (6 positional arguments).

    Backward differentiates the dense forward with torch.autograd."""

    @staticmethod
    def forward(ctx, q, k, v, causal, sm_scale, theta):
        cd = torch.float32 if q.dtype in (torch.float16, torch.bfloat16) else q.dtype
        ctx.save_for_backward(q, k, v)
        ctx.args = (causal, sm_scale, theta, cd)
        return corope_gqa_forward(q, k, v, causal, sm_scale, theta, cd)

    @staticmethod
    def backward(ctx, grad_out):
        q, k, v = (t.detach().clone().requires_grad_(True) for t in ctx.saved_tensors)
        causal, sm_scale, theta, cd = ctx.args
        with torch.enable_grad():
            o = corope_gqa_forward(q, k, v, causal, sm_scale, theta, cd)
            dq, dk, dv = torch.autograd.grad(o, (q, k, v), grad_out.to(o.dtype))
        return dq, dk, dv, None, None, None


attention_pytorch = _CoRopeOracle.apply
