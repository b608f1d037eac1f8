"""Pins for the RoPE-attention oracle (CPU only).

Each test checks the oracle against something that is NOT its own formula: a closed
form in higher precision, a library routine, an independent brute-force program, an
algebraic invariant, or torch.autograd."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import seeded
from oracle import rope_attn_oracle as O


# ----------------------------------------------------------------------------- a1 freqs
@pytest.mark.parametrize("D,N,theta", [(64, 128, 10000.0), (128, 512, 10000.0), (32, 17, 500.0)])
def test_freqs_closed_form(D, N, theta):
    c, s = O.precompute_freqs_cis(D, N, theta)
    assert c.shape == (N, D) and s.shape == (N, D) and c.dtype == torch.float32
    # closed form in fp64; the fp32 angle m*theta_i carries ~|angle| * 2^-24 of error
    i = np.arange(D // 2, dtype=np.float64)
    ang = np.arange(N, dtype=np.float64)[:, None] * theta ** (-2.0 * i / D)[None, :]
    tol = 4e-7 * max(N, 8)
    assert np.abs(c[:, :D // 2].numpy() - np.cos(ang)).max() < tol
    assert np.abs(s[:, :D // 2].numpy() - np.sin(ang)).max() < tol
    # invariants: position 0 is the identity, unit modulus, second half duplicates the first
    assert torch.all(c[0] == 1) and torch.all(s[0] == 0)
    assert torch.allclose(c * c + s * s, torch.ones_like(c), atol=1e-6)
    assert torch.equal(c[:, :D // 2], c[:, D // 2:]) and torch.equal(s[:, :D // 2], s[:, D // 2:])


def test_freqs_rejects_odd_dim():
    with pytest.raises(AssertionError):
        O.precompute_freqs_cis(33, 8, 10000.0)


# -------------------------------------------------------------------------- a2 rotation
def test_rotation_is_complex_multiplication():
    D, N = 64, 96
    x = seeded((2, 3, N, D), 1, torch.float64)
    c, s = O.precompute_freqs_cis(D, N, 10000.0, dtype=torch.float64)
    y = O.apply_rotary_emb(x, c, s)
    z = torch.complex(x[..., :D // 2], x[..., D // 2:]) * torch.complex(c[:, :D // 2], s[:, :D // 2])
    assert torch.allclose(y[..., :D // 2], z.real, atol=1e-12)
    assert torch.allclose(y[..., D // 2:], z.imag, atol=1e-12)
    # pair norms are preserved and -sin undoes the rotation (what the backward relies on)
    n_in = x[..., :D // 2] ** 2 + x[..., D // 2:] ** 2
    n_out = y[..., :D // 2] ** 2 + y[..., D // 2:] ** 2
    assert torch.allclose(n_in, n_out, atol=1e-12)
    assert torch.allclose(O.apply_rotary_emb(y, c, -s), x, atol=1e-6)


def test_rotate_half_sign_and_order():
    x = torch.arange(8.0).view(1, 8)
    assert torch.equal(O.rotate_half(x), torch.tensor([[-4.0, -5, -6, -7, 0, 1, 2, 3]]))


def test_relative_position_property():
    """(R_m q).(R_n k) depends on m-n only: shifting every position leaves O unchanged."""
    B, H, N, D = 1, 2, 48, 32
    q, k, v = (seeded((B, H, N, D), s, torch.float64) for s in (3, 4, 5))
    # fp64 tables (the fp32-angle tables of precompute_freqs_cis would limit this to ~1e-6)
    i = np.arange(D // 2)
    ang = torch.tensor(np.arange(N + 7)[:, None] * 10000.0 ** (-2.0 * i / D)[None, :])
    c = torch.cat([ang.cos(), ang.cos()], -1)
    s = torch.cat([ang.sin(), ang.sin()], -1)
    o0, _, _ = O.rope_attn_forward(q, k, v, True, 0.3, c[:N], s[:N], torch.float64)
    o7, _, _ = O.rope_attn_forward(q, k, v, True, 0.3, c[7:], s[7:], torch.float64)
    assert torch.allclose(o0, o7, atol=1e-10)


# --------------------------------------------------------------------- a3 attention fwd
@pytest.mark.parametrize("causal", [False, True])
def test_identity_rotation_reduces_to_sdpa(causal):
    """cos=1, sin=0 is plain attention -- the reference's own pytest uses this case."""
    B, H, N, D = 2, 3, 64, 32
    q, k, v = (seeded((B, H, N, D), s, torch.float64, 0.5) for s in (20, 21, 22))
    one, zero = torch.ones(N, D, dtype=torch.float64), torch.zeros(N, D, dtype=torch.float64)
    o, lse, _ = O.rope_attn_forward(q, k, v, causal, 0.5, one, zero, torch.float64)
    ref = F.scaled_dot_product_attention(q, k, v, is_causal=causal, scale=0.5)
    assert torch.allclose(o, ref, atol=1e-12)
    sc = (q @ k.transpose(-1, -2)) * 0.5
    if causal:
        sc = sc.masked_fill(torch.triu(torch.ones(N, N, dtype=torch.bool), 1), float("-inf"))
    assert torch.allclose(lse, torch.logsumexp(sc, -1), atol=1e-12)


@pytest.mark.parametrize("causal", [False, True])
def test_rope_path_is_sdpa_of_rotated_inputs(causal):
    B, H, N, D = 1, 2, 80, 64
    q, k, v = (seeded((B, H, N, D), s, torch.float64) for s in (7, 8, 9))
    c, s = O.precompute_freqs_cis(D, N, 10000.0, dtype=torch.float64)
    zq = torch.complex(q[..., :32], q[..., 32:]) * torch.complex(c[:, :32], s[:, :32])
    zk = torch.complex(k[..., :32], k[..., 32:]) * torch.complex(c[:, :32], s[:, :32])
    qr, kr = torch.cat([zq.real, zq.imag], -1), torch.cat([zk.real, zk.imag], -1)
    ref = F.scaled_dot_product_attention(qr, kr, v, is_causal=causal, scale=0.125)
    o, _, _ = O.rope_attn_forward(q, k, v, causal, 0.125, c, s, torch.float64)
    assert torch.allclose(o, ref, atol=1e-12)


@pytest.mark.parametrize("B,H,N,D,causal", [(1, 1, 16, 8, True), (2, 2, 33, 16, True), (1, 2, 24, 8, False)])
def test_forward_vs_brute_force(brute, B, H, N, D, causal):
    q, k, v = (seeded((B, H, N, D), s, torch.float64) for s in (11, 12, 13))
    c, s = O.precompute_freqs_cis(D, N, 10000.0, dtype=torch.float64)
    o, lse, _ = O.rope_attn_forward(q, k, v, causal, 1 / math.sqrt(D), c, s, torch.float64)
    bo, bl = brute.rope_attn(q.numpy(), k.numpy(), v.numpy(), c[:, :D // 2].numpy(), s[:, :D // 2].numpy(),
                             causal, 1 / math.sqrt(D))
    assert np.abs(o.numpy() - bo).max() < 1e-12
    assert np.abs(lse.numpy() - bl).max() < 1e-12


def test_forward_invariants():
    B, H, N, D = 1, 2, 40, 16
    q, k, v = (seeded((B, H, N, D), s) for s in (1, 2, 3))
    c, s = O.precompute_freqs_cis(D, N)
    o, _, (_, _, _, w) = O.rope_attn_forward(q, k, v, True, 0.25, c, s)
    assert torch.allclose(o[:, :, 0], v[:, :, 0], atol=1e-6)          # row 0 attends to key 0 only
    assert torch.allclose(w.sum(-1), torch.ones(B, H, N), atol=1e-6)   # convex combination of V rows
    assert torch.all(w >= 0) and torch.all(torch.triu(w, 1) == 0)


def test_blocked_forms_match_dense():
    B, H, N, D = 2, 2, 96, 32
    q, k, v, g = (seeded((B, H, N, D), s) for s in (1, 2, 3, 4))
    c, s = O.precompute_freqs_cis(D, N)
    o, lse, saved = O.rope_attn_forward(q, k, v, True, 0.2, c, s)
    dq, dk, dv = O.rope_attn_backward(saved, g, True, 0.2, c, s)
    ob, lb = O.rope_attn_forward_blocked(q, k, v, True, 0.2, c, s, row_block=40)
    assert torch.allclose(o, ob, atol=1e-6) and torch.allclose(lse, lb, atol=1e-6)
    rows = torch.tensor([0, 5, 95, 31])
    osub, lsub = O.rope_attn_forward_blocked(q, k, v, True, 0.2, c, s, rows=rows)
    assert torch.allclose(o[:, :, rows], osub, atol=1e-6) and torch.allclose(lse[:, :, rows], lsub, atol=1e-6)
    o2, l2, dq2, dk2, dv2, delta = O.rope_attn_fwd_bwd_blocked(q, k, v, g, True, 0.2, c, s)
    for a, b in ((o, o2), (lse, l2), (dq, dq2), (dk, dk2), (dv, dv2)):
        assert torch.allclose(a, b, atol=1e-6)
    assert torch.allclose(delta, (o * g).sum(-1), atol=1e-6)


# --------------------------------------------------------------------- a4 attention bwd
@pytest.mark.parametrize("causal", [False, True])
def test_backward_vs_autograd(causal):
    B, H, N, D = 2, 2, 48, 32
    q, k, v = (seeded((B, H, N, D), s, torch.float64).requires_grad_(True) for s in (1, 2, 3))
    g = seeded((B, H, N, D), 4, torch.float64)
    c, s = O.precompute_freqs_cis(D, N, dtype=torch.float64)
    # independent forward for autograd: rotation as complex product + library SDPA
    h = D // 2
    rot = torch.complex(c[:, :h], s[:, :h])
    zq = torch.complex(q[..., :h], q[..., h:]) * rot
    zk = torch.complex(k[..., :h], k[..., h:]) * rot
    ref = F.scaled_dot_product_attention(torch.cat([zq.real, zq.imag], -1), torch.cat([zk.real, zk.imag], -1), v,
                                         is_causal=causal, scale=0.3)
    rq, rk, rv = torch.autograd.grad(ref, (q, k, v), g)
    _, _, saved = O.rope_attn_forward(q.detach(), k.detach(), v.detach(), causal, 0.3, c, s, torch.float64)
    dq, dk, dv = O.rope_attn_backward(saved, g, causal, 0.3, c, s)
    assert torch.allclose(dq, rq, atol=1e-11) and torch.allclose(dk, rk, atol=1e-11)
    assert torch.allclose(dv, rv, atol=1e-11)


def test_function_twin_gradcheck_and_signature():
    B, H, N, D = 1, 1, 6, 4
    q, k, v = (seeded((B, H, N, D), s, torch.float64).requires_grad_(True) for s in (5, 6, 7))
    c, s = O.precompute_freqs_cis(D, N, dtype=torch.float64)
    assert torch.autograd.gradcheck(lambda a, b, d: O.attention_pytorch(a, b, d, True, 0.5, c, s), (q, k, v),
                                    eps=1e-6, atol=1e-6)
    out = O.attention_pytorch(q, k, v, True, 0.5, c, s)
    grads = torch.autograd.grad(out.sum(), (q, k, v))
    assert all(t.shape == (B, H, N, D) for t in grads)


def test_delta_identity():
    """rowsum(P * dP) == rowsum(O * dO): ties the preprocess pass to the dense softmax backward."""
    B, H, N, D = 1, 2, 32, 16
    q, k, v, g = (seeded((B, H, N, D), s, torch.float64) for s in (1, 2, 3, 4))
    c, s = O.precompute_freqs_cis(D, N, dtype=torch.float64)
    o, _, (_, _, _, w) = O.rope_attn_forward(q, k, v, True, 0.25, c, s, torch.float64)
    dP = torch.einsum("bhqd,bhkd->bhqk", g, v)
    assert torch.allclose((w * dP).sum(-1), (o * g).sum(-1), atol=1e-12)


def test_flop_model():
    # figures quoted for the benchmark shapes: 4*B*H*N^2*D, halved when causal, x2.5 backward
    assert O.attention_flops(2, 32, 4096, 128, "fwd", True) == pytest.approx(2.749e11, rel=1e-3)
    assert O.attention_flops(2, 32, 4096, 128, "bwd", True) == pytest.approx(6.872e11, rel=1e-3)
    assert O.attention_flops(4, 8, 512, 64, "fwd", True) == pytest.approx(1.074e9, rel=1e-3)
