"""Pins for the Co-RoPE GQA oracle (CPU only): brute force, the zero-leader bridge to the
RoPE-attention oracle, head bookkeeping, mileage invariants and autograd."""
import math

import numpy as np
import pytest
import torch

from conftest import seeded
from oracle import corope_gqa_oracle as C
from oracle import rope_attn_oracle as R


# tiny shapes the reference's own scripts use: compare_corope.py:152 and corope_attn_gqa_pytorch.py:309-321
@pytest.mark.parametrize("B,Hq,Hkv,N,D,scale", [(1, 4, 2, 32, 64, 1.0), (2, 4, 2, 64, 32, 32 ** -0.5), (1, 3, 3, 20, 8, 0.5),
                                              (1, 6, 2, 17, 16, 0.25)])
def test_forward_vs_brute_force(brute, B, Hq, Hkv, N, D, scale):
    q = seeded((B, Hq, N, D), 42, torch.float64)
    k = seeded((B, Hkv, N, D), 43, torch.float64)
    v = seeded((B, Hkv, N, D), 44, torch.float64)
    w = C.corope_inv_freq(D, 10000.0, dtype=torch.float64)
    o, aux = C.corope_gqa_forward(q, k, v, True, scale, 10000.0, torch.float64, return_aux=True)
    bo, bdelta = brute.corope(q.numpy(), k.numpy(), v.numpy(), w.numpy(), scale, want_delta=True)
    assert np.abs(o.numpy() - bo).max() < 1e-10
    G = Hq // Hkv
    tri = np.tril(np.ones((N, N), dtype=bool))
    d_or = aux["delta"][:, ::G].numpy()
    assert np.abs(np.where(tri, d_or - bdelta, 0)).max() < 1e-10


def test_inv_freq_closed_form():
    w = C.corope_inv_freq(128, 10000.0)
    ref = 10000.0 ** (-2.0 * np.arange(64) / 128)
    assert np.abs(w.numpy() / ref - 1).max() < 1e-6 and w[0] == 1.0


def test_zero_leader_reduces_to_rope_attention():
    """q_leader = 0 -> every gate is 1/2 -> delta_ij = (i-j)/2 -> the other heads of the group are ordinary
    RoPE attention at positions m/2, and the leader itself (all scores 0) is the causal running mean of V."""
    B, Hq, Hkv, N, D = 1, 4, 2, 40, 32
    G = Hq // Hkv
    q = seeded((B, Hq, N, D), 1, torch.float64)
    k = seeded((B, Hkv, N, D), 2, torch.float64)
    v = seeded((B, Hkv, N, D), 3, torch.float64)
    q[:, ::G] = 0
    o = C.corope_gqa_forward(q, k, v, True, 0.3, 10000.0, torch.float64)
    w = C.corope_inv_freq(D, 10000.0, dtype=torch.float64)
    ang = (torch.arange(N, dtype=torch.float64) / 2).unsqueeze(1) * w.unsqueeze(0)
    cos, sin = torch.cat([ang.cos()] * 2, -1), torch.cat([ang.sin()] * 2, -1)
    kx, vx = k.repeat_interleave(G, 1), v.repeat_interleave(G, 1)
    ref, _, _ = R.rope_attn_forward(q, kx, vx, True, 0.3, cos, sin, torch.float64)
    followers = [h for h in range(Hq) if h % G]
    assert torch.allclose(o[:, followers], ref[:, followers], atol=1e-10)
    run_mean = torch.cumsum(vx, 2) / torch.arange(1, N + 1, dtype=torch.float64).view(1, 1, N, 1)
    assert torch.allclose(o[:, ::G], run_mean[:, ::G], atol=1e-12)


def test_group_bookkeeping():
    """With G=1 every head is its own leader; a G=2 call must equal the G=1 call on explicitly expanded K/V whenever
    the two heads of a group carry the same queries (then follower == leader)."""
    B, Hkv, N, D = 1, 2, 24, 16
    qh = seeded((B, Hkv, N, D), 5, torch.float64)
    k = seeded((B, Hkv, N, D), 6, torch.float64)
    v = seeded((B, Hkv, N, D), 7, torch.float64)
    o1 = C.corope_gqa_forward(qh, k, v, True, 0.4, 10000.0, torch.float64)
    q2 = qh.repeat_interleave(2, 1)
    o2 = C.corope_gqa_forward(q2, k, v, True, 0.4, 10000.0, torch.float64)
    assert torch.allclose(o2[:, 0::2], o1, atol=1e-12) and torch.allclose(o2[:, 1::2], o1, atol=1e-12)
    # a follower's output must change with the leader's queries but not with another group's
    q3 = q2.clone(); q3[:, 2] += 1.0
    o3 = C.corope_gqa_forward(q3, k, v, True, 0.4, 10000.0, torch.float64)
    assert torch.allclose(o3[:, :2], o2[:, :2], atol=1e-12) and not torch.allclose(o3[:, 3], o2[:, 3], atol=1e-6)


def test_mileage_invariants():
    B, Hq, Hkv, N, D = 1, 4, 2, 48, 16
    q, k, v = seeded((B, Hq, N, D), 1), seeded((B, Hkv, N, D), 2), seeded((B, Hkv, N, D), 3)
    o, aux = C.corope_gqa_forward(q, k, v, True, 0.25, 10000.0, torch.float64, return_aux=True)
    d = aux["delta"]
    i = torch.arange(N)
    assert torch.all(torch.diagonal(d, dim1=-2, dim2=-1).abs() < 1e-12)
    low = torch.tril(torch.ones(N, N, dtype=torch.bool))
    gap = (i[:, None] - i[None, :]).double()
    assert torch.all(d[..., low] >= -1e-12) and torch.all((d <= gap + 1e-12)[..., low])
    step = d[..., :, :-1] - d[..., :, 1:]                    # non-increasing in j inside the causal region
    assert torch.all(step[..., low[:, 1:]] >= -1e-12)
    assert torch.allclose(o[:, :, 0], v.repeat_interleave(2, 1)[:, :, 0].double(), atol=1e-12)
    assert torch.allclose(aux["weights"].sum(-1), torch.ones(B, Hq, N, dtype=torch.float64), atol=1e-12)


def test_rows_form_matches_dense():
    B, Hq, Hkv, N, D = 2, 4, 2, 40, 16
    q, k, v = seeded((B, Hq, N, D), 1), seeded((B, Hkv, N, D), 2), seeded((B, Hkv, N, D), 3)
    o = C.corope_gqa_forward(q, k, v, True, 0.25, 10000.0)
    rows = torch.tensor([0, 1, 17, 39])
    sub = C.corope_gqa_forward_rows(q, k, v, True, 0.25, 10000.0, rows, row_block=3)
    assert torch.allclose(o[:, :, rows], sub, atol=2e-6)


def test_validation_errors():
    q, k = torch.zeros(1, 4, 8, 8), torch.zeros(1, 2, 8, 8)
    with pytest.raises(ValueError):
        C.corope_gqa_forward(q, k, k, False, 1.0, 1e4)
    with pytest.raises(ValueError):
        C.corope_gqa_forward(q, torch.zeros(1, 3, 8, 8), torch.zeros(1, 3, 8, 8), True, 1.0, 1e4)
    with pytest.raises(ValueError):
        C.corope_gqa_forward(q, k, torch.zeros(1, 2, 8, 4), True, 1.0, 1e4)
    with pytest.raises(ValueError):
        C.corope_gqa_forward(q[0], k[0], k[0], True, 1.0, 1e4)


def test_function_twin_backward_is_autograd():
    B, Hq, Hkv, N, D = 1, 2, 1, 6, 4
    q = seeded((B, Hq, N, D), 1, torch.float64).requires_grad_(True)
    k = seeded((B, Hkv, N, D), 2, torch.float64).requires_grad_(True)
    v = seeded((B, Hkv, N, D), 3, torch.float64).requires_grad_(True)
    assert torch.autograd.gradcheck(lambda a, b, c: C.attention_pytorch(a, b, c, True, 0.5, 100.0), (q, k, v),
                                    eps=1e-6, atol=1e-6)


@pytest.mark.parametrize("B,Hq,Hkv,N,D,scale,theta", [(1, 4, 2, 24, 16, 0.5, 100.0), (2, 3, 1, 17, 8, 1.0, 10.0),
                                                     (1, 2, 2, 33, 32, 32 ** -0.5, 10000.0)])
def test_closed_form_backward_matches_autograd(B, Hq, Hkv, N, D, scale, theta):
    """The decomposition the GPU backward uses (rotated key / rotated query sums, the running sum of G over the keys for the
    gate path) against autograd through the pinned dense forward, in fp64."""
    g = torch.Generator().manual_seed(11)
    q = torch.randn(B, Hq, N, D, generator=g, dtype=torch.float64)
    k, v = (torch.randn(B, Hkv, N, D, generator=g, dtype=torch.float64) for _ in range(2))
    go = torch.randn(B, Hq, N, D, generator=g, dtype=torch.float64)
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    ref = torch.autograd.grad(C.corope_gqa_forward(qa, ka, va, True, scale, theta, torch.float64), (qa, ka, va), go)
    got = C.corope_gqa_backward_manual(q, k, v, go, scale, theta)
    for name, a, b in zip(("dq", "dk", "dv"), got, ref):
        assert (a - b).abs().max() <= 1e-10 * max(1.0, b.abs().max()), name
