"""GPU parity of the Co-RoPE GQA backward against autograd through the dense CPU oracle (through the C ABI).

The oracle's gradients come from torch.autograd over its dense fp64 forward, which is how the reference checks its
own manual backward (corope-exp/corope_attn_gqa_pytorch.py:326-355).  Bar: max-abs <= 2e-2 for the bf16 gradients,
scaled by sqrt(G) for dK and dV, which sum G heads' contributions before the one rounding."""
import math

import pytest
import torch

from conftest import bf16_round, seeded
from oracle import corope_gqa_oracle as C

pytestmark = pytest.mark.gpu
TOL = 2e-2


def _inputs(B, Hq, Hkv, N, D, seed=42):
    return (bf16_round(seeded((B, Hq, N, D), seed)), bf16_round(seeded((B, Hkv, N, D), seed + 1)),
            bf16_round(seeded((B, Hkv, N, D), seed + 2)), bf16_round(seeded((B, Hq, N, D), seed + 3)))


def _oracle_grads(q, k, v, d_o, scale, theta):
    cd = torch.float64 if q.shape[2] <= 160 else torch.float32   # the dense form holds (B, Hq, N, N, D/2) temporaries
    q, k, v = (t.to(cd).clone().requires_grad_(True) for t in (q, k, v))   # (.to is a no-op for fp32 inputs: never mark the caller's tensor)
    o = C.corope_gqa_forward(q, k, v, True, scale, theta, cd)
    return [g.float() for g in torch.autograd.grad(o, (q, k, v), d_o.to(cd))]


def _gpu_grads(pkg, q, k, v, d_o, scale, theta):
    dev = torch.device("cuda:0")
    qg, kg, vg = (t.to(dev, torch.bfloat16).requires_grad_(True) for t in (q, k, v))
    o = pkg.corope_attention(qg, kg, vg, True, scale, theta)
    o.backward(d_o.to(dev, torch.bfloat16))
    torch.cuda.synchronize()
    return [t.grad.float().cpu() for t in (qg, kg, vg)]


def _compare(got, ref, G):
    for name, a, b, bar in zip(("dQ", "dK", "dV"), got, ref, (TOL, TOL * math.sqrt(G), TOL * math.sqrt(G))):
        err = (a - b).abs()
        print(f"  {name} max-abs {err.max():.3e} mean-abs {err.mean():.3e} (max |ref| {b.abs().max():.3f})", flush=True)
        assert torch.isfinite(a).all()
        assert err.max() <= bar, name


# (B, Hq, Hkv, N, D): every group size, ragged lengths around the 16/32/64 tile edges, both head dims
CASES = [(1, 4, 2, 32, 64), (2, 4, 2, 64, 64), (1, 2, 2, 96, 64), (1, 6, 2, 100, 64), (1, 8, 2, 130, 128),
         (1, 8, 1, 150, 64), (2, 5, 1, 77, 128), (1, 3, 1, 64, 128), (1, 7, 1, 65, 64), (1, 4, 1, 1, 64),
         (1, 1, 1, 33, 128), (1, 4, 2, 384, 64), (1, 4, 1, 449, 128), (1, 8, 1, 100, 128), (1, 7, 1, 70, 128),
         # head dims below the kernels' own run padded to 64 (32 is the shape of the reference's self-check,
         # corope_attn_gqa_pytorch.py:309-321)
         (2, 4, 2, 64, 32), (1, 6, 3, 130, 32), (1, 4, 1, 77, 16)]


@pytest.mark.parametrize("B,Hq,Hkv,N,D", CASES)
def test_corope_backward_parity(pkg, B, Hq, Hkv, N, D):
    print(f"case B={B} Hq={Hq} Hkv={Hkv} N={N} D={D}", flush=True)
    q, k, v, d_o = _inputs(B, Hq, Hkv, N, D)
    scale = 1 / math.sqrt(D)
    _compare(_gpu_grads(pkg, q, k, v, d_o, scale, 10000.0), _oracle_grads(q, k, v, d_o, scale, 10000.0), Hq // Hkv)


def test_corope_backward_unit_scale_small_theta(pkg):
    """sm_scale = 1 and a small base: fast rotations make the path through the gates a large part of dQ and dK.
    dO is halved so that the gradients stay below 4, where half a bf16 step of the result alone is under 8e-3."""
    q, k, v, d_o = _inputs(1, 4, 2, 48, 64, seed=7)
    q, k, d_o = bf16_round(q * 0.3), bf16_round(k * 0.3), d_o * 0.5
    _compare(_gpu_grads(pkg, q, k, v, d_o, 1.0, 100.0), _oracle_grads(q, k, v, d_o, 1.0, 100.0), 2)


def test_corope_backward_hot_softmax(pkg):
    """sm_scale = 1 on unit-variance inputs (the reference's comparison script, compare_corope.py:23): scores of +-20, rows
    dominated by one or two keys.  dO is scaled down so that the gradients stay of order one; the bar is the usual one."""
    q, k, v, d_o = _inputs(1, 4, 2, 64, 64, seed=21)
    d_o = bf16_round(d_o * 0.125)
    _compare(_gpu_grads(pkg, q, k, v, d_o, 1.0, 10000.0), _oracle_grads(q, k, v, d_o, 1.0, 10000.0), 2)


@pytest.mark.parametrize("trend", ["growing", "shrinking"])
def test_corope_score_trend_along_the_sweep(pkg, trend):
    """The kernels sweep a row's keys from the diagonal towards key 0 and move the reference value of their exponentials
    only when a score rises well above it.  Key norms that grow (resp. shrink) towards key 0 make the scores rise chunk
    after chunk (the reference moves again and again) or fall away (it stays at the first chunk's maximum while the
    weights become tiny): forward and all gradients against the oracle in both regimes."""
    B, Hq, Hkv, N, D = 1, 4, 2, 320, 64
    q, k, v, d_o = _inputs(B, Hq, Hkv, N, D, seed=33)
    ramp = torch.linspace(3.0, 0.5, N) if trend == "growing" else torch.linspace(0.3, 2.0, N)
    k = bf16_round(k * ramp[None, None, :, None])
    d_o = bf16_round(d_o * 0.25)
    scale = 1 / math.sqrt(D)
    print(f"case trend={trend}", flush=True)
    dev = torch.device("cuda:0")
    o = pkg.corope_attention(*(t.to(dev, torch.bfloat16) for t in (q, k, v)), True, scale, 10000.0).float().cpu()
    ro = C.corope_gqa_forward(q.double(), k.double(), v.double(), True, scale, 10000.0, torch.float64).float()
    print(f"  O max-abs {(o - ro).abs().max():.3e}", flush=True)
    assert torch.isfinite(o).all() and (o - ro).abs().max() <= TOL
    _compare(_gpu_grads(pkg, q, k, v, d_o, scale, 10000.0), _oracle_grads(q, k, v, d_o, scale, 10000.0), Hq // Hkv)


def test_corope_backward_gate_path_is_material_and_right(pkg):
    """On this input the gradient through the leader's gates is a large part of dQ and dK (the oracle with the
    position offsets cut out of the graph differs by far more than the bar), so parity here pins that path; a
    central finite difference through the dense forward pins the oracle's own gradient for one leader coordinate."""
    q, k, v, d_o = _inputs(1, 4, 2, 48, 64, seed=7)
    q, k, d_o = bf16_round(q * 0.3), bf16_round(k * 0.3), d_o * 0.5
    full = _oracle_grads(q, k, v, d_o, 1.0, 100.0)
    qd, kd, vd = (t.double().requires_grad_(True) for t in (q, k, v))
    o = C.corope_gqa_forward(qd, kd, vd, True, 1.0, 100.0, torch.float64, detach_gates=True)
    cut = [g.float() for g in torch.autograd.grad(o, (qd, kd, vd), d_o.double())]
    assert (full[0] - cut[0]).abs().max() > 10 * TOL and (full[1] - cut[1]).abs().max() > 10 * TOL
    assert torch.equal(full[0][:, 1::2], cut[0][:, 1::2])   # only the leaders' queries feed the gates
    got = _gpu_grads(pkg, q, k, v, d_o, 1.0, 100.0)
    _compare(got, full, 2)
    eps, idx = 1e-4, (0, 0, 40, 5)
    qp, qm = q.double(), q.double()
    qp[idx] += eps
    qm[idx] -= eps

    def loss(qq):
        return (C.corope_gqa_forward(qq, k.double(), v.double(), True, 1.0, 100.0, torch.float64) * d_o.double()).sum()

    fd = float((loss(qp) - loss(qm)) / (2 * eps))
    print(f"  finite difference {fd:.5f}, autograd {float(full[0][idx]):.5f}, gpu {float(got[0][idx]):.5f}")
    assert abs(fd - float(full[0][idx])) <= 1e-5 * max(1.0, abs(fd))
    assert abs(fd - float(got[0][idx])) <= TOL


def test_corope_backward_caller_workspace_and_reuse(pkg):
    """A caller-owned workspace filled with garbage gives the same gradients, whether it holds every group's matrices
    (one pass), some of them (the groups are walked in passes of as many as fit) or a single group's; one that cannot
    hold a single group's is refused."""
    mod = pkg.corope_gqa
    dev = torch.device("cuda:0")
    B, Hq, Hkv, N, D = 2, 6, 3, 70, 64
    q, k, v, d_o = (t.to(dev, torch.bfloat16) for t in _inputs(B, Hq, Hkv, N, D, seed=3))
    need = mod.backward_workspace_bytes(B, Hq, Hkv, N, D)
    packed = sum(64 * (i // 64 + 1) for i in range(N))          # rows hold the keys j <= i, padded to 64-key chunks
    assert need == 4 * (packed * (2 * B * Hkv + 3 * B * Hq) + B * Hkv * N * D)   # + the leader's fp32 dq rows
    a = mod.corope_gqa_backward(q, k, v, d_o, 0.125, 1e4)
    ws = torch.full((need // 4 + 64,), float("nan"), device=dev)
    b = mod.corope_gqa_backward(q, k, v, d_o, 0.125, 1e4, workspace=ws)
    torch.cuda.synchronize()
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    one = mod.backward_min_workspace_bytes(B, Hq, Hkv, N, D)
    assert one * B * Hkv == need
    for groups in (1, 2, 4):              # 6 groups in passes of 1, of 2, and of 4 + 2
        ws.fill_(float("nan"))
        c = mod.corope_gqa_backward(q, k, v, d_o, 0.125, 1e4, workspace=ws[: groups * one // 4 + 3])
        torch.cuda.synchronize()
        for x, y in zip(a, c):
            assert torch.equal(x, y), groups
    with pytest.raises(ValueError):
        mod.corope_gqa_backward(q, k, v, d_o, 0.125, 1e4, workspace=ws[: one // 4 - 1])


def test_corope_backward_keeps_its_own_workspace_between_calls(pkg, monkeypatch):
    """Without a caller's workspace the operator uses one buffer per device and stream, sized by the shape and a cap alone: the second
    call allocates nothing new, a smaller cap walks the groups in passes with the same gradients, release frees it."""
    mod = pkg.corope_gqa
    dev = torch.device("cuda:0")
    B, Hq, Hkv, N, D = 2, 6, 3, 70, 64
    q, k, v, d_o = (t.to(dev, torch.bfloat16) for t in _inputs(B, Hq, Hkv, N, D, seed=5))
    mod.release_backward_workspace()
    key = (dev.index, torch.cuda.current_stream(dev).cuda_stream)
    a = mod.corope_gqa_backward(q, k, v, d_o, 0.125, 1e4)
    ws = mod._workspaces[key]
    assert ws.numel() == mod.backward_workspace_bytes(B, Hq, Hkv, N, D)
    b = mod.corope_gqa_backward(q, k, v, d_o, 0.125, 1e4)
    assert mod._workspaces[key].data_ptr() == ws.data_ptr() and len(mod._workspaces) == 1
    one = mod.backward_min_workspace_bytes(B, Hq, Hkv, N, D)
    mod.release_backward_workspace(dev)
    assert not mod._workspaces
    monkeypatch.setattr(mod, "BACKWARD_WORKSPACE_CAP_BYTES", 2 * one + 5)
    c = mod.corope_gqa_backward(q, k, v, d_o, 0.125, 1e4)
    assert mod._workspaces[key].numel() == 2 * one
    torch.cuda.synchronize()
    for x, y, z in zip(a, b, c):
        assert torch.equal(x, y) and torch.equal(x, z)
    mod.release_backward_workspace()


def test_corope_random_shapes_forward_and_backward(pkg):
    """A seeded sweep over batch, group size, head dim, ragged lengths, temperature and rotation base: forward and
    backward in one go, each tensor against the dense oracle with the bar of conftest.within_bar (2e-2, or one bf16 step
    of the value where it exceeds 2.56; dK and dV scaled by sqrt(G) as above)."""
    import random
    from conftest import within_bar
    rnd = random.Random(5)
    dev = torch.device("cuda:0")
    for case in range(16):
        B, Hkv, G, D = rnd.choice([1, 2]), rnd.choice([1, 2, 3]), rnd.randint(1, 8), rnd.choice([64, 128])
        N = rnd.choice([1, 2, 31, 63, 64, 65, 100, 127, 128, 129, 190])
        scale, theta = rnd.choice([1 / math.sqrt(D), 0.25, 0.05]), rnd.choice([100.0, 10000.0, 500000.0])
        Hq = Hkv * G
        print(f"case {case}: B={B} Hq={Hq} Hkv={Hkv} N={N} D={D} scale={scale:.3f} theta={theta}", flush=True)
        q, k, v, d_o = _inputs(B, Hq, Hkv, N, D, seed=1000 + 4 * case)
        d_o = bf16_round(d_o * 0.5)
        cd = torch.float64 if N <= 130 else torch.float32
        qr, kr, vr = (t.to(cd).clone().requires_grad_(True) for t in (q, k, v))
        o_ref = C.corope_gqa_forward(qr, kr, vr, True, scale, theta, cd)
        g_ref = torch.autograd.grad(o_ref, (qr, kr, vr), d_o.to(cd))
        qg, kg, vg = (t.to(dev, torch.bfloat16).requires_grad_(True) for t in (q, k, v))
        o = pkg.corope_attention(qg, kg, vg, True, scale, theta)
        o.backward(d_o.to(dev, torch.bfloat16))
        torch.cuda.synchronize()
        checks = [("O", o.detach(), o_ref.detach(), TOL)]
        checks += [(n, t.grad, r, TOL * (1.0 if n == "dQ" else math.sqrt(G))) for n, t, r in zip(("dQ", "dK", "dV"), (qg, kg, vg), g_ref)]
        for name, got, ref, tol in checks:
            ok, err = within_bar(got.float().cpu(), ref.float(), tol)
            assert torch.isfinite(got).all() and ok, (case, name, err)


@pytest.mark.parametrize("with_o", [True, False])
@pytest.mark.parametrize("B,Hq,Hkv,N,D", [(1, 4, 2, 130, 64), (1, 8, 2, 100, 128)])
def test_corope_backward_does_not_depend_on_the_scale_of_dO(pkg, B, Hq, Hkv, N, D, with_o):
    """Upstream gradients of a mean-reduced loss (1e-6 and below) and unnormalised ones (1e3): the backward is linear in
    dO, and a power-of-two factor commutes with every rounding in it (the fp16 weights of the dQ sums are normalised per
    row by a power of two of |dO_i|), so grad(2^k dO) == 2^k grad(dO) bit for bit -- and both match the oracle."""
    mod = pkg.corope_gqa
    dev = torch.device("cuda:0")
    q, k, v, d_o = _inputs(B, Hq, Hkv, N, D, seed=11)
    scale = 1 / math.sqrt(D)
    qd, kd, vd, gd = (t.to(dev, torch.bfloat16) for t in (q, k, v, d_o))
    out = pkg.corope_attention(qd, kd, vd, True, scale, 10000.0) if with_o else None
    base = [t.float().cpu() for t in mod.corope_gqa_backward(qd, kd, vd, gd, scale, 10000.0, out=out)]
    _compare(base, _oracle_grads(q, k, v, d_o, scale, 10000.0), Hq // Hkv)
    for kexp in (-24, -20, 10, 14):      # 6e-8, 1e-6, 1e3, 1.6e4
        f = 2.0 ** kexp
        got = [t.float().cpu() for t in mod.corope_gqa_backward(qd, kd, vd, (gd.float() * f).to(torch.bfloat16), scale, 10000.0,
                                                                  out=out)]
        torch.cuda.synchronize()
        for name, a, b in zip(("dQ", "dK", "dV"), got, base):
            assert torch.isfinite(a).all(), (name, kexp)
            assert torch.equal(a, b * f), f"{name} at dO x 2^{kexp}: max rel diff {((a - b * f).abs() / (b.abs() * f + 1e-30)).max():.3e}"


def _f16_round(x):
    return x.to(torch.float16).float()


@pytest.mark.parametrize("B,Hq,Hkv,N,D", [(1, 4, 2, 32, 64), (1, 6, 2, 100, 64), (1, 8, 2, 130, 128), (2, 5, 1, 77, 128),
                                           (1, 4, 1, 449, 128), (2, 4, 2, 64, 32)])
def test_corope_backward_parity_fp16(pkg, B, Hq, Hkv, N, D):
    """fp16 tensors, the dtype of the reference's callers (corope-exp/compare_corope.py:18), forward and backward: the same
    kernels built for fp16 elements, against the oracle on the fp16-rounded inputs, at the bf16 bar (fp16 carries three
    mantissa bits more)."""
    print(f"case fp16 B={B} Hq={Hq} Hkv={Hkv} N={N} D={D}", flush=True)
    q, k, v, d_o = (_f16_round(t) for t in _inputs(B, Hq, Hkv, N, D, seed=11))
    scale = 1 / math.sqrt(D)
    dev = torch.device("cuda:0")
    qg, kg, vg = (t.to(dev, torch.float16).requires_grad_(True) for t in (q, k, v))
    o = pkg.corope_attention(qg, kg, vg, True, scale, 10000.0)
    o.backward(d_o.to(dev, torch.float16))
    torch.cuda.synchronize()
    assert all(t.grad.dtype == torch.float16 for t in (qg, kg, vg))
    ro = C.corope_gqa_forward(q.double(), k.double(), v.double(), True, scale, 10000.0, torch.float64).float()
    print(f"  O max-abs {(o.float().cpu() - ro).abs().max():.3e}", flush=True)
    assert (o.float().cpu() - ro).abs().max() <= TOL
    _compare([t.grad.float().cpu() for t in (qg, kg, vg)], _oracle_grads(q, k, v, d_o, scale, 10000.0), Hq // Hkv)


@pytest.mark.parametrize("kexp", [-8, 5])
def test_corope_backward_fp16_scaled_upstream_gradient(pkg, kexp):
    """fp16 tensors with an upstream gradient of 2^-8 and 2^5 times unit size (fp16's own range leaves room for little
    more): the gradients stay finite and match the oracle at the bar scaled by the same factor."""
    B, Hq, Hkv, N, D = 1, 4, 2, 130, 64
    f = 2.0 ** kexp
    q, k, v, d_o = (_f16_round(t) for t in _inputs(B, Hq, Hkv, N, D, seed=11))
    d_o = _f16_round(d_o * f)
    scale = 1 / math.sqrt(D)
    dev = torch.device("cuda:0")
    qg, kg, vg = (t.to(dev, torch.float16).requires_grad_(True) for t in (q, k, v))
    pkg.corope_attention(qg, kg, vg, True, scale, 10000.0).backward(d_o.to(dev, torch.float16))
    torch.cuda.synchronize()
    ref = _oracle_grads(q, k, v, d_o, scale, 10000.0)
    G = Hq // Hkv
    for name, t, b, bar in zip(("dQ", "dK", "dV"), (qg, kg, vg), ref, (TOL, TOL * math.sqrt(G), TOL * math.sqrt(G))):
        a = t.grad.float().cpu()
        err = (a - b).abs().max()
        print(f"  {name} at dO x 2^{kexp}: max-abs {err:.3e} (bar {bar * f:.3e}, max |ref| {b.abs().max():.3e})", flush=True)
        assert torch.isfinite(a).all() and err <= bar * f, name


def test_corope_more_heads_than_a_grid_axis(pkg):
    """B8200 Hq8 Hkv1 N16 D64: 65600 query heads, more than the 65535 a grid axis holds; the backward walks the groups in
    passes.  The first and the last group against the same groups run on their own."""
    mod = pkg.corope_gqa
    dev = torch.device("cuda:0")
    B, Hq, Hkv, N, D = 8200, 8, 1, 16, 64
    g = torch.Generator(device=dev).manual_seed(3)
    q, d_o = (torch.randn((B, Hq, N, D), device=dev, dtype=torch.bfloat16, generator=g) for _ in range(2))
    k, v = (torch.randn((B, Hkv, N, D), device=dev, dtype=torch.bfloat16, generator=g) for _ in range(2))
    o = pkg.corope_attention(q, k, v, True, 0.125, 1e4)
    grads = mod.corope_gqa_backward(q, k, v, d_o, 0.125, 1e4)
    torch.cuda.synchronize()
    for b in (0, 4100, B - 1):
        sl = slice(b, b + 1)
        o1 = pkg.corope_attention(q[sl], k[sl], v[sl], True, 0.125, 1e4)
        g1 = mod.corope_gqa_backward(q[sl], k[sl], v[sl], d_o[sl], 0.125, 1e4)
        torch.cuda.synchronize()
        assert torch.equal(o[sl], o1), b
        for a, r in zip(grads, g1):
            assert torch.equal(a[sl], r), b
    mod.release_backward_workspace()
