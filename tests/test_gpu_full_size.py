"""Parity at the benchmark's full sizes (C3, C4, C5), checked on sampled query rows (attention rows are independent
given K and V), on whole heads for the gradients, and through size-independent properties."""
import math

import pytest
import torch

from conftest import bf16_round, seeded, within_bar
from oracle import corope_gqa_oracle as C
from oracle import rope_attn_oracle as O

pytestmark = pytest.mark.gpu
TOL = 2e-2
LN2 = math.log(2.0)


def _rows(N, n, seed):
    g = torch.Generator().manual_seed(seed)
    r = torch.randperm(N, generator=g)[:n]
    return torch.unique(torch.cat([r, torch.tensor([0, 1, 63, 64, N // 2, N - 2, N - 1])]))


def test_c3_forward_backward(pkg):
    """B2 H32 N4096 D128 causal: O/LSE on sampled rows of every head; dQ/dK/dV on eight whole heads and, for dV, through a
    sum identity on all 64."""
    B, H, N, D = 2, 32, 4096, 128
    dev = torch.device("cuda:0")
    q, k, v, g = (bf16_round(seeded((B, H, N, D), 42 + i)) for i in range(4))
    c, s = O.precompute_freqs_cis(D, N)
    scale = 1 / math.sqrt(D)
    qd, kd, vd = (t.to(dev, torch.bfloat16).requires_grad_(True) for t in (q, k, v))
    o, M = pkg.rope_attn_forward_with_lse(qd.detach(), kd.detach(), vd.detach(), True, scale, c.to(dev), s.to(dev))
    out = pkg.attention(qd, kd, vd, True, scale, c.to(dev), s.to(dev))
    out.backward(g.to(dev, torch.bfloat16))
    torch.cuda.synchronize()
    assert torch.equal(out.detach(), o)
    o, M = o.float().cpu(), M.cpu()
    rows = _rows(N, 96, 1)
    ro, rl = O.rope_attn_forward_blocked(q, k, v, True, scale, c, s, rows=rows)
    e_o, e_l = (o[:, :, rows] - ro).abs().max().item(), (M[:, :, rows] * LN2 - rl).abs().max().item()
    print(f"  C3 O max-abs {e_o:.3e}, LSE max-abs {e_l:.3e} on {rows.numel()} rows x {B * H} heads", flush=True)
    assert e_o <= TOL and e_l <= TOL
    assert torch.equal(o[:, :, 0], v[:, :, 0])                                   # row 0 attends to key 0 only
    dq, dk, dv = (t.grad.float().cpu() for t in (qd, kd, vd))
    # every head: the key-wise sum of dV is the query-wise sum of dO (the rows of P sum to one), so a key block that was
    # skipped, done twice or given another head's operands shows in its head's sum
    colsum_err = (dv.sum(2) - g.sum(2)).abs().max().item()
    print(f"  C3 sum_j dV_j against sum_i dO_i over all {B * H} heads: max-abs {colsum_err:.3e}", flush=True)
    assert colsum_err <= 0.25       # 4096 bf16-rounded rows of magnitude ~0.1-1 per sum
    # whole heads against the oracle: eight of them, one per residue of the head index modulo 8 that the workgroups'
    # item lists are dealt by
    for (b, h) in ((0, 0), (0, 9), (0, 18), (0, 27), (1, 4), (1, 13), (1, 22), (1, 31)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        _, _, rdq, rdk, rdv, _ = O.rope_attn_fwd_bwd_blocked(q[sl], k[sl], v[sl], g[sl], True, scale, c, s)
        for name, a, r in (("dQ", dq[sl], rdq), ("dK", dk[sl], rdk), ("dV", dv[sl], rdv)):
            err = (a - r).abs()
            print(f"  C3 head ({b},{h}) {name}: max-abs {err.max():.3e} mean-abs {err.mean():.3e}", flush=True)
            assert within_bar(a, r, TOL)[0], name
    # linearity of the backward in dO: grad(2 dO) == 2 grad(dO) exactly (power-of-two scaling commutes with rounding)
    qd.grad = kd.grad = vd.grad = None
    out2 = pkg.attention(qd, kd, vd, True, scale, c.to(dev), s.to(dev))
    out2.backward((2 * g).to(dev, torch.bfloat16))
    torch.cuda.synchronize()
    assert torch.equal(qd.grad.float().cpu(), 2 * dq) and torch.equal(vd.grad.float().cpu(), 2 * dv)


def test_c4_long_context_forward(pkg):
    """B1 H8 N65536 D128 causal forward on sampled rows."""
    B, H, N, D = 1, 8, 65536, 128
    dev = torch.device("cuda:0")
    q, k, v = (bf16_round(seeded((B, H, N, D), 7 + i)) for i in range(3))
    c, s = O.precompute_freqs_cis(D, N)
    scale = 1 / math.sqrt(D)
    o, M = pkg.rope_attn_forward_with_lse(q.to(dev, torch.bfloat16), k.to(dev, torch.bfloat16),
                                          v.to(dev, torch.bfloat16), True, scale, c.to(dev), s.to(dev))
    torch.cuda.synchronize()
    o, M = o.float().cpu(), M.cpu()
    rows = _rows(N, 48, 2)
    ro, rl = O.rope_attn_forward_blocked(q, k, v, True, scale, c, s, rows=rows)
    e_o, e_l = (o[:, :, rows] - ro).abs().max().item(), (M[:, :, rows] * LN2 - rl).abs().max().item()
    print(f"  C4 O max-abs {e_o:.3e}, LSE max-abs {e_l:.3e} on {rows.numel()} rows x {H} heads", flush=True)
    assert torch.isfinite(o).all() and e_o <= TOL and e_l <= TOL


def test_c5_corope_forward(pkg):
    """B2 Hq32 Hkv8 N4096 D128 Co-RoPE forward on sampled rows of every head."""
    B, Hq, Hkv, N, D = 2, 32, 8, 4096, 128
    dev = torch.device("cuda:0")
    q = bf16_round(seeded((B, Hq, N, D), 3))
    k, v = bf16_round(seeded((B, Hkv, N, D), 4)), bf16_round(seeded((B, Hkv, N, D), 5))
    scale = 1 / math.sqrt(D)
    o = pkg.corope_attention(q.to(dev, torch.bfloat16), k.to(dev, torch.bfloat16), v.to(dev, torch.bfloat16), True,
                             scale, 10000.0)
    torch.cuda.synchronize()
    o = o.float().cpu()
    rows = _rows(N, 9, 3)
    ref = C.corope_gqa_forward_rows(q, k, v, True, scale, 10000.0, rows, torch.float32, row_block=16)
    err = (o[:, :, rows] - ref).abs()
    print(f"  C5 O max-abs {err.max():.3e} mean-abs {err.mean():.3e} on {rows.numel()} rows x {B * Hq} heads", flush=True)
    assert torch.isfinite(o).all() and err.max() <= TOL
    assert torch.equal(o[:, :, 0], v.repeat_interleave(Hq // Hkv, 1)[:, :, 0])


def test_corope_long_hot_rows(pkg):
    """2048 keys at sm_scale = 0.5 (scores of +-15) with key norms rising towards key 0: over a row's 32 chunks the
    reference value of the exponentials has to move again and again.  Sampled rows against the oracle; mean-abs bar as for
    the other hot cases (bf16 inputs at this temperature), finite everywhere."""
    B, Hq, Hkv, N, D = 1, 4, 2, 2048, 64
    dev = torch.device("cuda:0")
    q = bf16_round(seeded((B, Hq, N, D), 13))
    k, v = bf16_round(seeded((B, Hkv, N, D), 14)), bf16_round(seeded((B, Hkv, N, D), 15))
    k = bf16_round(k * torch.linspace(1.6, 0.6, N)[None, None, :, None])
    o = pkg.corope_attention(q.to(dev, torch.bfloat16), k.to(dev, torch.bfloat16), v.to(dev, torch.bfloat16), True, 0.5, 10000.0)
    torch.cuda.synchronize()
    o = o.float().cpu()
    rows = _rows(N, 12, 5)
    ref = C.corope_gqa_forward_rows(q, k, v, True, 0.5, 10000.0, rows, torch.float32, row_block=16)
    err = (o[:, :, rows] - ref).abs()
    print(f"  long hot rows: O max-abs {err.max():.3e} mean-abs {err.mean():.3e}", flush=True)
    assert torch.isfinite(o).all()
    assert err.max() <= 0.15 and err.mean() <= 5e-3


def test_c5_corope_backward(pkg):
    """B2 Hq32 Hkv8 N4096 D128 Co-RoPE backward: dQ of sampled rows against autograd through the row-sampled oracle
    (a query row's output depends on no other query row), dK and dV of one group's last 1024 keys against autograd through
    the oracle over the query rows that see them (rows before key j contribute nothing to key j: causal, and the mileage
    of a row sums gates of keys up to the row itself), and two size-independent identities for dK and dV as a whole:
    sum_j dv_j = sum_{h,i} dO^h_i per group (softmax rows sum to one), and sum q.dq = sum k.dk per group (scores and
    gates depend on q and k only through products q.k, so scaling q up and k down by the same factor changes nothing)."""
    mod = pkg.corope_gqa
    B, Hq, Hkv, N, D = 2, 32, 8, 4096, 128
    G = Hq // Hkv
    dev = torch.device("cuda:0")
    q, d_o = bf16_round(seeded((B, Hq, N, D), 3)), bf16_round(seeded((B, Hq, N, D), 6))
    k, v = bf16_round(seeded((B, Hkv, N, D), 4)), bf16_round(seeded((B, Hkv, N, D), 5))
    scale = 1 / math.sqrt(D)
    print("  C5 backward: launching", flush=True)
    dq, dk, dv = (t.float().cpu() for t in mod.corope_gqa_backward(*(t.to(dev, torch.bfloat16) for t in (q, k, v, d_o)),
                                                                     scale, 10000.0))
    torch.cuda.synchronize()
    assert all(torch.isfinite(t).all() for t in (dq, dk, dv))

    rows = _rows(N, 3, 7)
    qa = q.clone().requires_grad_(True)
    out = C.corope_gqa_forward_rows(qa, k, v, True, scale, 10000.0, rows, torch.float32, row_block=16)
    (ref_dq,) = torch.autograd.grad(out, qa, d_o[:, :, rows])
    err = (dq[:, :, rows] - ref_dq[:, :, rows]).abs()
    print(f"  C5 dQ max-abs {err.max():.3e} mean-abs {err.mean():.3e} on {rows.numel()} rows x {B * Hq} heads "
          f"(max |ref| {ref_dq[:, :, rows].abs().max():.3f})", flush=True)
    assert err.max() <= TOL

    # one whole group's last keys: every query row that sees them, 64 rows at a time
    b, kv, first = B - 1, Hkv // 2, N - 1024
    qs, dos = q[b:b + 1, kv * G:(kv + 1) * G], d_o[b:b + 1, kv * G:(kv + 1) * G]
    kx, vx = (t[b:b + 1, kv:kv + 1].clone().requires_grad_(True) for t in (k, v))
    for r0 in range(first, N, 64):
        blk = C.corope_gqa_forward_rows(qs[:, :, :r0 + 64], kx[:, :, :r0 + 64], vx[:, :, :r0 + 64], True, scale, 10000.0,
                                        torch.arange(r0, r0 + 64), torch.float32, row_block=64)
        blk.backward(dos[:, :, r0:r0 + 64])
    for name, got, ref in (("dK", dk, kx.grad), ("dV", dv, vx.grad)):
        err = (got[b, kv, first:] - ref[0, 0, first:]).abs()
        print(f"  C5 {name} max-abs {err.max():.3e} mean-abs {err.mean():.3e} on the last {N - first} keys of group "
              f"(batch {b}, kv head {kv}) (max |ref| {ref[0, 0, first:].abs().max():.3f})", flush=True)
        assert err.max() <= TOL * math.sqrt(G), name     # sums over the group's G heads

    ulp = 2.0 ** -9
    dv_sum, do_sum = dv.double().sum(2), d_o.double().view(B, Hkv, G, N, D).sum((2, 3))
    bound = 8 * ulp * dv.double().pow(2).sum(2).sqrt()          # N independent roundings of dv rows
    print(f"  C5 sum_j dv - sum dO: max {float((dv_sum - do_sum).abs().max()):.3e} (bound min {float(bound.min()):.3e})", flush=True)
    assert ((dv_sum - do_sum).abs() <= bound + 1e-3 * do_sum.abs()).all()

    qdq = (q.double() * dq.double()).view(B, Hkv, G, N, D)
    kdk = k.double() * dk.double()
    lhs, rhs = qdq.sum((2, 3, 4)), kdk.sum((2, 3))
    bound = 8 * ulp * (qdq.pow(2).sum((2, 3, 4)) + kdk.pow(2).sum((2, 3))).sqrt()
    print(f"  C5 sum q.dq vs sum k.dk per group: max diff {float((lhs - rhs).abs().max()):.3e}, "
          f"|sum| up to {float(lhs.abs().max()):.3e}, bound min {float(bound.min()):.3e}", flush=True)
    assert ((lhs - rhs).abs() <= bound + 2e-3 * lhs.abs()).all()


def test_tensors_of_more_than_2_31_elements(pkg):
    """B66 H128 N2048 D128: 8448 (batch, head) slabs, 2.2e9 elements (4.4 GB) per tensor, so the offsets of the last slabs
    do not fit 32 bits.  The first slab, one in the middle and the last two are held against the oracle, forward and
    backward, and against the same slabs run on their own."""
    B, H, N, D = 66, 128, 2048, 128
    dev = torch.device("cuda:0")
    assert B * H * N * D > 2 ** 31
    gen = torch.Generator(device=dev).manual_seed(7)
    qd, kd, vd, gd = (torch.randn((B, H, N, D), device=dev, dtype=torch.bfloat16, generator=gen) for _ in range(4))
    c, s = O.precompute_freqs_cis(D, N)
    cd, sd = c.to(dev), s.to(dev)
    scale = 1 / math.sqrt(D)
    for t in (qd, kd, vd):
        t.requires_grad_(True)
    out = pkg.attention(qd, kd, vd, True, scale, cd, sd)
    out.backward(gd)
    torch.cuda.synchronize()
    for (b, h) in ((0, 0), (32, 65), (65, 126), (65, 127)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        q, k, v, g = (t.detach()[sl].float().cpu() for t in (qd, kd, vd, gd))
        ro, _, rdq, rdk, rdv, _ = O.rope_attn_fwd_bwd_blocked(q, k, v, g, True, scale, c, s)
        q1, k1, v1 = (t.detach()[sl].clone().requires_grad_(True) for t in (qd, kd, vd))
        o1 = pkg.attention(q1, k1, v1, True, scale, cd, sd)
        o1.backward(gd[sl].clone())
        for name, a, r, alone in (("O", out.detach()[sl], ro, o1.detach()), ("dQ", qd.grad[sl], rdq, q1.grad),
                                  ("dK", kd.grad[sl], rdk, k1.grad), ("dV", vd.grad[sl], rdv, v1.grad)):
            ok, err = within_bar(a.float().cpu(), r, TOL)[:2]
            d_alone = (a.float() - alone.float()).abs().max().item()
            print(f"  slab ({b},{h}) {name}: max-abs {err:.3e} against the oracle, {d_alone:.1e} against the slab alone", flush=True)
            assert ok, (b, h, name)
            assert d_alone <= 2e-2, (b, h, name)


def test_corope_tensors_of_more_than_2_31_elements(pkg):
    """Co-RoPE at B66 Hq128 Hkv32 N2048 D128: q, O, dO and dQ hold 2.2e9 elements each, so the offsets of the last heads do
    not fit 32 bits (and the backward walks its workspace in slices of groups).  The first group, one in the middle and
    the last are held against the same groups run on their own, forward and backward, and sampled rows of the last
    group's output against the oracle."""
    mod = pkg.corope_gqa
    B, Hq, Hkv, N, D = 66, 128, 32, 2048, 128
    G = Hq // Hkv
    dev = torch.device("cuda:0")
    assert B * Hq * N * D > 2 ** 31
    gen = torch.Generator(device=dev).manual_seed(11)
    qd, gd = (torch.randn((B, Hq, N, D), device=dev, dtype=torch.bfloat16, generator=gen) for _ in range(2))
    kd, vd = (torch.randn((B, Hkv, N, D), device=dev, dtype=torch.bfloat16, generator=gen) for _ in range(2))
    scale = 1 / math.sqrt(D)
    print("  launching the forward", flush=True)
    out = pkg.corope_attention(qd, kd, vd, True, scale, 10000.0)
    torch.cuda.synchronize()
    print("  launching the backward", flush=True)
    dq, dk, dv = mod.corope_gqa_backward(qd, kd, vd, gd, scale, 10000.0)
    torch.cuda.synchronize()
    for (b, kv) in ((0, 0), (31, 17), (B - 1, Hkv - 1)):
        hs, sl = (slice(b, b + 1), slice(kv * G, (kv + 1) * G)), (slice(b, b + 1), slice(kv, kv + 1))
        q1, g1, k1, v1 = qd[hs].clone(), gd[hs].clone(), kd[sl].clone(), vd[sl].clone()
        o1 = pkg.corope_attention(q1, k1, v1, True, scale, 10000.0)
        dq1, dk1, dv1 = mod.corope_gqa_backward(q1, k1, v1, g1, scale, 10000.0)
        torch.cuda.synchronize()
        for name, a, alone in (("O", out[hs], o1), ("dQ", dq[hs], dq1), ("dK", dk[sl], dk1), ("dV", dv[sl], dv1)):
            d = (a.float() - alone.float()).abs().max().item()
            print(f"  group ({b},{kv}) {name}: {d:.1e} against the group alone", flush=True)
            assert torch.isfinite(a.float()).all() and d <= TOL, (b, kv, name)
    rows = _rows(N, 5, 9)
    hs, sl = (slice(B - 1, B), slice(Hq - G, Hq)), (slice(B - 1, B), slice(Hkv - 1, Hkv))
    ref = C.corope_gqa_forward_rows(qd[hs].float().cpu(), kd[sl].float().cpu(), vd[sl].float().cpu(), True, scale, 10000.0,
                                    rows, torch.float32, row_block=16)
    err = (out[hs].float().cpu()[:, :, rows] - ref).abs().max().item()
    print(f"  last group: O max-abs {err:.3e} against the oracle on {rows.numel()} rows", flush=True)
    assert err <= TOL
