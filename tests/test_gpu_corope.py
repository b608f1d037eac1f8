"""GPU parity of the Co-RoPE GQA forward against the CPU oracle (through the C ABI).

Bar: max-abs <= 2e-2 for the bf16 output against the oracle evaluated in fp64/fp32 on the same bf16-rounded
inputs.  Small shapes use the dense oracle; long sequences use its row-sampled form."""
import math

import pytest
import torch

from conftest import bf16_round, seeded
from oracle import corope_gqa_oracle as C

pytestmark = pytest.mark.gpu
TOL = 2e-2


def _inputs(B, Hq, Hkv, N, D, seed=42):
    return (bf16_round(seeded((B, Hq, N, D), seed)), bf16_round(seeded((B, Hkv, N, D), seed + 1)),
            bf16_round(seeded((B, Hkv, N, D), seed + 2)))


def _run(pkg, q, k, v, scale, theta):
    dev = torch.device("cuda:0")
    o = pkg.corope_attention(q.to(dev, torch.bfloat16), k.to(dev, torch.bfloat16), v.to(dev, torch.bfloat16), True,
                             scale, theta)
    torch.cuda.synchronize()
    return o.float().cpu()


# (B, Hq, Hkv, N, D): the reference's compare_corope.py shape first, then every group size and ragged lengths
CASES = [(1, 4, 2, 32, 64), (2, 4, 2, 64, 64), (1, 2, 2, 96, 64), (1, 6, 2, 100, 64), (1, 8, 2, 130, 128),
         (1, 8, 1, 257, 64), (2, 5, 1, 77, 128), (1, 6, 1, 64, 128), (1, 7, 1, 65, 64), (1, 4, 1, 1, 64),
         (2, 8, 2, 512, 128)]


@pytest.mark.parametrize("B,Hq,Hkv,N,D", CASES)
def test_corope_forward_parity(pkg, B, Hq, Hkv, N, D):
    print(f"case B={B} Hq={Hq} Hkv={Hkv} N={N} D={D}", flush=True)
    q, k, v = _inputs(B, Hq, Hkv, N, D)
    scale = 1 / math.sqrt(D)
    o = _run(pkg, q, k, v, scale, 10000.0)
    if N <= 130:
        ref = C.corope_gqa_forward(q, k, v, True, scale, 10000.0, torch.float64).float()
    else:
        ref = C.corope_gqa_forward_rows(q, k, v, True, scale, 10000.0, torch.arange(N), torch.float32)
    err = (o - ref).abs()
    print(f"  O max-abs {err.max():.3e} mean-abs {err.mean():.3e}")
    assert torch.isfinite(o).all()
    assert err.max() <= TOL


def test_corope_unit_scale_small_theta(pkg):
    """sm_scale = 1 and a small base (fast rotations), as in the reference's comparison script (sm_scale=1.0)."""
    q, k, v = _inputs(1, 4, 2, 32, 64, seed=7)
    q, k = bf16_round(q * 0.3), bf16_round(k * 0.3)
    o = _run(pkg, q, k, v, 1.0, 100.0)
    ref = C.corope_gqa_forward(q, k, v, True, 1.0, 100.0, torch.float64).float()
    assert (o - ref).abs().max() <= TOL


def test_corope_zero_leader_matches_rope_kernel(pkg):
    """With a zero leader every gate is 1/2, so the follower heads equal RoPE attention at positions m/2:
    the Co-RoPE kernel and the RoPE-attention kernel must then agree with each other."""
    B, Hq, Hkv, N, D = 1, 4, 2, 256, 64
    G = Hq // Hkv
    q, k, v = _inputs(B, Hq, Hkv, N, D, seed=11)
    q[:, ::G] = 0
    scale = 1 / math.sqrt(D)
    o = _run(pkg, q, k, v, scale, 10000.0)
    w = C.corope_inv_freq(D, 10000.0)
    ang = (torch.arange(N, dtype=torch.float32) / 2).unsqueeze(1) * w.unsqueeze(0)
    cos, sin = torch.cat([ang.cos()] * 2, -1), torch.cat([ang.sin()] * 2, -1)
    dev = torch.device("cuda:0")
    kx, vx = k.repeat_interleave(G, 1), v.repeat_interleave(G, 1)
    o_rope, _ = pkg.rope_attn_forward_with_lse(q.to(dev, torch.bfloat16), kx.to(dev, torch.bfloat16),
                                                vx.to(dev, torch.bfloat16), True, scale, cos.to(dev), sin.to(dev))
    followers = [h for h in range(Hq) if h % G]
    assert (o[:, followers] - o_rope.float().cpu()[:, followers]).abs().max() <= TOL


def test_corope_validation_errors(pkg):
    dev = torch.device("cuda:0")
    q = torch.zeros(1, 4, 64, 64, device=dev, dtype=torch.bfloat16)
    k = torch.zeros(1, 2, 64, 64, device=dev, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        pkg.corope_attention(q, k, k, False, 1.0, 1e4)
    with pytest.raises(ValueError):
        pkg.corope_attention(q, k[:, :, :32], k[:, :, :32], True, 1.0, 1e4)
    with pytest.raises(ValueError):
        pkg.corope_attention(torch.zeros(1, 18, 64, 64, device=dev, dtype=torch.bfloat16), k, k, True, 1.0, 1e4)
    with pytest.raises(ValueError):
        pkg.corope_attention(q.float(), k.float(), k.float(), True, 1.0, 1e4)


@pytest.mark.parametrize("scale", [None, 1.0])
@pytest.mark.parametrize("B,Hq,Hkv,N,D", [(1, 4, 2, 32, 64), (1, 6, 2, 100, 64), (1, 8, 2, 130, 128), (2, 8, 2, 512, 128)])
def test_corope_forward_fp16(pkg, B, Hq, Hkv, N, D, scale):
    """fp16 tensors, the dtype of the reference's kernel and comparison script (compare_corope.py:18, whose shape comes
    first and which runs at sm_scale = 1): the same kernel built for fp16 elements, against the oracle on the same
    fp16-rounded inputs.  Bar: max-abs <= 2e-2 at 1/sqrt(D); at sm_scale = 1 (logits with a standard deviation of 8 to 11)
    max <= 0.15 and mean <= 5e-3 as for the other hot cases.  (The fp16 backward: test_gpu_corope_bwd.py.)"""
    print(f"case fp16 B={B} Hq={Hq} Hkv={Hkv} N={N} D={D} scale={scale}", flush=True)
    q, k, v = (t.to(torch.float16).float() for t in (seeded((B, Hq, N, D), 5), seeded((B, Hkv, N, D), 6), seeded((B, Hkv, N, D), 7)))
    sc = 1 / math.sqrt(D) if scale is None else scale
    dev = torch.device("cuda:0")
    qd = q.to(dev, torch.float16).requires_grad_(True)
    o = pkg.corope_attention(qd, k.to(dev, torch.float16), v.to(dev, torch.float16), True, sc, 10000.0)
    torch.cuda.synchronize()
    assert o.dtype == torch.float16
    if N <= 130:
        ref = C.corope_gqa_forward(q, k, v, True, sc, 10000.0, torch.float64).float()
    else:
        ref = C.corope_gqa_forward_rows(q, k, v, True, sc, 10000.0, torch.arange(N), torch.float32)
    err = (o.float().cpu() - ref).abs()
    print(f"  O max-abs {err.max():.3e} mean-abs {err.mean():.3e}")
    assert torch.isfinite(o).all()
    if scale is None:
        assert err.max() <= TOL
    else:
        assert err.max() <= 0.15 and err.mean() <= 5e-3
