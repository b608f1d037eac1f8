"""Writes the golden fixtures in this directory (small .npz files: inputs + expected outputs).

The reference repository stores no golden vectors for this path, so these are produced here from programs that
are independent of the PyTorch oracle they pin:
  * forward outputs and natural-log LSE: the fp64 brute-force C program oracle/brute_force.c;
  * RoPE-attention gradients: torch.autograd (fp64) through a complex-multiplication rotation + library SDPA;
  * Co-RoPE gradients: central finite differences of the brute-force program's own forward (fp64, every coordinate of
    the smallest case, a sample of coordinates of the others, which otherwise hold torch.autograd through the dense oracle
    after that sample has confirmed it).
Expected outputs are stored rounded to fp32.  Inputs are N(0,1) draws from a seeded CPU generator, rounded to bf16 so that the GPU kernels see them exactly.

Run from the repository root:  python tests/golden/make_golden.py
"""
import math
import os
import sys

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from conftest import bf16_round, seeded  # noqa: E402


def _load_brute():
    import ctypes, subprocess
    so = os.path.join(ROOT, "oracle", "libbrute_force.so")
    if not os.path.exists(so):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    lib = ctypes.CDLL(so)
    dp = ctypes.POINTER(ctypes.c_double)
    lib.bf_rope_attn_fwd.argtypes = [dp] * 5 + [ctypes.c_int] * 5 + [ctypes.c_double, dp, dp]
    lib.bf_corope_gqa_fwd.argtypes = [dp] * 4 + [ctypes.c_int] * 5 + [ctypes.c_double, dp, dp]
    return lib, (lambda a: a.ctypes.data_as(dp))


def rope_case(name, B, H, N, D, causal, seed):
    lib, ptr = _load_brute()
    q, k, v, g = (bf16_round(seeded((B, H, N, D), seed + i)).double() for i in range(4))
    h = D // 2
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2).float() / D))
    ang = torch.outer(torch.arange(N, dtype=torch.float32), inv)          # fp32 angles, like the reference's table
    cos, sin = torch.cos(ang), torch.sin(ang)
    scale = 1 / math.sqrt(D)
    qn, kn, vn = (np.ascontiguousarray(t.numpy()) for t in (q, k, v))
    cn, sn = np.ascontiguousarray(cos.double().numpy()), np.ascontiguousarray(sin.double().numpy())
    o, lse = np.empty_like(qn), np.empty((B, H, N))
    assert lib.bf_rope_attn_fwd(ptr(qn), ptr(kn), ptr(vn), ptr(cn), ptr(sn), B, H, N, D, int(causal), scale, ptr(o), ptr(lse)) == 0
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    rot = torch.complex(cos.double(), sin.double())
    zq = torch.complex(qa[..., :h], qa[..., h:]) * rot
    zk = torch.complex(ka[..., :h], ka[..., h:]) * rot
    ref = F.scaled_dot_product_attention(torch.cat([zq.real, zq.imag], -1), torch.cat([zk.real, zk.imag], -1), va,
                                         is_causal=causal, scale=scale)
    assert np.abs(ref.detach().numpy() - o).max() < 1e-12
    dq, dk, dv = torch.autograd.grad(ref, (qa, ka, va), g)
    np.savez_compressed(os.path.join(HERE, name), q=qn.astype(np.float32), k=kn.astype(np.float32), v=vn.astype(np.float32),
                        do=g.numpy().astype(np.float32), cos=cos.numpy(), sin=sin.numpy(), causal=np.array(causal),
                        sm_scale=np.array(scale), o=o.astype(np.float32), lse=lse.astype(np.float32),
                        dq=dq.numpy().astype(np.float32), dk=dk.numpy().astype(np.float32), dv=dv.numpy().astype(np.float32))


def corope_case(name, B, Hq, Hkv, N, D, scale, theta, seed, fd_all=False, fd_samples=48):
    from oracle import corope_gqa_oracle as C
    lib, ptr = _load_brute()
    q = bf16_round(seeded((B, Hq, N, D), seed)).double().numpy()
    k = bf16_round(seeded((B, Hkv, N, D), seed + 1)).double().numpy()
    v = bf16_round(seeded((B, Hkv, N, D), seed + 2)).double().numpy()
    g = bf16_round(seeded((B, Hq, N, D), seed + 3)).double().numpy()
    inv = (1.0 / (theta ** (torch.arange(0, D, 2).float() / D))).double().numpy()   # fp32 expression, as the reference
    o = np.empty_like(q)
    assert lib.bf_corope_gqa_fwd(ptr(q), ptr(k), ptr(v), ptr(inv), B, Hq, Hkv, N, D, scale, ptr(o), None) == 0

    def loss(qq, kk, vv):       # sum(O * dO) through the brute-force program
        out = np.empty_like(qq)
        assert lib.bf_corope_gqa_fwd(ptr(qq), ptr(kk), ptr(vv), ptr(inv), B, Hq, Hkv, N, D, scale, ptr(out), None) == 0
        return float((out * g).sum())

    def fd(which, idx, eps=1e-5):
        args = [q.copy(), k.copy(), v.copy()]
        args[which][idx] += eps
        up = loss(*args)
        args[which][idx] -= 2 * eps
        return (up - loss(*args)) / (2 * eps)

    qa, ka, va = (torch.from_numpy(t).clone().requires_grad_(True) for t in (q, k, v))
    auto = [t.numpy() for t in torch.autograd.grad(C.corope_gqa_forward(qa, ka, va, True, scale, theta, torch.float64),
                                                   (qa, ka, va), torch.from_numpy(g))]
    grads = [np.array(a) for a in auto]
    rng = np.random.default_rng(seed)
    for which, ref in enumerate(auto):
        coords = list(np.ndindex(ref.shape)) if fd_all else [tuple(rng.integers(0, n) for n in ref.shape) for _ in range(fd_samples)]
        for idx in coords:
            d = fd(which, idx)
            assert abs(d - ref[idx]) <= 2e-6 * max(1.0, abs(ref[idx])), (name, which, idx, d, ref[idx])
            if fd_all:
                grads[which][idx] = d
    np.savez_compressed(os.path.join(HERE, name), q=q.astype(np.float32), k=k.astype(np.float32), v=v.astype(np.float32),
                        do=g.astype(np.float32), sm_scale=np.array(scale), theta=np.array(theta), o=o.astype(np.float32),
                        dq=grads[0].astype(np.float32), dk=grads[1].astype(np.float32), dv=grads[2].astype(np.float32))


if __name__ == "__main__":
    rope_case("rope_B1_H2_N128_D64_causal.npz", 1, 2, 128, 64, True, 100)
    rope_case("rope_B1_H1_N256_D128_causal.npz", 1, 1, 256, 128, True, 200)
    rope_case("rope_B1_H2_N96_D64_full.npz", 1, 2, 96, 64, False, 300)
    # the two tiny shapes the reference's own Co-RoPE scripts use (compare_corope.py:152; corope_attn_gqa_pytorch.py:309-321)
    corope_case("corope_B1_Hq4_Hkv2_N32_D64.npz", 1, 4, 2, 32, 64, 1.0, 10000.0, 400, fd_all=True)
    corope_case("corope_B2_Hq4_Hkv2_N64_D32.npz", 2, 4, 2, 64, 32, 32 ** -0.5, 10000.0, 500)
    corope_case("corope_B1_Hq8_Hkv2_N96_D128.npz", 1, 8, 2, 96, 128, 128 ** -0.5, 10000.0, 600)
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
