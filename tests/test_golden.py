"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py from the fp64 brute-force program and
fp64 autograd): the oracle must reproduce them on CPU, the HIP kernels on the GPU."""
import glob
import os

import numpy as np
import pytest
import torch

from conftest import within_bar
from oracle import corope_gqa_oracle as C
from oracle import rope_attn_oracle as O

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
ROPE = sorted(glob.glob(os.path.join(HERE, "rope_*.npz")))
COROPE = sorted(glob.glob(os.path.join(HERE, "corope_*.npz")))


def _t(a):
    return torch.from_numpy(np.asarray(a))


def test_fixtures_present():
    assert len(ROPE) >= 3 and len(COROPE) >= 3


@pytest.mark.parametrize("path", ROPE, ids=os.path.basename)
def test_oracle_reproduces_rope_fixture(path):
    z = np.load(path)
    q, k, v, g = (_t(z[n]).double() for n in ("q", "k", "v", "do"))
    D = q.shape[-1]
    cos, sin = (torch.cat([_t(z[n])] * 2, -1).double() for n in ("cos", "sin"))
    causal, scale = bool(z["causal"]), float(z["sm_scale"])
    o, lse, saved = O.rope_attn_forward(q, k, v, causal, scale, cos, sin, torch.float64)
    dq, dk, dv = O.rope_attn_backward(saved, g, causal, scale, cos, sin)
    for name, got in (("o", o), ("lse", lse), ("dq", dq), ("dk", dk), ("dv", dv)):
        assert (got - _t(z[name]).double()).abs().max() < 2e-6, name
    # the fp32 run (what the GPU parity tests compare against) stays within fp32 round-off of it
    o32, _, _ = O.rope_attn_forward(q.float(), k.float(), v.float(), causal, scale, cos.float(), sin.float())
    assert (o32.double() - _t(z["o"]).double()).abs().max() < 1e-4
    # the table handed to the kernels is the one the fixture was built from
    c2, s2 = O.precompute_freqs_cis(D, q.shape[2])
    assert torch.equal(c2[:, :D // 2], _t(z["cos"])) and torch.equal(s2[:, :D // 2], _t(z["sin"]))


@pytest.mark.parametrize("path", COROPE, ids=os.path.basename)
def test_oracle_reproduces_corope_fixture(path):
    z = np.load(path)
    q, k, v = (_t(z[n]).double() for n in ("q", "k", "v"))
    o = C.corope_gqa_forward(q, k, v, True, float(z["sm_scale"]), float(z["theta"]), torch.float64)
    assert (o - _t(z["o"]).double()).abs().max() < 2e-6
    rows = torch.arange(q.shape[2])
    o_rows = C.corope_gqa_forward_rows(q.float(), k.float(), v.float(), True, float(z["sm_scale"]), float(z["theta"]), rows)
    assert (o_rows.double() - _t(z["o"]).double()).abs().max() < 1e-4
    # gradients: the fixture's come from finite differences of the brute-force program (see make_golden.py)
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    do = _t(z["do"]).double()
    auto = torch.autograd.grad(C.corope_gqa_forward(qa, ka, va, True, float(z["sm_scale"]), float(z["theta"]), torch.float64),
                               (qa, ka, va), do)
    manual = C.corope_gqa_backward_manual(q, k, v, do, float(z["sm_scale"]), float(z["theta"]))
    for name, a, m in zip(("dq", "dk", "dv"), auto, manual):
        ref = _t(z[name]).double()
        tol = 1e-5 * max(1.0, float(ref.abs().max()))     # the fixture is stored in fp32
        assert (a - ref).abs().max() <= tol and (m - ref).abs().max() <= tol, name


@pytest.mark.gpu
@pytest.mark.parametrize("path", ROPE, ids=os.path.basename)
def test_kernels_reproduce_rope_fixture(pkg, path):
    z = np.load(path)
    dev = torch.device("cuda:0")
    q, k, v = (_t(z[n]).to(dev, torch.bfloat16).requires_grad_(True) for n in ("q", "k", "v"))
    cos, sin = _t(z["cos"]).to(dev), _t(z["sin"]).to(dev)          # half-width (N, D/2) tables
    o = pkg.attention(q, k, v, bool(z["causal"]), float(z["sm_scale"]), cos, sin)
    o.backward(_t(z["do"]).to(dev, torch.bfloat16))
    torch.cuda.synchronize()
    for name, got in (("o", o), ("dq", q.grad), ("dk", k.grad), ("dv", v.grad)):
        ok, err = within_bar(got.detach().float().cpu(), _t(z[name]))
        print(f"  {os.path.basename(path)} {name}: max-abs {err:.3e}")
        assert ok, name


@pytest.mark.gpu
@pytest.mark.parametrize("path", COROPE, ids=os.path.basename)   # the D = 32 fixture runs padded to the kernels' D = 64
def test_kernel_reproduces_corope_fixture(pkg, path):
    z = np.load(path)
    dev = torch.device("cuda:0")
    q, k, v = (_t(z[n]).to(dev, torch.bfloat16).requires_grad_(True) for n in ("q", "k", "v"))
    o = pkg.corope_attention(q, k, v, True, float(z["sm_scale"]), float(z["theta"]))
    o.backward(_t(z["do"]).to(dev, torch.bfloat16))
    torch.cuda.synchronize()
    err = (o.detach().float().cpu() - _t(z["o"])).abs().max().item()
    print(f"  {os.path.basename(path)} o: max-abs {err:.3e}")
    assert err <= 2e-2
    group = q.shape[1] // k.shape[1]
    for name, got in (("dq", q.grad), ("dk", k.grad), ("dv", v.grad)):
        ok, err = within_bar(got.float().cpu(), _t(z[name]), 2e-2 * (1.0 if name == "dq" else group ** 0.5))
        print(f"  {os.path.basename(path)} {name}: max-abs {err:.3e}")
        assert ok, name
