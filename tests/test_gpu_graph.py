"""The operators under HIP graph capture: the library calls no allocator, memset or synchronisation, so a forward +
backward recorded once must replay with the same results as eager launches, on fresh inputs, several times, with
eager work in between."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _capture_and_replay(run, inputs, make_inputs):
    """run(*inputs) -> tensors to compare (recorded into a graph); make_inputs(i) -> fresh values for replay i."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):            # warm-up off the default stream, as graph capture wants it
        for _ in range(2):
            for t in inputs:
                t.grad = None
            run(*inputs)
    torch.cuda.current_stream().wait_stream(side)
    for t in inputs:
        t.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = run(*inputs)
    for i in range(3):
        fresh = make_inputs(i)
        with torch.no_grad():
            for t, f in zip(inputs, fresh):
                t.copy_(f)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.detach().clone() for o in outs]
        eager_in = [f.clone().requires_grad_(t.requires_grad) for t, f in zip(inputs, fresh)]
        want = run(*eager_in)                # eager launches between the replays
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b.detach()), f"replay {i}"


def test_rope_attention_replays_in_a_graph(pkg):
    dev = torch.device("cuda:0")
    B, H, N, D = 1, 4, 1024, 128
    cos, sin = pkg.precompute_freqs_cis(D, N, 10000.0, device=dev)
    gen = torch.Generator(device="cpu").manual_seed(3)

    def make(i):
        return [torch.randn(B, H, N, D, generator=gen).to(dev, torch.bfloat16) for _ in range(4)]

    def run(q, k, v, d_o):
        o = pkg.attention(q, k, v, True, 1 / math.sqrt(D), cos, sin)
        dq, dk, dv = torch.autograd.grad(o, (q, k, v), d_o)
        return o, dq, dk, dv

    inputs = [t.requires_grad_(j < 3) for j, t in enumerate(make(-1))]
    _capture_and_replay(run, inputs, make)


def test_corope_attention_replays_in_a_graph(pkg):
    dev = torch.device("cuda:0")
    B, Hq, Hkv, N, D = 1, 4, 2, 200, 64
    gen = torch.Generator(device="cpu").manual_seed(4)

    def make(i):
        shapes = [(B, Hq, N, D), (B, Hkv, N, D), (B, Hkv, N, D), (B, Hq, N, D)]
        return [torch.randn(*s, generator=gen).to(dev, torch.bfloat16) for s in shapes]

    def run(q, k, v, d_o):
        o = pkg.corope_attention(q, k, v, True, 0.125, 10000.0)
        dq, dk, dv = torch.autograd.grad(o, (q, k, v), d_o)
        return o, dq, dk, dv

    inputs = [t.requires_grad_(j < 3) for j, t in enumerate(make(-1))]
    _capture_and_replay(run, inputs, make)
