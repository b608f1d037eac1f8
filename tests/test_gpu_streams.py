"""Calls on two streams of one device at the same time: the kernels share no state between launches (static item lists,
no atomics) and the Python operators keep none that two streams could meet in (the Co-RoPE backward's cached scratch is
per stream), so each stream's results are those of the same call made alone."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _alone_and_together(make_inputs, run, rounds=3):
    """run(inputs) -> tensors.  Both streams (default priority) are fed `rounds` calls on inputs of their own without any
    synchronisation in between; every result is compared with the same call made on the default stream afterwards."""
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    inputs = [[make_inputs(10 * s + r) for r in range(rounds)] for s in range(2)]
    torch.cuda.synchronize()
    got = [[None] * rounds for _ in range(2)]
    for r in range(rounds):
        for s, stream in enumerate(streams):
            with torch.cuda.stream(stream):
                got[s][r] = run(inputs[s][r])
    torch.cuda.synchronize()
    for s in range(2):
        for r in range(rounds):
            want = run(inputs[s][r])
            torch.cuda.synchronize()
            for a, b in zip(got[s][r], want):
                assert torch.equal(a, b), (s, r)


def test_rope_attention_on_two_streams(pkg):
    dev = torch.device("cuda:0")
    B, H, N, D = 2, 8, 2048, 128
    c, s = pkg.precompute_freqs_cis(D, N, 10000.0, device=dev)

    def make_inputs(seed):
        g = torch.Generator(device=dev).manual_seed(seed)
        return [torch.randn((B, H, N, D), device=dev, dtype=torch.bfloat16, generator=g) for _ in range(4)]

    def run(ts):
        q, k, v = (t.detach().clone().requires_grad_(True) for t in ts[:3])
        o = pkg.attention(q, k, v, True, 1 / math.sqrt(D), c, s)
        o.backward(ts[3])
        return o.detach(), q.grad, k.grad, v.grad

    _alone_and_together(make_inputs, run)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_corope_attention_on_two_streams(pkg, dtype):
    dev = torch.device("cuda:0")
    B, Hq, Hkv, N, D = 1, 8, 2, 1024, 64

    def make_inputs(seed):
        g = torch.Generator(device=dev).manual_seed(seed)
        return [torch.randn((B, h, N, D), device=dev, dtype=dtype, generator=g) for h in (Hq, Hkv, Hkv, Hq)]

    def run(ts):
        q, k, v = (t.detach().clone().requires_grad_(True) for t in ts[:3])
        o = pkg.corope_attention(q, k, v, True, 1 / math.sqrt(D), 10000.0)
        o.backward(ts[3])
        return o.detach(), q.grad, k.grad, v.grad

    pkg.corope_gqa.release_backward_workspace()
    _alone_and_together(make_inputs, run)
    # one cached scratch per stream that ran a backward (two side streams and the default one)
    assert len({key for key in pkg.corope_gqa._workspaces if key[0] == 0}) == 3
    pkg.corope_gqa.release_backward_workspace("cuda")
    assert not pkg.corope_gqa._workspaces
