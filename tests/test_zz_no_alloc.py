"""The forward entry point that allocates nothing (corope_rope_attn_fwd_noalloc) against corope_rope_attn_fwd_ws: same
kernels, the rotated K in the library's built-in buffer instead of a caller's workspace.  Through the C ABI, bit for
bit, on two calls in a row of which the second is smaller (the buffer keeps the first call's contents)."""
import math

import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu


def _run_pair(pkg, shape, causal, seed):
    lib = pkg._lib.load()
    dev = torch.device("cuda:0")
    B, H, N, D = shape
    q, k, v = (seeded(shape, seed + i, torch.bfloat16).to(dev) for i in range(3))
    cos, sin = pkg.precompute_freqs_cis(D, N, 10000.0, device=dev)
    scale = 1 / math.sqrt(D)
    stream = torch.cuda.current_stream().cuda_stream
    nbytes = lib.corope_rope_attn_fwd_workspace_bytes(B, H, N, D)
    assert 0 < nbytes <= lib.corope_rope_attn_fwd_noalloc_max_bytes()
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    o_ws, o_na = torch.zeros_like(q), torch.ones_like(q)
    m_ws = torch.zeros(B, H, N, device=dev)
    m_na = torch.ones(B, H, N, device=dev)
    args = (q.data_ptr(), k.data_ptr(), v.data_ptr(), cos.data_ptr(), sin.data_ptr(), cos.stride(0))
    tail = (B, H, N, D, scale, int(causal))
    rc = lib.corope_rope_attn_fwd_ws(*args, o_ws.data_ptr(), m_ws.data_ptr(), *tail, ws.data_ptr(), nbytes, stream)
    assert rc == 0, pkg._lib.last_error()
    torch.cuda.synchronize()
    # a first call may set kernel attributes and look up the buffer's address; the one after it is the one measured:
    # neither torch's allocator nor the device's free memory (which a hipMalloc inside the library would lower) may move
    rc = lib.corope_rope_attn_fwd_noalloc(*args, o_na.data_ptr(), m_na.data_ptr(), *tail, stream)
    assert rc == 0, pkg._lib.last_error()
    torch.cuda.synchronize()
    o_na.fill_(1)
    m_na.fill_(1)
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(dev), torch.cuda.mem_get_info(dev)[0]
    rc = lib.corope_rope_attn_fwd_noalloc(*args, o_na.data_ptr(), m_na.data_ptr(), *tail, stream)
    assert rc == 0, pkg._lib.last_error()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before and torch.cuda.mem_get_info(dev)[0] == free_before
    assert torch.equal(o_na, o_ws), f"O differs at {shape}: {(o_na.float() - o_ws.float()).abs().max().item():.3e}"
    assert torch.equal(m_na, m_ws), f"row statistics differ at {shape}"


def test_noalloc_forward_matches_workspace_forward_twice(pkg):
    # larger call first, then a smaller one with other data: whatever the first call left in the buffer must not matter
    _run_pair(pkg, (2, 4, 1500, 128), True, seed=11)
    _run_pair(pkg, (1, 3, 333, 64), True, seed=23)
    _run_pair(pkg, (1, 2, 200, 128), False, seed=31)


def test_noalloc_forward_refuses_sizes_beyond_its_buffer(pkg):
    lib = pkg._lib.load()
    limit = lib.corope_rope_attn_fwd_noalloc_max_bytes()
    assert limit == 65 << 20
    B, H, N, D = 4, 32, 4096, 128            # twice the metric shape: 128 MiB of rotated K
    assert lib.corope_rope_attn_fwd_workspace_bytes(B, H, N, D) > limit
    # refused on sizes alone, before any pointer is looked at or any HIP call is made
    rc = lib.corope_rope_attn_fwd_noalloc(None, None, None, None, None, D, None, None, B, H, N, D, 0.1, 1, None)
    assert rc == pkg._lib.E_UNSUPPORTED
    assert "bytes of scratch" in pkg._lib.last_error()
    assert lib.corope_rope_attn_fwd_workspace_bytes(2, 32, 4096, 128) <= limit   # the metric shape fits


def test_noalloc_forward_replays_in_a_graph(pkg):
    """What the entry point is for: recorded into a HIP graph after one warm call outside the capture (kernel attributes,
    the buffer's address), replayed on fresh inputs with eager calls in between, bit-equal to the workspace forward."""
    lib = pkg._lib.load()
    dev = torch.device("cuda:0")
    B, H, N, D = 1, 4, 1100, 128
    cos, sin = pkg.precompute_freqs_cis(D, N, 10000.0, device=dev)
    scale = 1 / math.sqrt(D)
    q, k, v = (seeded((B, H, N, D), 40 + i, torch.bfloat16).to(dev) for i in range(3))
    o, o_ref = torch.empty_like(q), torch.empty_like(q)
    m, m_ref = torch.empty(B, H, N, device=dev), torch.empty(B, H, N, device=dev)
    nbytes = lib.corope_rope_attn_fwd_workspace_bytes(B, H, N, D)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    args = (q.data_ptr(), k.data_ptr(), v.data_ptr(), cos.data_ptr(), sin.data_ptr(), cos.stride(0))
    tail = (B, H, N, D, scale, 1)

    def call(stream):
        assert lib.corope_rope_attn_fwd_noalloc(*args, o.data_ptr(), m.data_ptr(), *tail, stream) == 0, pkg._lib.last_error()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(torch.cuda.current_stream().cuda_stream)
    for i in range(3):
        for t, sd in ((q, 50), (k, 60), (v, 70)):
            t.copy_(seeded((B, H, N, D), sd + i, torch.bfloat16))
        o.zero_()
        graph.replay()
        torch.cuda.synchronize()
        rc = lib.corope_rope_attn_fwd_ws(*args, o_ref.data_ptr(), m_ref.data_ptr(), *tail, ws.data_ptr(), nbytes,
                                         torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(o, o_ref) and torch.equal(m, m_ref), f"replay {i}"
