"""Co-RoPE grouped-query attention (forward and backward, bfloat16 or float16) behind the reference's call surface.

``attention(q, k, v, causal, sm_scale, theta[, warp_specialize])`` mirrors the reference's
``_attention.apply`` (corope-exp/flash_attn_co_rope_gqa_triton.py:403-456, :580), including its validation
errors (:407-425).  Forward and backward are hand-written gfx950 kernels reached through the C ABI.  The reference's
own "fused" operator falls back to a dense PyTorch backward with (B, Hq, N, N, D/2) temporaries (:459-577); the
backward here produces the same gradients from q, k, v and dO with N*N/2 fp32 scalars per matrix and head of scratch memory
(``backward_workspace_bytes`` says how much)."""
from __future__ import annotations

import torch

from . import _lib
from .rope_attn import _PADDED_D, gather_halves, spread_halves


class _CoRopeGqaAttn(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, causal, sm_scale, theta, warp_specialize=False):
        if not causal:
            raise ValueError("CoRoPE fused kernel supports causal=True only.")
        if q.ndim != 4 or k.ndim != 4 or v.ndim != 4:
            raise ValueError("Expected q, k, v to have shape (batch, heads, seqlen, dim).")
        if k.shape != v.shape:
            raise ValueError("k and v must share the same shape in GQA.")
        if q.shape[0] != k.shape[0] or q.shape[2] != k.shape[2] or q.shape[3] != k.shape[3]:
            raise ValueError("k must align with q along batch/sequence/head_dim.")
        B, Hq, N, D = q.shape
        Hkv = k.shape[1]
        if Hq % Hkv != 0:
            raise ValueError("Number of query heads must be divisible by KV heads.")
        if Hq // Hkv > 8:
            raise ValueError(f"CoRoPE backbone currently limits group_size <= 8 (got {Hq // Hkv}).")
        if not (q.is_cuda and k.is_cuda and v.is_cuda):
            raise ValueError("Co-RoPE attention runs on the GPU only: q, k, v must be on a HIP device")
        if not (q.dtype == k.dtype == v.dtype and q.dtype in (torch.bfloat16, torch.float16)):
            raise ValueError(f"q, k, v must all be bfloat16 or all float16 (got {q.dtype}, {k.dtype}, {v.dtype})")
        lib = _lib.load()
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        o = torch.empty_like(q)
        with torch.cuda.device(q.device):
            fwd = lib.corope_gqa_fwd_f16 if q.dtype == torch.float16 else lib.corope_gqa_fwd
            rc = fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), B, Hq, Hkv, N, D,
                     float(sm_scale), float(theta), torch.cuda.current_stream(q.device).cuda_stream)
        _lib.check(rc, "corope_gqa_fwd")
        # what the reference keeps (:451), minus inv_freq (theta is enough), plus the output: the backward takes a
        # reference value for its row sums from it (accuracy of dQ on sharply peaked rows; not needed mathematically)
        ctx.save_for_backward(q, k, v, o)
        ctx.group_size = Hq // Hkv
        ctx.sm_scale = sm_scale
        ctx.theta = theta
        ctx.causal = causal
        return o

    @staticmethod
    def backward(ctx, grad_output):
        q, k, v, o = ctx.saved_tensors
        dq, dk, dv = corope_gqa_backward(q, k, v, grad_output, ctx.sm_scale, ctx.theta, out=o)
        return dq, dk, dv, None, None, None, None


def backward_workspace_bytes(B, Hq, Hkv, N, D):
    """Scratch memory for a backward that handles all groups in one pass: (2 * B * Hkv + 3 * B * Hq) packed
    lower-triangular N x N fp32 matrices (about N * N / 2 + 32 * N values each), plus B * Hkv * N * D values."""
    n = _lib.load().corope_gqa_bwd_workspace_bytes(B, Hq, Hkv, N, D)
    if n < 0:
        raise ValueError(_lib.last_error() or "unsupported Co-RoPE shape")
    return n


def backward_min_workspace_bytes(B, Hq, Hkv, N, D):
    """The smallest scratch the backward accepts: one (batch, key/value head) group's matrices."""
    n = _lib.load().corope_gqa_bwd_min_workspace_bytes(B, Hq, Hkv, N, D)
    if n < 0:
        raise ValueError(_lib.last_error() or "unsupported Co-RoPE shape")
    return n


# The backward's scratch when the caller brings none: one buffer per device and stream, kept between calls and grown when
# a call needs more, holding as many groups' matrices as fit BACKWARD_WORKSPACE_CAP_BYTES (never less than one group; all
# groups in one pass is fastest: at B2 Hq32 Hkv8 N4096 D128 7.1 GiB and 14 ms, against 31 ms with a quarter of that).  The
# size depends on the shape and the cap only, not on what else is resident.  Per stream, because calls on two streams of a
# device may run at the same time and torch's allocator only orders a buffer's reuse on the stream it was allocated on.
BACKWARD_WORKSPACE_CAP_BYTES = 8 << 30
_workspaces = {}   # (device index, stream handle) -> uint8 tensor


def _cached_workspace(device, B, Hq, Hkv, N, D):
    one, full = backward_min_workspace_bytes(B, Hq, Hkv, N, D), backward_workspace_bytes(B, Hq, Hkv, N, D)
    want = min(full, max(1, BACKWARD_WORKSPACE_CAP_BYTES // one) * one)
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < want:
        _workspaces.pop(key, None)
        ws = None                      # the old buffer goes back to the allocator before the larger one is asked for
        try:
            ws = torch.empty(want, dtype=torch.uint8, device=device)
        except torch.cuda.OutOfMemoryError:
            if want > one:
                try:
                    ws = torch.empty(one, dtype=torch.uint8, device=device)
                except torch.cuda.OutOfMemoryError:
                    ws = None
        if ws is None:
            raise MemoryError(f"Co-RoPE backward at B={B} Hq={Hq} Hkv={Hkv} N={N} D={D} needs at least {one} bytes of scratch "
                              f"(one key/value group; {full} for all groups in one pass) and {device} does not have them")
        _workspaces[key] = ws
    return ws


def release_backward_workspace(device=None):
    """Gives the cached scratch of the backward (of one device, or of all) back to torch's allocator."""
    if device is None:
        _workspaces.clear()
    else:
        index = torch.device(device).index
        if index is None:
            index = torch.cuda.current_device()
        for key in [k for k in _workspaces if k[0] == index]:
            del _workspaces[key]


def corope_gqa_backward(q, k, v, grad_output, sm_scale, theta, workspace=None, out=None):
    """(dq, dk, dv) of the Co-RoPE GQA attention for upstream gradient ``grad_output`` (reference :459-577).

    ``workspace`` may be a caller-owned uint8/float tensor of at least ``backward_min_workspace_bytes`` bytes (the groups
    are then processed in passes of as many as fit; ``backward_workspace_bytes`` holds them all); without one a buffer
    cached per device and stream is used (``BACKWARD_WORKSPACE_CAP_BYTES``, ``release_backward_workspace``); ``out`` the
    forward's output for the same inputs (optional: it only steadies the rounding of dQ on sharply peaked rows)."""
    lib = _lib.load()
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    q, k, v, d_o = q.contiguous(), k.contiguous(), v.contiguous(), grad_output.to(q.dtype).contiguous()
    out_c = None if out is None else out.contiguous()
    o_ptr = None if out_c is None else out_c.data_ptr()
    if workspace is None:
        workspace = _cached_workspace(q.device, B, Hq, Hkv, N, D)
    have = workspace.numel() * workspace.element_size()
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    with torch.cuda.device(q.device):
        bwd = lib.corope_gqa_bwd_f16 if q.dtype == torch.float16 else lib.corope_gqa_bwd
        rc = bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o_ptr, d_o.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                 dv.data_ptr(), B, Hq, Hkv, N, D, float(sm_scale), float(theta), workspace.data_ptr(),
                 have, torch.cuda.current_stream(q.device).cuda_stream)
    _lib.check(rc, "corope_gqa_bwd")
    return dq, dk, dv


def attention(q, k, v, causal, sm_scale, theta, warp_specialize=False):
    """The reference's ``attention = _attention.apply`` (corope-exp/flash_attn_co_rope_gqa_triton.py:580): positional
    arguments in its order.  Head dims 64 and 128 go to the kernels as they are.  16 and 32 -- the reference's own
    self-check runs at 32 (corope_attn_gqa_pytorch.py:309-321) -- run at D = 64 with each half of a row padded with zeros:
    the rotation pairs and every dot product keep their values, and the inverse frequencies theta^(-2d/D) of the pairs
    that carry data are those of theta^(64/D) at D = 64."""
    d = q.shape[-1] if q.ndim == 4 else 0
    if d in _PADDED_D and k.ndim == 4 and v.ndim == 4 and k.shape[-1] == d and v.shape[-1] == d:
        o = _CoRopeGqaAttn.apply(spread_halves(q, 64), spread_halves(k, 64), spread_halves(v, 64), causal, sm_scale,
                                 float(theta) ** (64 // d), warp_specialize)
        return gather_halves(o, d)
    return _CoRopeGqaAttn.apply(q, k, v, causal, sm_scale, theta, warp_specialize)


def corope_attn_gqa(q, k, v, sm_scale=None, theta=10000.0, causal=True):
    """Keyword-friendly form: ``sm_scale`` defaults to 1/sqrt(D)."""
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    return attention(q, k, v, causal, sm_scale, theta)
