"""Fused RoPE flash-attention behind the reference's call surface.

``attention(q, k, v, causal, sm_scale, freqs_cos, freqs_sin[, warp_specialize])`` is positional-only, exactly
like the reference's ``attention = _attention.apply`` (fused-rope/fused_rope_attn.py:652-780); the last argument is
accepted and ignored (it selects a Triton code path there).  ``fused_rope_attn`` is a keyword-friendly wrapper.

Forward and backward run hand-written gfx950 kernels through the C ABI in ``include/corope_amd.h``; there is no
other implementation behind this module.  Tensors are bfloat16 or float16 (the reference's dtype, fused_rope_attn.py:236;
the same kernel sources built for fp16 elements)."""
from __future__ import annotations

import ctypes

import torch

from . import _lib

_SUPPORTED_D = (64, 128, 256)
# 256 (the largest head dim of the reference, fused_rope_attn.py:661) runs one wave per SIMD: the single-launch forward
# kernel (on a rotated key copy from the rotated path's lengths on) and separate dQ, dV and dK kernels.
_ROTATED_PATH_MAX_D = 256
# Head dims of the reference (fused_rope_attn.py:661) below the kernels' own: run at D = 64 with each half of a row padded
# with zeros (the rotation pairs column j with column j + D/2, so the halves must stay the starts of the new halves).
_PADDED_D = (16, 32)


def spread_halves(x, d_to):
    """(..., D) -> (..., d_to): [x[:D/2], 0, x[D/2:], 0]; zero columns add nothing to any dot product."""
    d = x.shape[-1]
    h, z = d // 2, x.new_zeros(x.shape[:-1] + ((d_to - d) // 2,))
    return torch.cat([x[..., :h], z, x[..., h:], z], dim=-1)


def gather_halves(y, d):
    """Inverse of spread_halves on the columns that carry data."""
    h, hp = d // 2, y.shape[-1] // 2
    return torch.cat([y[..., :h], y[..., hp:hp + h]], dim=-1)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_ptr(t):
    """The current HIP stream of t's device as an integer handle (the short way when this torch has it: at the small
    shapes the operator is bound by the host, and torch.cuda.current_stream() builds a Python object per call)."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def _on_device(t):
    """Context in which t's device is the current one; nothing to enter when it already is."""
    return _NO_GUARD if torch.cuda.current_device() == t.device.index else torch.cuda.device(t.device)


def _check_inputs(q, k, v, freqs_cos, freqs_sin):
    # shape constraints of the reference (fused_rope_attn.py:657-661)
    assert q.dim() == 4 and k.dim() == 4 and v.dim() == 4, "q, k, v must be (B, H, N, D)"
    d = q.shape[-1]
    assert d == k.shape[-1] and d == v.shape[-1], "q, k, v must share the head dim"
    # grouped-query attention (an extension: the reference requires one shape): k, v may have fewer heads
    assert k.shape == v.shape, "k and v must share one shape"
    assert q.shape[0] == k.shape[0] and q.shape[2:] == k.shape[2:], "q and k must agree in batch, sequence and head dim"
    assert q.shape[1] % k.shape[1] == 0, "the number of query heads must be a multiple of the number of key/value heads"
    if d not in _SUPPORTED_D:
        raise ValueError(f"head dim {d} not built for gfx950 (kernels: {_SUPPORTED_D}; padded to 64: {_PADDED_D})")
    if not (q.is_cuda and k.is_cuda and v.is_cuda and freqs_cos.is_cuda and freqs_sin.is_cuda):
        raise ValueError("fused RoPE attention runs on the GPU only: all tensors must be on a HIP device")
    if not (q.dtype == k.dtype == v.dtype and q.dtype in (torch.bfloat16, torch.float16)):
        raise ValueError(f"q, k, v must all be bfloat16 or all float16 (got {q.dtype}, {k.dtype}, {v.dtype})")
    n = q.shape[2]
    for name, f in (("freqs_cos", freqs_cos), ("freqs_sin", freqs_sin)):
        if f.dim() != 2 or f.shape[0] < n or f.shape[1] < d // 2:
            raise ValueError(f"{name} must be (N, D) or (N, D/2) with N >= {n}, got {tuple(f.shape)}")


def _freq_table(f):
    """fp32 table with unit column stride and a row stride the kernels accept."""
    if f.dtype != torch.float32:
        f = f.float()
    if f.stride(1) != 1 or f.stride(0) % 4 != 0 or f.data_ptr() % 16 != 0:
        f = f.contiguous()
        if f.stride(0) % 4 != 0:
            f = torch.nn.functional.pad(f, (0, 4 - f.shape[1] % 4)).contiguous()
    return f


# Shapes from which the operator rotates its operands ahead of the attention kernels: K once into a scratch buffer for
# the forward (every K tile is otherwise rotated again by each query block of its head), and, when a gradient will be asked
# for, q and k once for the backward (fused dK+dV, no tables in its loops).  Measured crossover on MI355X, the same for both:
# N * D = 65536 (N = 512 at D = 128, N = 1024 at D = 64); below it every kernel rotates its own tiles.
TWO_LAUNCH_MIN_N = 1024
TRAIN_ROTATED_MIN_ND = 65536


# fp16 tensors, forward of a call that will be differentiated: "exact" = the single-launch kernel's bookkeeping, which
# keeps P and V in fp16 (O within 1.2e-2 of the fp32 oracle at the reference's verification temperature sm_scale = 0.5,
# gradients within its 0.15 / 5e-3 thresholds), from the rotated path's lengths on run on a key copy rotated beforehand;
# "fast" = the pipelined forward (bf16 probabilities against a V converted to bf16 on its way into LDS: as fast as with
# bf16 tensors, O within one bf16 ulp), whose O carries bf16's rounding of V into delta = rowsum(O * dO) and through it
# into dQ and dK: up to 0.24 there instead of 0.05.  A forward that will not be differentiated always takes the fast form.
FP16_TRAINING_FORWARD = "exact"


def use_rotated_path(N, D, training):
    """Whether the operator rotates the operands ahead of the attention kernels at this shape."""
    return D <= _ROTATED_PATH_MAX_D and (N >= TWO_LAUNCH_MIN_N or N * D >= TRAIN_ROTATED_MIN_ND)


def _view_strides(t):
    """(batch, head, row) strides in elements if the kernels can read t where it lies -- last dimension contiguous, rows
    16-byte aligned and at least D apart, as the reference's forward reads q and k through their strides
    (fused_rope_attn.py:709-710) -- else None."""
    sb, sh, sn, sd = t.stride()
    d = t.shape[-1]
    if sd != 1 or sn < d or min(sb, sh) < 0 or sb % 8 or sh % 8 or sn % 8 or t.data_ptr() % 16 or t.shape[2] * sn * 2 >= 1 << 32:
        return None
    return (ctypes.c_int64 * 3)(sb, sh, sn)


def _forward(q, k, v, causal, sm_scale, freqs_cos, freqs_sin, two_launch=None, keep_rotated=False):
    """Runs the forward kernels; returns (o, M, fc, fs, rotated) with the tables in the form the kernels were given.
    ``rotated`` is (q_rot, k_rot) when ``keep_rotated`` was asked for and the two-launch path ran, else None.
    q, k, v may be strided views (a (B, N, H, D) tensor seen as (B, H, N, D), a slice of a fused projection): they are read
    where they lie when their layout allows it, else copied."""
    lib = _lib.load()
    fc, fs = _freq_table(freqs_cos), _freq_table(freqs_sin)
    if fc.stride(0) != fs.stride(0):
        fc, fs = fc.contiguous(), fs.contiguous()
    B, H, N, D = q.shape
    strides = None
    if not (q.is_contiguous() and k.is_contiguous() and v.is_contiguous()):
        strides = tuple(_view_strides(t) for t in (q, k, v))
        if any(st is None for st in strides) or D > _ROTATED_PATH_MAX_D:
            q, k, v, strides = q.contiguous(), k.contiguous(), v.contiguous(), None
    o = torch.empty(q.shape, device=q.device, dtype=q.dtype)
    M = torch.empty((B, H, N), device=q.device, dtype=torch.float32)
    if two_launch is None:
        two_launch = use_rotated_path(N, D, training=keep_rotated)
    rotated = None
    Hkv = k.shape[1]
    with _on_device(q):
        if strides is not None:
            fp16 = q.dtype == torch.float16
            # fp16 with gradients: P and V stay fp16 (no key-norm maxima: the single-launch kernel, on the rotated copy)
            exact = fp16 and keep_rotated and FP16_TRAINING_FORWARD != "fast"
            q_rot = torch.empty(q.shape, device=q.device, dtype=q.dtype) if (two_launch and keep_rotated) else None
            k_rot = torch.empty(k.shape, device=q.device, dtype=q.dtype) if two_launch else None
            kmax = torch.empty((B, Hkv, (N + 63) // 64), device=q.device, dtype=torch.float32) if (two_launch and not exact) else None
            rc = lib.corope_rope_attn_fwd_strided(q.data_ptr(), strides[0], k.data_ptr(), strides[1], v.data_ptr(), strides[2],
                                                  fc.data_ptr(), fs.data_ptr(), fc.stride(0), o.data_ptr(), M.data_ptr(),
                                                  q_rot.data_ptr() if q_rot is not None else None,
                                                  k_rot.data_ptr() if k_rot is not None else None,
                                                  kmax.data_ptr() if kmax is not None else None, B, H, Hkv, N, D,
                                                  float(sm_scale), int(bool(causal)), int(fp16), _stream_ptr(q))
            _lib.check(rc, "corope_rope_attn_fwd_strided")
            if q_rot is not None:
                rotated = (q_rot, k_rot)
        elif q.dtype == torch.float16:
            # the reference's dtype: one entry point covers the forms, grouped-query K/V included.  With key-norm maxima: the
            # pipelined kernel (bf16 probabilities against a V converted to bf16 on its way into LDS); without, for a forward
            # with gradients: the single-launch kernel on the rotated copy, P and V in fp16
            exact = keep_rotated and FP16_TRAINING_FORWARD != "fast"
            q_rot = torch.empty_like(q) if (two_launch and keep_rotated) else None
            k_rot = torch.empty_like(k) if two_launch else None
            kmax = torch.empty((B, Hkv, (N + 63) // 64), device=q.device, dtype=torch.float32) if (two_launch and not exact) else None
            rc = lib.corope_rope_attn_fwd_f16(q.data_ptr(), k.data_ptr(), v.data_ptr(), fc.data_ptr(), fs.data_ptr(),
                                              fc.stride(0), o.data_ptr(), M.data_ptr(),
                                              q_rot.data_ptr() if q_rot is not None else None,
                                              k_rot.data_ptr() if k_rot is not None else None,
                                              kmax.data_ptr() if kmax is not None else None, B, H, Hkv, N, D,
                                              float(sm_scale), int(bool(causal)), _stream_ptr(q))
            _lib.check(rc, "corope_rope_attn_fwd_f16")
            if q_rot is not None:
                rotated = (q_rot, k_rot)
        elif Hkv != H:   # grouped-query attention: one entry point covers the three forms
            q_rot = torch.empty_like(q) if (two_launch and keep_rotated) else None
            k_rot = torch.empty_like(k) if two_launch else None
            kmax = torch.empty((B, Hkv, (N + 63) // 64), device=q.device, dtype=torch.float32) if two_launch else None
            rc = lib.corope_rope_attn_fwd_gqa(q.data_ptr(), k.data_ptr(), v.data_ptr(), fc.data_ptr(), fs.data_ptr(),
                                              fc.stride(0), o.data_ptr(), M.data_ptr(),
                                              q_rot.data_ptr() if q_rot is not None else None,
                                              k_rot.data_ptr() if k_rot is not None else None,
                                              kmax.data_ptr() if kmax is not None else None, B, H, Hkv, N, D,
                                              float(sm_scale), int(bool(causal)), _stream_ptr(q))
            _lib.check(rc, "corope_rope_attn_fwd_gqa")
            if q_rot is not None:
                rotated = (q_rot, k_rot)
        elif two_launch and keep_rotated:
            q_rot, k_rot = torch.empty_like(q), torch.empty_like(k)
            kmax = torch.empty((B, H, (N + 63) // 64), device=q.device, dtype=torch.float32)
            rc = lib.corope_rope_attn_fwd_train(q.data_ptr(), k.data_ptr(), v.data_ptr(), fc.data_ptr(), fs.data_ptr(),
                                                fc.stride(0), o.data_ptr(), M.data_ptr(), q_rot.data_ptr(), k_rot.data_ptr(),
                                                kmax.data_ptr(), B, H, N, D, float(sm_scale), int(bool(causal)),
                                                _stream_ptr(q))
            _lib.check(rc, "corope_rope_attn_fwd_train")
            rotated = (q_rot, k_rot)
        elif two_launch:
            nbytes = lib.corope_rope_attn_fwd_workspace_bytes(B, H, N, D)
            if nbytes < 0:
                _lib.check(lib.corope_rope_attn_check(B, H, N, D, fc.stride(0), float(sm_scale), 0), "corope_rope_attn_check")
            ws = torch.empty(nbytes, device=q.device, dtype=torch.uint8)
            rc = lib.corope_rope_attn_fwd_ws(q.data_ptr(), k.data_ptr(), v.data_ptr(), fc.data_ptr(), fs.data_ptr(),
                                             fc.stride(0), o.data_ptr(), M.data_ptr(), B, H, N, D, float(sm_scale),
                                             int(bool(causal)), ws.data_ptr(), nbytes, _stream_ptr(q))
            _lib.check(rc, "corope_rope_attn_fwd_ws")
        else:
            rc = lib.corope_rope_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), fc.data_ptr(), fs.data_ptr(),
                                          fc.stride(0), o.data_ptr(), M.data_ptr(), B, H, N, D, float(sm_scale),
                                          int(bool(causal)), _stream_ptr(q))
            _lib.check(rc, "corope_rope_attn_fwd")
    return o, M, fc, fs, rotated


class _FusedRopeAttn(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, causal, sm_scale, freqs_cos, freqs_sin, warp_specialize=True):
        _check_inputs(q, k, v, freqs_cos, freqs_sin)
        B, H, N, D = q.shape
        training = any(ctx.needs_input_grad[:3])
        if training:
            v = v.contiguous()         # the backward kernels read v row-major; q and k they read as the forward left them
        # when a gradient will be asked for, the forward keeps its rotated q and k for the backward and the originals
        # are not saved (the reference saves q and k, fused_rope_attn.py:718, and re-rotates them in its backward)
        o, M, fc, fs, rotated = _forward(q, k, v, causal, sm_scale, freqs_cos, freqs_sin, keep_rotated=training)
        ctx.rotated = rotated is not None
        if ctx.rotated:
            ctx.save_for_backward(rotated[0], rotated[1], v, o, M, fc, fs)
        else:
            ctx.save_for_backward(q.contiguous(), k.contiguous(), v.contiguous(), o, M, fc, fs)
        ctx.sm_scale = float(sm_scale)
        ctx.HEAD_DIM = D
        ctx.causal = bool(causal)
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, M, fc, fs = ctx.saved_tensors
        lib = _lib.load()
        do = do.contiguous()
        if do.dtype != q.dtype:
            do = do.to(q.dtype)
        B, H, N, D = q.shape
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        delta = torch.empty_like(M)
        with _on_device(q):
            if q.dtype == torch.float16:
                ws, nbytes = None, 0
                if not ctx.rotated and use_rotated_path(N, D, training=True):   # rotate q and k once, then the kernels on the copies
                    nbytes = lib.corope_rope_attn_bwd_workspace_bytes(B, H, N, D)
                    ws = torch.empty(nbytes, device=q.device, dtype=torch.uint8)
                rc = lib.corope_rope_attn_bwd_f16(q.data_ptr(), k.data_ptr(), int(ctx.rotated), v.data_ptr(), o.data_ptr(), do.data_ptr(),
                                                  M.data_ptr(), delta.data_ptr(), fc.data_ptr(), fs.data_ptr(), fc.stride(0),
                                                  dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, H, k.shape[1], N, D,
                                                  ctx.sm_scale, int(ctx.causal), ws.data_ptr() if ws is not None else None,
                                                  nbytes, _stream_ptr(q))
            elif k.shape[1] != H:         # grouped-query attention
                rc = lib.corope_rope_attn_bwd_gqa(q.data_ptr(), k.data_ptr(), int(ctx.rotated), v.data_ptr(), o.data_ptr(),
                                                  do.data_ptr(), M.data_ptr(), delta.data_ptr(), fc.data_ptr(), fs.data_ptr(),
                                                  fc.stride(0), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, H,
                                                  k.shape[1], N, D, ctx.sm_scale, int(ctx.causal), _stream_ptr(q))
            elif ctx.rotated:           # q, k are the rotated copies the forward kept
                rc = lib.corope_rope_attn_bwd_prerotated(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                                         do.data_ptr(), M.data_ptr(), delta.data_ptr(), fc.data_ptr(),
                                                         fs.data_ptr(), fc.stride(0), dq.data_ptr(), dk.data_ptr(),
                                                         dv.data_ptr(), B, H, N, D, ctx.sm_scale, int(ctx.causal),
                                                         _stream_ptr(q))
            elif use_rotated_path(N, D, training=True):   # rotate q and k once, then run the kernels on the rotated copies
                nbytes = lib.corope_rope_attn_bwd_workspace_bytes(B, H, N, D)
                ws = torch.empty(nbytes, device=q.device, dtype=torch.uint8)
                rc = lib.corope_rope_attn_bwd_ws(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), do.data_ptr(),
                                                 M.data_ptr(), delta.data_ptr(), fc.data_ptr(), fs.data_ptr(),
                                                 fc.stride(0), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, H, N, D,
                                                 ctx.sm_scale, int(ctx.causal), ws.data_ptr(), nbytes, _stream_ptr(q))
            else:
                rc = lib.corope_rope_attn_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), do.data_ptr(),
                                              M.data_ptr(), delta.data_ptr(), fc.data_ptr(), fs.data_ptr(), fc.stride(0),
                                              dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, H, N, D, ctx.sm_scale,
                                              int(ctx.causal), _stream_ptr(q))
        _lib.check(rc, "corope_rope_attn_bwd")
        return dq, dk, dv, None, None, None, None, None


def attention(q, k, v, causal, sm_scale, freqs_cos, freqs_sin, warp_specialize=True):
    """The reference's ``attention = _attention.apply`` (fused-rope/fused_rope_attn.py:780): positional arguments in its
    order.  Head dims 64 and 128 go to the kernels as they are; 16 and 32 are padded to 64 around the same kernels (zero
    columns, tables padded with the identity rotation), which changes no value of the result."""
    d = q.shape[-1]
    if d in _PADDED_D and q.dim() == 4 and k.shape[-1] == d and v.shape[-1] == d:
        h, pad = d // 2, (64 - d) // 2
        fc = torch.cat([freqs_cos[:, :h].float(), freqs_cos.new_ones((freqs_cos.shape[0], pad), dtype=torch.float32)], dim=1)
        fs = torch.cat([freqs_sin[:, :h].float(), freqs_sin.new_zeros((freqs_sin.shape[0], pad), dtype=torch.float32)], dim=1)
        o = _FusedRopeAttn.apply(spread_halves(q, 64), spread_halves(k, 64), spread_halves(v, 64), causal, sm_scale, fc, fs,
                                 warp_specialize)
        return gather_halves(o, d)
    return _FusedRopeAttn.apply(q, k, v, causal, sm_scale, freqs_cos, freqs_sin, warp_specialize)


def fused_rope_attn(q, k, v, freqs_cos, freqs_sin, causal=True, sm_scale=None):
    """Keyword-friendly form: ``sm_scale`` defaults to 1/sqrt(D)."""
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    return attention(q, k, v, causal, sm_scale, freqs_cos, freqs_sin)


def rope_attn_forward_with_lse(q, k, v, causal, sm_scale, freqs_cos, freqs_sin, two_launch=None):
    """Forward only, returning (O, M) where M is the saved base-2 log-sum-exp statistic (B, H, N) fp32.
    ``two_launch`` forces (True / False) or leaves to the length rule (None) the choice of forward path."""
    _check_inputs(q, k, v, freqs_cos, freqs_sin)
    o, M, _, _, _ = _forward(q, k, v, causal, sm_scale, freqs_cos, freqs_sin, two_launch)
    return o, M


def rope_rotate(x, freqs_cos, freqs_sin, with_tile_max=False, scale=1.0):
    """``scale`` times the half-layout rotation of x (B, H, N, D) bf16 on the device (fp32 arithmetic, one rounding to
    bf16).  Returns y, or (y, tile_max) with the largest row norm of y in every 64-row tile, (B, H, ceil(N/64)) fp32.
    The pre-rotated operands of the backward kernels are ``rope_rotate(k, ...)`` and
    ``rope_rotate(q, ..., scale=sm_scale * log2(e))``."""
    _check_inputs(x, x, x, freqs_cos, freqs_sin)
    if x.dtype != torch.bfloat16:
        raise ValueError("the rotation pass is built for bfloat16 only")
    lib = _lib.load()
    x = x.contiguous()
    fc, fs = _freq_table(freqs_cos), _freq_table(freqs_sin)
    if fc.stride(0) != fs.stride(0):
        fc, fs = fc.contiguous(), fs.contiguous()
    B, H, N, D = x.shape
    y = torch.empty_like(x)
    tm = torch.empty((B, H, (N + 63) // 64), device=x.device, dtype=torch.float32) if with_tile_max else None
    with _on_device(x):
        rc = lib.corope_rope_rotate(x.data_ptr(), fc.data_ptr(), fs.data_ptr(), fc.stride(0), y.data_ptr(),
                                    tm.data_ptr() if with_tile_max else None, B, H, N, D, float(scale), _stream_ptr(x))
    _lib.check(rc, "corope_rope_rotate")
    return (y, tm) if with_tile_max else y
