#!/usr/bin/env python3
"""Benchmark of the fused RoPE flash-attention hot path on one MI355X.

One step = one forward + one backward of the operator (through its public torch.autograd.Function) on the
metric shape B2 H32 N4096 D128, causal, bf16, synthetic N(0,1) inputs resident in HBM.  Prints ONE JSON line:
whole-step TFLOP/s by the reference's FLOP model (4*B*H*N^2*D, halved for causal, x2.5 for the backward,
rotation FLOPs not counted), the roofline of the dominant kernel from per-launch HIP-event timings, and the CPU
oracle timed on the host cores as a baseline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2|c3|c4|c5] [--no-cpu-baseline]
                    [--parity | --no-parity] [--data normal|sink] [--phase-trace] [--sweep [--lanes] [--flush]]
                    [--mfma-rate] [--hbm-passes]

(c3 is the metric shape and the default; c2/c4 are the other RoPE-attention shapes; c5 is the Co-RoPE GQA forward,
with its backward timed beside it.)  --parity adds per-tensor errors against the CPU oracle to the line (outside the
timed region); --data sink times the same shape on attention-sink-like keys; --phase-trace splits the three attention
kernels into prologue / steady state / diagonal / epilogue from time stamps taken inside the kernels (needs the
trace build of the library that co-rope_amd/build.py makes beside the shipped one).
"""
import argparse
import importlib
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA peak used for every "fraction of peak" below
PEAK_HBM_GBS = 8000.0

# HBM bytes per launch (read + written) measured with rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE on this
# benchmark (summary and commands: profiles/rope_attn_c3_c4_hbm_traffic.md); FETCH_SIZE is scaled by 2.0 and WRITE_SIZE
# by 1.0, the factors a plain 1 GiB device copy gives for the same counters.
HBM_TRAFFIC_BYTES = {
    ("c3", "rope_attn_fwd"): int((305561 * 2.0 + 132096) * 1024),
    ("c3", "rope_attn_bwd_dq"): int((404872 * 2.0 + 91136) * 1024),
    ("c3", "rope_attn_bwd_dkdv"): int((312964 * 2.0 + 131072) * 1024),
    ("c4", "rope_attn_fwd"): int((1073484 * 2.0 + 243220) * 1024),
    # Co-RoPE at C5 (profiles/corope_gqa_c5_hbm_traffic.md): the forward kernel; the backward's six launches together
    ("c5", "corope_gqa_fwd"): int((70416 * 2.0 + 65536) * 1024),
    ("c5", "corope_gqa_bwd"): int(((2 * 22429 + 701939 + 48483 + 226967 + 298542) * 2.0
                                   + (2 * 188709 + 1422980 + 2364 + 2341 + 2341)) * 1024),
}

CONFIGS = {
    "c2": dict(B=4, H=8, N=1024, D=64, name="C2: fused RoPE flash-attention fwd+bwd B4 H8 N1024 D64 causal bf16"),
    "c3": dict(B=2, H=32, N=4096, D=128, name="C3: fused RoPE flash-attention fwd+bwd B2 H32 N4096 D128 causal bf16"),
    "c4": dict(B=1, H=8, N=65536, D=128, name="C4: fused RoPE flash-attention fwd B1 H8 N65536 D128 causal bf16"),
}


SETTLE_SECONDS = 0.1


def settle_clocks(step, torch):
    """Untimed: keeps running `step` until SETTLE_SECONDS of sustained load have passed.  The first ~50 ms after an idle
    period run at other clocks than what follows (the matrix kernels 3-10 % slower, the vector-bound ones a little faster),
    so a short --warmup alone would time the transient.  Returns the number of extra steps."""
    step()                       # first call: library load, kernel attributes, allocator growth
    torch.cuda.synchronize()
    n, t0 = 1, time.perf_counter()
    while time.perf_counter() - t0 < SETTLE_SECONDS:
        for _ in range(16):
            step()
        torch.cuda.synchronize()
        n += 16
    return n


def calc_sim(x, y):
    """The reference's similarity measure, 2 sum(xy) / sum(x^2 + y^2) in fp64 (utils.py:12-19): 1 for equal tensors."""
    x, y = x.double(), y.double()
    den = (x * x + y * y).sum()
    return 1.0 if float(den) == 0.0 else float(2 * (x * y).sum() / den)


def make_inputs(B, H, N, D, data, torch, seed=42):
    """q, k, v, dO (bf16-representable fp32, on the host).  "normal": N(0,1).  "sink": the same with an attention-sink
    first key (x8), one outlier key in 1000 (x16) and key norms growing 0.5 -> 2 along the sequence -- the per-tile norm
    bounds of the two-launch forward are then far above the scores that occur, and rise tile after tile."""
    g = torch.Generator().manual_seed(seed)
    q, k, v, do = (torch.randn(B, H, N, D, generator=g) for _ in range(4))
    if data == "sink":
        k = k * torch.linspace(0.5, 2.0, N).reshape(1, 1, N, 1)
        k[:, :, 0] *= 8
        k[:, :, 7::1000] *= 16
    elif data != "normal":
        sys.exit(f"bench.py: unknown --data {data}")
    return tuple(t.to(torch.bfloat16).float() for t in (q, k, v, do))


def err_stats(got, ref, torch):
    """max / mean / percentiles of |got - ref| as the reference's verification script prints them (verification.py:91-114)."""
    d = (got.float() - ref.float()).abs().flatten()
    if d.numel() > (1 << 24):        # torch.quantile refuses more than 2^24 elements: a fixed stride sample for the percentiles
        dq = d[:: d.numel() // (1 << 24) + 1]
    else:
        dq = d
    qs = torch.quantile(dq, torch.tensor([0.5, 0.95, 0.99]))
    return {"max_abs": float(d.max()), "mean_abs": float(d.mean()), "p50": float(qs[0]), "p95": float(qs[1]),
            "p99": float(qs[2]), "max_abs_ref": float(ref.abs().max()), "calc_sim": round(calc_sim(got, ref), 8),
            "n": int(d.numel())}


def sample_rows(N, n, torch, seed=1):
    g = torch.Generator().manual_seed(seed)
    r = torch.randperm(N, generator=g)[:n]
    return torch.unique(torch.cat([r, torch.tensor([0, 1, 63, 64, N // 2, N - 2, N - 1]).clamp(0, N - 1)]))


def rope_parity(pkg, cfg_name, q, k, v, do, cos, sin, scale, fwd_only, torch, quick=False):
    """Per-tensor errors of the HIP path against the fp32 CPU oracle on the same bf16-rounded inputs: O (and the row
    statistic) on sampled rows of every head, dQ / dK / dV on whole heads (all of them at C2, 8 at C3).  ``quick``: the
    sample every run of the benchmark carries in its line (32 rows of every head, 2 whole heads: seconds of host time)."""
    from oracle import rope_attn_oracle as O
    B, H, N, D = q.shape
    dev = torch.device("cuda:0")
    qd, kd, vd = (t.to(dev, torch.bfloat16).requires_grad_(not fwd_only) for t in (q, k, v))
    o = pkg.attention(qd, kd, vd, True, scale, cos, sin)
    if not fwd_only:
        o.backward(do.to(dev, torch.bfloat16))
    torch.cuda.synchronize()
    o = o.detach().float().cpu()
    rows = sample_rows(N, 25 if quick else (128 if N <= 8192 else 48), torch)
    c, s = cos.float().cpu(), sin.float().cpu()
    ro, _ = O.rope_attn_forward_blocked(q, k, v, True, scale, c, s, rows=rows)
    out = {"bar": "max-abs <= 2e-2 against the fp32 oracle (one bf16 ulp of the reference value where that is larger)",
           "O": dict(err_stats(o[:, :, rows], ro, torch), sample=f"{rows.numel()} rows x {B * H} heads")}
    if not fwd_only:
        heads = [(b, h) for b in range(B) for h in range(H)]
        if quick:
            heads = [heads[len(heads) // 3], heads[-1]]
        elif len(heads) > 32:
            heads = heads[:: len(heads) // 8][:8]
        acc = {n: ([], []) for n in ("dQ", "dK", "dV")}
        for (b, h) in heads:
            sl = (slice(b, b + 1), slice(h, h + 1))
            _, _, rdq, rdk, rdv, _ = O.rope_attn_fwd_bwd_blocked(q[sl], k[sl], v[sl], do[sl], True, scale, c, s)
            for n, t, r in (("dQ", qd, rdq), ("dK", kd, rdk), ("dV", vd, rdv)):
                acc[n][0].append(t.grad[sl].float().cpu())
                acc[n][1].append(r)
        for n, (got, ref) in acc.items():
            out[n] = dict(err_stats(torch.cat(got), torch.cat(ref), torch), sample=f"{len(heads)} whole heads of {B * H}")
    return out


def corope_parity(pkg, q, k, v, do, o_gpu, grads_gpu, scale, theta, torch):
    """Per-tensor errors of the Co-RoPE kernels against the fp32 CPU oracle: O and dQ on sampled query rows of every head
    (a query row's output depends on no other query row, so autograd through the row-sampled oracle gives its dQ), dK and
    dV of one whole (batch, key/value head) group, accumulated by autograd over all its query rows, 64 at a time."""
    from oracle import corope_gqa_oracle as C
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    dq_g, dk_g, dv_g = grads_gpu
    rows = sample_rows(N, 9, torch, seed=3)
    qa = q.clone().requires_grad_(True)
    ref = C.corope_gqa_forward_rows(qa, k, v, True, scale, theta, rows, torch.float32, row_block=16)
    (ref_dq,) = torch.autograd.grad(ref, qa, do[:, :, rows])
    out = {"bar": "max-abs <= 2e-2 against the fp32 oracle (dK, dV: x sqrt(group size), sums over the group's heads)",
           "O": dict(err_stats(o_gpu[:, :, rows], ref.detach(), torch), sample=f"{rows.numel()} rows x {B * Hq} heads"),
           "dQ": dict(err_stats(dq_g[:, :, rows], ref_dq[:, :, rows], torch), sample=f"{rows.numel()} rows x {B * Hq} heads")}
    b, kv = B - 1, Hkv // 2                       # one whole group
    qs, dos = q[b:b + 1, kv * G:(kv + 1) * G], do[b:b + 1, kv * G:(kv + 1) * G]
    kx, vx = (t[b:b + 1, kv:kv + 1].clone().requires_grad_(True) for t in (k, v))
    for r0 in range(0, N, 64):
        hi = min(r0 + 64, N)
        blk = C.corope_gqa_forward_rows(qs[:, :, :hi], kx[:, :, :hi], vx[:, :, :hi], True, scale, theta,
                                        torch.arange(r0, hi), torch.float32, row_block=64)
        blk.backward(dos[:, :, r0:hi])
    out["dK"] = dict(err_stats(dk_g[b:b + 1, kv:kv + 1], kx.grad, torch), sample=f"group (batch {b}, kv head {kv}), all {N} keys")
    out["dV"] = dict(err_stats(dv_g[b:b + 1, kv:kv + 1], vx.grad, torch), sample=f"group (batch {b}, kv head {kv}), all {N} keys")
    return out


def attention_flops(B, H, N, D, mode, causal=True):
    total = 4.0 * B * H * N * N * D * (0.5 if causal else 1.0)
    return total * (2.5 if mode == "bwd" else 1.0)


def cpu_baseline():
    """The oracle (an eager-PyTorch port of the reference's rope_attn_pytorch path) at the reference's CPU-runnable
    configuration: B4 H8 N512 D64 fp32, forward + backward."""
    import torch
    from oracle import rope_attn_oracle as O
    B, H, N, D = 4, 8, 512, 64
    g = torch.Generator().manual_seed(0)
    q, k, v, do = (torch.randn(B, H, N, D, generator=g) for _ in range(4))
    cos, sin = O.precompute_freqs_cis(D, N)
    scale = 1 / math.sqrt(D)

    def step():
        _, _, saved = O.rope_attn_forward(q, k, v, True, scale, cos, sin)
        O.rope_attn_backward(saved, do, True, scale, cos, sin)

    for _ in range(2):
        step()
    times = []
    t_end = time.perf_counter() + 15.0
    while len(times) < 5 or (time.perf_counter() < t_end and len(times) < 40):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    flops = attention_flops(B, H, N, D, "fwd") + attention_flops(B, H, N, D, "bwd")
    return {"value": round(flops / med * 1e-12, 5), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "kind": "port", "ms_per_step": round(med * 1e3, 3),
            "sample": f"oracle fwd+bwd at B4 H8 N512 D64 fp32 causal, median of {len(times)} reps after 2 warm-ups, "
                      f"os.cpu_count()={os.cpu_count()}"}


# the 19 shapes of the reference's comparison harness (fused-rope/bench_compare.py:323-350): (B, H, N, D, name), causal
SWEEP = [(4, 8, 512, 64, "Small-512"), (4, 8, 1024, 64, "Small-1K"), (2, 8, 2048, 64, "Small-2K"),
         (2, 8, 4096, 64, "Small-4K"), (1, 8, 8192, 64, "Small-8K"),
         (4, 32, 512, 128, "Llama7B-512"), (4, 32, 1024, 128, "Llama7B-1K"), (2, 32, 2048, 128, "Llama7B-2K"),
         (2, 32, 4096, 128, "Llama7B-4K"), (1, 32, 8192, 128, "Llama7B-8K"), (1, 32, 16384, 128, "Llama7B-16K"),
         (2, 64, 512, 128, "Llama70B-512"), (2, 64, 1024, 128, "Llama70B-1K"), (1, 64, 2048, 128, "Llama70B-2K"),
         (1, 64, 4096, 128, "Llama70B-4K"), (1, 32, 8192, 128, "Llama70B-8K"),
         (1, 16, 32768, 128, "Long-32K"), (1, 8, 65536, 128, "Long-64K"), (1, 4, 131072, 128, "Long-128K")]


def sweep_protocol(N):
    """(warm-up, measurement) in milliseconds for a sequence length: the reference harness's table
    (fused-rope/bench_compare.py:390-401), whose timer takes both as durations, not counts."""
    if N >= 262144:
        return 20, 30
    if N >= 131072:
        return 25, 50
    if N >= 65536:
        return 50, 100
    if N >= 32768:
        return 50, 150
    if N >= 8192:
        return 100, 200
    return 100, 300


def timed_reps(fn, N, torch, flush_buf=None):
    """(median, min, max) ms of fn over repetitions timed one by one with HIP events, as the reference harness's timer does
    (fused-rope/bench_compare.py:30-58): the duration of one call is estimated from 5 calls, then warm-up and measurement
    run for the durations sweep_protocol gives (the warm-up never shorter than SETTLE_SECONDS of sustained load, so that
    every shape and lane is timed at settled clocks, like the headline line).  flush_buf: a buffer larger than every cache,
    overwritten by a fill kernel before each timed call (that timer's cold-cache protocol); None: calls back to back."""
    warm_ms, rep_ms = sweep_protocol(N)
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        fn()
    e1.record()
    torch.cuda.synchronize()
    est = max(e0.elapsed_time(e1) / 5, 1e-3)
    n_warm = max(1, int(max(warm_ms, SETTLE_SECONDS * 1e3) / est))
    n_rep = max(5, min(1000, int(rep_ms / est)))
    for _ in range(n_warm):
        fn()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_rep)]
    for a, b in evs:
        if flush_buf is not None:
            flush_buf.zero_()
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    t = sorted(a.elapsed_time(b) for a, b in evs)
    return statistics.median(t), t[0], t[-1]


def bench_sweep(args):
    """Forward and backward-only times (HIP-event timings, backward with the forward graph retained, as the reference's
    harness does) for the reference's 19 shapes; one JSON line per shape: median / min / max of back-to-back calls at
    settled clocks and, with --flush, of calls that each start on flushed caches."""
    import torch
    pkg = importlib.import_module("corope_amd")
    dev = torch.device("cuda:0")
    flush_buf = torch.empty(512 << 20, dtype=torch.uint8, device=dev) if args.flush else None
    dtype = torch.float16 if args.dtype == "fp16" else torch.bfloat16
    pkg.rope_attn.FP16_TRAINING_FORWARD = args.fp16_forward
    shapes = [s for s in SWEEP if args.only is None or s[4] in args.only.split(",")]
    if args.shape is not None:
        B, H, N, D = (int(x) for x in args.shape.split(","))
        shapes = [(B, H, N, D, f"B{B}-H{H}-N{N}-D{D}")]
    for (B, H, N, D, name) in shapes:
        sm_scale = args.sm_scale if args.sm_scale is not None else 0.5   # the reference harness's value
        g = torch.Generator().manual_seed(0)
        q, k, v, do = (torch.randn(B, H, N, D, generator=g).to(dev, dtype) for _ in range(4))
        cos, sin = pkg.rope_freqs_device(D, N, 10000.0, device=dev)
        q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
        stats = {}

        def timed(fn, key=None):
            med, lo, hi = timed_reps(fn, N, torch)
            if key is not None:
                stats[key + "_min_ms"], stats[key + "_max_ms"] = round(lo, 4), round(hi, 4)
                if flush_buf is not None:
                    fm, fl, fh = timed_reps(fn, N, torch, flush_buf)
                    stats[key + "_flushed_ms"] = round(fm, 4)
                    stats[key + "_flushed_min_ms"], stats[key + "_flushed_max_ms"] = round(fl, 4), round(fh, 4)
            return med

        f_ms = timed(lambda: pkg.attention(q, k, v, True, sm_scale, cos, sin), "fwd")
        o = pkg.attention(q, k, v, True, sm_scale, cos, sin)

        def clear_grads():   # otherwise every call after the first also runs three accumulate-into-.grad kernels
            q.grad = k.grad = v.grad = None

        b_ms = timed(lambda: (clear_grads(), o.backward(do, retain_graph=True)), "bwd")
        ff, fb = attention_flops(B, H, N, D, "fwd"), attention_flops(B, H, N, D, "bwd")
        row = {"config": name, "B": B, "H": H, "N": N, "D": D, "dtype": args.dtype, "sm_scale": sm_scale, "fwd_ms": round(f_ms, 4),
               "fwd_tflops": round(ff / f_ms * 1e-9, 1), "bwd_ms": round(b_ms, 4), "bwd_tflops": round(fb / b_ms * 1e-9, 1)}
        row.update(stats)
        if args.lanes:
            # the reference harness's comparison lanes (fused-rope/bench_compare.py:98-260), on this GPU:
            #   unfused = a separate rotation pass over q and k, then the same attention kernels with identity tables
            #             (backward: those kernels plus the inverse rotation of dq and dk, timed as two more passes);
            #   sdpa    = the same rotation passes, then PyTorch's scaled_dot_product_attention.
            qd, kd, vd = q.detach(), k.detach(), v.detach()
            one, zero = torch.ones_like(cos), torch.zeros_like(sin)
            rot_ms = timed(lambda: (pkg.rope_rotate(qd, cos, sin), pkg.rope_rotate(kd, cos, sin)))
            qr = pkg.rope_rotate(qd, cos, sin).requires_grad_(True)
            kr = pkg.rope_rotate(kd, cos, sin).requires_grad_(True)
            uf_ms = rot_ms + timed(lambda: pkg.attention(qr, kr, v, True, sm_scale, one, zero))
            ou = pkg.attention(qr, kr, v, True, sm_scale, one, zero)

            def clear_rot_grads():
                qr.grad = kr.grad = v.grad = None

            ub_ms = rot_ms + timed(lambda: (clear_rot_grads(), ou.backward(do, retain_graph=True)))
            row.update({"unfused_fwd_ms": round(uf_ms, 4), "unfused_bwd_ms": round(ub_ms, 4),
                        "fwd_speedup_vs_unfused": round(uf_ms / f_ms, 3), "bwd_speedup_vs_unfused": round(ub_ms / b_ms, 3),
                        "calc_sim_vs_unfused": round(calc_sim(o.detach(), ou.detach()), 8)})
            try:
                sdpa = torch.nn.functional.scaled_dot_product_attention
                sf_ms = rot_ms + timed(lambda: sdpa(qr, kr, v, is_causal=True, scale=sm_scale))
                osd = sdpa(qr, kr, v, is_causal=True, scale=sm_scale)
                sb_ms = rot_ms + timed(lambda: (clear_rot_grads(), osd.backward(do, retain_graph=True)))
                row.update({"sdpa_fwd_ms": round(sf_ms, 4), "sdpa_bwd_ms": round(sb_ms, 4),
                            "fwd_speedup_vs_sdpa": round(sf_ms / f_ms, 3), "bwd_speedup_vs_sdpa": round(sb_ms / b_ms, 3)})
                del osd
            except Exception as e:   # a shape PyTorch's kernels do not take on this build
                row["sdpa_error"] = type(e).__name__
            del qr, kr, ou
        print(json.dumps(row), flush=True)
        del q, k, v, do, o


def bench_corope(args):
    """C5: Co-RoPE GQA forward, B2 Hq32 Hkv8 N4096 D128 bf16 causal.  VALU/transcendental-bound: reported as ms,
    attention-equivalent TFLOP/s and (sin, cos) pairs per second, not as an MFMA fraction."""
    import torch
    pkg = importlib.import_module("corope_amd")
    lib = pkg._lib.load()
    dev = torch.device("cuda:0")
    B, Hq, Hkv, N, D = 2, 32, 8, 4096, 128
    scale = 1 / math.sqrt(D)
    g = torch.Generator().manual_seed(42)
    q = torch.randn(B, Hq, N, D, generator=g).to(dev, torch.bfloat16)
    k, v = (torch.randn(B, Hkv, N, D, generator=g).to(dev, torch.bfloat16) for _ in range(2))
    o = torch.empty_like(q)
    stream = torch.cuda.current_stream().cuda_stream

    def step():
        rc = lib.corope_gqa_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), B, Hq, Hkv, N, D, scale, 10000.0, stream)
        if rc != 0:
            sys.exit(pkg._lib.last_error())

    settle_steps = settle_clocks(step, torch)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    evs[0].record()
    for i in range(args.steps):
        step()
        evs[i + 1].record()
    torch.cuda.synchronize()
    kms = sum(evs[i].elapsed_time(evs[i + 1]) for i in range(args.steps)) / args.steps
    flops = attention_flops(B, Hq, N, D, "fwd")
    pairs = B * Hkv * N * (N + 1) / 2 * D / 2

    # backward (dq, dk, dv from q, k, v, dO): same shape, caller-owned workspace
    do = torch.randn(B, Hq, N, D, generator=g).to(dev, torch.bfloat16)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    ws_bytes = lib.corope_gqa_bwd_workspace_bytes(B, Hq, Hkv, N, D)
    wsp = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)

    def bwd_step():
        rc = lib.corope_gqa_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), do.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                                dv.data_ptr(), B, Hq, Hkv, N, D, scale, 10000.0, wsp.data_ptr(), ws_bytes, stream)
        if rc != 0:
            sys.exit(pkg._lib.last_error())

    bsteps = max(3, args.steps // 3)

    def time_bwd():
        for _ in range(2):
            bwd_step()
        bev = [torch.cuda.Event(enable_timing=True) for _ in range(bsteps + 1)]
        bev[0].record()
        for i in range(bsteps):
            bwd_step()
            bev[i + 1].record()
        torch.cuda.synchronize()
        return sum(bev[i].elapsed_time(bev[i + 1]) for i in range(bsteps)) / bsteps

    bms = time_bwd()
    # the same backward with less scratch: the groups are then walked in passes of as many as fit
    full_bytes, one = ws_bytes, lib.corope_gqa_bwd_min_workspace_bytes(B, Hq, Hkv, N, D)
    by_workspace = {}
    for groups in (4, 1):
        ws_bytes = groups * one
        by_workspace[f"{groups} of {B * Hkv} groups per pass, {ws_bytes / 2**30:.2f} GiB"] = round(time_bwd(), 4)
    ws_bytes = full_bytes
    # issue slots per (sin, cos) pair, counted as for the forward (a transcendental = 2 slots): scores kernel 11 + 4 (phase
    # 2, unpack 2, rotate 4, pack 1, LDS 2; sin, cos); dk kernel 8 + 4 (phase 2, rotate-accumulate 4, gate path 2; sin, cos);
    # the per-head sums run on the matrix cores
    bwd_instr = pairs * (15 + 12)
    # VALU roofline: 256 CUs x 4 SIMDs x 16 lanes x 2.4 GHz issue slots/s.  Per (sin, cos) pair the forward needs 14 slots:
    # 10 full-rate instructions (phase 2, unpack 2, rotate 4, pack 1, LDS 1) and two transcendentals, which issue at half
    # the rate (measured on this chip: v_sin_f32 16.0 T lanes/s against 33.3 for v_fma_f32), so 2 slots each; the per-head
    # dot products run on the matrix cores
    fwd_instr = pairs * 14
    out = {"metric": "Co-RoPE GQA fwd, B2 Hq32 Hkv8 N4096 D128 causal", "value": round(flops / (ms * 1e-3) * 1e-12, 2),
           "unit": "TFLOP/s (attention-equivalent)", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "settle_steps": settle_steps,
           "dtype": "bf16", "data": "synthetic",
           "config": {"workload": "C5: Co-RoPE GQA attention fwd B2 Hq32 Hkv8 N4096 D128 causal bf16", "theta": 10000.0},
           "sincos_pairs_per_s": round(pairs / (kms * 1e-3), 1), "kernel_ms": round(kms, 4),
           "roofline": {"bound": "valu", "kernel": "corope_gqa_fwd", "achieved": round(fwd_instr / (kms * 1e-3) * 1e-12, 3),
                        "peak": round(256 * 4 * 16 * 2.4e9 * 1e-12, 3), "unit": "T issue slots/s",
                        "frac": round(fwd_instr / (kms * 1e-3) / (256 * 4 * 16 * 2.4e9), 4),
                        "traffic": HBM_TRAFFIC_BYTES[("c5", "corope_gqa_fwd")]},
           "backward": {"ms": round(bms, 4), "steps": bsteps, "workspace_gib": round(ws_bytes / 2**30, 2), "ms_by_workspace": by_workspace,
                        "sincos_pairs_per_s": round(2 * pairs / (bms * 1e-3), 1),
                        "tflops_attention_equivalent": round(2.5 * flops / (bms * 1e-3) * 1e-12, 2),
                        "roofline": {"bound": "valu", "kernel": "corope_gqa_bwd (6 launches)",
                                     "achieved": round(bwd_instr / (bms * 1e-3) * 1e-12, 3),
                                     "peak": round(256 * 4 * 16 * 2.4e9 * 1e-12, 3), "unit": "T issue slots/s",
                                     "frac": round(bwd_instr / (bms * 1e-3) / (256 * 4 * 16 * 2.4e9), 4),
                                     "traffic": HBM_TRAFFIC_BYTES[("c5", "corope_gqa_bwd")]}},
           "cpu_baseline": None}
    if args.parity:
        torch.cuda.synchronize()
        out["parity"] = corope_parity(pkg, q.float().cpu(), k.float().cpu(), v.float().cpu(), do.float().cpu(), o.float().cpu(),
                                      tuple(t.float().cpu() for t in (dq, dk, dv)), scale, 10000.0, torch)
    print(json.dumps(out))


def bench_hbm_passes(args):
    """The two HBM-bound passes of the chosen RoPE shape (rotation of K with per-tile norms; delta = rowsum(O * dO)) beside a
    plain device copy of the same tensor, each timed two ways: back to back (operands largely resident in the 256 MB
    last-level cache from the previous call) and with a 1 GiB buffer overwritten before every call (nothing resident).
    Inside a training step the passes run between those two extremes.  Prints a markdown table."""
    import torch
    pkg = importlib.import_module("corope_amd")
    lib = pkg._lib.load()
    dev = torch.device("cuda:0")
    cfg = CONFIGS[args.config]
    B, H, N, D = cfg["B"], cfg["H"], cfg["N"], cfg["D"]
    k, o, do, _ = (t.to(dev, torch.bfloat16) for t in make_inputs(B, H, N, D, "normal", torch))
    c, s = pkg.precompute_freqs_cis(D, N, 10000.0, device=dev)
    kr = torch.empty_like(k)
    kmax = torch.empty(B, H, (N + 63) // 64, device=dev, dtype=torch.float32)
    delta = torch.empty(B, H, N, device=dev, dtype=torch.float32)
    st = torch.cuda.current_stream().cuda_stream
    flush = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    ops = [("plain copy of one tensor (torch copy_)", lambda: kr.copy_(k), 2 * k.numel() * 2),
           ("rope_rotate_k (read K, write rotated K + tile norms)",
            lambda: lib.corope_rope_rotate(k.data_ptr(), c.data_ptr(), s.data_ptr(), c.stride(0), kr.data_ptr(), kmax.data_ptr(),
                                           B, H, N, D, 1.0, st), 2 * k.numel() * 2 + kmax.numel() * 4),
           ("rope_attn_bwd_preprocess (read O and dO, write delta)",
            lambda: lib.corope_rope_attn_bwd_preprocess(o.data_ptr(), do.data_ptr(), delta.data_ptr(), B, H, N, D, st),
            2 * k.numel() * 2 + delta.numel() * 4)]
    print(f"Workload: {cfg['name']}\n\n| pass | bytes | back to back: us | GB/s | of 8 TB/s | caches flushed before every call: us | GB/s | of 8 TB/s |\n"
          "|---|---|---|---|---|---|---|---|")
    for name, fn, by in ops:
        for _ in range(50):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(300):
            fn()
        e1.record()
        torch.cuda.synchronize()
        warm = e0.elapsed_time(e1) / 300
        ts = []
        for _ in range(40):
            flush.zero_()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1))
        cold = statistics.median(ts)
        print(f"| {name} | {by / 1e6:.1f} MB | {warm * 1e3:.1f} | {by / warm * 1e-6:.0f} | {by / warm * 1e-6 / PEAK_HBM_GBS:.2f} | "
              f"{cold * 1e3:.1f} | {by / cold * 1e-6:.0f} | {by / cold * 1e-6 / PEAK_HBM_GBS:.2f} |")


def forward_ms(pkg, q, k, v, cos, sin, scale, torch, reps=100):
    """Average duration of the operator's forward (all its launches) over `reps` back-to-back calls, HIP events."""
    for _ in range(20):
        pkg.rope_attn_forward_with_lse(q, k, v, True, scale, cos, sin)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        pkg.rope_attn_forward_with_lse(q, k, v, True, scale, cos, sin)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def bench_phase_trace(args):
    """Where the time of the forward, dQ and dK+dV kernels goes at the chosen shape: the kernels of the trace build stamp
    the constant 100 MHz counter at the phase boundaries of every item they work on (one lane of the wave that sees every
    tile) and the core-clock counter around its tile loop.  Prints a markdown table (one traced step in the middle of a run
    of steps)."""
    import ctypes
    import numpy as np
    import torch
    pkg = importlib.import_module("corope_amd")
    try:
        lib = pkg._lib.load_trace()
    except pkg._lib.CoRopeLibraryError as e:
        sys.exit(f"bench.py: {e}")
    dev = torch.device("cuda:0")
    cfg = CONFIGS[args.config]
    B, H, N, D = cfg["B"], cfg["H"], cfg["N"], cfg["D"]
    scale = 1 / math.sqrt(D)
    q, k, v, do = (t.to(dev, torch.bfloat16) for t in make_inputs(B, H, N, D, args.data, torch))
    c, s = pkg.precompute_freqs_cis(D, N, 10000.0, device=dev)
    st, fs = torch.cuda.current_stream().cuda_stream, c.stride(0)
    o, qr, kr, dq, dk, dv = (torch.empty_like(q) for _ in range(6))
    M = torch.empty(B, H, N, device=dev, dtype=torch.float32)
    delta = torch.empty_like(M)
    kmax = torch.empty(B, H, (N + 63) // 64, device=dev, dtype=torch.float32)
    P = lambda t: t.data_ptr()
    launches = [
        ("rope_rotate_k", lambda: lib.corope_rope_rotate(P(k), P(c), P(s), fs, P(kr), P(kmax), B, H, N, D, 1.0, st)),
        ("rope_attn_fwd", lambda: lib.corope_rope_attn_fwd_prerotated(P(q), P(kr), P(kmax), P(v), P(c), P(s), fs, P(o), P(M), P(qr),
                                                                      B, H, N, D, scale, 1, st)),
        ("rope_attn_bwd_dq", lambda: lib.corope_rope_attn_bwd_dq_prerotated(P(qr), P(kr), P(v), P(o), P(do), P(M), P(delta), P(c),
                                                                            P(s), fs, P(dq), B, H, N, D, scale, 1, st)),
        ("rope_attn_bwd_dkdv", lambda: lib.corope_rope_attn_bwd_dkdv_prerotated(P(qr), P(kr), P(v), P(do), P(M), P(delta), P(c), P(s),
                                                                                fs, P(dk), P(dv), B, H, N, D, scale, 1, st)),
    ]
    lib.corope_debug_trace(None)
    for _ in range(60):          # settle the clocks
        for n, f in launches:
            assert f() == 0, n
    torch.cuda.synchronize()
    n_wg = B * H * ((N + 127) // 128)     # room for the forms with 128-row items as well
    bufs = {n: torch.zeros(n_wg * 16, dtype=torch.int64, device=dev) for n, _ in launches[1:]}
    for rep in range(3):         # the traced step sits between untraced ones
        for n, f in launches:
            lib.corope_debug_trace(bufs[n].data_ptr() if (n in bufs and rep == 1) else None)
            assert f() == 0, n
    torch.cuda.synchronize()
    lib.corope_debug_trace(None)

    def row(label, x):
        x = np.asarray(x, dtype=float)
        return f"| {label} | {x.mean():.2f} | {np.percentile(x, 10):.2f} | {np.percentile(x, 50):.2f} | {np.percentile(x, 90):.2f} | {x.max():.2f} |"

    print(f"Workload: {cfg['name']}, data {args.data}; times in microseconds per item (256 rows) unless said otherwise.\n")
    for name, buf in bufs.items():
        a = buf.cpu().numpy().reshape(-1, 16)
        if args.trace_dump:
            np.save(os.path.join(args.trace_dump, f"trace_{name}_{args.data}.npy"), a)
        a = a[a[:, 0] != 0]
        t = a[:, :14].astype(np.float64) * 0.01
        t = np.where(a[:, :14] != 0, t - t[:, 0].min(), np.nan)
        hw, xcc = a[:, 14] & 0xffffffff, (a[:, 14] >> 32) & 0xf
        cu_key = xcc * 1000 + ((hw >> 13) & 7) * 100 + ((hw >> 12) & 1) * 16 + ((hw >> 8) & 0xf)
        ntile = a[:, 15].astype(float)
        dkdv = name.endswith("dkdv")
        gaps, busy = [], []
        for kk in set(cu_key):
            idx = np.where(cu_key == kk)[0]
            idx = idx[np.argsort(t[idx, 0])]
            gaps += [t[j, 0] - t[i, 6] for i, j in zip(idx[:-1], idx[1:])]
            busy.append(sum(t[i, 6] - t[i, 0] for i in idx))
        span = np.nanmax(t[:, 6])
        ghz = a[:, 7] / ((a[:, 5] - (a[:, 1] if name != "rope_attn_fwd" else a[:, 2])) * 10.0)
        print(f"### {name}: {len(a)} items on {len(set(cu_key))} CUs, {len(a) / len(set(cu_key)):.1f} per CU, "
              f"launch span {span:.1f} us, mean busy time per CU {np.mean(busy):.1f} us\n")
        print("| phase | mean | p10 | p50 | p90 | max |\n|---|---|---|---|---|---|")
        print(row("whole item", t[:, 6] - t[:, 0]))
        print(row("gap to the next item on the same CU", gaps))
        print(row("prologue (previous item's stores issued -> operand rows in registers)", t[:, 1] - t[:, 0]))
        big = ntile > 5
        if dkdv:      # the key block's diagonal query tiles come first
            print(row("first tile", t[:, 3] - t[:, 1]))
            print(row("diagonal tiles 2-4, per tile", (t[big, 4] - t[big, 3]) / 3))
            print(row("steady state, per tile (64 queries x 256 keys)", (t[big, 5] - t[big, 4]) / (ntile[big] - 4)))
        else:
            if name == "rope_attn_fwd":
                print(row("key-norm bounds of the wave's tiles", t[:, 2] - t[:, 1]))
                print(row("first tile (with its exact pass)", t[:, 3] - t[:, 2]))
                print(row("tiles examined twice, fraction of the wave's tiles", a[:, 13] / ntile))
            else:
                print(row("first tile", t[:, 3] - t[:, 1]))
            print(row("steady state, per tile (256 queries x 64 keys)", (t[big, 4] - t[big, 3]) / (ntile[big] - 5)))
            print(row("diagonal block, per tile (4 tiles, waves drop out)", (t[:, 5] - t[:, 4]) / 4))
        print(row("epilogue (last tile -> stores issued, next rows requested)", t[:, 6] - t[:, 5]))
        print(row("shader clock in the tile loop [GHz]", ghz))
        per_cu = len(a) / len(set(cu_key))
        edge = np.nanmean(t[:, 1] - t[:, 0]) + np.nanmean(t[:, 6] - t[:, 5]) + np.mean(gaps)
        print(f"\nPer CU: {per_cu:.0f} items x {edge:.1f} us of prologue + epilogue + gap = {per_cu * edge:.0f} us "
              f"of {np.mean(busy):.0f} us ({100 * per_cu * edge / np.mean(busy):.0f} %).\n")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # defaults long enough for the clocks to settle: the first ~50 ms of sustained load run 3-10 % slower than what follows
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--config", default="c3", choices=sorted(CONFIGS) + ["c5"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--sweep", action="store_true",
                    help="time the reference harness's 19 shapes instead (one JSON line per shape)")
    ap.add_argument("--lanes", action="store_true",
                    help="with --sweep: also time the unfused lanes (separate rotation + identity-table attention, PyTorch SDPA)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp16"], help="with --sweep: element type of q, k, v, dO")
    ap.add_argument("--fp16-forward", default="exact", choices=["exact", "fast"],
                    help="with --sweep --dtype fp16: rope_attn.FP16_TRAINING_FORWARD (the forward of a differentiated call)")
    ap.add_argument("--sm-scale", type=float, default=None, help="with --sweep: softmax scale instead of the reference harness's 0.5")
    ap.add_argument("--shape", default=None, help="with --sweep: one shape B,H,N,D of your own instead of the 19 (e.g. 2,16,4096,256)")
    ap.add_argument("--only", default=None, help="with --sweep: comma-separated names of the shapes to run")
    ap.add_argument("--flush", action="store_true",
                    help="with --sweep: also time every call on flushed caches (a 512 MiB buffer overwritten before each call)")
    ap.add_argument("--parity", action="store_true",
                    help="the larger parity sample (the line always carries per-tensor errors against the CPU oracle on a small one)")
    ap.add_argument("--no-parity", action="store_true", help="leave the per-tensor errors out of the line")
    ap.add_argument("--data", default="normal", choices=["normal", "sink"],
                    help="synthetic inputs: N(0,1), or attention-sink-like keys (see make_inputs)")
    ap.add_argument("--phase-trace", action="store_true",
                    help="split the attention kernels of the chosen RoPE config into phases (trace build of the library)")
    ap.add_argument("--trace-dump", default=None, metavar="DIR",
                    help="with --phase-trace: also save the raw stamps of every kernel (one row of 16 per item) as .npy files there")
    ap.add_argument("--hbm-passes", action="store_true",
                    help="time the rotation and dO.O passes of the chosen RoPE shape beside a plain device copy, with warm and "
                         "with flushed caches (markdown table)")
    ap.add_argument("--mfma-rate", action="store_true",
                    help="build (if stale) and run bench_mfma_rate.hip: what the matrix pipes sustain on this machine, by operand "
                         "source, instruction shape and accompanying vector work (markdown tables)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy (for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs on ONE GPU (every (batch, head) is independent, so the path would shard over "
                 "batch x heads without any exchange); run it with --gpus 1")

    if args.mfma_rate:
        import subprocess
        src, exe = os.path.join(ROOT, "bench_mfma_rate.hip"), os.path.join(ROOT, "bench_mfma_rate")
        if not os.path.exists(exe) or os.path.getmtime(exe) < os.path.getmtime(src):
            importlib.import_module("corope_amd.build").build_program(src, exe)
        return sys.exit(subprocess.run([exe]).returncode)
    if args.copy_calibration:
        import torch
        a = torch.empty(1 << 29, dtype=torch.bfloat16, device="cuda:0").normal_()
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)          # reads 1 GiB, writes 1 GiB per launch
        torch.cuda.synchronize()
        del a, b
    if args.sweep:
        return bench_sweep(args)
    if args.config == "c5":
        return bench_corope(args)
    if args.phase_trace:
        return bench_phase_trace(args)
    if args.hbm_passes:
        return bench_hbm_passes(args)
    import torch
    pkg = importlib.import_module("corope_amd")
    lib = pkg._lib.load()
    dev = torch.device("cuda:0")
    cfg = CONFIGS[args.config]
    B, H, N, D = cfg["B"], cfg["H"], cfg["N"], cfg["D"]
    fwd_only = args.config == "c4"
    scale = 1 / math.sqrt(D)
    host = make_inputs(B, H, N, D, args.data, torch)
    q, k, v, do = (t.to(dev, torch.bfloat16) for t in host)
    cos, sin = pkg.precompute_freqs_cis(D, N, 10000.0, device=dev)
    if not fwd_only:
        q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)

    def step():
        o = pkg.attention(q, k, v, True, scale, cos, sin)
        if not fwd_only:
            o.backward(do)
            q.grad = k.grad = v.grad = None
        return o

    settle_steps = settle_clocks(step, torch)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    f_fwd, f_bwd = attention_flops(B, H, N, D, "fwd"), (0.0 if fwd_only else attention_flops(B, H, N, D, "bwd"))
    value = (f_fwd + f_bwd) / (ms_per_step * 1e-3) * 1e-12

    # ---- per-kernel launch durations: HIP events on the launch stream, straight through the C ABI ----------------
    stream = torch.cuda.current_stream().cuda_stream
    o = torch.empty_like(q)
    M = torch.empty(B, H, N, device=dev, dtype=torch.float32)
    delta = torch.empty_like(M)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    qp, kp, vp, dop = q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr()
    cp, sp, fs = cos.data_ptr(), sin.data_ptr(), cos.stride(0)
    rotated = pkg.rope_attn.use_rotated_path(N, D, training=not fwd_only)
    if rotated:   # the forward the operator takes at this shape: rotate K, then attention
        k_rot, q_rot = torch.empty_like(k), torch.empty_like(q)
        kmax = torch.empty(B, H, (N + 63) // 64, device=dev, dtype=torch.float32)
        launches = [("rope_rotate_k", lambda: lib.corope_rope_rotate(kp, cp, sp, fs, k_rot.data_ptr(), kmax.data_ptr(),
                                                                     B, H, N, D, 1.0, stream)),
                    ("rope_attn_fwd", lambda: lib.corope_rope_attn_fwd_prerotated(
                        qp, k_rot.data_ptr(), kmax.data_ptr(), vp, cp, sp, fs, o.data_ptr(), M.data_ptr(),
                        None if fwd_only else q_rot.data_ptr(), B, H, N, D, scale, 1, stream))]
    else:
        launches = [("rope_attn_fwd", lambda: lib.corope_rope_attn_fwd(qp, kp, vp, cp, sp, fs, o.data_ptr(), M.data_ptr(),
                                                                      B, H, N, D, scale, 1, stream))]
    if not fwd_only:
        if rotated:   # the backward the operator takes at this shape: on the rotated q, k the forward kept; the dQ kernel
            qr, kr = q_rot.data_ptr(), k_rot.data_ptr()   # computes delta on its way, the fused dK+dV kernel follows
            launches += [
                ("rope_attn_bwd_dq", lambda: lib.corope_rope_attn_bwd_dq_prerotated(
                    qr, kr, vp, o.data_ptr(), dop, M.data_ptr(), delta.data_ptr(), cp, sp, fs, dq.data_ptr(), B, H, N, D,
                    scale, 1, stream)),
                ("rope_attn_bwd_dkdv", lambda: lib.corope_rope_attn_bwd_dkdv_prerotated(
                    qr, kr, vp, dop, M.data_ptr(), delta.data_ptr(), cp, sp, fs, dk.data_ptr(), dv.data_ptr(), B, H, N, D,
                    scale, 1, stream)),
            ]
        else:
            launches += [
                ("rope_attn_bwd_preprocess", lambda: lib.corope_rope_attn_bwd_preprocess(
                    o.data_ptr(), dop, delta.data_ptr(), B, H, N, D, stream)),
                ("rope_attn_bwd_dv", lambda: lib.corope_rope_attn_bwd_dv(qp, kp, dop, M.data_ptr(), cp, sp, fs, dv.data_ptr(),
                                                                        B, H, N, D, scale, 1, stream)),
                ("rope_attn_bwd_dk", lambda: lib.corope_rope_attn_bwd_dk(qp, kp, vp, dop, M.data_ptr(), delta.data_ptr(),
                                                                        cp, sp, fs, dk.data_ptr(), B, H, N, D, scale, 1, stream)),
                ("rope_attn_bwd_dq", lambda: lib.corope_rope_attn_bwd_dq(qp, kp, vp, dop, M.data_ptr(), delta.data_ptr(),
                                                                        cp, sp, fs, dq.data_ptr(), B, H, N, D, scale, 1, stream)),
            ]
    # the launches of a step in step order, back to back over all iterations with no host synchronisation in between: the
    # matrix pipes run at a power-limited clock, and a pause per iteration lets every kernel run 4-7 % faster than it
    # does inside a training step
    durs = {n: [] for n, _ in launches}
    all_evs = [[torch.cuda.Event(enable_timing=True) for _ in range(len(launches) + 1)]
               for _ in range(args.warmup + args.steps)]
    for evs in all_evs:
        evs[0].record()
        for i, (name, fn) in enumerate(launches):
            rc = fn()
            if rc != 0:
                sys.exit(f"{name} failed: {pkg._lib.last_error()}")
            evs[i + 1].record()
    torch.cuda.synchronize()
    for evs in all_evs[args.warmup:]:
        for i, (name, _) in enumerate(launches):
            durs[name].append(evs[i].elapsed_time(evs[i + 1]))
    avg = {n: sum(d) / len(d) for n, d in durs.items()}
    # algorithmic FLOPs per launch (the reference's model: forward 2 matmul units, backward 5): fused dK+dV kernel 4 units
    # (the counted S recompute, dP, dV, dK) -- as two launches: dV 2 units, dK 2 units (its own S recompute is overhead on
    # top of the model); dQ kernel 1 unit (dQ; its S and dP recomputes are overhead); the preprocess pass is HBM-bound.
    unit = 2.0 * B * H * N * N * D * 0.5
    alg = {"rope_attn_fwd": 2 * unit, "rope_attn_bwd_dkdv": 4 * unit, "rope_attn_bwd_dv": 2 * unit, "rope_attn_bwd_dk": 2 * unit,
           "rope_attn_bwd_dq": 1 * unit}
    kernels = {}
    for n, ms in avg.items():
        if n in alg:
            tf = alg[n] / (ms * 1e-3) * 1e-12
            kernels[n] = {"ms": round(ms, 4), "tflops": round(tf, 1), "frac_of_peak": round(tf / PEAK_BF16_TFLOPS, 4)}
        else:   # HBM-bound passes: two (B,H,N,D) bf16 tensors moved (read o, do / read k, write k_rot) plus small extras
            by = 2.0 * B * H * N * D * 2 + B * H * N * 4
            kernels[n] = {"ms": round(ms, 4), "gbs": round(by / (ms * 1e-3) * 1e-9, 1),
                          "frac_of_hbm_peak": round(by / (ms * 1e-3) * 1e-9 / PEAK_HBM_GBS, 4)}
    dom = max((n for n in avg if n in alg), key=lambda n: avg[n])
    dom_tf = alg[dom] / (avg[dom] * 1e-3) * 1e-12
    traffic = HBM_TRAFFIC_BYTES.get((args.config, dom))
    roofline = {"bound": "mfma", "kernel": dom, "achieved": round(dom_tf, 1), "peak": PEAK_BF16_TFLOPS,
                "unit": "TFLOP/s", "frac": round(dom_tf / PEAK_BF16_TFLOPS, 4), "traffic": traffic,
                "avg_launch_ms": round(avg[dom], 4)}
    fwd_ms = avg["rope_attn_fwd"] + avg.get("rope_rotate_k", 0.0)
    fwd_tf = alg["rope_attn_fwd"] / (fwd_ms * 1e-3) * 1e-12
    out = {
        "metric": f"RoPE-attn {'fwd' if fwd_only else 'fwd+bwd'} TFLOPS & % bf16 MFMA peak, B{B} H{H} N{N} D{D} causal",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "settle_steps": settle_steps,
        "dtype": "bf16", "data": "synthetic" if args.data == "normal" else "synthetic (attention-sink keys)",
        "config": {"workload": cfg["name"], "B": B, "H": H, "N": N, "D": D, "causal": True,
                   "sm_scale": "1/sqrt(D)", "rope_base": 10000.0},
        "frac_of_bf16_peak": round(value / PEAK_BF16_TFLOPS, 4),
        "fwd": {"ms": round(fwd_ms, 4), "tflops": round(fwd_tf, 1),
                "frac_of_peak": round(fwd_tf / PEAK_BF16_TFLOPS, 4)},
        "kernels": kernels, "roofline": roofline,
    }
    if not fwd_only:
        bwd_ms = sum(ms for n, ms in avg.items() if n not in ("rope_rotate_k", "rope_attn_fwd"))
        bwd_tf = f_bwd / (bwd_ms * 1e-3) * 1e-12
        out["bwd"] = {"ms": round(bwd_ms, 4), "tflops": round(bwd_tf, 1), "frac_of_peak": round(bwd_tf / PEAK_BF16_TFLOPS, 4)}
    # the dO.O pass (delta = rowsum(O o dO)) on its own: at this shape the dQ kernel computes delta on its way, so the pass is
    # not one of the step's launches; timed here for its HBM rate (two (B,H,N,D) bf16 tensors read, (B,H,N) fp32 written)
    if not fwd_only and "rope_attn_bwd_preprocess" not in kernels:
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(51)]
        for i in range(-5, 50):
            lib.corope_rope_attn_bwd_preprocess(o.data_ptr(), dop, delta.data_ptr(), B, H, N, D, stream)
            if i >= -1:
                evs[i + 1].record()
        torch.cuda.synchronize()
        ms = sum(evs[i].elapsed_time(evs[i + 1]) for i in range(50)) / 50
        by = 2.0 * B * H * N * D * 2 + B * H * N * 4
        kernels["rope_attn_bwd_preprocess (standalone: not a launch of the step at this shape)"] = {
            "ms": round(ms, 4), "gbs": round(by / (ms * 1e-3) * 1e-9, 1), "frac_of_hbm_peak": round(by / (ms * 1e-3) * 1e-9 / PEAK_HBM_GBS, 4)}
    if args.data != "normal":
        # the same forward on N(0,1) inputs, timed the same way, beside the line's own
        hq, hk, hv, _ = make_inputs(B, H, N, D, "normal", torch)
        out["fwd_ms_by_data"] = {args.data: round(forward_ms(pkg, q.detach(), k.detach(), v.detach(), cos, sin, scale, torch), 4),
                                 "normal": round(forward_ms(pkg, *(t.to(dev, torch.bfloat16) for t in (hq, hk, hv)), cos, sin,
                                                            scale, torch), 4)}
    # per-tensor errors against the CPU oracle, outside the timed region (--parity: the larger sample; --no-parity: none)
    if not args.no_parity:
        out["parity"] = rope_parity(pkg, args.config, host[0], host[1], host[2], host[3], cos, sin, scale, fwd_only, torch,
                                    quick=not args.parity)
    out["cpu_baseline"] = None if args.no_cpu_baseline else cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
