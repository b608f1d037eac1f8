"""Builds libcorope_amd.so (gfx950 HIP kernels + C ABI) in-tree with hipcc.

Run as ``python co-rope_amd/build.py`` or call ``build()``; the result lands in
``co-rope_amd/lib/libcorope_amd.so`` and is what ``_lib.load()`` opens."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libcorope_amd.so")

SOURCES = ["abi.hip", "rope_freqs.hip", "rope_rotate.hip", "rope_attn_fwd.hip", "rope_attn_fwd_pipe.hip", "rope_attn_bwd_pre.hip", "rope_attn_bwd.hip", "corope_gqa_fwd.hip", "corope_gqa_bwd.hip"]

# -packed-fp32-ops is switched off: packed fp32 VALU forms are not used by these kernels.
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-value",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unknown-attributes",
               "-Wno-ignored-optimization-argument", "-Wno-unused-command-line-argument"]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _compile(src, extra):
    obj = os.path.join(LIBDIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    return obj, err


def build(verbose=False, extra_flags=()):
    os.makedirs(LIBDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        results = list(ex.map(lambda s: _compile(s, list(extra_flags)), SOURCES))
    if verbose:
        for (_, err), s in zip(results, SOURCES):
            if err.strip():
                print(f"--- {s}\n{err}", file=sys.stderr)
    objs = [o for o, _ in results]
    r = subprocess.run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, extra_flags=sys.argv[1:]))
