"""Builds libcorope_amd.so (gfx950 HIP kernels + C ABI) in-tree with hipcc.

Run as ``python co-rope_amd/build.py`` or call ``build()``; the result lands in
``co-rope_amd/lib/libcorope_amd.so`` and is what ``_lib.load()`` opens.  Beside it, for measurement only:
``libcorope_amd_trace.so`` (the same sources with -DCOROPE_TRACE: the attention kernels stamp a clock at their phase
boundaries into a buffer ``bench.py --phase-trace`` hands them, and a call forces kernel forms for the tests).
``build_program`` compiles a stand-alone HIP program with the same flags (``bench.py --mfma-rate`` uses it)."""
from __future__ import annotations

import glob
import os
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

try:
    from .check_isa import ASM_MFMA_IN_SOURCE, check_asm_mfma
except ImportError:   # run as a script
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from check_isa import ASM_MFMA_IN_SOURCE, check_asm_mfma

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libcorope_amd.so")
TRACE_LIB = os.path.join(LIBDIR, "libcorope_amd_trace.so")

# compiled a second time with -DCOROPE_F16 (fp16 elements, namespace corope_f16)
F16_SOURCES = ["rope_rotate.hip", "rope_attn_fwd.hip", "rope_attn_fwd_pipe.hip", "rope_attn_bwd_pre.hip", "rope_attn_bwd.hip", "corope_gqa_fwd.hip",
               "corope_gqa_bwd.hip"]

SOURCES = ["abi.hip", "rope_freqs.hip", "rope_rotate.hip", "rope_attn_fwd.hip", "rope_attn_fwd_pipe.hip", "rope_attn_fwd_pipe_acc.hip", "rope_attn_bwd_pre.hip", "rope_attn_bwd.hip", "corope_gqa_fwd.hip", "corope_gqa_bwd.hip"]



def isa_checked(src):
    """Whether a source issues matrix-core instructions from asm statements (itself or through the helpers of common.hpp):
    the generated assembly of every variant of such a source is checked (check_isa.py)."""
    with open(os.path.join(CSRC, src)) as f:
        return ASM_MFMA_IN_SOURCE.search(f.read()) is not None


# -packed-fp32-ops is switched off: packed fp32 VALU forms are not used by these kernels.
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-value",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unknown-attributes",
               "-Wno-ignored-optimization-argument", "-Wno-unused-command-line-argument"]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _compile(src, extra, suffix=""):
    obj = os.path.join(LIBDIR, os.path.splitext(src)[0] + suffix + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    noise = "is not a recognized feature for this target"
    if not isa_checked(src):
        r = subprocess.run(cmd, capture_output=True, text=True)
        problems = []
    else:   # the compiler's intermediate files, among them the device assembly, land in a directory of their own
        with tempfile.TemporaryDirectory(prefix="corope_build_") as tmp:
            r = subprocess.run(cmd + ["--save-temps"], capture_output=True, text=True, cwd=tmp)
            problems = []
            if r.returncode == 0:
                asm = glob.glob(os.path.join(tmp, "*-hip-amdgcn-*.s"))
                if not asm:
                    raise RuntimeError(f"no device assembly of {src}{suffix} to check")
                for path in asm:
                    with open(path) as f:
                        problems += check_asm_mfma(f.read(), src + suffix)
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if problems:
        raise RuntimeError("asm-issued matrix-core results touched too early:\n" + "\n".join(problems))
    return obj, err


def _link(objs, out, shared=True):
    r = subprocess.run([_hipcc(), "--offload-arch=gfx950", *(["-shared", "-fPIC"] if shared else []), *objs, "-o", out],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link of {out} failed:\n{r.stderr}")
    return out


def build(verbose=False, extra_flags=(), extras=True):
    """Compiles every source.  ``extras``: also the trace variant of the library."""
    os.makedirs(LIBDIR, exist_ok=True)
    jobs = [(s, list(extra_flags), "") for s in SOURCES] + [(s, list(extra_flags) + ["-DCOROPE_F16"], ".f16") for s in F16_SOURCES]
    if extras:
        jobs += [(s, j[1] + ["-DCOROPE_TRACE"], j[2] + ".trace") for j in list(jobs) for s in [j[0]]]
    with ThreadPoolExecutor(max_workers=8) as ex:
        results = list(ex.map(lambda j: _compile(*j), jobs))
    if verbose:
        for (_, err), j in zip(results, jobs):
            if err.strip():
                print(f"--- {j[0]}{j[2]}\n{err}", file=sys.stderr)
    n = len(SOURCES) + len(F16_SOURCES)
    _link([o for o, _ in results[:n]], LIB)
    if extras:
        _link([o for o, _ in results[n:2 * n]], TRACE_LIB)
    return LIB


def build_program(source, out):
    """Compiles one stand-alone HIP program (a measurement tool beside bench.py) for gfx950."""
    flags = [f for f in HIPCC_FLAGS if f != "-fPIC"]
    r = subprocess.run([_hipcc(), *flags, "-I", os.path.dirname(HERE), source, "-o", out], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {source}:\n{r.stderr}")
    return out


if __name__ == "__main__":
    print(build(verbose=True, extra_flags=sys.argv[1:]))
