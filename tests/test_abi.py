"""CPU-only checks of the drop-in boundary: the shared library loads, exports every symbol the header declares,
validates its arguments before touching HIP, and the Python layer keeps the reference's call surface."""
import ctypes
import inspect
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "corope_amd.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(corope_[a-z_0-9]+)\s*\(", text)))


def test_header_symbols_are_exported_and_typed(pkg):
    lib = pkg._lib.load()
    names = _declared_symbols()
    assert "corope_rope_attn_fwd" in names and "corope_gqa_fwd" in names and len(names) >= 10
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
    assert sorted(pkg._lib.SIGNATURES) == names, "ctypes table and header disagree"
    assert lib.corope_amd_version() == pkg._lib.ABI_VERSION


def test_header_cites_reference_for_each_entry_point():
    text = open(HEADER).read()
    for fn in ("corope_rope_freqs", "corope_rope_attn_fwd", "corope_rope_attn_bwd_preprocess", "corope_rope_attn_bwd_dv",
               "corope_rope_attn_bwd_dk", "corope_rope_attn_bwd_dkdv",
               "corope_rope_attn_bwd_dq", "corope_rope_attn_bwd", "corope_gqa_fwd"):
        before = text[:text.index(f"int {fn}(")]
        comment = before[before.rindex("/*"):]
        assert re.search(r"\.py:\d+", comment), f"{fn}: no reference file:line in its comment"


@pytest.mark.parametrize("args,code", [
    ((2, 32, 4096, 128, 128, 0.088, 0), 0),
    ((4, 8, 1024, 64, 32, 0.125, 1), 0),
    ((1, 1, 77, 128, 64, 1.0, 0), 0),
    ((0, 8, 128, 64, 64, 1.0, 0), -1),
    ((1, 8, -5, 64, 64, 1.0, 0), -1),
    ((1, 8, 128, 32, 32, 1.0, 0), -2),
    ((1, 8, 128, 256, 256, 1.0, 0), 0),
    ((1, 8, 128, 512, 256, 1.0, 0), -2),
    ((1, 8, 128, 64, 16, 1.0, 0), -1),      # table narrower than D/2
    ((1, 8, 128, 64, 66, 1.0, 0), -1),      # row stride not a multiple of 4 floats
    ((1, 8, 128, 64, 64, 0.0, 0), -1),
    ((1, 8, 128, 64, 64, float("nan"), 0), -1),
    ((1, 1, 1 << 24, 128, 64, 1.0, 0), -2),   # one (batch, head) slab of 4 GiB: past the 32-bit staging offsets
    ((1, 1, 1 << 22, 128, 256, 1.0, 0), -2),  # cos/sin table of 4 GiB
    ((1, 1, 1 << 22, 128, 64, 1.0, 0), 0),
    ((1 << 16, 1 << 15, 1, 64, 32, 1.0, 0), -2),    # 2^31 (batch, head) slabs of one row: more workgroups than a grid axis takes
])
def test_rope_attn_check_codes(pkg, args, code):
    lib = pkg._lib.load()
    assert lib.corope_rope_attn_check(*args) == code
    assert (pkg._lib.last_error() == "") == (code == 0)


@pytest.mark.parametrize("args,code", [
    ((2, 32, 8, 4096, 128, 0.088, 10000.0), 0),
    ((1, 7, 1, 65, 64, 1.0, 100.0), 0),
    ((1, 6, 4, 64, 64, 1.0, 1e4), -1),      # Hq not a multiple of Hkv
    ((1, 18, 2, 64, 64, 1.0, 1e4), -2),     # group of 9
    ((1, 4, 2, 64, 32, 1.0, 1e4), -2),
    ((1, 4, 2, 64, 64, 1.0, 0.0), -1),
    ((1, 4, 2, 0, 64, 1.0, 1e4), -1),
    ((64, 64, 64, 1 << 19, 64, 1.0, 1e4), -2),   # B * Hkv * N rows do not fit one grid axis
    ((1, 1, 1, 1 << 24, 128, 1.0, 1e4), -2),     # a slab beyond 32-bit byte offsets
])
def test_corope_check_codes(pkg, args, code):
    assert pkg._lib.load().corope_gqa_check(*args) == code


def test_null_and_misaligned_pointers_are_rejected_before_any_launch(pkg):
    lib = pkg._lib.load()
    buf = ctypes.create_string_buffer(4096)
    base = (ctypes.addressof(buf) + 15) & ~15
    ok, odd = base, base + 2
    rc = lib.corope_rope_attn_fwd(ok, ok, None, ok, ok, 64, ok, ok, 1, 1, 8, 64, 1.0, 1, None)
    assert rc == -1 and "null" in pkg._lib.last_error()
    rc = lib.corope_rope_attn_fwd(ok, odd, ok, ok, ok, 64, ok, ok, 1, 1, 8, 64, 1.0, 1, None)
    assert rc == -3 and "aligned" in pkg._lib.last_error()
    rc = lib.corope_rope_attn_bwd_preprocess(ok, None, ok, 1, 1, 8, 64, None)
    assert rc == -1
    rc = lib.corope_gqa_fwd(ok, ok, ok, odd, 1, 2, 1, 8, 64, 1.0, 1e4, None)
    assert rc == -3
    with pytest.raises(ValueError):
        pkg._lib.check(rc, "corope_gqa_fwd")


def test_composite_entry_points_check_every_argument_before_the_first_launch(pkg):
    """The entry points that make several launches look at ALL their arguments first: a null or misaligned pointer that
    only the last launch would use is refused with a BADARG / ALIGN status (a launch attempted here, without a GPU, would
    come back as a LAUNCH status instead)."""
    lib = pkg._lib.load()
    buf = ctypes.create_string_buffer(4096)
    ok = (ctypes.addressof(buf) + 15) & ~15
    tail = (1, 1, 8, 64, 1.0, 1)
    # corope_rope_attn_bwd(q, k, v, o, d_o, lse, delta, cos, sin, stride, dq, dk, dv, ...): dq is used by the last launch
    rc = lib.corope_rope_attn_bwd(ok, ok, ok, ok, ok, ok, ok, ok, ok, 64, None, ok, ok, *tail, None)
    assert rc == -1 and "null" in pkg._lib.last_error()
    rc = lib.corope_rope_attn_bwd(ok, ok, ok, ok, ok, ok, ok, ok, ok, 64, ok + 2, ok, ok, *tail, None)
    assert rc == -3 and "aligned" in pkg._lib.last_error()
    # the same on rotated operands: dk / dv belong to the second launch
    rc = lib.corope_rope_attn_bwd_prerotated(ok, ok, ok, ok, ok, ok, ok, ok, ok, 64, ok, ok, None, *tail, None)
    assert rc == -1 and "null" in pkg._lib.last_error()
    rc = lib.corope_rope_attn_bwd_prerotated(ok, ok, ok, ok, ok, ok, ok, ok, ok, 64, ok, ok + 4, ok, *tail, None)
    assert rc == -3
    # with a workspace: the rotation passes come first, dq last
    need = lib.corope_rope_attn_bwd_workspace_bytes(1, 1, 8, 64)
    rc = lib.corope_rope_attn_bwd_ws(ok, ok, ok, ok, ok, ok, ok, ok, ok, 64, None, ok, ok, *tail, ok, need, None)
    assert rc == -1 and "null" in pkg._lib.last_error()
    rc = lib.corope_rope_attn_bwd_ws(ok, ok, ok, ok, ok, ok, ok, ok, ok, 64, ok, ok, ok, *tail, ok, need - 1, None)
    assert rc == -1 and "workspace" in pkg._lib.last_error()
    # dK+dV as two launches: v and dk belong to the second
    rc = lib.corope_rope_attn_bwd_dkdv(ok, ok, None, ok, ok, ok, ok, ok, 64, ok, ok, *tail, None)
    assert rc == -1 and "null" in pkg._lib.last_error()
    # training forward: o and lse belong to the second launch (the first rotates K)
    rc = lib.corope_rope_attn_fwd_train(ok, ok, ok, ok, ok, 64, None, ok, ok, ok, ok, *tail, None)
    assert rc == -1 and "null" in pkg._lib.last_error()
    rc = lib.corope_rope_attn_fwd_train(ok, ok, ok, ok, ok, 64, ok, ok + 8, ok, ok, ok, *tail, None)
    assert rc == -3
    # grouped-query forward with a rotation pass: q belongs to the second launch
    rc = lib.corope_rope_attn_fwd_gqa(None, ok, ok, ok, ok, 64, ok, ok, None, ok, ok, 1, 4, 2, 8, 64, 1.0, 1, None)
    assert rc == -1 and "null" in pkg._lib.last_error()
    # the forward that allocates nothing refuses oversized shapes and bad pointers alike without a launch
    rc = lib.corope_rope_attn_fwd_noalloc(ok, ok, ok, ok, ok, 64, ok, None, *tail, None)
    assert rc == -1 and "null" in pkg._lib.last_error()
    rc = lib.corope_rope_attn_fwd_noalloc(ok, ok, ok, ok, ok, 128, ok, ok, 4, 32, 4096, 128, 1.0, 1, None)
    assert rc == -2 and "scratch" in pkg._lib.last_error()


def test_no_entry_point_changes_later_calls(pkg):
    """The shipped library exports nothing that forces kernel forms (its measurement build does, for the tests)."""
    lib = pkg._lib.load()
    for name in ("corope_amd_set_tile_rows", "corope_debug_set_forms", "corope_debug_trace"):
        assert not hasattr(lib, name), name
    trace = pkg._lib.load_trace()
    assert trace.corope_debug_set_forms(64, 0) == -1 and trace.corope_debug_set_forms(0, 48) == -1
    assert trace.corope_debug_set_forms(128, 64) == 0 and trace.corope_debug_set_forms(0, 0) == 0


def test_grouped_query_argument_checks(pkg):
    """Head-count and pointer checks of the grouped-query entry points happen before any launch."""
    lib = pkg._lib.load()
    ok = 4096
    rc = lib.corope_rope_attn_fwd_gqa(ok, ok, ok, ok, ok, 64, ok, ok, None, None, None, 1, 6, 4, 8, 64, 1.0, 1, None)
    assert rc == -1 and "multiple" in pkg._lib.last_error()
    rc = lib.corope_rope_attn_fwd_gqa(ok, ok, ok, ok, ok, 64, ok, ok, ok, None, None, 1, 8, 2, 8, 64, 1.0, 1, None)
    assert rc == -1 and "q_rot without k_rot" in pkg._lib.last_error()
    rc = lib.corope_rope_attn_fwd_gqa(ok, ok, ok, ok, ok, 64, ok, ok, None, ok, None, 1, 8, 2, 8, 64, 1.0, 1, None)
    assert rc == -1 and "tile_kmax" in pkg._lib.last_error()
    rc = lib.corope_rope_attn_bwd_gqa(ok, ok, 1, ok, ok, ok, ok, ok, ok, ok, 64, ok, ok, ok, 1, 8, 3, 8, 64, 1.0, 1, None)
    assert rc == -1 and "multiple" in pkg._lib.last_error()
    rc = lib.corope_rope_attn_bwd_gqa(ok, ok, 1, ok, ok, ok, ok, ok, ok, ok, 64, ok, None, ok, 1, 8, 2, 8, 64, 1.0, 1, None)
    assert rc == -1 and "null" in pkg._lib.last_error()


def test_corope_backward_argument_checks(pkg):
    """Workspace size query and the checks corope_gqa_bwd makes before any launch (no GPU needed)."""
    lib = pkg._lib.load()
    packed = lambda n: sum(64 * (i // 64 + 1) for i in range(n))   # one lower-triangular matrix, rows padded to 64 keys
    assert lib.corope_gqa_bwd_workspace_bytes(2, 32, 8, 4096, 128) == 4 * (packed(4096) * (2 * 16 + 3 * 64) + 16 * 4096 * 128)
    assert lib.corope_gqa_bwd_workspace_bytes(1, 4, 2, 33, 64) == 4 * (packed(33) * (2 * 2 + 3 * 4) + 2 * 33 * 64)
    assert packed(4096) == 4096 * 4096 // 2 + 32 * 4096
    assert lib.corope_gqa_bwd_workspace_bytes(1, 5, 2, 33, 64) == -1      # Hq not a multiple of Hkv
    assert lib.corope_gqa_bwd_workspace_bytes(1, 18, 2, 33, 64) == -1     # group size 9
    assert lib.corope_gqa_bwd_workspace_bytes(1, 4, 2, 33, 96) == -1      # head dim not built
    buf = ctypes.create_string_buffer(4096)
    ok = (ctypes.addressof(buf) + 15) & ~15
    # the smallest accepted workspace holds one (batch, kv head) group: the full figure divided by the number of groups
    assert lib.corope_gqa_bwd_min_workspace_bytes(2, 32, 8, 4096, 128) * 16 == lib.corope_gqa_bwd_workspace_bytes(2, 32, 8, 4096, 128)
    assert lib.corope_gqa_bwd_min_workspace_bytes(1, 5, 2, 33, 64) == -1
    need = lib.corope_gqa_bwd_min_workspace_bytes(1, 4, 2, 8, 64)
    assert 2 * need == lib.corope_gqa_bwd_workspace_bytes(1, 4, 2, 8, 64)
    args = lambda ws, nbytes, dq=ok, o=None: (ok, ok, ok, o, ok, dq, ok, ok, 1, 4, 2, 8, 64, 0.125, 1e4, ws, nbytes, None)
    assert lib.corope_gqa_bwd(*args(None, need)) == -1 and "null" in pkg._lib.last_error()
    assert lib.corope_gqa_bwd(*args(ok, need, dq=ok + 2)) == -3 and "aligned" in pkg._lib.last_error()
    assert lib.corope_gqa_bwd(*args(ok, need - 4)) == -1 and "workspace" in pkg._lib.last_error()
    assert lib.corope_gqa_bwd(*args(ok, need, o=ok + 2)) == -3 and "aligned" in pkg._lib.last_error()   # o is optional, not sloppy
    rc = lib.corope_gqa_bwd(ok, ok, ok, None, ok, ok, ok, ok, 1, 18, 2, 8, 64, 0.125, 1e4, ok, 1 << 40, None)
    assert rc == -2 and "group size" in pkg._lib.last_error()


def test_rope_freqs_argument_checks(pkg):
    lib = pkg._lib.load()
    buf = ctypes.create_string_buffer(4096)
    ok = (ctypes.addressof(buf) + 15) & ~15
    assert lib.corope_rope_freqs(ok, ok, 0, 64, 64, 64, 0, 1e4, None) == -1
    assert lib.corope_rope_freqs(ok, ok, 8, 64, 48, 64, 0, 1e4, None) == -1      # width neither D nor D/2
    assert lib.corope_rope_freqs(ok, ok, 8, 64, 64, 32, 0, 1e4, None) == -1      # stride < width
    assert lib.corope_rope_freqs(ok, None, 8, 64, 64, 64, 0, 1e4, None) == -1
    assert lib.corope_rope_freqs(ok, ok, 8, 64, 64, 64, -1, 1e4, None) == -1
    with pytest.raises(ValueError):
        pkg.rope_freqs_device(64, 8, device="cpu")


def test_python_surface_matches_reference_order(pkg):
    # reference: forward(ctx, q, k, v, causal, sm_scale, freqs_cos, freqs_sin, warp_specialize=True)
    from importlib import import_module
    ra = import_module("co-rope_amd.rope_attn")
    cg = import_module("co-rope_amd.corope_gqa")
    assert list(inspect.signature(ra._FusedRopeAttn.forward).parameters) == [
        "ctx", "q", "k", "v", "causal", "sm_scale", "freqs_cos", "freqs_sin", "warp_specialize"]
    assert list(inspect.signature(cg._CoRopeGqaAttn.forward).parameters) == [
        "ctx", "q", "k", "v", "causal", "sm_scale", "theta", "warp_specialize"]
    assert list(inspect.signature(pkg.fused_rope_attn).parameters) == [
        "q", "k", "v", "freqs_cos", "freqs_sin", "causal", "sm_scale"]


def test_host_validation_raises_without_a_gpu(pkg):
    q = torch.zeros(1, 2, 16, 64, dtype=torch.bfloat16)
    c = torch.ones(16, 64)
    with pytest.raises(ValueError):          # CPU tensors: there is no CPU fallback
        pkg.attention(q, q, q, True, 0.125, c, c)
    with pytest.raises(AssertionError):      # mismatched head dims, as the reference asserts
        pkg.attention(q, q[..., :32], q, True, 0.125, c, c)
    with pytest.raises(ValueError):
        pkg.attention(torch.zeros(1, 2, 16, 32, dtype=torch.bfloat16), torch.zeros(1, 2, 16, 32, dtype=torch.bfloat16),
                      torch.zeros(1, 2, 16, 32, dtype=torch.bfloat16), True, 0.1, c, c)
    k = torch.zeros(1, 1, 16, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        pkg.corope_attention(q, k, k, False, 1.0, 1e4)          # non-causal
    with pytest.raises(ValueError):
        pkg.corope_attention(q, k, k[:, :, :8], True, 1.0, 1e4)  # k/v shape mismatch
    with pytest.raises(ValueError):
        pkg.corope_attention(q[0], k[0], k[0], True, 1.0, 1e4)   # rank
    with pytest.raises(ValueError):
        pkg.corope_attention(torch.zeros(1, 3, 16, 64, dtype=torch.bfloat16), torch.zeros(1, 2, 16, 64, dtype=torch.bfloat16),
                             torch.zeros(1, 2, 16, 64, dtype=torch.bfloat16), True, 1.0, 1e4)
    with pytest.raises(ValueError):
        pkg.corope_attention(q, k, k, True, 1.0, 1e4)            # CPU tensors


def test_freqs_match_oracle(pkg):
    from oracle import rope_attn_oracle as O
    c, s = pkg.precompute_freqs_cis(128, 300, 10000.0, device="cpu")
    rc, rs = O.precompute_freqs_cis(128, 300, 10000.0)
    assert torch.equal(c, rc) and torch.equal(s, rs) and c.shape == (300, 128)


def test_missing_library_fails_loudly(pkg, monkeypatch):
    monkeypatch.setattr(pkg._lib, "_lib", None)
    monkeypatch.setattr(pkg._lib, "LIB_PATH", "/nonexistent/libcorope_amd.so")
    with pytest.raises(pkg._lib.CoRopeLibraryError):
        pkg._lib.load()


def test_strided_forward_argument_checks(pkg):
    """Strides are checked before any launch: multiples of 8 elements, rows at least D apart, slices below 4 GiB."""
    import ctypes
    lib = pkg._lib.load()
    ok = 4096
    arr = lambda *x: (ctypes.c_int64 * 3)(*x)
    good = arr(8 * 64 * 100, 64, 8 * 64)
    tail = (ok, ok, 64, ok, ok, None, None, None, 1, 8, 8, 100, 64, 1.0, 1, 0, None)
    for bad in (arr(8 * 64 * 100, 64, 32), arr(8 * 64 * 100, 60, 8 * 64), arr(-512, 64, 512), arr(0, 0, 1 << 31)):
        rc = lib.corope_rope_attn_fwd_strided(ok, bad, ok, good, ok, good, *tail)
        assert rc in (-1, -2) and "stride" in pkg._lib.last_error(), list(bad)
    assert lib.corope_rope_attn_fwd_strided(ok, None, ok, good, ok, good, *tail) == -1
    assert lib.corope_rope_attn_fwd_strided(ok, good, ok, good, ok + 2, good, *tail) == -3


def test_alias_names_the_same_modules():
    """``corope_amd`` is an alias of the package in the directory ``co-rope_amd``: importing a submodule through either
    name gives the one module object whose globals the package's functions read (a second copy would have thresholds
    and switches of its own, and setting them would change nothing)."""
    from importlib import import_module
    pkg = import_module("corope_amd")
    for sub in ("rope_attn", "corope_gqa", "_lib", "freqs"):
        assert import_module("corope_amd." + sub) is import_module("co-rope_amd." + sub) is getattr(pkg, sub), sub
    assert pkg.attention.__globals__ is pkg.rope_attn.__dict__
