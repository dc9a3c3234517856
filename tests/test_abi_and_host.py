"""CPU-side checks: the C-ABI library loads and exports every symbol the header declares (no compute calls), the Python
binding table matches the header, and the host-side model plumbing (flat parameter groups, token generator, FLOP
count) behaves."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tfb_kernels.h")


def _declared():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    decls = {}
    for m in re.finditer(r"\b(int|long)\s+(tfb_\w+)\s*\(([^;]*?)\)\s*;", src, flags=re.S):
        args = [a.strip() for a in m.group(3).split(",") if a.strip() and a.strip() != "void"]
        decls[m.group(2)] = (m.group(1), args)
    return decls


def test_header_declares_entry_points():
    d = _declared()
    assert len(d) >= 25
    for name in ("tfb_gemm_bf16", "tfb_attn_fwd", "tfb_attn_bwd", "tfb_mlp8_fwd", "tfb_mlp8_bwd", "tfb_lmhead_fwd",
                 "tfb_rmsnorm_fwd", "tfb_loss_bwd", "tfb_adamw"):
        assert name in d


def test_library_exports_every_declared_symbol():
    from trainium_frontier_them_bones_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built (run __graft_entry__.build())")
    L = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared():
        assert hasattr(L, name), name


def test_binding_table_matches_header():
    from trainium_frontier_them_bones_amd import _lib
    d = _declared()
    assert set(_lib.SIGNATURES) == set(d)
    for name, (ret, args) in d.items():
        sig = _lib.SIGNATURES[name]
        assert len(sig) == len(args), name
        for a, c in zip(args, sig):
            if "*" in a:
                assert c in (ctypes.c_void_p, _lib._lp, _lib._fp), (name, a)
            elif a.startswith("float"):
                assert c is ctypes.c_float, (name, a)
            elif a.startswith("long"):
                assert c is ctypes.c_long, (name, a)
            else:
                assert c is ctypes.c_int, (name, a)


def test_ops_refuse_cpu_tensors():
    from trainium_frontier_them_bones_amd import ops
    with pytest.raises(RuntimeError):
        ops.matmul(torch.zeros(128, 64, dtype=torch.bfloat16), torch.zeros(64, 128, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError):
        ops.rmsnorm_fwd(torch.zeros(4, 64, dtype=torch.bfloat16))


def test_flat_params_layout_and_tokens():
    from trainium_frontier_them_bones_amd.model import FlatParams, GPTConfig, zipf_tokens
    fp = FlatParams({"a": (3, 5), "b": (7,), "c": (2, 8)}, torch.float32, "cpu")
    assert fp.offsets["a"] == (0, 15) and fp.offsets["b"][0] == 16 and fp.offsets["c"][0] == 24 and fp.numel == 40
    fp.load("b", torch.arange(7.0))
    assert torch.equal(fp.params["b"].detach().float(), torch.arange(7.0)) and fp.master[16:23].tolist() == list(range(7))
    assert fp.params["a"].grad_buf.shape == (3, 5) and fp.params["a"].grad_buf.dtype == torch.float32
    x, y = zipf_tokens(4, 64, 1000, seed=1)
    x2, _ = zipf_tokens(4, 64, 1000, seed=1)
    assert torch.equal(x, x2) and torch.equal(x[:, 1:], y[:, :-1]) and int(x.max()) < 1000
    cnt = torch.bincount(zipf_tokens(64, 512, 1000, seed=2)[0].reshape(-1), minlength=1000)
    assert cnt[0] > cnt[10] > cnt[200]            # Zipfian: low ids dominate
    cfg = GPTConfig()
    assert cfg.head_dim == 64


def test_bench_flop_formula():
    import bench
    from trainium_frontier_them_bones_amd.model import GPTConfig
    assert abs(bench.flops_per_token(GPTConfig()) / 1e6 - 773.8) < 0.5    # 773.8 MFLOP/token -> 25.36 TFLOP per 32768-token step


def test_every_entry_point_is_reached_from_the_host_layer():
    """Each exported kernel entry point is called by the package's host code (ops / autograd / the reference-named layers)
    or, for the plain forwarding forms, by a test: nothing in the header is dead."""
    import glob
    import os
    from trainium_frontier_them_bones_amd import _lib
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    host = "".join(open(f).read() for f in glob.glob(os.path.join(root, "trainium_frontier_them_bones_amd", "*.py"))
                   if not f.endswith("_lib.py"))
    tests = "".join(open(f).read() for f in glob.glob(os.path.join(root, "tests", "test_gpu_*.py")))
    for name in _lib.SIGNATURES:
        assert ('"%s"' % name) in host or ("." + name + "(") in host or name in tests, name


def test_amax_hint_is_void_after_an_in_place_update():
    """The amax partials a producer hangs on a gradient tensor are used only while the tensor still holds what they were
    taken from: the same memory, and no in-place write since (autograd may accumulate a second gradient into it)."""
    import torch
    from trainium_frontier_them_bones_amd import autograd as A
    t = torch.randn(8, 4)
    am = torch.tensor([float(t.abs().max())])
    A._attach_amax(t, am)
    assert A._amax_hint(t, t.reshape(8, 4)) is am
    assert A._amax_hint(t, t.clone()) is None                 # a copy is other memory
    old = A.USE_AMAX_HINT
    A.USE_AMAX_HINT = False
    try:
        assert A._amax_hint(t, t) is None
    finally:
        A.USE_AMAX_HINT = old
    t.add_(1.0)
    assert A._amax_hint(t, t) is None                         # written to since: the partials are void
    assert A._amax_hint(torch.randn(3), torch.randn(3)) is None


def test_every_entry_point_rejects_null_pointers_and_empty_shapes_on_the_host():
    """Argument checks come before any device work: with every pointer NULL an entry point answers "bad argument" (or
    "unsupported shape" where the sizes are looked at first), and with dummy non-null pointers and all sizes zero it answers
    with one of the two as well; no call reaches a kernel launch (status 3), so this runs without a GPU."""
    import ctypes
    from trainium_frontier_them_bones_amd import _lib
    L = _lib.lib()
    plain = _lib._LONG_RESULT | {"tfb_norm_bwd_blocks", "tfb_resmix_bwd_blocks"}      # size queries: no status to check
    for name, sig in _lib.SIGNATURES.items():
        if name in plain:
            continue
        for null in (True, False):
            args = []
            for t in sig:
                if t is _lib._vp:
                    args.append(None if null else 0x1000)          # never dereferenced on the host
                elif t is _lib._lp:
                    args.append(None if null else (ctypes.c_long * 4)())
                elif t is _lib._fp:
                    args.append(None if null else (ctypes.c_float * 16)())
                elif t is _lib._f:
                    args.append(0.0)
                else:
                    args.append(0)
            assert getattr(L, name)(*args) in (1, 2), (name, null)
