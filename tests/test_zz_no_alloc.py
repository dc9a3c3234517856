"""The attention backward entry point that allocates nothing (tfb_attn_bwd_static: its row-statistic scratch is a static
device array inside the library) against tfb_attn_bwd with caller-owned scratch: same kernels, so the gradients must be
equal bit for bit. Two calls in a row, the second on a smaller input (the array keeps the first call's contents), and
the size guard. Collected last: it must pass alone in a fresh process and after every other test."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(dev):
    from trainium_frontier_them_bones_amd import ops as _ops
    return _ops


def _case(ops, dev, B, H, T, D, seed, fused):
    g = torch.Generator().manual_seed(seed)
    if fused:
        # q, k, v as thirds of one [B, T, 3 H D] projection (token-major), gradients into thirds of one dqkv buffer
        qkv = torch.randn(B, T, 3 * H * D, generator=g).bfloat16().to(dev)
        q, k, v = (t.view(B, T, H, D) for t in qkv.split(H * D, dim=-1))
        layout = "bthd"
    else:
        q, k, v = (torch.randn(B, H, T, D, generator=g).bfloat16().to(dev) for _ in range(3))
        layout = "bhtd"
    do = torch.randn(B, T, H, D, generator=g).bfloat16().to(dev)
    scale = D ** -0.5
    o, lse = ops.attn_fwd(q, k, v, scale, layout=layout)
    if fused:
        want = torch.empty(B, T, 3 * H * D, dtype=torch.bfloat16, device=dev)
        got = torch.full_like(want, float("nan"))
        wq, wk, wv = (t.view(B, T, H, D) for t in want.split(H * D, dim=-1))
        gq, gk, gv = (t.view(B, T, H, D) for t in got.split(H * D, dim=-1))
    else:
        wq, wk, wv = (torch.empty(B, H, T, D, dtype=torch.bfloat16, device=dev) for _ in range(3))
        gq, gk, gv = (torch.full((B, H, T, D), float("nan"), dtype=torch.bfloat16, device=dev) for _ in range(3))
    ops.attn_bwd(q, k, v, o, do, lse, scale, layout=layout, dq=wq, dk=wk, dv=wv, out_layout=layout)
    before = torch.cuda.memory_allocated(dev)
    ops.attn_bwd_static(q, k, v, o, do, lse, scale, gq, gk, gv, layout=layout, out_layout=layout)
    assert torch.cuda.memory_allocated(dev) == before                        # the wrapper made no tensor either
    torch.cuda.synchronize()
    for a, b, name in ((gq, wq, "dq"), (gk, wk, "dk"), (gv, wv, "dv")):
        assert torch.isfinite(a.float()).all(), name
        assert torch.equal(a, b), name
    return q, k, v, o, do, lse, scale, layout, (gq, gk, gv)


def test_attn_bwd_static_matches_attn_bwd_on_two_calls_in_a_row(ops, dev):
    print("attn_bwd_static: B4 H6 T1024 D64 seed 71, then B2 H3 T256 D64 seed 72, then D128", flush=True)
    _case(ops, dev, 4, 6, 1024, 64, 71, fused=True)
    _case(ops, dev, 2, 3, 256, 64, 72, fused=False)        # smaller: the array still holds the first call's statistics
    _case(ops, dev, 1, 2, 256, 128, 73, fused=False)       # the D = 128 kernels read the same scratch


def test_attn_bwd_static_captured_into_a_hip_graph(ops, dev):
    """After one eager call (which resolves the static array's address and the kernels' LDS attributes), the entry point is
    captured into a HIP graph: three replays on new inputs, with eager calls and synchronisations between them, each
    equal to tfb_attn_bwd's gradients bit for bit."""
    B, H, T, D = 2, 4, 512, 64
    g = torch.Generator().manual_seed(81)

    def fresh():
        q, k, v = (torch.randn(B, H, T, D, generator=g).bfloat16().to(dev) for _ in range(3))
        do = torch.randn(B, T, H, D, generator=g).bfloat16().to(dev)
        o, lse = ops.attn_fwd(q, k, v, 0.125)
        return q, k, v, o, do, lse

    static = fresh()
    outs = tuple(torch.empty(B, H, T, D, dtype=torch.bfloat16, device=dev) for _ in range(3))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.attn_bwd_static(*static, 0.125, *outs)            # the warm-up the capture needs
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.attn_bwd_static(*static, 0.125, *outs)
    for rep in range(3):
        print("attn_bwd_static graph replay %d" % rep, flush=True)
        new = fresh()
        want = tuple(torch.empty(B, H, T, D, dtype=torch.bfloat16, device=dev) for _ in range(3))
        ops.attn_bwd(*new, 0.125, dq=want[0], dk=want[1], dv=want[2])   # eager work between the replays
        torch.cuda.synchronize()
        for s_, n_ in zip(static, new):
            s_.copy_(n_)
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(outs, want):
            assert torch.equal(a, b)


def test_attn_bwd_host_checks_reject_mismatched_tensors(ops, dev):
    q, k, v = (torch.zeros(1, 2, 256, 64, dtype=torch.bfloat16, device=dev) for _ in range(3))
    o = torch.zeros(1, 256, 2, 64, dtype=torch.bfloat16, device=dev)
    lse = torch.zeros(1, 2, 256, dtype=torch.float32, device=dev)
    outs = tuple(torch.zeros(1, 2, 256, 64, dtype=torch.bfloat16, device=dev) for _ in range(3))
    with pytest.raises(ValueError):
        ops.attn_bwd_static(q, k, v, o, o, lse[:, :1], 0.125, *outs)               # lse too short
    with pytest.raises(ValueError):
        ops.attn_bwd_static(q, k, v, o, o, lse.double(), 0.125, *outs)             # lse not fp32
    with pytest.raises(ValueError):
        ops.attn_bwd_static(q, k[:, :1], v, o, o, lse, 0.125, *outs)               # k with fewer heads
    with pytest.raises(ValueError):
        ops.attn_bwd(q, k, v, o.permute(0, 2, 1, 3), o, lse, 0.125)                # o not [B, T, H, D]
    with pytest.raises(ValueError):
        ops.attn_bwd_static(q, k, v, o, o, lse, 0.125, outs[0], outs[1], outs[2][:, :, :128])   # dv too short


def test_attn_bwd_static_refuses_sizes_beyond_its_array(ops, dev):
    from trainium_frontier_them_bones_amd import _lib
    max_rows = ops.attn_bwd_static_max_rows()
    assert max_rows == 1 << 20
    # B * H * T one row block beyond the maximum: refused on the host before any launch (the tensors are never read,
    # so small stand-ins with the right dtype are enough and no memory of that size is needed)
    B, H, T, D = 1, 1, int(max_rows) + 128, 64
    t = torch.zeros(1, 1, 128, D, dtype=torch.bfloat16, device=dev)
    lse = torch.zeros(1, 1, 128, dtype=torch.float32, device=dev)
    st = _lib.lib().tfb_attn_bwd_static(
        ops._p(t), ops._bht(t, "bhtd"), ops._p(t), ops._bht(t, "bhtd"), ops._p(t), ops._bht(t, "bhtd"), ops._p(t),
        ops._bht(t, "bhtd"), ops._p(t), ops._bht(t, "bhtd"), ops._p(t), ops._bht(t, "bhtd"), ops._p(t), ops._bht(t, "bhtd"),
        ops._p(t), ops._bht(t, "bhtd"), ops._p(lse), B, H, T, D, 0.125, None)
    assert st == 4
    with pytest.raises(_lib.TfbError):
        _lib.call("tfb_attn_bwd_static", ops._p(t), ops._bht(t, "bhtd"), ops._p(t), ops._bht(t, "bhtd"), ops._p(t),
                  ops._bht(t, "bhtd"), ops._p(t), ops._bht(t, "bhtd"), ops._p(t), ops._bht(t, "bhtd"), ops._p(t),
                  ops._bht(t, "bhtd"), ops._p(t), ops._bht(t, "bhtd"), ops._p(t), ops._bht(t, "bhtd"), ops._p(lse), B, H, T, D,
                  0.125, None)
