"""Parity of the HIP kernels (called through the C-ABI) against the CPU oracle on the same seeded inputs.
Tolerances: bit-exact for integer / byte work (fp8 bytes, weight packs, gathers, power-of-two scales); rel-L2 <= 5e-3
for bf16 paths and <= 2e-2 for fp8 paths; losses within 1e-3 relative."""
import math

import pytest
import torch

from helpers import fp8_table, rel_l2

pytestmark = pytest.mark.gpu

BF16_TOL = 5e-3
FP8_TOL = 2e-2


@pytest.fixture(scope="module")
def ops():
    from trainium_frontier_them_bones_amd import ops as _ops
    return _ops


def _g(seed):
    return torch.Generator().manual_seed(seed)


# ------------------------------------------------------------------------------------------ GEMM
@pytest.mark.parametrize("shape", [(128, 128, 64), (256, 384, 512), (1024, 768, 768), (768, 768, 8192), (128, 256, 16384)])
@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_gemm_layouts(ops, dev, shape, ta, tb):
    M, N, K = shape
    g = _g(M + N + K)
    a = torch.randn((K, M) if ta else (M, K), generator=g).bfloat16()
    b = torch.randn((N, K) if tb else (K, N), generator=g).bfloat16()
    ref = (a.float().t() if ta else a.float()) @ (b.float().t() if tb else b.float())
    c = ops.matmul(a.to(dev), b.to(dev), ta, tb)
    assert rel_l2(c, ref.bfloat16()) < 1e-3 and rel_l2(c, ref) < BF16_TOL
    base = torch.randn(M, N, generator=g)
    c32 = ops.matmul(a.to(dev), b.to(dev), ta, tb, out=base.to(dev).clone(), accumulate=True)
    assert rel_l2(c32, ref + base) < 1e-5
    cb = ops.matmul(a.to(dev), b.to(dev), ta, tb, out=base.bfloat16().to(dev), accumulate=True)
    assert rel_l2(cb, ref + base.bfloat16().float()) < BF16_TOL


def test_gemm_rejects_bad_shapes(ops, dev):
    from trainium_frontier_them_bones_amd._lib import TfbError
    with pytest.raises(TfbError) as e:
        ops.matmul(torch.zeros(100, 64, dtype=torch.bfloat16, device=dev), torch.zeros(64, 128, dtype=torch.bfloat16, device=dev))
    assert e.value.status == 1


# ------------------------------------------------------------------------------------------ norms / elementwise
@pytest.mark.parametrize("C", [256, 768, 1024, 2048])
@pytest.mark.parametrize("weighted", [False, True])
def test_rmsnorm_fwd_bwd(ops, dev, C, weighted):
    from oracle import norm as O
    g = _g(C)
    N = 512 + 4
    x, r, gy, gs = (torch.randn(N, C, generator=g).bfloat16() for _ in range(4))
    w = (1 + 0.02 * torch.randn(C, generator=g)).bfloat16() if weighted else None
    eps = 1e-6 if weighted else O.RMS_EPS
    s, y, inv = ops.rmsnorm_fwd(x.to(dev), None if w is None else w.to(dev), eps, res=r.to(dev))
    so, yo, invo = O.add_rmsnorm(x, r, w, eps)
    assert torch.equal(s.cpu(), so)
    assert (y.cpu() != yo).float().mean().item() < 1e-3 and rel_l2(y, yo) < 1e-3       # at most rare 1-ulp flips
    assert rel_l2(inv, invo) < 1e-6
    dx, dw = ops.rmsnorm_bwd(gy.to(dev), s, inv, None if w is None else w.to(dev), gs.to(dev))
    dxo, dwo = O.add_rmsnorm_backward(gs, gy, so, invo, w)
    assert rel_l2(dx, dxo) < 1e-3
    if weighted:
        assert rel_l2(dw, dwo) < 1e-4
    _, y1, _ = ops.rmsnorm_fwd(x.to(dev), None if w is None else w.to(dev), eps)
    assert rel_l2(y1, O.rmsnorm(x, w, eps)[0]) < 1e-3


def test_norm_with_fp8_cast_and_projections_with_residual_equal_the_separate_passes(ops, dev):
    """The folded forms (norm that also writes the next GEMM's e4m3 operand; projections and the MLP with the residual add
    in their store) against the separate passes they replace, bit for bit, and against the oracle's composition."""
    from oracle import mlp8 as OM, norm as ON
    g = _g(33)
    M, d, F = 512, 768, 3072
    x, res = (torch.randn(M, d, generator=g).bfloat16() for _ in range(2))
    w = (1 + 0.02 * torch.randn(d, generator=g)).bfloat16()
    xd, rd, wd = x.to(dev), res.to(dev), w.to(dev)
    # norm + cast
    for r_ in (None, rd):
        s0, y0, inv0 = ops.rmsnorm_fwd(xd, wd, 1e-6, res=r_)
        s1, y1, inv1, y8 = ops.rmsnorm_fwd_q(xd, wd, 1e-6, res=r_, y8_scale=4.0)
        assert torch.equal(s0, s1) and torch.equal(y0, y1) and torch.equal(inv0, inv1)
        assert torch.equal(y8, ops.quant_fp8(y0, 4.0, ops.FMT_E4M3))
        assert torch.equal(y8.cpu().view(torch.float8_e4m3fn).float(), (y0.cpu().float() * 4.0).to(torch.float8_e4m3fn).float())
    # bf16 projection + residual
    wo = (0.02 * torch.randn(d, d, generator=g)).bfloat16().to(dev)
    assert torch.equal(ops.matmul_res(xd, wo, rd, trans_b=True), ops.matmul(xd, wo, trans_b=True) + rd)
    assert torch.equal(ops.matmul_res(xd, wo, rd), ops.matmul(xd, wo) + rd)
    # fp8 projection + residual
    x8 = ops.quant_fp8(xd, 4.0, ops.FMT_E4M3)
    sw = torch.tensor([64.0, 1.0 / 64.0], device=dev)
    w8 = ops.quant_fp8(wo, sw[0:1], ops.FMT_E4M3)
    assert torch.equal(ops.gemm_fp8_res(x8, w8, rd, None, sw[1:2], 0.25), ops.gemm_fp8(x8, w8, ops.FMT_E4M3, None, sw[1:2], 0.25) + rd)
    # fp8 MLP from the norm's bytes, residual in the second GEMM's store
    wf = (0.02 * torch.randn(F, d, generator=g)).bfloat16()
    wp = (0.02 * torch.randn(d, F, generator=g)).bfloat16()
    row = ops.mlp8_forward_scales(wf.to(dev), wp.to(dev))
    pack = ops.mlp8_precast(wf.to(dev), wp.to(dev), row)
    _, h, _, h8 = ops.rmsnorm_fwd_q(xd, wd, 1e-6, y8_scale=4.0)
    y_sep, r_sep = ops.mlp8_fwd(h, pack, row, F)
    y_fold, r_fold = ops.mlp8_fwd(h, pack, row, F, x8=h8, res=xd)
    assert torch.equal(r_fold, r_sep) and torch.equal(y_fold, y_sep + xd)
    ho = ON.rmsnorm(x, w, 1e-6)[0]
    yo, _ = OM.forward(ho, wf, wp, OM.forward_scales(wf, wp))
    assert rel_l2(y_fold, (yo + x).bfloat16()) < FP8_TOL
    from trainium_frontier_them_bones_amd._lib import TfbError
    with pytest.raises(TfbError):
        ops.matmul_res(xd[:100], wo, rd[:100], trans_b=True)                      # rows % 128 != 0


def test_norm_weight_gradients_finished_in_one_launch(ops, dev):
    """rmsnorm_bwd(part=...) + norm_dw_finish equals the per-call weight gradient bit for bit (same partials, same
    order of summation), also when added into."""
    g = _g(21)
    rows, C, n = 2048, 768, 3
    xs = [torch.randn(rows, C, generator=g).bfloat16().to(dev) for _ in range(n)]
    gys = [torch.randn(rows, C, generator=g).bfloat16().to(dev) for _ in range(n)]
    w = (1 + 0.02 * torch.randn(C, generator=g)).bfloat16().to(dev)
    parts = torch.empty(n, ops.norm_bwd_blocks(rows), C, dtype=torch.float32, device=dev)
    want, dxs = [], []
    for i in range(n):
        _, _, inv = ops.rmsnorm_fwd(xs[i], w, 1e-6)
        dx, dw = ops.rmsnorm_bwd(gys[i], xs[i], inv, w)
        dx2, none = ops.rmsnorm_bwd(gys[i], xs[i], inv, w, part=parts[i])
        assert none is None and torch.equal(dx, dx2)
        want.append(dw)
    out = torch.full((n, C), 7.0, dtype=torch.float32, device=dev)
    ops.norm_dw_finish(parts, out, rows)
    assert torch.equal(out, torch.stack(want))
    ops.norm_dw_finish(parts, out, rows, accumulate=True)
    assert torch.equal(out, 2 * torch.stack(want))


def test_block_head(ops, dev):
    from oracle import norm as O
    g = _g(11)
    x, x0, sk, g1, g2 = (torch.randn(1024, 768, generator=g).bfloat16() for _ in range(5))
    gains = torch.tensor([0.9, 0.25, -0.4])
    for skip in (None, sk):
        xn, xnorm, inv = ops.block_head_fwd(x.to(dev), x0.to(dev), gains.to(dev), None if skip is None else skip.to(dev))
        o = O.block_head(x, x0, gains[0], gains[1], skip, gains[2])
        assert torch.equal(xn.cpu(), o[0]) and rel_l2(xnorm, o[1]) < 1e-3
        dx, dx0, dsk, dg = ops.block_head_bwd(g1.to(dev), g2.to(dev), x.to(dev), x0.to(dev), xn, inv, gains.to(dev),
                                              None if skip is None else skip.to(dev))
        ob = O.block_head_backward(g1, g2, x, x0, o[0], o[2], gains[0], gains[1], skip, gains[2])
        assert rel_l2(dx, ob[0]) < 1e-3 and rel_l2(dx0, ob[1]) < 1e-3
        assert abs(dg[0].item() - ob[3].item()) < 1e-3 * abs(ob[3].item()) + 0.05
        assert abs(dg[1].item() - ob[4].item()) < 1e-3 * abs(ob[4].item()) + 0.05
        if skip is not None:
            assert rel_l2(dsk, ob[2]) < 1e-3 and abs(dg[2].item() - ob[5].item()) < 1e-3 * abs(ob[5].item()) + 0.05


def test_relu2_rope_resmix_embedding_bit_exact(ops, dev):
    from oracle import attention as OA
    from oracle import norm as O
    g = _g(12)
    x, gy = (torch.randn(512, 3072, generator=g).bfloat16() for _ in range(2))
    assert torch.equal(ops.relu2(x.to(dev)).cpu(), O.relu2(x))
    assert torch.equal(ops.relu2_bwd(x.to(dev), gy.to(dev)).cpu(), O.relu2_backward(x, gy))
    h = O.relu2(x)
    assert rel_l2(ops.relu2_bwd_from_h(h.to(dev), gy.to(dev)), O.relu2_backward_from_h(h, gy)) < 1e-3
    B, T, H, D = 2, 256, 4, 64
    qkv = torch.randn(B, T, 3 * H * D, generator=g).bfloat16()
    cos, sin = OA.rope_tables(T, D)
    qd = qkv.to(dev).clone()
    ops.rope_(qd, cos.to(dev), sin.to(dev), T, 2 * H, D)
    ref = qkv.clone()
    ref[..., : 2 * H * D] = OA.rope(qkv[..., : 2 * H * D].reshape(B, T, 2 * H, D), cos, sin).reshape(B, T, 2 * H * D)
    assert torch.equal(qd.cpu(), ref)                      # the v third is untouched, q and k rotate bit-exactly
    gback = qd.clone()
    ops.rope_(gback, cos.to(dev), sin.to(dev), T, 2 * H, D, inverse=True)
    want = ref.clone()
    want[..., : 2 * H * D] = OA.rope_backward(ref[..., : 2 * H * D].reshape(B, T, 2 * H, D), cos, sin).reshape(B, T, 2 * H * D)
    assert torch.equal(gback.cpu(), want)
    gx, xx, x0 = (torch.randn(4096, 768, generator=g).bfloat16() for _ in range(3))
    ab = torch.tensor([0.9, 0.3])
    dx, dx0, dab = ops.resmix_bwd(gx.to(dev), xx.to(dev), x0.to(dev), ab.to(dev))
    r = O.resmix_backward(gx, xx, x0, ab[0], ab[1])
    assert torch.equal(dx.cpu(), r[0]) and torch.equal(dx0.cpu(), r[1])
    assert abs(dab[0].item() - r[2].item()) < 1e-3 * abs(r[2].item()) + 0.05
    idx = torch.randint(0, 1000, (4, 128), generator=g)
    idx[0, :64] = 7                                          # heavy collisions
    w = torch.randn(1000, 768, generator=g).bfloat16()
    assert torch.equal(ops.embedding_fwd(idx.to(dev), w.to(dev)).cpu(), w[idx])
    assert torch.equal(ops.embedding_fwd(idx.int().to(dev), w.to(dev)).cpu(), w[idx])
    dy = torch.randn(4, 128, 768, generator=g).bfloat16()
    dw = ops.fill_f32_(torch.empty(1000, 768, device=dev), 0.0)
    ops.embedding_bwd(idx.to(dev), dy.to(dev), dw)
    want = torch.zeros(1000, 768).index_add_(0, idx.reshape(-1), dy.float().reshape(-1, 768))
    assert rel_l2(dw, want) < 1e-6
    # ragged row count, int32 ids, accumulation into a non-zero dW, Zipf-like skew
    idx2 = (torch.rand(1237, generator=g) ** 4 * 1000).long().clamp_(0, 999)
    dy2 = torch.randn(1237, 768, generator=g).bfloat16()
    ops.embedding_bwd(idx2.int().to(dev), dy2.to(dev), dw)
    want.index_add_(0, idx2, dy2.float())
    assert rel_l2(dw, want) < 1e-6
    # the plain atomic entry point gives the same sums; every row on one token and every row on its own token
    dwa = ops.fill_f32_(torch.empty(1000, 768, device=dev), 0.0)
    ops.embedding_bwd(idx.to(dev), dy.to(dev), dwa, grouped=False)
    ops.embedding_bwd(idx2.to(dev), dy2.to(dev), dwa, grouped=False)
    assert rel_l2(dwa, want) < 1e-6
    for ids in (torch.full((512,), 3, dtype=torch.long), torch.randperm(1000, generator=g)[:512]):
        dy3 = torch.randn(512, 768, generator=g).bfloat16()
        w3 = torch.zeros(1000, 768).index_add_(0, ids, dy3.float())
        for grouped in (True, False):
            d3 = ops.fill_f32_(torch.empty(1000, 768, device=dev), 0.0)
            ops.embedding_bwd(ids.to(dev), dy3.to(dev), d3, grouped=grouped)
            assert rel_l2(d3, w3) < 1e-6
    # ids outside [0, V) are never addresses: zero rows forward, no gradient backward, every other row unchanged
    bad = idx2.clone()
    bad[::7] = 1000
    bad[3::11] = -5
    bad[5::13] = 1 << 40
    ok = (bad >= 0) & (bad < 1000)
    e = ops.embedding_fwd(bad.to(dev), w.to(dev)).cpu()
    assert torch.equal(e[ok], w[bad[ok]]) and not e[~ok].any()
    wantb = torch.zeros(1000, 768).index_add_(0, bad[ok], dy2.float()[ok])
    for grouped in (True, False):
        d4 = ops.fill_f32_(torch.empty(1000, 768, device=dev), 0.0)
        ops.embedding_bwd(bad.to(dev), dy2.to(dev), d4, grouped=grouped)
        assert rel_l2(d4, wantb) < 1e-6


def test_adamw(ops, dev):
    from oracle import optim as O
    g = _g(13)
    n = 1 << 18
    p = torch.randn(n, generator=g)
    m, v = torch.zeros(n), torch.zeros(n)
    pd, md, vd = p.to(dev), m.to(dev), v.to(dev)
    p16 = torch.empty(n, dtype=torch.bfloat16, device=dev)
    for step in (1, 2, 3):
        gr = torch.randn(n, generator=g).bfloat16()
        ops.adamw_(pd, gr.to(dev), md, vd, step, 3e-4, 0.9, 0.95, 1e-8, 0.1, p16)
        O.adamw_step(p, gr, m, v, step, 3e-4, 0.9, 0.95, 1e-8, 0.1)
    assert (pd.cpu() - p).abs().max().item() < 5e-7 and rel_l2(md, m) < 1e-6 and rel_l2(vd, v) < 1e-6
    assert torch.equal(p16.cpu(), pd.cpu().bfloat16())
    # sizes that are not a multiple of four (one-element gains, odd vectors): the kernel's element-wise tail
    for n in (1, 3, 1027):
        p = torch.randn(n, generator=g)
        m, v = torch.zeros(n), torch.zeros(n)
        pd, md, vd = p.to(dev), m.to(dev), v.to(dev)
        p16 = torch.empty(n, dtype=torch.bfloat16, device=dev)
        for step in (1, 2):
            gr = torch.randn(n, generator=g)
            ops.adamw_(pd, gr.to(dev), md, vd, step, 3e-4, 0.9, 0.95, 1e-8, 0.1, p16)
            O.adamw_step(p, gr, m, v, step, 3e-4, 0.9, 0.95, 1e-8, 0.1)
        assert (pd.cpu() - p).abs().max().item() < 5e-7 and (md.cpu() - m).abs().max().item() < 1e-6
        assert (vd.cpu() - v).abs().max().item() < 1e-6 and torch.equal(p16.cpu(), pd.cpu().bfloat16())


# ------------------------------------------------------------------------------------------ fp8 MLP
def test_fp8_casts_exhaustive_against_format_tables(ops, dev):
    from oracle import mlp8 as O
    allb = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    allb = allb[torch.isfinite(allb.float())]
    allb = torch.cat([allb, torch.zeros((-allb.numel()) % 8, dtype=torch.bfloat16)])
    for fmt, name, lim in ((0, "e4m3fn", 448.0), (1, "e5m2", 57344.0)):
        table = fp8_table(name)
        for sc in (1.0, 4.0, 0.03125, 2048.0):
            q = ops.quant_fp8(allb.to(dev), sc, fmt).cpu()
            v = allb.float() * sc
            ok = v.abs() <= lim
            assert torch.equal(q[ok], O.fp8_bytes(v, fmt)[ok])             # every bf16 value: bytes equal torch's cast
            dec = table[q.long()]
            assert bool(((dec[ok] - v[ok].double()).abs() <= (v[ok].double().abs() * 2.0 ** -3 + 2.0 ** -10)).all())
            sat = table[q[~ok].long()].abs()
            assert bool((sat == lim).all())                               # beyond the range: saturates
        s = torch.tensor([0.5], device=dev)
        assert torch.equal(ops.quant_fp8(allb.to(dev), s, fmt).cpu(), ops.quant_fp8(allb.to(dev), 0.5, fmt).cpu())
        # a NaN stays a NaN through the cast (as torch's), it is not turned into the format's largest value
        nan = torch.full((16,), float("nan"), dtype=torch.bfloat16)
        nan[::2] = 1.0
        qn = ops.quant_fp8(nan.to(dev), 1.0, fmt).cpu().view(torch.float8_e5m2 if fmt else torch.float8_e4m3fn).float()
        assert bool(torch.isnan(qn[1::2]).all()) and bool((qn[::2] == 1.0).all())


@pytest.mark.parametrize("shape", [(256, 256, 512), (1024, 768, 3072), (384, 1024, 2816 - 2816 % 256)])
@pytest.mark.parametrize("limit", [240.0, 448.0])
def test_mlp8_scales_precast_forward_backward(ops, dev, shape, limit):
    from oracle import mlp8 as O
    M, d, F = shape
    g = _g(M + d + F)
    x = torch.randn(M, d, generator=g).bfloat16()
    wf = (0.02 * torch.randn(F, d, generator=g)).bfloat16()
    wp = (0.02 * torch.randn(d, F, generator=g)).bfloat16()
    dy = torch.randn(M, d, generator=g).bfloat16()
    row_o = O.forward_scales(wf, wp, limit)
    xd, wfd, wpd, dyd = x.to(dev), wf.to(dev), wp.to(dev), dy.to(dev)
    row = ops.mlp8_forward_scales(wfd, wpd, limit)
    pow2_cols = [0, 1, 2, 3, 4, 11, 12, 13, 14, 15]
    assert torch.equal(row.cpu()[pow2_cols], row_o[pow2_cols])              # scales and amax: exact
    assert torch.allclose(row.cpu()[9:11], row_o[9:11], rtol=1e-5)         # norms: fp32 summation order
    w8 = ops.mlp8_precast(wfd, wpd, row)
    a8 = O.fp8_bytes(wf.float() * row_o[0], 0)
    b8 = O.fp8_bytes(wp.float() * row_o[3], 0)
    for got, want in zip(w8.cpu(), (a8, a8.t(), b8, b8.t())):
        assert torch.equal(got, want.reshape(-1))
    y, r = ops.mlp8_fwd(xd, w8, row, F)
    yo, ro = O.forward(x, wf, wp, row_o)
    assert rel_l2(r, ro) < 2e-3 and rel_l2(y, yo) < FP8_TOL
    rowb_o = O.backward_scales(dy, row_o)
    rowb = ops.mlp8_backward_scales(dyd, row)
    assert torch.equal(rowb.cpu()[5:9], rowb_o[5:9])
    dx, h, dpre = ops.mlp8_bwd(dyd, r, w8, rowb)
    dxo, ho, dpo = O.backward(dy, r.cpu(), wf, wp, rowb_o)
    assert torch.equal(h.cpu(), ho) and rel_l2(dpre, dpo) < 2e-3 and rel_l2(dx, dxo) < FP8_TOL
    dwfo, dwpo = O.weight_grads(dy, x, h.cpu(), dpre.cpu())
    assert rel_l2(ops.matmul(dpre, xd, trans_a=True), dwfo) < BF16_TOL
    assert rel_l2(ops.mlp_dw_proj(dyd, r), dwpo) < BF16_TOL
    acc = torch.randn(d, F, generator=g)
    got = ops.mlp_dw_proj(dyd, r, out=acc.to(dev).clone(), accumulate=True)
    assert rel_l2(got, (dy.float().t() @ ho.float()) + acc) < 1e-4
    st = ops.amax_scale(dyd, 28672.0, -40, 60).cpu()
    assert st[0].item() == rowb_o[5].item() and st[2].item() == dy.float().abs().max().item()


@pytest.mark.parametrize("shape", [(256, 256, 512), (1024, 768, 3072), (4096, 768, 3072)])
@pytest.mark.parametrize("limit", [240.0, 448.0])
def test_mlp8_fp8_weight_grads(ops, dev, shape, limit):
    """tfb_mlp8_bwd_q + tfb_mlp8_dw8 against the oracle's fp8 weight gradients; the operand bytes bit for bit."""
    from oracle import mlp8 as O
    from helpers import fp8_table
    M, d, F = shape
    g = _g(7 * M + d + F)
    x = torch.randn(M, d, generator=g).bfloat16()
    wf = (0.02 * torch.randn(F, d, generator=g)).bfloat16()
    wp = (0.02 * torch.randn(d, F, generator=g)).bfloat16()
    dy = torch.randn(M, d, generator=g).bfloat16()
    xd, wfd, wpd, dyd = x.to(dev), wf.to(dev), wp.to(dev), dy.to(dev)
    row = ops.mlp8_forward_scales(wfd, wpd, limit)
    w8 = ops.mlp8_precast(wfd, wpd, row)
    y, r, x8 = ops.mlp8_fwd(xd, w8, row, F, want_x8=True)
    rowb = ops.mlp8_backward_scales(dyd, row)
    dx, dpre, dp8, hq8, dy8 = ops.mlp8_bwd_q(dyd, r, w8, rowb, limit)
    dx0, _, dpre0 = ops.mlp8_bwd(dyd, r, w8, rowb, want_h=False)
    assert torch.equal(dx, dx0) and torch.equal(dpre, dpre0)                       # the extra output changes nothing else
    rb = rowb.cpu()
    s_dp, s_h, s_dy = (rb[O.COL[k]] for k in ("s_dp", "s_h", "s_dy"))
    hb = (r.cpu().float() * r.cpu().float()).bfloat16()
    assert torch.equal(x8.cpu(), O.fp8_bytes(x.float() * 4.0, 0))
    assert torch.equal(dy8.cpu(), O.fp8_bytes(dy.float() * s_dy, 1))
    assert torch.equal(dp8.cpu(), O.fp8_bytes(dpre.cpu().float() * s_dp, 1))
    assert torch.equal(hq8.cpu(), O.fp8_bytes(torch.clamp_max(hb.float() * s_h, limit), 0))
    dw_fc, dw_proj = ops.mlp8_dw8(x8, dp8, hq8, dy8, rowb)
    # the oracle on the same saved activations (r and dpre as the device produced them)
    o_fc, o_pj = O.weight_grads_fp8(x, dy, hb, dpre.cpu(), rb, e4m3_limit=limit)
    assert rel_l2(dw_fc, o_fc) < 2e-3 and rel_l2(dw_proj, o_pj) < 2e-3             # summation order + one bf16 rounding
    # and through the byte tables, in fp64
    t4, t5 = fp8_table("e4m3fn"), fp8_table("e5m2")
    ref_fc = (t5[dp8.cpu().long()].t() @ t4[x8.cpu().long()]) / float(s_dp * 4.0)
    ref_pj = (t5[dy8.cpu().long()].t() @ t4[hq8.cpu().long()]) / float(s_dy * s_h)
    assert rel_l2(dw_fc, ref_fc) < 3e-3 and rel_l2(dw_proj, ref_pj) < 3e-3
    # within the fp8 budget of the bf16 weight gradients
    b_fc, b_pj = O.weight_grads(dy, x, hb, dpre.cpu())
    assert rel_l2(dw_fc, b_fc) < 0.08 and rel_l2(dw_proj, b_pj) < 0.08
    # fp32 outputs, accumulated into
    acc_fc = torch.randn(F, d, generator=g)
    acc_pj = torch.randn(d, F, generator=g)
    a_fc, a_pj = ops.mlp8_dw8(x8, dp8, hq8, dy8, rowb, dw_fc=acc_fc.to(dev).clone(), dw_proj=acc_pj.to(dev).clone(), accumulate=True)
    assert rel_l2(a_fc, ref_fc + acc_fc) < 1e-4 and rel_l2(a_pj, ref_pj + acc_pj) < 1e-4


def test_mlp8_activation_scale_from_the_device(ops, dev):
    """The activation scale as a device scalar (the per-tensor amax scale, never read back by the host) gives the layer
    the host-float path's outputs and gradients bit for bit: scale row, forward, backward and both fp8 weight gradients."""
    from trainium_frontier_them_bones_amd import autograd as A
    M, d, F = 1024, 256, 512
    g = _g(4242)
    x = (3.0 * torch.randn(M, d, generator=g)).bfloat16().to(dev)
    wf = (0.02 * torch.randn(F, d, generator=g)).bfloat16().to(dev)
    wp = (0.02 * torch.randn(d, F, generator=g)).bfloat16().to(dev)
    dy = torch.randn(M, d, generator=g).bfloat16().to(dev)
    sc = ops.amax_scale(x, 448.0, -20, 20)
    host = float(sc[0].item())
    assert host > 0 and host == 2.0 ** round(torch.log2(torch.tensor(host)).item())      # a power of two
    outs = []
    for x_scale in (host, sc[0:1]):
        xl, wfl, wpl = (t.clone().requires_grad_(True) for t in (x, wf, wp))
        st = A.Mlp8State(e4m3_limit=448.0, x_scale=x_scale, dw_fp8=True)
        st.refresh(wfl, wpl)
        y = A.Mlp8Fn.apply(xl, wfl, wpl, st)
        y.backward(dy)
        outs.append((st.row, y.detach(), xl.grad, wfl.grad, wpl.grad))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    with pytest.raises(ValueError):
        ops.mlp8_forward_scales(wf, wp, 448.0, sc)                                       # three elements: not a scalar


def test_norm_that_writes_only_the_bytes_the_mlp_reads(ops, dev):
    """RMSNormPassFn(bytes_only) -> Mlp8Fn with fp8 weight gradients: the norm's bf16 rows are not written (the tensor handed
    on is a storage-less NaN placeholder) and outputs and gradients equal the path that writes them, bit for bit."""
    from trainium_frontier_them_bones_amd import autograd as A
    M, d, F = 1024, 256, 512
    g = _g(515)
    x = torch.randn(4, M // 4, d, generator=g).bfloat16().to(dev)
    nw = (1 + 0.1 * torch.randn(d, generator=g)).bfloat16().to(dev)
    wf = (0.02 * torch.randn(F, d, generator=g)).bfloat16().to(dev)
    wp = (0.02 * torch.randn(d, F, generator=g)).bfloat16().to(dev)
    dy = torch.randn(4, M // 4, d, generator=g).bfloat16().to(dev)
    outs = []
    for bytes_only in (False, True):
        xl, nl, wfl, wpl = (t.clone().requires_grad_(True) for t in (x, nw, wf, wp))
        st = A.Mlp8State(dw_fp8=True)
        st.refresh(wfl, wpl)
        s, h, h8 = A.RMSNormPassFn.apply(xl, nl, 1e-6, st.x_scale, bytes_only)
        if bytes_only:
            assert h.shape == x.shape and h.stride() == (0, 0, 0) and bool(torch.isnan(h).all())
        y = A.Mlp8Fn.apply(h, wfl, wpl, st, h8, s)
        y.backward(dy)
        outs.append((y.detach(), xl.grad, nl.grad, wfl.grad, wpl.grad))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    with pytest.raises(ValueError):
        A.RMSNormPassFn.apply(x, nw, 1e-6, None, True)
    # the one-node form (parameter-free norm, x + MLP(norm(x))) with fp8 weight gradients writes no bf16 rows either and
    # equals the two-node composition that does
    eps = 2.0 ** -23
    res = []
    for fused in (True, False):
        xl, wfl, wpl = (t.clone().requires_grad_(True) for t in (x.reshape(M, d), wf, wp))
        st = A.Mlp8State(dw_fp8=True)
        st.refresh(wfl, wpl)
        if fused:
            y = A.NrMlpFn.apply(xl, wfl, wpl, st, eps)
        else:
            s, h, h8 = A.RMSNormPassFn.apply(xl, None, eps, st.x_scale, False)
            y = A.Mlp8Fn.apply(h, wfl, wpl, st, h8, s)
        y.backward(dy.reshape(M, d))
        res.append((y.detach(), xl.grad, wfl.grad, wpl.grad))
    for a, b in zip(*res):
        assert torch.equal(a, b)


def test_norm_backward_hands_its_amax_to_the_mlp_backward(ops, dev):
    """rmsnorm_bwd(want_amax): the partials' maximum is amax of the dx it wrote, bit for bit, and the scale row taken from
    them equals the one taken from a pass over dx. Through autograd (two norm + fp8 MLP blocks in a row, so that the first
    block's MLP receives the second block's norm gradient): gradients with the hand-over equal those without it."""
    from trainium_frontier_them_bones_amd import autograd as A
    M, d, F = 1024, 256, 512
    g = _g(616)
    x = torch.randn(M, d, generator=g).bfloat16().to(dev)
    gy = torch.randn(M, d, generator=g).bfloat16().to(dev)
    gs = (torch.randn(M, d, generator=g) * torch.logspace(-2, 1, M)[:, None]).bfloat16().to(dev)
    nw = (1 + 0.1 * torch.randn(d, generator=g)).bfloat16().to(dev)
    _, _, inv = ops.rmsnorm_fwd(x, nw, 1e-6)
    dx0, dw0 = ops.rmsnorm_bwd(gy, x, inv, nw, gs)
    dx1, dw1, am = ops.rmsnorm_bwd(gy, x, inv, nw, gs, want_amax=True)
    assert torch.equal(dx0, dx1) and torch.equal(dw0, dw1)
    assert float(am.max()) == float(dx1.float().abs().max()) and am.numel() == ops.norm_bwd_blocks(M)
    wf = (0.02 * torch.randn(F, d, generator=g)).bfloat16().to(dev)
    wp = (0.02 * torch.randn(d, F, generator=g)).bfloat16().to(dev)
    row = ops.mlp8_forward_scales(wf, wp)
    assert torch.equal(ops.mlp8_backward_scales(dx1, row), ops.mlp8_backward_scales(dx1, row, am))

    def two_blocks(hint, skip=False):
        old = A.USE_AMAX_HINT
        A.USE_AMAX_HINT = hint
        try:
            xl = x.clone().requires_grad_(True)
            ps = [t.clone().requires_grad_(True) for t in (nw, wf, wp, nw, wf, wp)]
            h = xl
            mids = []
            for b in range(2):
                n_, f_, p_ = ps[3 * b:3 * b + 3]
                st = A.Mlp8State(dw_fp8=True)
                st.refresh(f_, p_)
                s_, y_, y8_ = A.RMSNormPassFn.apply(h, n_, 1e-6, st.x_scale, True)
                h = A.Mlp8Fn.apply(y_, f_, p_, st, y8_, s_)
                mids.append(h)
            if skip:                           # the first block's output has a second reader: its gradient is a sum
                h = h + 0.5 * mids[0]
            h.backward(gy)
            return [xl.grad] + [t.grad for t in ps]
        finally:
            A.USE_AMAX_HINT = old

    seen = []
    real = ops.mlp8_backward_scales
    ops.mlp8_backward_scales = lambda dy2, row_, amax_part=None: (seen.append(amax_part is not None), real(dy2, row_, amax_part))[1]
    try:
        with_hint = two_blocks(True)
        assert seen == [False, True]           # the last block's dy comes from outside, the first block's from the norm backward
        without = two_blocks(False)
        assert seen == [False, True, False, False]
    finally:
        ops.mlp8_backward_scales = real
    for a, b in zip(with_hint, without):
        assert torch.equal(a, b)
    # with a second reader of the first block's output, autograd sums two gradients for it and may do so in place in the
    # tensor the norm backward wrote: partials taken before the sum must not be used for it
    for a, b in zip(two_blocks(True, skip=True), two_blocks(False, skip=True)):
        assert torch.equal(a, b)


def test_mlp8_layer_replayed_as_a_hip_graph(ops, dev):
    """The fp8 MLP layer with everything per-step inside (amax activation scale on the device, scale row, weight packs,
    forward, backward, fp8 weight gradients) recorded once as a HIP graph: three replays on new inputs, with eager runs
    of the same layer and synchronisations between them, each equal to the eager result bit for bit."""
    from trainium_frontier_them_bones_amd import autograd as A
    M, d, F = 1024, 256, 512
    g = _g(77)

    def fresh():
        return ((2.0 * torch.randn(M, d, generator=g)).bfloat16().to(dev), (0.02 * torch.randn(F, d, generator=g)).bfloat16().to(dev),
                (0.02 * torch.randn(d, F, generator=g)).bfloat16().to(dev), torch.randn(M, d, generator=g).bfloat16().to(dev))

    def layer(x, wf, wp, dy):
        xl, wfl, wpl = (t.detach().requires_grad_(True) for t in (x, wf, wp))
        st = A.Mlp8State(e4m3_limit=448.0, x_scale=ops.amax_scale(xl.detach(), 448.0, -20, 20)[0:1], dw_fp8=True)
        st.refresh(wfl, wpl)
        y = A.Mlp8Fn.apply(xl, wfl, wpl, st)
        y.backward(dy)
        return y.detach(), xl.grad, wfl.grad, wpl.grad

    static = fresh()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            layer(*static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = layer(*static)
    for _ in range(3):
        new = fresh()
        want = [t.clone() for t in layer(*new)]          # eager work between the replays
        torch.cuda.synchronize()
        for s_, n_ in zip(static, new):
            s_.copy_(n_)
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(outs, want):
            assert torch.equal(a, b)


def test_mlp8_refresh_of_all_layers_equals_per_layer_calls(ops, dev):
    g = _g(31)
    L, d, F = 3, 256, 512
    per = 2 * F * d + 1024                                                 # w_fc, w_proj and some other parameters
    flat = (0.05 * torch.randn(L * per, generator=g)).bfloat16().to(dev)
    wfc = [flat[i * per:i * per + F * d].view(F, d) for i in range(L)]
    wpj = [flat[i * per + F * d:i * per + 2 * F * d].view(d, F) for i in range(L)]
    rows, w8 = ops.mlp8_refresh_layers(wfc[0], wpj[0], per, L, 448.0, 4.0)
    for i in range(L):
        row = ops.mlp8_forward_scales(wfc[i], wpj[i], 448.0, 4.0)
        assert torch.equal(rows[i], row)
        assert torch.equal(w8[i], ops.mlp8_precast(wfc[i], wpj[i], row))


def test_mlp8_full_size_properties(ops, dev):
    """configuration 3 of BASELINE.json sizes: exact equivariance under a permutation of the tokens and agreement of 512-row slices
    with the oracle."""
    from oracle import mlp8 as O
    M, d, F = 16384, 768, 3072
    g = _g(3)
    x = torch.randn(M, d, generator=g).bfloat16()
    wf = (0.02 * torch.randn(d, F, generator=g)).bfloat16().t().contiguous()      # W_up [768, 3072] -> [F, d]
    wp = (0.02 * torch.randn(F, d, generator=g)).bfloat16().t().contiguous()      # W_down [3072, 768] -> [d, F]
    dy = torch.randn(M, d, generator=g).bfloat16()
    xd, wfd, wpd, dyd = x.to(dev), wf.to(dev), wp.to(dev), dy.to(dev)
    row = ops.mlp8_forward_scales(wfd, wpd)
    w8 = ops.mlp8_precast(wfd, wpd, row)
    y, r = ops.mlp8_fwd(xd, w8, row, F)
    row_o = O.forward_scales(wf, wp)
    yo, ro = O.forward(x[:512], wf, wp, row_o)
    assert rel_l2(y[:512], yo) < FP8_TOL and rel_l2(r[:512], ro) < 2e-3
    perm = torch.randperm(M, generator=g).to(dev)
    y2, r2 = ops.mlp8_fwd(xd[perm].contiguous(), w8, row, F)
    assert torch.equal(r2, r[perm]) and torch.equal(y2, y[perm])                   # tokens are independent: exact equivariance
    rowb = ops.mlp8_backward_scales(dyd, row)
    dx, _, dpre = ops.mlp8_bwd(dyd, r, w8, rowb, want_h=False)
    dxo, _, dpo = O.backward(dy[-512:], r[-512:].cpu(), wf, wp, O.backward_scales(dy, row_o))
    assert rel_l2(dx[-512:], dxo) < FP8_TOL and rel_l2(dpre[-512:], dpo) < 2e-3
    assert torch.isfinite(dx.float()).all() and torch.isfinite(y.float()).all()


@pytest.mark.parametrize("M,Ms,F", [(2048, 1920, 3072), (8192, 8064, 768), (5632, 5504, 1280)])
def test_mlp8_weight_stationary_kernel_equals_the_tiled_kernel(ops, dev, M, Ms, F):
    """With d_model = 768 the up-projection and the dH GEMM of a batch of a multiple of 512 tokens run the weight-stationary
    kernel (weights in registers, tokens streamed), any other batch the 128 x 128 tiled kernel. Tokens are independent, so
    the rows the two batches share must come out bit for bit the same: r, y, dx, dpre, h, and the fp8 bytes handed to the
    weight gradients. M is a multiple of 512 (weight-stationary), Ms = M - 128 is not (tiled); the shapes give runs of equal
    and of unequal length per workgroup, with and without panel borders inside a run."""
    d = 768
    g = _g(768 + F)
    x = torch.randn(M, d, generator=g).bfloat16().to(dev)
    wf = (0.02 * torch.randn(F, d, generator=g)).bfloat16().to(dev)
    wp = (0.02 * torch.randn(d, F, generator=g)).bfloat16().to(dev)
    dy = torch.randn(M, d, generator=g).bfloat16().to(dev)
    row = ops.mlp8_forward_scales(wf, wp, 448.0)
    w8 = ops.mlp8_precast(wf, wp, row)
    y, r = ops.mlp8_fwd(x, w8, row, F)
    ys, rs = ops.mlp8_fwd(x[:Ms].contiguous(), w8, row, F)
    assert torch.equal(r[:Ms], rs) and torch.equal(y[:Ms], ys)
    rowb = ops.mlp8_backward_scales(dy, row)
    dx, h, dpre = ops.mlp8_bwd(dy, r, w8, rowb)
    dxs, hs, dps = ops.mlp8_bwd(dy[:Ms].contiguous(), rs, w8, rowb)
    assert torch.equal(dpre[:Ms], dps) and torch.equal(h[:Ms], hs) and torch.equal(dx[:Ms], dxs)
    dxq, _, dp8, hq8, _ = ops.mlp8_bwd_q(dy, r, w8, rowb, 448.0, want_dpre=False)
    dxqs, _, dp8s, hq8s, _ = ops.mlp8_bwd_q(dy[:Ms].contiguous(), rs, w8, rowb, 448.0, want_dpre=False)
    assert torch.equal(dp8[:Ms], dp8s) and torch.equal(hq8[:Ms], hq8s) and torch.equal(dxq[:Ms], dxqs) and torch.equal(dxq, dx)


@pytest.mark.parametrize("fmt", [0, 1])
def test_fp8_projection_weight_stationary_kernel_equals_the_tiled_kernel(ops, dev, fmt):
    """tfb_gemm_fp8 / tfb_gemm_fp8_res with a contraction of 768 bytes: a batch of a multiple of 512 tokens runs the
    weight-stationary kernel, a shorter one the tiled kernel; the rows they share are equal bit for bit (e4m3 activations and
    e5m2 gradients, plain store and the store with the residual add)."""
    M, Ms, K, N = 2048, 1920, 768, 2304
    g = _g(99 + fmt)
    a8 = ops.quant_fp8(torch.randn(M, K, generator=g).bfloat16().to(dev), 4.0, fmt)
    b8 = ops.quant_fp8((0.05 * torch.randn(N, K, generator=g)).bfloat16().to(dev), 64.0, 0)
    dq = torch.tensor([1.0 / 256.0], device=dev)
    y = ops.gemm_fp8(a8, b8, fmt, dq_a=dq, dq=0.5)
    ys = ops.gemm_fp8(a8[:Ms].contiguous(), b8, fmt, dq_a=dq, dq=0.5)
    assert torch.equal(y[:Ms], ys)
    want = (a8.view(torch.float8_e5m2 if fmt else torch.float8_e4m3fn).float() @ b8.view(torch.float8_e4m3fn).float().t()) / 512.0
    assert rel_l2(y, want) < BF16_TOL
    if fmt == 0:
        res = torch.randn(M, N, generator=g).bfloat16().to(dev)
        z = ops.gemm_fp8_res(a8, b8, res, dq_a=dq, dq=0.5)
        zs = ops.gemm_fp8_res(a8[:Ms].contiguous(), b8, res[:Ms].contiguous(), dq_a=dq, dq=0.5)
        assert torch.equal(z[:Ms], zs) and torch.equal(z, (res.float() + y.float()).bfloat16())


@pytest.mark.parametrize("shape", [(512, 256, 512), (16384, 768, 3072)])
def test_mlp8_as_the_benchmark_times_it(ops, dev, shape):
    """Configuration 3 of BASELINE.json in the form bench.py times: OCP e4m3 at 448, the activation scale from the tensor's
    amax (a power of two, left on the device), all six GEMMs in fp8 (weight gradients from the bytes the other GEMMs
    multiplied), through the autograd wrapper. Against the oracle with the same limit and the same activation scale:
    y and dx on two 512-row slices (2e-2), both weight gradients over all rows (2e-2)."""
    from oracle import mlp8 as O
    from trainium_frontier_them_bones_amd import autograd as A
    M, d, F = shape
    g = _g(20263)
    x = torch.randn(M, d, generator=g).bfloat16()
    wf = (0.02 * torch.randn(d, F, generator=g)).bfloat16().t().contiguous()      # W_up [d, F] -> [F, d]
    wp = (0.02 * torch.randn(F, d, generator=g)).bfloat16().t().contiguous()      # W_down [F, d] -> [d, F]
    dy = torch.randn(M, d, generator=g).bfloat16()
    xl, wfl, wpl = (t.to(dev).requires_grad_(True) for t in (x, wf, wp))
    st = A.Mlp8State(e4m3_limit=448.0, dw_fp8=True)
    sc = ops.amax_scale(xl.detach(), 448.0, -20, 20)
    st.x_scale = sc[0:1]
    st.refresh(wfl, wpl)
    y = A.Mlp8Fn.apply(xl, wfl, wpl, st)
    y.backward(dy.to(dev))
    # the oracle's activation scale: the largest power of two s with amax(x) s <= 448
    xs, _ = O.pow2_floor_scale(x.float().abs().amax(), 448.0, -20, 20)
    assert float(sc[0].item()) == float(xs)
    xs = float(xs)
    row_o = O.forward_scales(wf, wp, 448.0, xs)
    assert torch.equal(st.row.cpu()[[0, 1, 2, 3, 4]], row_o[[0, 1, 2, 3, 4]])
    yo, ro = O.forward(x, wf, wp, row_o, xs)
    rowb_o = O.backward_scales(dy, row_o)
    dxo, ho, dpo = O.backward(dy, ro, wf, wp, rowb_o)
    for sl in (slice(0, 512), slice(M - 512, M)):
        assert rel_l2(y[sl], yo[sl]) < FP8_TOL and rel_l2(xl.grad[sl], dxo[sl]) < FP8_TOL
    o_fc, o_pj = O.weight_grads_fp8(x, dy, ho, dpo, rowb_o, x_scale=xs, e4m3_limit=448.0)
    assert rel_l2(wfl.grad, o_fc) < FP8_TOL and rel_l2(wpl.grad, o_pj) < FP8_TOL
    # and within the fp8 budget of the plain bf16 layer (the reference's off-device expression)
    b_fc, b_pj = O.weight_grads(dy, x, ho, dpo)
    assert rel_l2(wfl.grad, b_fc) < 0.08 and rel_l2(wpl.grad, b_pj) < 0.08


@pytest.mark.parametrize("ta,tb", [(False, True), (False, False), (True, False), (True, True)])
def test_gemm_long_contraction_in_every_operand_layout(ops, dev, ta, tb):
    """Long contractions over at least 64 output tiles of 256 x 256 run the persistent kernel in all four operand layouts
    (k-contiguous and k-strided operands, the latter through the transposing LDS reads), here with the k range cut into
    four work items per tile and finished through the fp32 workspace: against the fp32 product of the same bf16 values,
    also accumulated into an fp32 output and scaled by a device scalar; and without a split (one round of tiles), bit-equal
    to the same product assembled from narrow column slices on the 128 x 128 kernel where that one does not split either."""
    g = _g(17 + 2 * ta + tb)
    for (M, N, K) in ((4096, 1024, 8192), (4096, 4096, 8192)):
        a = torch.randn((K, M) if ta else (M, K), generator=g).bfloat16()
        b = torch.randn((N, K) if tb else (K, N), generator=g).bfloat16()
        ref = (a.float().t() if ta else a.float())[:512] @ (b.float().t() if tb else b.float())
        ad, bd = a.to(dev), b.to(dev)
        c = ops.matmul(ad, bd, trans_a=ta, trans_b=tb)
        assert rel_l2(c[:512], ref) < BF16_TOL
        if N == 1024:
            acc = torch.randn(M, N, generator=g)
            al = torch.tensor([0.5], device=dev)
            got = ops.matmul(ad, bd, trans_a=ta, trans_b=tb, out=acc.to(dev).clone(), accumulate=True, alpha=al)
            assert rel_l2(got[:512], 0.5 * ref + acc[:512]) < 1e-4


@pytest.mark.parametrize("shape", [(2304, 768, 8192), (768, 768, 32768), (768, 3072, 16384), (1024, 512, 20480)])
def test_gemm_long_contraction_over_few_tiles(ops, dev, shape):
    """Weight-gradient shapes: a token contraction of at least 128 k-tiles over fewer than 64 output tiles of 256 x 256 runs the
    persistent kernel with one k range per workgroup (27 tiles: 8 ranges; 9 tiles: 24 uneven ranges of 21 or 22 k-tiles; 36
    tiles: 7 ranges; 8 tiles: 32 ranges of 10 k-tiles are too short, so fewer), the partial tiles summed through the fp32
    workspace: against the fp32 product of the same bf16 values, fresh, accumulated into an fp32 buffer, and scaled."""
    M, N, K = shape
    g = _g(M + 3 * N + K)
    a = torch.randn(K, M, generator=g).bfloat16()
    b = torch.randn(K, N, generator=g).bfloat16()
    ad, bd = a.to(dev), b.to(dev)
    ref = (ad.float().t() @ bd.float()).cpu()
    c = ops.matmul(ad, bd, trans_a=True)
    assert rel_l2(c, ref) < BF16_TOL
    acc = torch.randn(M, N, generator=g)
    al = torch.tensor([0.25], device=dev)
    got = ops.matmul(ad, bd, trans_a=True, out=acc.to(dev).clone(), accumulate=True, alpha=al)
    assert rel_l2(got, 0.25 * ref + acc) < 1e-4
    # the other operand order of the same contraction (k-strided P against k-contiguous Q)
    c2 = ops.matmul(ad, bd.t().contiguous(), trans_a=True, trans_b=True)
    assert rel_l2(c2, ref) < BF16_TOL


@pytest.mark.parametrize("shape", [(2048, 1024, 1024, 128), (512, 4096, 1536, 128), (8192, 256, 1984, 128)])
def test_gemm_256_tile_kernel_equals_the_128_tile_kernel(ops, dev, shape):
    """A product large enough for the persistent 256 x 256 kernel (both operands k-contiguous, 16 to 31 k-tiles: long enough
    for that kernel, short enough that no k-split is chosen) equals, bit for bit, the same product assembled from column
    slices too narrow for it (which run the 128 x 128 kernel): the two kernels add the same terms in the same order. Also
    against the fp64 product, with the residual add in the store and with the device scalar factor."""
    M, N, K, w = shape
    g = _g(M + N + K)
    a = torch.randn(M, K, generator=g).bfloat16().to(dev)
    b = torch.randn(N, K, generator=g).bfloat16().to(dev)
    c = ops.matmul(a, b, trans_b=True)
    parts = [ops.matmul(a, b[n0:n0 + w].contiguous(), trans_b=True) for n0 in range(0, N, w)]
    assert torch.equal(c, torch.cat(parts, dim=1))
    ref = a[:256].double() @ b.double().t()
    assert rel_l2(c[:256], ref) < BF16_TOL
    # the same product with either operand stored k-strided (the transposing LDS reads feed the same sums)
    at, bt = a.t().contiguous(), b.t().contiguous()
    assert torch.equal(ops.matmul(at, b, trans_a=True, trans_b=True), c)
    assert torch.equal(ops.matmul(a, bt), c)
    assert torch.equal(ops.matmul(at, bt, trans_a=True), c)
    res = torch.randn(M, N, generator=g).bfloat16().to(dev)
    assert torch.equal(ops.matmul_res(a, b, res, trans_b=True), (c.float() + res.float()).bfloat16())
    al = torch.tensor([0.37], device=dev)
    assert rel_l2(ops.matmul(a, b, trans_b=True, alpha=al)[:256], 0.37 * ref) < BF16_TOL


# ------------------------------------------------------------------------------------------ attention
@pytest.mark.parametrize("shape", [(1, 2, 128, 64), (2, 3, 512, 64), (1, 1, 1024, 64), (1, 2, 256, 128), (2, 1, 512, 128)])
def test_attention_fwd_bwd(ops, dev, shape):
    from oracle import attention as O
    B, H, T, D = shape
    g = _g(T + H)
    q, k, v = (torch.randn(B, H, T, D, generator=g).bfloat16() for _ in range(3))
    do = torch.randn(B, T, H, D, generator=g).bfloat16()
    scale = 1.0 / math.sqrt(D)
    o, lse = ops.attn_fwd(q.to(dev), k.to(dev), v.to(dev), scale)
    oo, lo = O.forward(q, k, v, scale)
    assert rel_l2(o, oo) < BF16_TOL and rel_l2(lse, lo) < 1e-4
    assert rel_l2(o, O.sdpa_reference(q, k, v, scale)) < BF16_TOL             # and against the library routine
    dq, dk, dv = ops.attn_bwd(q.to(dev), k.to(dev), v.to(dev), o, do.to(dev), lse, scale)
    dqo, dko, dvo = O.backward(q, k, v, o.cpu(), do, lse.cpu(), scale)
    assert rel_l2(dq, dqo) < BF16_TOL and rel_l2(dk, dko) < BF16_TOL and rel_l2(dv, dvo) < BF16_TOL


@pytest.mark.parametrize("ramp", [0.5, 3.0, 12.0])
def test_attention_growing_row_maximum(ops, dev, ramp):
    """Scores whose row maximum keeps growing along the keys (slowly, by a few powers of two per tile, and by far more
    than the range of one tile): the forward's reference point of the exponentials has to follow at every rate, and the
    output and log-sum-exp must not depend on when it does."""
    from oracle import attention as O
    B, H, T, D = 1, 2, 1024, 64
    g = _g(31)
    q = torch.randn(B, H, T, D, generator=g).abs().bfloat16()
    k = torch.randn(B, H, T, D, generator=g).abs()
    k = (k * (1.0 + ramp * torch.arange(T).float()[None, None, :, None] / T)).bfloat16()   # q.k > 0 and growing with the key
    k[:, :, 700:] *= 0.25                                                                    # ... then far below the maximum
    v = torch.randn(B, H, T, D, generator=g).bfloat16()
    o, lse = ops.attn_fwd(q.to(dev), k.to(dev), v.to(dev), 0.125)
    oo, lo = O.forward(q, k, v, 0.125)
    assert torch.isfinite(o.float()).all() and torch.isfinite(lse).all()
    assert rel_l2(o, oo) < BF16_TOL and rel_l2(lse, lo) < 1e-4
    assert rel_l2(o, O.sdpa_reference(q, k, v, 0.125)) < BF16_TOL


@pytest.mark.parametrize("shape,nw", [((1, 2, 1024, 64), 1), ((2, 2, 1024, 64), 3), ((1, 2, 1024, 64), 4), ((1, 1, 768, 128), 2),
                                      ((1, 2, 512, 128), 4), ((1, 1, 512, 64), 9)])
def test_attention_tile_band(ops, dev, shape, nw):
    """The reference's windowed layers (band_mask, K/nki_attn_bandpro.py:1654): a query of 128-token tile i sees the keys
    k <= q of tiles i - nw + 1 .. i. Forward and backward against the oracle with the same mask; a band as wide as the
    sequence equals the full causal kernels bit for bit."""
    from oracle import attention as O
    B, H, T, D = shape
    g = _g(T + D + nw)
    q, k, v = (torch.randn(B, H, T, D, generator=g).bfloat16() for _ in range(3))
    do = torch.randn(B, T, H, D, generator=g).bfloat16()
    scale = 1.0 / math.sqrt(D)
    qd, kd, vd, dod = q.to(dev), k.to(dev), v.to(dev), do.to(dev)
    o, lse = ops.attn_fwd(qd, kd, vd, scale, band=nw)
    oo, lo = O.forward(q, k, v, scale, band_tiles=nw)
    assert rel_l2(o, oo) < BF16_TOL and rel_l2(lse, lo) < 1e-4
    dq, dk, dv = ops.attn_bwd(qd, kd, vd, o, dod, lse, scale, band=nw)
    dqo, dko, dvo = O.backward(q, k, v, o.cpu(), do, lse.cpu(), scale, band_tiles=nw)
    assert rel_l2(dq, dqo) < BF16_TOL and rel_l2(dk, dko) < BF16_TOL and rel_l2(dv, dvo) < BF16_TOL
    if nw * 128 >= T:
        o2, lse2 = ops.attn_fwd(qd, kd, vd, scale)
        dq2, dk2, dv2 = ops.attn_bwd(qd, kd, vd, o2, dod, lse2, scale)
        assert torch.equal(o, o2) and torch.equal(lse, lse2) and torch.equal(dq, dq2) and torch.equal(dk, dk2) and torch.equal(dv, dv2)
    else:
        # keys before the band do not matter: perturbing them changes nothing for the last tile's queries
        k2, v2 = kd.clone(), vd.clone()
        first = T - nw * 128
        k2[:, :, :first] += 1.0
        v2[:, :, :first] -= 1.0
        o3, _ = ops.attn_fwd(qd, k2, v2, scale, band=nw)
        assert torch.equal(o3[:, T - 128:], o[:, T - 128:])


def test_attention_strided_qkv_and_rejects(ops, dev):
    from oracle import attention as O
    from trainium_frontier_them_bones_amd._lib import TfbError
    B, H, T, D = 2, 4, 256, 64
    g = _g(5)
    qkv = torch.randn(B, T, 3 * H * D, generator=g).bfloat16()
    do = torch.randn(B, T, H, D, generator=g).bfloat16()
    qd = qkv.to(dev)
    q, k, v = (t.view(B, T, H, D) for t in qd.split(H * D, dim=-1))
    o, lse = ops.attn_fwd(q, k, v, 0.125, layout="bthd")
    q4, k4, v4 = (t.reshape(B, T, H, D).permute(0, 2, 1, 3) for t in qkv.split(H * D, dim=-1))
    oo, lo = O.forward(q4, k4, v4, 0.125)
    assert rel_l2(o, oo) < BF16_TOL
    dqkv = torch.empty_like(qd)
    dq, dk, dv = (t.view(B, T, H, D) for t in dqkv.split(H * D, dim=-1))
    ops.attn_bwd(q, k, v, o, do.to(dev), lse, 0.125, "bthd", dq, dk, dv, "bthd")
    dqo, dko, dvo = O.backward(q4, k4, v4, o.cpu(), do, lse.cpu(), 0.125)
    want = torch.cat([t.permute(0, 2, 1, 3).reshape(B, T, H * D) for t in (dqo, dko, dvo)], dim=-1)
    assert rel_l2(dqkv, want) < BF16_TOL
    # inverse RoPE fused into the backward stores == the separate rotation pass over the bf16 gradient, bit for bit
    cos, sin = O.rope_tables(T, D)
    cosd, sind = cos.to(dev), sin.to(dev)
    unfused = dqkv.clone()
    ops.rope_(unfused.view(B * T, 3 * H * D), cosd, sind, T, 2 * H, D, inverse=True)
    fused = torch.empty_like(qd)
    fq, fk, fv = (t.view(B, T, H, D) for t in fused.split(H * D, dim=-1))
    ops.attn_bwd(q, k, v, o, do.to(dev), lse, 0.125, "bthd", fq, fk, fv, "bthd", rope=(cosd, sind))
    assert torch.equal(fused, unfused)
    with pytest.raises(TfbError):
        ops.attn_fwd(q[:, :100], k[:, :100], v[:, :100], 0.125, layout="bthd")       # T % 128 != 0


def test_attention_full_size_properties(ops, dev):
    """configuration 2 of BASELINE.json (B16 H12 T2048 D64, RoPE'd q and k): two (b, h) pairs against the oracle, causality by
    perturbing the future, and dV with dO = 1 equal to the column sums of P."""
    from oracle import attention as O
    B, H, T, D = 16, 12, 2048, 64
    g = _g(2)
    q, k, v = (torch.randn(B, H, T, D, generator=g) for _ in range(3))
    cos, sin = O.rope_tables(T, D, 10000.0, torch.float32)
    q = O.rope(q.transpose(1, 2), cos, sin).transpose(1, 2).bfloat16().contiguous()
    k = O.rope(k.transpose(1, 2), cos, sin).transpose(1, 2).bfloat16().contiguous()
    v = v.bfloat16()
    do = torch.randn(B, T, H, D, generator=g).bfloat16()
    qd, kd, vd, dod = q.to(dev), k.to(dev), v.to(dev), do.to(dev)
    o, lse = ops.attn_fwd(qd, kd, vd, 0.125)
    dq, dk, dv = ops.attn_bwd(qd, kd, vd, o, dod, lse, 0.125)
    for (b, h) in ((0, 0), (15, 11)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        oo, lo = O.forward(q[sl], k[sl], v[sl], 0.125)
        assert rel_l2(o[b:b + 1, :, h:h + 1], oo) < BF16_TOL
        dqo, dko, dvo = O.backward(q[sl], k[sl], v[sl], o[b:b + 1, :, h:h + 1].cpu(), do[b:b + 1, :, h:h + 1], lse[sl].cpu(), 0.125)
        assert rel_l2(dq[sl], dqo) < BF16_TOL and rel_l2(dk[sl], dko) < BF16_TOL and rel_l2(dv[sl], dvo) < BF16_TOL
    k2, v2 = kd.clone(), vd.clone()
    k2[:, :, 1500:] += 1.0
    v2[:, :, 1500:] -= 1.0
    o2, _ = ops.attn_fwd(qd, k2, v2, 0.125)
    assert torch.equal(o2[:, :1500], o[:, :1500])
    ones = torch.ones_like(dod)
    _, _, dv1 = ops.attn_bwd(qd, kd, vd, o, ones, lse, 0.125)
    p = torch.exp((q[3, 5].float() @ k[3, 5].float().t()) * 0.125 - lse[3, 5].cpu()[:, None]).bfloat16().float() * O.mask(T)
    assert rel_l2(dv1[3, 5, :, 0], p.sum(0)) < BF16_TOL


@pytest.mark.parametrize("T,nw", [(2048, 0), (4096, 0), (2048, 4), (4096, 4)])
def test_attention_head_dim_128_at_the_reference_lengths(ops, dev, T, nw):
    """Head dimension 128 (the reference's own models) at the sequence lengths the reference runs it on, B2 H6: two
    (batch, head) pairs against the oracle, forward and backward, the full causal triangle and a band of four tiles."""
    from oracle import attention as O
    B, H, D = 2, 6, 128
    g = _g(T + nw)
    q, k, v = (torch.randn(B, H, T, D, generator=g).bfloat16() for _ in range(3))
    do = torch.randn(B, T, H, D, generator=g).bfloat16()
    scale = 1.0 / math.sqrt(D)
    qd, kd, vd, dod = q.to(dev), k.to(dev), v.to(dev), do.to(dev)
    band = nw if nw else None
    if nw:
        o, lse = ops.attn_fwd(qd, kd, vd, scale, band=nw)
        dq, dk, dv = ops.attn_bwd(qd, kd, vd, o, dod, lse, scale, band=nw)
    else:
        o, lse = ops.attn_fwd(qd, kd, vd, scale)
        dq, dk, dv = ops.attn_bwd(qd, kd, vd, o, dod, lse, scale)
    for (b, h) in ((0, 1), (1, 5)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        oo, lo = O.forward(q[sl], k[sl], v[sl], scale, band_tiles=band)
        assert rel_l2(o[b:b + 1, :, h:h + 1], oo) < BF16_TOL and rel_l2(lse[sl], lo) < 1e-4
        dqo, dko, dvo = O.backward(q[sl], k[sl], v[sl], o[b:b + 1, :, h:h + 1].cpu(), do[b:b + 1, :, h:h + 1], lse[sl].cpu(),
                                   scale, band_tiles=band)
        assert rel_l2(dq[sl], dqo) < BF16_TOL and rel_l2(dk[sl], dko) < BF16_TOL and rel_l2(dv[sl], dvo) < BF16_TOL



# ------------------------------------------------------------------------------------------ loss head
@pytest.mark.parametrize("cap", [15.0, None])
def test_loss_fwd_bwd(ops, dev, cap):
    from oracle import loss as O
    g = _g(21)
    N, V = 512, 8192
    x = (3 * torch.randn(N, V, generator=g)).bfloat16()
    t = torch.randint(0, V, (N,), generator=g)
    t[5] = -1
    t[9] = V                                                                   # beyond the vocabulary: ignored too, never an address
    t[11] = 1 << 40
    w = O.row_weights(t, "mean", V)
    rows, lse = ops.loss_fwd(x.to(dev), t.to(dev), cap, w.to(dev))
    assert float(rows[9]) == 0.0 and float(rows[11]) == 0.0
    ro, lo = O.loss_rows(x, t, cap)
    assert rel_l2(rows, ro * w) < 1e-5 and rel_l2(lse, lo) < 1e-6
    assert abs(rows.sum().item() - O.fused_loss(x, t, "mean", cap).item()) < 1e-3 * O.fused_loss(x, t, "mean", cap).item()
    t32 = t.clamp(max=V).int()
    rows32, _ = ops.loss_fwd(x.to(dev), t32.to(dev), cap, w.to(dev))
    assert torch.equal(rows32, rows)
    grow = torch.rand(N, generator=g) / N
    d = ops.loss_bwd(x.to(dev), t.to(dev), lse, grow.to(dev), cap)
    assert rel_l2(d, O.loss_backward(x, t, lo, grow, cap)) < BF16_TOL
    assert float(d[5].float().abs().max()) == 0.0                              # the ignored row gets no gradient
    assert float(d[9].float().abs().max()) == 0.0 and float(d[11].float().abs().max()) == 0.0


def test_lmhead_config1(ops, dev):
    """configuration 1 of BASELINE.json at full size through the autograd layer: RMSNorm -> LM-head GEMM (+lse) -> CE, fwd + bwd."""
    from oracle import loss as O
    from trainium_frontier_them_bones_amd import autograd as A
    g = _g(20261)
    N, d, V = 8192, 768, 32768
    x = torch.randn(N, d, generator=g).bfloat16()
    nw = (1 + 0.02 * torch.randn(d, generator=g)).bfloat16()
    W = (0.02 * torch.randn(V, d, generator=g)).bfloat16()
    t = torch.randint(0, V, (N,), generator=g)
    xd = x.to(dev).requires_grad_(True)
    nd = nw.to(dev).requires_grad_(True)
    Wd = W.to(dev).requires_grad_(True)
    loss = A.LmHeadLossFn.apply(A.RMSNormFn.apply(xd, nd, 1e-6), Wd, t.to(dev), 0.0, "mean")
    loss.backward()
    lo, saved = O.lmhead_loss(x, nw, W, t, 1e-6, None)
    assert abs(loss.item() - lo.item()) < 1e-3 * lo.item()
    dx, dnw, dW = O.lmhead_loss_backward(x, nw, W, t, saved, 1e-6, None)
    assert rel_l2(xd.grad, dx) < BF16_TOL and rel_l2(Wd.grad, dW) < BF16_TOL and rel_l2(nd.grad, dnw) < BF16_TOL


@pytest.mark.parametrize("V", [1024, 32768, 50304, 65536])
@pytest.mark.parametrize("cap,idx", [(0.0, torch.int64), (15.0, torch.int32)])
def test_loss_forward_and_backward_in_one_pass_equal_the_two_kernels(ops, dev, V, cap, idx):
    """tfb_loss_fwd_bwd against tfb_loss_fwd + tfb_loss_bwd with grow = the row weights: row losses, lse and the gradient
    written in place of the logits, bit for bit; ignored rows (target < 0 or >= V) give zero loss and a zero gradient row."""
    g = _g(900 + V)
    N = 192
    x = (3.0 * torch.randn(N, V, generator=g)).bfloat16().to(dev)
    t = torch.randint(0, V, (N,), generator=g).to(idx)
    t[3], t[100] = -1, V + 7
    t = t.to(dev)
    w = torch.rand(N, generator=g).to(dev)
    rows0, lse0 = ops.loss_fwd(x, t, cap, w)
    d0 = ops.loss_bwd(x, t, lse0, w, cap)
    y = x.clone()
    rows1, lse1 = ops.loss_fwd_bwd(y, t, w, cap)
    assert torch.equal(rows0, rows1) and torch.equal(lse0, lse1) and torch.equal(d0, y)
    assert float(rows1[3]) == 0.0 and float(y[3].float().abs().max()) == 0.0 and float(y[100].float().abs().max()) == 0.0
    y2 = x.clone()
    rows2, _ = ops.loss_fwd_bwd(y2, t, None, cap)                                   # no row weights: weight one
    assert torch.equal(y2, ops.loss_bwd(x, t, lse0, torch.ones_like(w), cap))


def test_lmhead_loss_node_with_an_upstream_gradient(ops, dev):
    """LmHeadLossFn under an upstream gradient of one equals, bit for bit, the composition of the separate calls (GEMM, loss rows and
    lse, dlogits in place, two gradient GEMMs); under another upstream gradient (a scaled loss) the gradients follow the oracle's."""
    from oracle import loss as O
    from trainium_frontier_them_bones_amd import autograd as A
    g = _g(41)
    N, d, V = 1024, 256, 8192
    x = torch.randn(N, d, generator=g).bfloat16()
    W = (0.05 * torch.randn(V, d, generator=g)).bfloat16()
    t = torch.randint(0, V, (N,), generator=g)
    t[17] = -1
    xd, Wd, td = x.to(dev).requires_grad_(True), W.to(dev).requires_grad_(True), t.to(dev)
    loss = A.LmHeadLossFn.apply(xd, Wd, td, 15.0, "mean")
    loss.backward()
    valid = (td >= 0).float()
    w = valid / valid.sum()
    logits = ops.matmul(xd.detach(), Wd.detach(), trans_b=True)
    rows, lse = ops.loss_fwd(logits, td, 15.0, w)
    dl = ops.loss_bwd(logits, td, lse, w, 15.0, inplace=True)
    assert torch.equal(loss.detach(), rows.sum())
    assert torch.equal(xd.grad, ops.matmul(dl, Wd.detach())) and torch.equal(Wd.grad, ops.matmul(dl, xd.detach(), trans_a=True))
    gx, gw = xd.grad.clone(), Wd.grad.clone()
    xd.grad = Wd.grad = None
    (0.37 * A.LmHeadLossFn.apply(xd, Wd, td, 15.0, "mean")).backward()
    assert rel_l2(xd.grad, 0.37 * gx.float()) < BF16_TOL and rel_l2(Wd.grad, 0.37 * gw.float()) < BF16_TOL
    _, lse_o = O.loss_rows(F_linear(x, W), t, 15.0)
    grow = 0.37 * O.row_weights(t, "mean", V)
    dlo = O.loss_backward(F_linear(x, W), t, lse_o, grow, 15.0)
    assert rel_l2(xd.grad, dlo.float() @ W.float()) < BF16_TOL and rel_l2(Wd.grad, dlo.float().t() @ x.float()) < BF16_TOL


def F_linear(x, W):
    return (x.float() @ W.float().t()).bfloat16()


def test_lmhead_softcap_matches_materialised_path(ops, dev):
    g = _g(22)
    N, d, V = 1024, 768, 32768
    x = torch.randn(N, d, generator=g).bfloat16().to(dev)
    W = (0.05 * torch.randn(V, d, generator=g)).bfloat16().to(dev)
    t = torch.randint(0, V, (N,), generator=g).to(dev)
    logits, rows, lse = ops.lmhead_fwd(x, W, t, 15.0)
    assert torch.equal(logits, ops.matmul(x, W, trans_b=True))
    rows2, lse2 = ops.loss_fwd(logits, t, 15.0)
    assert rel_l2(rows, rows2) < 1e-5 and rel_l2(lse, lse2) < 1e-6


def test_lmhead_loss_with_every_target_ignored_and_with_one_valid_row(ops, dev):
    """ignore_index rows carry neither loss nor gradient: with all of them ignored the mean loss and every gradient are
    exactly zero; with one valid row the loss is that row's cross-entropy (torch's on the kernel's own logits)."""
    from trainium_frontier_them_bones_amd import autograd as A
    g = _g(23)
    N, d, V = 256, 256, 1024
    x = torch.randn(N, d, generator=g).bfloat16().to(dev).requires_grad_(True)
    W = (0.05 * torch.randn(V, d, generator=g)).bfloat16().to(dev).requires_grad_(True)
    t = torch.full((N,), -1, dtype=torch.long, device=dev)
    loss = A.LmHeadLossFn.apply(x, W, t, 15.0, "mean")
    loss.backward()
    assert loss.item() == 0.0 and float(x.grad.float().abs().max()) == 0.0 and float(W.grad.float().abs().max()) == 0.0
    x.grad = W.grad = None
    t[77] = 5
    loss = A.LmHeadLossFn.apply(x, W, t, 15.0, "mean")
    loss.backward()
    z = 15.0 * torch.tanh(ops.matmul(x.detach(), W.detach(), trans_b=True)[77].float() / 15.0)
    want = torch.nn.functional.cross_entropy(z[None], t[77:78])
    assert abs(loss.item() - want.item()) < 1e-3 * want.item()
    rows = x.grad.float().abs().sum(1)
    assert float(rows[77]) > 0 and float(rows.sum() - rows[77]) == 0.0          # only the valid row has a gradient


def test_qkv_rope_projection_fused_equals_unfused(ops, dev):
    """The projection with the rotary embedding in its epilogue, and the autograd node built on it, against the
    separate GEMM / rotation / attention launches: bit for bit."""
    from oracle import attention as O
    from trainium_frontier_them_bones_amd import autograd as A
    B, T, H, D, Cin = 2, 256, 4, 64, 256
    g = _g(21)
    x = torch.randn(B, T, Cin, generator=g).bfloat16().to(dev)
    w = (0.05 * torch.randn(3 * H * D, Cin, generator=g)).bfloat16().to(dev)
    cos, sin = (t.to(dev) for t in O.rope_tables(T, D))
    fused = ops.qkv_rope(x.view(B * T, Cin), w, cos, sin, T, 2 * H * D)
    plain = ops.matmul(x.view(B * T, Cin), w, trans_b=True)
    ops.rope_(plain, cos, sin, T, 2 * H, D)
    assert torch.equal(fused, plain)
    go = torch.randn(B, T, H * D, generator=g).bfloat16().to(dev)
    x1, w1 = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    y1 = A.QkvRopeAttentionFn.apply(x1, w1, cos, sin, H, 0.125)
    y1.backward(go)
    x2, w2 = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    y2 = A.RopeAttentionFn.apply(A.LinearFn.apply(x2, w2), cos, sin, H, 0.125)
    y2.backward(go)
    assert torch.equal(y1, y2) and torch.equal(x1.grad, x2.grad) and torch.equal(w1.grad, w2.grad)


# ------------------------------------------------------------------------------------------ Muon Newton-Schulz
# Five chained iterations amplify one-ulp bf16 flips: two evaluations of the ORACLE that differ only in the order of the
# fp32 sums (fp32 against fp64 accumulation) already differ by 5e-3 .. 7e-3 rel-L2 (tests/test_oracle_muon.py pins that
# figure), so the five-iteration result is held to 2e-2 and every single iteration to the bf16 bar of 5e-3. The reference
# states the same about its own kernel ("within the bf16 band, not bitwise", round2/source/kernels/nki_nsk.py:55-57).
NS_TOL = 2e-2
@pytest.mark.parametrize("shape", [(3, 768, 256), (2, 256, 768), (1, 384, 384)])
def test_newton_schulz_stack(ops, dev, shape):
    """tfb_ns5 against the oracle's restatement of the reference kernel's arithmetic (same rounding points; the fp32
    accumulation order is free), tall, wide and square stacks."""
    from oracle import muon as O
    K, r, c = shape
    g = torch.randn(K, r, c, generator=_g(r + c)) * 0.02
    d = O.muon_denominator(g)
    y, v = ops.ns5(g.to(dev), d.to(dev))
    yo, vo = O.ns5(g, d)
    assert y.shape == (K, r, c) and v.shape == (K, max(r, c))
    assert rel_l2(y, yo) < NS_TOL
    assert rel_l2(v, vo) < NS_TOL
    # one real iteration at a time (the other four made the identity by a = 1, b = c = 0: B = 0, X' = X): the bf16 bar
    ident = (1.0, 0.0, 0.0)
    for it in range(5):
        co = (O.NS_COEFFS[it],) + (ident,) * 4
        y1, _ = ops.ns5(g.to(dev), d.to(dev), co)
        y1o, _ = O.ns5(g, d, co)
        assert rel_l2(y1, y1o) < BF16_TOL, it
    assert rel_l2(v, y.float().square().sum(dim=-1 if r >= c else -2)) < 1e-6        # v is the row statistic of the y returned


def test_newton_schulz_full_size_properties(ops, dev):
    """The 12 MLP matrices of the benchmark model in one call (K 12, 3072 x 768): singular values inside the Polar Express
    band, the same singular vectors as the input (cosine with the SVD polar factor), and the wide stack equal to the
    transposed tall one bit for bit."""
    from oracle import muon as O
    from trainium_frontier_them_bones_amd._lib import TfbError
    K, M, N = 12, 3072, 768
    g = torch.randn(K, M, N, generator=_g(77)) * 0.02
    d = O.muon_denominator(g)
    gd, dd = g.to(dev), d.to(dev)
    y, v = ops.ns5(gd, dd)
    sv = torch.linalg.svdvals(y[5].float())
    assert sv.min().item() > 0.6 and sv.max().item() < 1.3
    x0 = O.x0_of(g[5], d.reshape(-1)[5]).to(dev).float()
    u, _, vh = torch.linalg.svd(x0, full_matrices=False)
    polar = u @ vh
    cos = (y[5].float() * polar).sum() / (y[5].float().norm() * polar.norm())
    assert cos.item() > 0.97
    yw, vw = ops.ns5(gd.transpose(1, 2).contiguous(), dd)
    assert torch.equal(yw, y.transpose(1, 2)) and torch.equal(vw, v)
    yo, _ = O.ns5(g[:1], d[:1])
    assert rel_l2(y[:1], yo) < NS_TOL
    with pytest.raises(TfbError):
        ops.ns5(gd[:, :100].contiguous(), dd)                                         # rows % 128 != 0


def test_autograd_nodes_do_not_corrupt_what_autograd_cannot_see(ops, dev):
    """RopeAttentionFn leaves its input qkv untouched (the rotation goes into a buffer of its own); LmHeadLossFn, where its
    backward overwrites the saved logits with their gradient, refuses a second backward instead of returning garbage."""
    from trainium_frontier_them_bones_amd import autograd as A
    from oracle import attention as OA
    g = _g(31)
    B, T, H, D = 2, 256, 4, 64
    qkv = torch.randn(B, T, 3 * H * D, generator=g).bfloat16().to(dev).requires_grad_(True)
    before = qkv.detach().clone()
    cos, sin = OA.rope_tables(T, D)
    out = A.RopeAttentionFn.apply(qkv, cos.to(dev), sin.to(dev), H, 0.125)
    assert torch.equal(qkv.detach(), before)
    out.sum().backward()
    assert torch.equal(qkv.detach(), before) and bool(torch.isfinite(qkv.grad.float()).all())
    # beyond the one-pass loss kernel's vocabulary limit the node saves the logits and overwrites them in its backward
    V = 65536 + 128
    x = torch.randn(128, 128, generator=g).bfloat16().to(dev).requires_grad_(True)
    W = (0.05 * torch.randn(V, 128, generator=g)).bfloat16().to(dev).requires_grad_(True)
    t = torch.randint(0, V, (128,), generator=g).to(dev)
    loss = A.LmHeadLossFn.apply(x, W, t, 0.0, "mean")
    loss.backward(retain_graph=True)
    with pytest.raises(RuntimeError):
        loss.backward()
    # within it the saved tensor is the gradient itself, and a second backward accumulates the same gradients again
    x = torch.randn(256, 256, generator=g).bfloat16().to(dev).requires_grad_(True)
    W = (0.05 * torch.randn(1024, 256, generator=g)).bfloat16().to(dev).requires_grad_(True)
    t = torch.randint(0, 1024, (256,), generator=g).to(dev)
    loss = A.LmHeadLossFn.apply(x, W, t, 0.0, "mean")
    loss.backward(retain_graph=True)
    gx, gw = x.grad.clone(), W.grad.clone()
    x.grad = W.grad = None
    loss.backward()
    assert torch.equal(x.grad, gx) and torch.equal(W.grad, gw)


@pytest.mark.parametrize("V", [32768, 50304])
def test_embedding_backward_at_full_size_on_a_zipf_batch(ops, dev, V):
    """The grouped embedding backward at the benchmark's size (32768 rows of 768, Zipf(1.1) ids): with the vocabulary's
    counters in LDS (V = 32768: per-workgroup histogram, placement without atomics) and on the per-row path a larger
    vocabulary takes (V = 50304: its counters do not fit), both against index_add_ in fp32 and against the plain atomic
    entry point; int64 and int32 ids, ids outside [0, V) dropped."""
    from trainium_frontier_them_bones_amd.model import zipf_tokens
    idx, _ = zipf_tokens(16, 2048, V, seed=9)
    idx = idx.reshape(-1).clone()
    idx[5::97] = V + 3
    idx[11::89] = -1
    ok = (idx >= 0) & (idx < V)
    g = torch.Generator().manual_seed(2)
    dy = torch.randn(idx.numel(), 768, generator=g).bfloat16()
    want = torch.zeros(V, 768).index_add_(0, idx[ok], dy.float()[ok])
    for ids in (idx, idx.int()):
        dw = ops.fill_f32_(torch.empty(V, 768, device=dev), 0.0)
        ops.embedding_bwd(ids.to(dev), dy.to(dev), dw)
        assert rel_l2(dw, want) < 1e-6
    dwa = ops.fill_f32_(torch.empty(V, 768, device=dev), 0.0)
    ops.embedding_bwd(idx.to(dev), dy.to(dev), dwa, grouped=False)
    assert rel_l2(dwa, want) < 1e-6
    assert int((want.abs().sum(1) > 0).sum()) > 3000 and int(torch.bincount(idx[ok]).max()) > 1000   # many tokens, one very hot



def test_loss_row_weights_equal_the_host_expression(ops, dev):
    """tfb_loss_row_weights: (t >= 0) / max(1, count) for the mean, (t >= 0) for the sum, bit for bit what the compare /
    cast / sum / clamp / divide chain gives; int64 and int32 targets, lengths off every stride of the kernel, no row valid."""
    g = _g(4242)
    for n in (1, 63, 1024, 4097, 32768, 100003):
        for dt in (torch.int64, torch.int32):
            t = torch.randint(0, 1000, (n,), generator=g).to(dt)
            t[torch.rand(n, generator=g) < 0.3] = -1
            t = t.to(dev)
            valid = (t >= 0).to(torch.float32)
            assert torch.equal(ops.loss_row_weights(t, "mean"), valid / valid.sum().clamp_min(1.0))
            assert torch.equal(ops.loss_row_weights(t, "sum"), valid)
    none = torch.full((777,), -1, dtype=torch.int64, device=dev)
    assert torch.equal(ops.loss_row_weights(none, "mean"), torch.zeros(777, device=dev))
    # with the vocabulary size given, a target at or beyond it is a row without a loss: it counts neither in the numerator
    # nor in the mean's denominator (the loss kernels give such a row 0)
    t = torch.tensor([3, 999, 1000, -1, 5000, 0], dtype=torch.int64, device=dev)
    want = torch.tensor([1, 1, 0, 0, 0, 1], dtype=torch.float32, device=dev)
    assert torch.equal(ops.loss_row_weights(t, "mean", 1000), want / 3.0)
    assert torch.equal(ops.loss_row_weights(t, "sum", 1000), want)


def test_lm_head_loss_without_grad_takes_the_forward_only_path(ops, dev):
    """Under torch.no_grad() the LM-head wrapper runs the GEMM with the log-sum-exp in its epilogue (no dlogits pass) even when
    its inputs are parameters; the loss equals the training path's."""
    from trainium_frontier_them_bones_amd import autograd as A
    g = _g(123)
    x = torch.randn(256, 128, generator=g).bfloat16().to(dev).requires_grad_(True)
    W = (0.05 * torch.randn(512, 128, generator=g)).bfloat16().to(dev).requires_grad_(True)
    t = torch.randint(0, 512, (256,), generator=g).to(dev)
    calls = []
    real = ops.loss_fwd_bwd
    ops.loss_fwd_bwd = lambda *a, **k: (calls.append(1), real(*a, **k))[1]
    try:
        train = A.LmHeadLossFn.apply(x, W, t, 0.0, "mean")
        assert calls == [1]
        with torch.no_grad():
            ev = A.LmHeadLossFn.apply(x, W, t, 0.0, "mean")
        assert calls == [1]
    finally:
        ops.loss_fwd_bwd = real
    assert abs(train.item() - ev.item()) < 1e-5 * abs(train.item())


def test_mean_loss_with_a_target_beyond_the_vocabulary(ops, dev):
    """A target id >= V is a row without a loss: the mean divides by the rows that have one. LM-head wrapper against the
    oracle's mean and against F.cross_entropy over the rows that count."""
    from oracle import loss as O
    from trainium_frontier_them_bones_amd import autograd as A
    g = _g(99)
    N, d, V = 256, 128, 512
    x = torch.randn(N, d, generator=g).bfloat16()
    W = (0.05 * torch.randn(V, d, generator=g)).bfloat16()
    t = torch.randint(0, V, (N,), generator=g)
    t[7] = V + 3
    t[100] = -1
    logits = (x.float() @ W.float().t()).bfloat16()
    want = O.fused_loss(logits, t, "mean", None)
    keep = (t >= 0) & (t < V)
    ref = torch.nn.functional.cross_entropy(logits.float()[keep], t[keep])
    assert abs(want.item() - ref.item()) < 1e-5
    got = A.LmHeadLossFn.apply(x.to(dev).requires_grad_(True), W.to(dev).requires_grad_(True), t.to(dev), 0.0, "mean")
    assert abs(got.item() - want.item()) < 1e-3 * want.item()
