"""Pins oracle/norm.py, oracle/loss.py, oracle/optim.py against library routines, autograd and closed forms."""
import math

import torch
import torch.nn.functional as F

from oracle import loss as OL
from oracle import norm as ON
from oracle import optim as OO
from helpers import rel_l2


def test_rmsnorm_matches_library():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(64, 768, generator=g).bfloat16()
    w = (1 + 0.02 * torch.randn(768, generator=g)).bfloat16()
    y, inv = ON.rmsnorm(x, w, 1e-6)
    ref = F.rms_norm(x.float(), (768,), w.float(), 1e-6)
    assert rel_l2(y, ref) < 4e-3
    y0, _ = ON.rmsnorm(x, None, ON.RMS_EPS)
    assert torch.equal(y0, F.rms_norm(x, (768,), None, ON.RMS_EPS))
    assert torch.allclose(inv, torch.rsqrt(x.float().pow(2).mean(-1) + 1e-6))


def test_rmsnorm_backward_is_autograd_and_orthogonal():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(32, 256, generator=g).bfloat16()
    w = (1 + 0.1 * torch.randn(256, generator=g)).bfloat16()
    gy = torch.randn(32, 256, generator=g).bfloat16()
    _, inv = ON.rmsnorm(x, w, 1e-6)
    dx, dw = ON.rmsnorm_backward(gy, x, inv, w)
    xd, wd = x.double().requires_grad_(True), w.double().requires_grad_(True)
    (xd * torch.rsqrt(xd.pow(2).mean(-1, keepdim=True) + 1e-6) * wd).backward(gy.double())
    assert rel_l2(dx, xd.grad) < 1e-5 and rel_l2(dw, wd.grad) < 1e-5
    _, inv0 = ON.rmsnorm(x, None, 0.0)
    dx0, _ = ON.rmsnorm_backward(gy, x, inv0, None)
    assert float((dx0 * x.float()).sum(-1).abs().max()) < 1e-3    # J^T g is orthogonal to x when eps = 0


def test_block_head_and_tail_match_eager_autograd():
    g = torch.Generator().manual_seed(2)
    x, x0, sk = (torch.randn(16, 128, generator=g).bfloat16() for _ in range(3))
    l1, l2, l3 = torch.tensor(0.9), torch.tensor(0.25), torch.tensor(-0.4)
    x_new, x_norm, inv = ON.block_head(x, x0, l1, l2, sk, l3)
    # the U-net skip joins the stream BEFORE the block head (round1/source/train.py:5644-5647: s = x + l3 * skip, then
    # head(s, x0)): x_new = l1 (x + l3 skip) + l2 x0, not l1 x + l2 x0 + l3 skip
    assert rel_l2(x_new, 0.9 * (x.float() - 0.4 * sk.float()) + 0.25 * x0.float()) < 4e-3
    assert rel_l2(x_new, 0.9 * x.float() + 0.25 * x0.float() - 0.4 * sk.float()) > 1e-2
    eager_s = x + l3.to(x.dtype) * sk                                   # the reference's eager chain, bf16 step by step
    assert rel_l2(x_new, ON.block_head(eager_s, x0, l1, l2)[0]) < 6e-3
    assert torch.equal(x_norm, F.rms_norm(x_new, (128,), None, ON.RMS_EPS))
    gn, gm = torch.randn(16, 128, generator=g).bfloat16(), torch.randn(16, 128, generator=g).bfloat16()
    dx, dx0, dsk, d1, d2, d3 = ON.block_head_backward(gn, gm, x, x0, x_new, inv, l1, l2, sk, l3)
    xs = [t.double().requires_grad_(True) for t in (x, x0, sk)]
    ls = [t.double().requires_grad_(True) for t in (l1, l2, l3)]
    v = ls[0] * (xs[0] + ls[2] * xs[2]) + ls[1] * xs[1]
    n = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + ON.RMS_EPS)
    (v * gn.double()).sum().backward(retain_graph=True)
    (n * gm.double()).sum().backward()
    assert rel_l2(dx, xs[0].grad) < 1e-2 and rel_l2(dx0, xs[1].grad) < 1e-2 and rel_l2(dsk, xs[2].grad) < 1e-2
    # gain gradients are sums of ~2000 signed products of O(1): the bf16 rounding of x_new inside G leaves ~1e-2 absolute
    assert abs(d1.item() - ls[0].grad.item()) < 2e-2 * abs(ls[0].grad.item()) + 5e-2
    assert abs(d2.item() - ls[1].grad.item()) < 2e-2 * abs(ls[1].grad.item()) + 5e-2
    assert abs(d3.item() - ls[2].grad.item()) < 2e-2 * abs(ls[2].grad.item()) + 5e-2
    # with the old (wrong) association the l3 gradient would lack the factor l1 = 0.9 and dskip the factor l1
    assert abs(d3.item() / 0.9 - ls[2].grad.item()) > abs(d3.item() - ls[2].grad.item())
    s, y, inv = ON.add_rmsnorm(x, x0)
    assert torch.equal(s, x + x0) and torch.equal(y, F.rms_norm(s, (128,), None, ON.RMS_EPS))


def test_relu2_family():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(8, 256, generator=g).bfloat16()
    gy = torch.randn(8, 256, generator=g).bfloat16()
    assert torch.equal(ON.relu2(x), F.relu(x).square())
    xr = x.float().requires_grad_(True)
    F.relu(xr).square().backward(gy.float())
    assert rel_l2(ON.relu2_backward(x, gy), xr.grad) < 4e-3
    assert rel_l2(ON.relu2_backward_from_h(ON.relu2(x), gy), xr.grad) < 1e-2


def test_loss_matches_cross_entropy_and_autograd():
    g = torch.Generator().manual_seed(4)
    N, V = 64, 512
    x = (3 * torch.randn(N, V, generator=g)).bfloat16()
    t = torch.randint(0, V, (N,), generator=g)
    t[3] = -1
    for cap in (15.0, None):
        s = (cap * torch.tanh(x.float() / cap)) if cap else x.float()
        rows, lse = OL.loss_rows(x, t, cap)
        ref = F.cross_entropy(s, t, ignore_index=-1, reduction="none")
        assert torch.allclose(rows, ref, atol=1e-5)
        assert abs(OL.fused_loss(x, t, "mean", cap).item() - F.cross_entropy(s, t, ignore_index=-1).item()) < 1e-5
        xr = x.float().requires_grad_(True)
        sr = (cap * torch.tanh(xr / cap)) if cap else xr
        F.cross_entropy(sr, t, ignore_index=-1).backward()
        d = OL.loss_backward(x.float(), t, lse, OL.row_weights(t, "mean"), cap)
        assert rel_l2(d, xr.grad) < 1e-5
        if cap:
            th = torch.tanh(x.float() / cap)
            assert float((d / (1 - th * th)).sum(-1).abs().max()) < 1e-6     # sum_v dlogits / (1 - t^2) = 0


def test_loss_uniform_logits_is_log_vocab():
    t = torch.randint(0, 1000, (16,))
    assert abs(OL.fused_loss(torch.zeros(16, 1000), t, "mean", 15.0).item() - math.log(1000)) < 1e-5


def test_lmhead_composition_matches_autograd():
    g = torch.Generator().manual_seed(5)
    N, d, V = 128, 64, 256
    x = torch.randn(N, d, generator=g).bfloat16()
    nw = (1 + 0.02 * torch.randn(d, generator=g)).bfloat16()
    W = (0.05 * torch.randn(V, d, generator=g)).bfloat16()
    t = torch.randint(0, V, (N,), generator=g)
    loss, saved = OL.lmhead_loss(x, nw, W, t)
    dx, dnw, dW = OL.lmhead_loss_backward(x, nw, W, t, saved)
    xd, nd, Wd = (a.double().requires_grad_(True) for a in (x, nw, W))
    h = xd * torch.rsqrt(xd.pow(2).mean(-1, keepdim=True) + 1e-6) * nd
    ref = F.cross_entropy(h @ Wd.t(), t)
    ref.backward()
    assert abs(loss.item() - ref.item()) < 1e-3 * ref.item()
    assert rel_l2(dx, xd.grad) < 2e-2 and rel_l2(dW, Wd.grad) < 2e-2 and rel_l2(dnw, nd.grad) < 2e-2


def test_adamw_against_torch_and_first_step_closed_form():
    g = torch.Generator().manual_seed(6)
    p0 = torch.randn(1000, generator=g)
    p = p0.clone()
    m, v = torch.zeros(1000), torch.zeros(1000)
    ref = torch.nn.Parameter(p0.clone())
    opt = torch.optim.AdamW([ref], lr=1e-2, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    for step in range(1, 6):
        gr = torch.randn(1000, generator=g)
        if step == 1:
            want = p0 * (1 - 1e-2 * 0.1) - 1e-2 * gr / (gr.abs() + 1e-8)
        OO.adamw_step(p, gr, m, v, step, 1e-2, 0.9, 0.95, 1e-8, 0.1)
        if step == 1:
            assert torch.allclose(p, want, atol=1e-6)
        ref.grad = gr.clone()
        opt.step()
        assert torch.allclose(p, ref.detach(), atol=2e-6)


def test_resmix_backward_sums():
    g = torch.Generator().manual_seed(7)
    gg, x, x0 = (torch.randn(64, 128, generator=g).bfloat16() for _ in range(3))
    dx, dx0, da, db = ON.resmix_backward(gg, x, x0, torch.tensor(0.9), torch.tensor(0.3))
    assert rel_l2(dx, 0.9 * gg.float()) < 4e-3 and rel_l2(dx0, 0.3 * gg.float()) < 4e-3
    assert abs(da.item() - (gg.float() * x.float()).sum().item()) < 0.5


def test_multi_target_and_label_smoothed_rows_against_cross_entropy_and_autograd():
    g = torch.Generator().manual_seed(9)
    N, V, K = 48, 256, 3
    x = (3 * torch.randn(N, V, generator=g)).bfloat16()
    tg = torch.randint(0, V, (K, N), generator=g)
    tg[1, 5] = -1
    tg[2, 7] = tg[0, 7]                       # two targets of a row may coincide
    rw = torch.rand(K, N, generator=g)
    for cap in (15.0, None):
        s = (cap * torch.tanh(x.float() / cap)) if cap else x.float()
        # (1) several targets: a weighted sum of the library's single-target rows
        rows, lse = OL.loss_multi_rows(x, tg, rw, cap)
        ref = sum(rw[k] * F.cross_entropy(s, tg[k], ignore_index=-1, reduction="none") for k in range(K))
        assert torch.allclose(rows, ref, atol=2e-5)
        # K = 1 and unit weights is the single-target oracle
        r1, l1 = OL.loss_multi_rows(x, tg[:1], torch.ones(1, N), cap)
        r0, l0 = OL.loss_rows(x, tg[0], cap)
        assert torch.allclose(r1, r0, atol=1e-6) and torch.equal(l1, l0)
        # (2) label smoothing: the library's label_smoothing on the softcapped logits
        for eps in (0.1, 0.3):
            rs, _ = OL.loss_multi_rows(x, tg[:1], torch.ones(1, N), cap, eps)
            assert torch.allclose(rs, F.cross_entropy(s, tg[0], reduction="none", label_smoothing=eps), atol=2e-5)
        # (3) gradients: autograd in fp64 of the same expressions
        for eps, kk in ((0.0, K), (0.2, 1), (0.2, K)):
            xd = x.double().requires_grad_(True)
            sd = (cap * torch.tanh(xd / cap)) if cap else xd
            lsed = torch.logsumexp(sd, -1)
            tot = 0
            for k in range(kk):
                valid = (tg[k] >= 0).double()
                pick = sd.gather(1, tg[k].clamp_min(0)[:, None]).squeeze(1)
                tot = tot + (rw[k].double() * valid * (lsed - (1 - eps) * pick - eps * sd.mean(-1)))
            gup = torch.rand(N, generator=g)
            (tot * gup.double()).sum().backward()
            _, lse_k = OL.loss_multi_rows(x, tg[:kk], rw[:kk], cap, eps)
            d = OL.loss_multi_backward(x.float(), tg[:kk], rw[:kk], lse_k, gup, cap, eps)
            assert rel_l2(d, xd.grad) < 1e-5


def test_mix_tail_is_the_eager_chain_and_its_autograd():
    """oracle/norm.py mix_tail / mix_tail_backward against the reference's unfused expression lam * shift1(x) -> tail_norm2
    written with library routines: the forward in bf16 arithmetic (bit for bit), the backward against fp64 autograd of
    the same chain (bf16 roundings bound the distance), the shift's adjoint identity, and lam = 0 (s1 = x, the norm's
    own backward)."""
    g = torch.Generator().manual_seed(11)
    B, T, C = 3, 16, 256
    x = torch.randn(B, T, C, generator=g).bfloat16()
    lam = torch.tensor(0.37).bfloat16()
    s1, y, inv = ON.mix_tail(x, lam.float())
    sh = torch.cat([torch.zeros_like(x[:, :1]), x[:, :-1]], dim=1)
    s_ref = x + lam * sh                                     # the eager bf16 ops: mul rounds, add rounds
    assert torch.equal(s1, s_ref)
    assert torch.equal(y, F.rms_norm(s_ref, (C,), None, ON.RMS_EPS))
    assert float(sh[:, 0].abs().max()) == 0.0 and torch.equal(sh[:, 1:], x[:, :-1])
    gy = torch.randn(B, T, C, generator=g).bfloat16()
    ge = torch.randn(B, T, C, generator=g).bfloat16()
    gx, dlam = ON.mix_tail_backward(x, s1, inv, lam.float(), gy, ge)
    xd = x.double().requires_grad_(True)
    ld = lam.double().requires_grad_(True)
    shd = torch.cat([torch.zeros_like(xd[:, :1]), xd[:, :-1]], dim=1)
    sd = xd + ld * shd
    yd = sd * torch.rsqrt(sd.pow(2).mean(-1, keepdim=True) + ON.RMS_EPS)
    (yd * gy.double()).sum().backward(retain_graph=True)
    (sd * ge.double()).sum().backward()
    assert rel_l2(gx, xd.grad) < 6e-3
    assert abs(float(dlam) - float(ld.grad)) < 2e-2 * abs(float(ld.grad)) + 0.5
    # the shift's adjoint: <shift1(x), g> = <x, shift1^T(g)>, with shift1^T(g)[t] = g[t + 1]
    gg = torch.randn(B, T, C, generator=g).double()
    nxt = torch.cat([gg[:, 1:], torch.zeros_like(gg[:, :1])], dim=1)
    assert abs(float((ON.shift1(x).double() * gg).sum() - (x.double() * nxt).sum())) < 1e-9
    # lam = 0: s1 = x and gx is the tail norm's own backward, dlam still the sum of g * shift1(x)
    s0, _, inv0 = ON.mix_tail(x, 0.0)
    assert torch.equal(s0, x)
    gx0, _ = ON.mix_tail_backward(x, s0, inv0, 0.0, gy, None)
    dx0, _ = ON.rmsnorm_backward(gy.reshape(-1, C), x.reshape(-1, C), inv0.reshape(-1), None)
    assert rel_l2(gx0.reshape(-1, C), dx0) < 4e-3
