"""The reference-named host functions (trainium_frontier_them_bones_amd/train_api.py) called the way the reference's
train.py calls them, checked against the oracle on the same seeded inputs. bf16 paths: rel-L2 <= 5e-3; fp8: <= 2e-2;
loss: <= 1e-3 relative."""
import math

import pytest
import torch

from helpers import rel_l2

pytestmark = pytest.mark.gpu

BF16_TOL, FP8_TOL, LOSS_TOL = 5e-3, 2e-2, 1e-3


def _g(seed):
    return torch.Generator().manual_seed(seed)


@pytest.fixture(scope="module")
def api():
    from trainium_frontier_them_bones_amd import train_api
    return train_api


def test_nki_attn_fn_and_rope_norm(api, dev):
    from oracle import attention as O
    B, H, T, D = 2, 3, 256, 64
    g = _g(1)
    q, k, v = (torch.randn(B, H, T, D, generator=g).bfloat16() for _ in range(3))
    go = torch.randn(B, T, H, D, generator=g).bfloat16()
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    y = api.nki_attn_fn(qd, kd, vd)                                       # scale=None -> 1 / sqrt(D)
    assert y.shape == (B, T, H, D)
    y.backward(go.to(dev))
    o, lse = O.forward(q, k, v, 1.0 / math.sqrt(D))
    dq, dk, dv = O.backward(q, k, v, o, go, lse, 1.0 / math.sqrt(D))
    assert rel_l2(y, o) < BF16_TOL
    assert rel_l2(qd.grad, dq) < BF16_TOL and rel_l2(kd.grad, dk) < BF16_TOL and rel_l2(vd.grad, dv) < BF16_TOL
    assert y.data_ptr() != qd.data_ptr() and torch.equal(qd.detach().cpu(), q)   # inputs untouched
    # rope_norm: [B, T, H, D] in, [B, H, T, D] out, tables in the reference's [1, T, 1, D/2] shape
    for Dh in (64, 128):
        x = torch.randn(B, T, H, Dh, generator=g).bfloat16()
        cos, sin = O.rope_tables(T, Dh)
        gy = torch.randn(B, H, T, Dh, generator=g).bfloat16()
        xd = x.to(dev).requires_grad_(True)
        yn = api.rope_norm(xd, cos.to(dev)[None, :, None, :], sin.to(dev)[None, :, None, :])
        assert yn.shape == (B, H, T, Dh)
        yn.backward(gy.to(dev))
        yo, r, inv = O.rope_norm(x, cos, sin)
        assert rel_l2(yn, yo.transpose(1, 2)) < 1e-3
        assert float((yn.detach().cpu().float() - yo.transpose(1, 2).float()).abs().max()) <= 2.0 ** -6   # one bf16 ulp near 2
        dxo = O.rope_norm_backward(gy.transpose(1, 2).contiguous(), r, inv, cos, sin)
        assert rel_l2(xd.grad, dxo) < 2e-3


@pytest.mark.parametrize("D", [64, 128])
def test_nki_rope_attention_with_qk_norm(api, dev, D):
    from oracle import attention as O
    B, T, H = 2, 256, 3
    C = H * D
    g = _g(2 + D)
    qkv = torch.randn(B, T, 3 * C, generator=g).bfloat16()
    go = torch.randn(B, T, H, D, generator=g).bfloat16()
    cos, sin = O.rope_tables(T, D)
    xd = qkv.to(dev).requires_grad_(True)
    y = api.nki_rope_attention(xd, cos.to(dev), sin.to(dev), H, scale=0.11)
    assert y.shape == (B, T, H, D)
    y.backward(go.to(dev))
    assert torch.equal(xd.detach().cpu(), qkv)                            # the fused projection output is not modified
    # oracle: the unfused chain rope_norm -> causal attention, and its backward
    q, k, v = (t.view(B, T, H, D) for t in qkv.split(C, dim=-1))
    qn, rq, iq = O.rope_norm(q, cos, sin)
    kn, rk, ik = O.rope_norm(k, cos, sin)
    q4, k4, v4 = (t.transpose(1, 2).contiguous() for t in (qn, kn, v))
    o, lse = O.forward(q4, k4, v4, 0.11)
    assert rel_l2(y, o) < BF16_TOL
    dq4, dk4, dv4 = O.backward(q4, k4, v4, o, go, lse, 0.11)
    dq = O.rope_norm_backward(dq4.transpose(1, 2).contiguous(), rq, iq, cos, sin)
    dk = O.rope_norm_backward(dk4.transpose(1, 2).contiguous(), rk, ik, cos, sin)
    want = torch.cat([dq.reshape(B, T, C), dk.reshape(B, T, C), dv4.transpose(1, 2).reshape(B, T, C)], dim=-1)
    assert rel_l2(xd.grad, want) < BF16_TOL
    # "None = not done": a head size the kernels do not take
    assert api.nki_rope_attention(torch.zeros(1, 128, 3 * 2 * 32, dtype=torch.bfloat16, device=dev), cos.to(dev), sin.to(dev), 2) is None


def test_fused_loss_family(api, dev):
    from oracle import loss as O
    g = _g(5)
    B, T, V, K = 2, 128, 1024, 3
    N = B * T
    x = (3 * torch.randn(B, T, V, generator=g)).bfloat16()
    t = torch.randint(0, V, (B, T), generator=g)
    t[0, 3] = -1
    for red in ("mean", "sum", "none"):
        xd = x.to(dev).requires_grad_(True)
        got = api.fused_loss(xd, t.to(dev), red)
        want = O.fused_loss(x, t, red, 15.0)
        if red == "none":
            assert got.shape == t.shape and rel_l2(got, want) < LOSS_TOL
            got.sum().backward()
        else:
            assert abs(got.item() - want.item()) < LOSS_TOL * abs(want.item())
            got.backward()
        rows, lse = O.loss_rows(x.reshape(N, V), t, 15.0)
        grow = O.row_weights(t, "mean") if red == "mean" else (t.reshape(-1) >= 0).float()
        assert rel_l2(xd.grad.reshape(N, V), O.loss_backward(x.reshape(N, V), t, lse, grow, 15.0)) < BF16_TOL
    # several targets per row (multi-token prediction)
    tg = torch.randint(0, V, (K, N), generator=g)
    tg[1, 7] = -1
    rw = torch.rand(K, N, generator=g)
    xd = x.to(dev).requires_grad_(True)
    got = api.fused_loss_multi(xd, tg.to(dev), rw.to(dev))
    rows, lse = O.loss_multi_rows(x.reshape(N, V), tg, rw, 15.0)
    assert abs(got.item() - rows.sum().item()) < LOSS_TOL * rows.sum().item()
    got.backward()
    assert rel_l2(xd.grad.reshape(N, V), O.loss_multi_backward(x.reshape(N, V), tg, rw, lse, torch.ones(N), 15.0)) < BF16_TOL
    assert api.fused_loss_multi(xd, tg.to(dev).repeat(4, 1), rw.to(dev).repeat(4, 1)) is None      # K = 12: not taken
    # label smoothing and per-token weights (R2's chunked_loss_mean)
    tok_w = 1.0 + torch.rand(B, T, generator=g)
    for smooth, eps in ((False, 0.0), (True, 0.1)):
        xd = x.to(dev).requires_grad_(True)
        got = api.chunked_loss_mean(xd, t.to(dev), smooth=smooth, tok_w=tok_w.to(dev), eps=eps)
        w = (O.row_weights(t, "mean") * tok_w.reshape(-1)).view(1, N)
        rows, lse = O.loss_multi_rows(x.reshape(N, V), t.view(1, N), w, 15.0, eps)
        assert abs(got.item() - rows.sum().item()) < LOSS_TOL * rows.sum().item()
        got.backward()
        want = O.loss_multi_backward(x.reshape(N, V), t.view(1, N), w, lse, torch.ones(N), 15.0, eps)
        assert rel_l2(xd.grad.reshape(N, V), want) < BF16_TOL
    s = 15.0 * torch.tanh(x.float().reshape(N, V) / 15.0)
    lib = torch.nn.functional.cross_entropy(s, t.reshape(-1), ignore_index=-1, label_smoothing=0.1)
    got = api.chunked_loss_mean(x.to(dev), t.to(dev), smooth=True, eps=0.1)
    assert abs(got.item() - lib.item()) < LOSS_TOL * lib.item()


def test_norm_blocks_and_relu2(api, dev):
    from oracle import norm as O
    g = _g(6)
    shape = (2, 128, 768)
    x, x0, sk, a, gn, gy = (torch.randn(*shape, generator=g).bfloat16() for _ in range(6))
    l1, l2, l3 = (torch.tensor([v]) for v in (0.9, 0.25, -0.4))
    ld = [t.to(dev).requires_grad_(True) for t in (l1, l2, l3)]
    xd, x0d, skd = (t.to(dev).requires_grad_(True) for t in (x, x0, sk))
    xn, xnorm = api.head_skip(xd, x0d, skd, *ld)
    (xn.float() * gn.to(dev).float()).sum().backward(retain_graph=True)
    (xnorm.float() * gy.to(dev).float()).sum().backward()
    o = O.block_head(x.view(-1, 768), x0.view(-1, 768), l1[0], l2[0], sk.view(-1, 768), l3[0])
    assert rel_l2(xn, o[0].view(shape)) < 1e-3 and rel_l2(xnorm, o[1].view(shape)) < 1e-3
    eager = (x + l3.to(x.dtype) * sk)                                   # R1:5646, then the block head
    assert rel_l2(xn, (l1 * eager.float() + l2 * x0.float())) < BF16_TOL
    ob = O.block_head_backward(gn.view(-1, 768), gy.view(-1, 768), x.view(-1, 768), x0.view(-1, 768), o[0], o[2], l1[0], l2[0],
                               sk.view(-1, 768), l3[0])
    assert rel_l2(xd.grad, ob[0].view(shape)) < BF16_TOL and rel_l2(x0d.grad, ob[1].view(shape)) < BF16_TOL
    assert rel_l2(skd.grad, ob[2].view(shape)) < BF16_TOL
    for got, want in zip(ld, ob[3:]):
        assert abs(got.grad.item() - want.item()) < 1e-3 * abs(want.item()) + 0.05
    xn2, xnorm2 = api.block_head(x.to(dev), x0.to(dev), l1.to(dev), l2.to(dev))
    o2 = O.block_head(x, x0, l1[0], l2[0])
    assert rel_l2(xn2, o2[0]) < 1e-3 and rel_l2(xnorm2, o2[1]) < 1e-3
    assert rel_l2(api.rmsnorm_fast(x.to(dev)), O.rmsnorm(x, None, O.RMS_EPS)[0]) < 1e-3
    s1, y = api.tail_norm2(x.to(dev), a.to(dev))
    so, yo, _ = O.add_rmsnorm(x, a)
    assert torch.equal(s1.cpu(), so) and rel_l2(y, yo) < 1e-3
    assert rel_l2(api.final_norm(x.to(dev), a.to(dev)), yo) < 1e-3
    assert torch.equal(api.relu_squared(x.to(dev)).cpu(), O.relu2(x))


def test_gemm_glue_and_mlp_fused8(api, dev):
    from oracle import mlp8 as O8
    g = _g(7)
    M, d, F = 384, 256, 512
    x = torch.randn(3, 128, d, generator=g).bfloat16()
    w = (0.05 * torch.randn(d, F, generator=g)).bfloat16()                # LinearT [in, out]
    xd, wd = x.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    h = api.fused_fc_relu2(xd, wd)
    ref = torch.relu(x.float().reshape(M, d) @ w.float()).bfloat16().float().square().bfloat16()
    assert h.shape == (3, 128, F) and rel_l2(h, ref.view(3, 128, F)) < BF16_TOL
    gh = torch.randn(3, 128, F, generator=g).bfloat16()
    h.backward(gh.to(dev))
    xf, wf = x.float().reshape(M, d).requires_grad_(True), w.float().requires_grad_(True)
    (torch.relu(xf @ wf).square() * gh.float().reshape(M, F)).sum().backward()
    assert rel_l2(xd.grad.reshape(M, d), xf.grad) < 1e-2 and rel_l2(wd.grad, wf.grad) < 1e-2
    # inplace=True: the weight gradient is summed into an existing w.grad, the op answers None for it
    wd2 = w.to(dev).requires_grad_(True)
    wd2.grad = torch.ones_like(wd2)
    api.fused_fc_relu2(x.to(dev), wd2, inplace=True).backward(gh.to(dev))
    assert rel_l2(wd2.grad, wf.grad + 1.0) < 1e-2
    a2, b2 = torch.randn(M, d, generator=g).bfloat16(), torch.randn(M, F, generator=g).bfloat16()
    assert rel_l2(api.nki_matmul(a2.to(dev), b2.to(dev), trans_a=True), a2.float().t() @ b2.float()) < BF16_TOL
    assert rel_l2(api.dw_matmul(a2.to(dev), b2.to(dev)), a2.float().t() @ b2.float()) < BF16_TOL
    assert api.dw_matmul(a2.to(dev)[:, :100].contiguous(), b2.to(dev)) is None
    # the fp8 MLP on a module with c_fc / c_proj, 300 tokens (padded to 384 inside)
    mlp = torch.nn.Module()
    mlp.c_fc = torch.nn.Linear(d, F, bias=False)
    mlp.c_proj = torch.nn.Linear(F, d, bias=False)
    wf8 = (0.05 * torch.randn(F, d, generator=g)).bfloat16()
    wp8 = (0.05 * torch.randn(d, F, generator=g)).bfloat16()
    mlp.c_fc.weight.data, mlp.c_proj.weight.data = wf8.clone(), wp8.clone()
    mlp = mlp.to(dev)
    xm = torch.randn(3, 100, d, generator=g).bfloat16()
    xmd = xm.to(dev).requires_grad_(True)
    y = api.mlp_fused8(mlp, xmd)
    row = O8.forward_scales(wf8, wp8)
    yo, ro = O8.forward(xm.reshape(300, d), wf8, wp8, row)
    assert y.shape == xm.shape and rel_l2(y.reshape(300, d), yo) < FP8_TOL
    gy = torch.randn(3, 100, d, generator=g).bfloat16()
    y.backward(gy.to(dev))
    gpad = torch.cat([gy.reshape(300, d), torch.zeros(84, d, dtype=torch.bfloat16)])   # the amax of dy ignores zero rows
    dxo, ho, dpo = O8.backward(gy.reshape(300, d), ro, wf8, wp8, O8.backward_scales(gpad, row))
    assert rel_l2(xmd.grad.reshape(300, d), dxo) < FP8_TOL
    dwf, dwp = O8.weight_grads(gy.reshape(300, d), xm.reshape(300, d), ho, dpo)
    assert rel_l2(mlp.c_fc.weight.grad, dwf) < FP8_TOL and rel_l2(mlp.c_proj.weight.grad, dwp) < FP8_TOL
    assert torch.equal(api.forward_scales(wf8.to(dev), wp8.to(dev)).cpu()[[0, 3, 13]], row[[0, 3, 13]])
    tile = api.sc_tile(api.forward_scales(wf8.to(dev), wp8.to(dev)))
    assert tile.shape == (128, 16) and torch.equal(tile[77].cpu()[[0, 3, 13]], row[[0, 3, 13]])
    assert api.shapes_apply8(384, 256, 512) and not api.shapes_apply8(300, 256, 512) and not api.shapes_apply8(384, 128, 512)


def test_nr_mlp_and_projection_with_residual(api, dev):
    """nr_mlp(mlp, x1) = x1 + MLP(rms_norm(x1)) (R2:9202) against the oracle's composition norm -> fp8 MLP -> add, forward
    and backward (the norm's backward plus the residual gradient, R2:9199), and the projection with its residual."""
    from oracle import mlp8 as O8, norm as ON
    g = _g(12)
    d, F = 256, 512
    mlp = torch.nn.Module()
    mlp.c_fc = torch.nn.Linear(d, F, bias=False)
    mlp.c_proj = torch.nn.Linear(F, d, bias=False)
    wf8 = (0.05 * torch.randn(F, d, generator=g)).bfloat16()
    wp8 = (0.05 * torch.randn(d, F, generator=g)).bfloat16()
    mlp.c_fc.weight.data, mlp.c_proj.weight.data = wf8.clone(), wp8.clone()
    mlp = mlp.to(dev)
    x1 = torch.randn(3, 100, d, generator=g).bfloat16()
    x1d = x1.to(dev).requires_grad_(True)
    xo = api.nr_mlp(mlp, x1d)
    x2 = x1.reshape(300, d)
    xn, inv = ON.rmsnorm(x2, None, ON.RMS_EPS)
    row = O8.forward_scales(wf8, wp8)
    yo, ro = O8.forward(xn, wf8, wp8, row)
    assert xo.shape == x1.shape and rel_l2(xo.reshape(300, d), (x2.float() + yo.float()).bfloat16()) < FP8_TOL
    assert rel_l2(xo.reshape(300, d).float() - x2.to(dev).float(), yo) < FP8_TOL          # the MLP term itself, not hidden by x1
    gy = torch.randn(3, 100, d, generator=g).bfloat16()
    xo.backward(gy.to(dev))
    gpad = torch.cat([gy.reshape(300, d), torch.zeros(84, d, dtype=torch.bfloat16)])
    dxn, ho, dpo = O8.backward(gy.reshape(300, d), ro, wf8, wp8, O8.backward_scales(gpad, row))
    gxo = ON.add_rmsnorm_backward(gy.reshape(300, d), dxn, x2, inv, None)[0]
    assert rel_l2(x1d.grad.reshape(300, d), gxo) < FP8_TOL
    assert rel_l2(x1d.grad.reshape(300, d).float() - gy.reshape(300, d).to(dev).float(),
                  gxo.float() - gy.reshape(300, d).float()) < 2 * FP8_TOL                  # the norm-path term alone
    dwf, dwp = O8.weight_grads(gy.reshape(300, d), xn, ho, dpo)
    assert rel_l2(mlp.c_fc.weight.grad, dwf) < FP8_TOL and rel_l2(mlp.c_proj.weight.grad, dwp) < FP8_TOL
    # projection + residual
    a = torch.randn(2, 128, d, generator=g).bfloat16()
    res = torch.randn(2, 128, d, generator=g).bfloat16()
    w = (0.05 * torch.randn(d, d, generator=g)).bfloat16()
    ad, rd, wd = (t.to(dev).requires_grad_(True) for t in (a, res, w))
    out = api.proj_residual(ad, wd, rd)
    want = ((a.float() @ w.float().t()).bfloat16().float() + res.float()).bfloat16()
    assert rel_l2(out, want) < 1e-3
    go = torch.randn(2, 128, d, generator=g).bfloat16()
    out.backward(go.to(dev))
    assert torch.equal(rd.grad.cpu(), go)
    assert rel_l2(ad.grad, go.float() @ w.float()) < BF16_TOL
    assert rel_l2(wd.grad, go.float().reshape(256, d).t() @ a.float().reshape(256, d)) < BF16_TOL


def test_embedding_fwd(api, dev):
    g = _g(8)
    V, C = 1024, 256
    w = torch.randn(V, C, generator=g).bfloat16()
    idx = torch.randint(0, V, (2, 128), generator=g)
    wd = w.to(dev).requires_grad_(True)
    e = api.embedding_fwd(idx.to(dev), wd, torch.bfloat16)
    assert torch.equal(e.cpu(), w[idx])
    gy = torch.randn(2, 128, C, generator=g).bfloat16()
    e.backward(gy.to(dev))
    want = torch.zeros(V, C).index_add_(0, idx.reshape(-1), gy.float().reshape(-1, C))
    assert rel_l2(wd.grad, want) < BF16_TOL


def test_nsk_both_stacks(api, dev):
    """nsk(ga, gb, d_a, d_b) (K/nki_nsk.py:370): the tall and the wide stack of one Muon step against the oracle's
    restatement of emulate_nsk; tolerance as explained in tests/test_gpu_kernels.py (chained iterations)."""
    from oracle import muon as O
    g = _g(13)
    ga = torch.randn(2, 512, 256, generator=g) * 0.02
    gb = torch.randn(3, 256, 512, generator=g) * 0.02
    da, db = O.muon_denominator(ga), O.muon_denominator(gb)
    ya, yb, va, vb = api.nsk(ga.to(dev), gb.to(dev), da.to(dev), db.to(dev))
    yao, vao = O.ns5(ga, da)
    ybo, vbo = O.ns5(gb, db)
    assert ya.shape == ga.shape and yb.shape == gb.shape and va.shape == (2, 512) and vb.shape == (3, 512)
    assert rel_l2(ya, yao) < 2e-2 and rel_l2(yb, ybo) < 2e-2 and rel_l2(va, vao) < 2e-2 and rel_l2(vb, vbo) < 2e-2
    e = api.nsk(ga.to(dev)[:0], gb.to(dev), da.to(dev)[:0], db.to(dev))
    assert e[0].shape == (0, 512, 256) and torch.equal(e[1], yb)


def test_head2_and_adamw_fused_step(api, dev):
    from oracle import norm as ON
    g = _g(14)
    s1, mo, x0, sk = (torch.randn(2, 128, 256, generator=g).bfloat16() for _ in range(4))
    l1, l2, l3 = torch.tensor([0.9]), torch.tensor([0.25]), torch.tensor([-0.4])
    d = lambda t: t.to(dev)
    # the pair form with an external skip, emitting the block input
    x_new, x_norm, x_in, x0p = api.head2((d(s1), d(mo)), d(x0), d(sk), d(l1), d(l2), d(l3), emit=True)
    xt = s1 + mo
    o = ON.block_head(xt.reshape(-1, 256), x0.reshape(-1, 256), l1[0], l2[0], sk.reshape(-1, 256), l3[0])
    assert torch.equal(x_in.cpu(), xt) and torch.equal(x_new.cpu().reshape(-1, 256), o[0]) and x0p.data_ptr() == x0p.data_ptr()
    assert rel_l2(x_norm.reshape(-1, 256), o[1]) < 1e-3
    # the self-skip form on a plain tensor, nothing emitted
    x_new2, _, none, _ = api.head2(d(xt), d(x0), api.SELF_SKIP, d(l1), d(l2), d(l3))
    o2 = ON.block_head(xt.reshape(-1, 256), x0.reshape(-1, 256), l1[0], l2[0], xt.reshape(-1, 256), l3[0])
    assert none is None and torch.equal(x_new2.cpu().reshape(-1, 256), o2[0])
    # AdamW: three steps against torch.optim.AdamW on the same parameters and gradients
    ps = [torch.randn(300, 64, generator=g), torch.randn(1000, generator=g), torch.randn(1, generator=g),
          torch.randn(3, generator=g)]                                         # one-element gains and odd sizes step too
    ref = [p.clone().requires_grad_(True) for p in ps]
    mine = [p.clone().to(dev).requires_grad_(True) for p in ps]
    kw = dict(lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    o_ref, o_mine = torch.optim.AdamW(ref, **kw), torch.optim.AdamW(mine, **kw)
    for step in range(3):
        for a, b in zip(ref, mine):
            gr = torch.randn(a.shape, generator=g)
            a.grad, b.grad = gr.clone(), gr.to(dev)
        o_ref.step()
        versions = [b._version for b in mine]
        assert api.adamw_fused_step(o_mine) is True
        assert all(b._version > v for b, v in zip(mine, versions))            # the raw kernel write is visible to autograd's counters
    for a, b in zip(ref, mine):
        assert rel_l2(b, a) < 1e-6
        assert rel_l2(o_mine.state[b]["exp_avg_sq"], o_ref.state[a]["exp_avg_sq"]) < 1e-6
    mine[0].grad = mine[0].grad.t().contiguous().t()                         # a strided gradient is not the kernel's layout: nothing is done
    before = mine[1].detach().clone()
    assert api.adamw_fused_step(o_mine) is False and torch.equal(mine[1].detach(), before)


def test_r1_fp8_rows(api, dev):
    """The fixed-scale fp8 rows of the reference's round1 sources (R1:2169 fused_fc_relu2_fp8, 4097 fused_fc_relu2_nn, 3728 c_proj, 3412 row_matmul,
    3486 dw_matmul, 2059 begin_step) against the oracle's restatement: each row alone, then the MLP forward + backward with
    the in-place weight-gradient convention."""
    from oracle import r1fp8 as O
    nn8 = api.nki_gemm_fp8_nn
    g = _g(15)
    M, d, F = 384, 256, 512
    x = torch.randn(M, d, generator=g).bfloat16()
    w1 = (0.5 * torch.randn(d, F, generator=g)).bfloat16()                  # LinearT [in, out]
    w2 = (0.05 * torch.randn(d, F, generator=g)).bfloat16()                 # [out, in]
    dy = (1e-7 * torch.randn(M, d, generator=g)).bfloat16()
    xd, w1d, w2d, dyd = (t.to(dev) for t in (x, w1, w2, dy))
    nn8.begin_step()
    pre = nn8.row_matmul(xd, w1d, 1)
    assert rel_l2(pre, O.row_matmul(x, w1, 1)) < 1e-3
    h = (torch.relu(pre.float()) * pre.float()).bfloat16()
    assert rel_l2(nn8.row_matmul(h, w2d, 2), O.row_matmul(h.cpu(), w2, 2)) < 1e-3
    assert rel_l2(nn8.row_matmul(dyd, w2d, 4), O.row_matmul(dy, w2, 4)) < 1e-3
    dpre = (1e-7 * torch.randn(M, F, generator=g)).bfloat16()
    assert rel_l2(nn8.row_matmul(dpre.to(dev), w1d, 3), O.row_matmul(dpre, w1, 3)) < 1e-3
    assert rel_l2(nn8.dw_matmul(xd, dpre.to(dev), 5), O.dw_matmul(x, dpre, 5)) < 1e-3
    assert rel_l2(nn8.dw_matmul(dyd, h, 6), O.dw_matmul(dy, h.cpu(), 6)) < 1e-3
    assert nn8.dw_matmul(xd.float(), dpre.to(dev), 5) is None and nn8.dw_matmul(xd[:100], dpre.to(dev)[:100], 5) is None
    # the weight cache: one fp8 copy per step, a new one after begin_step or after the parameter is written
    a = api.nki_gemm_fp8.quantised_weight(w1d, 64.0, False)
    assert api.nki_gemm_fp8.quantised_weight(w1d, 64.0, False) is a
    nn8.begin_step()
    assert api.nki_gemm_fp8.quantised_weight(w1d, 64.0, False) is not a
    # the MLP through the reference's two calls, inplace: gradients are summed into existing .grad tensors
    x3 = x.view(3, 128, d).to(dev).requires_grad_(True)
    p1, p2 = w1d.clone().requires_grad_(True), w2d.clone().requires_grad_(True)
    g1 = (1e-5 * torch.randn(d, F, generator=g)).bfloat16()              # what an earlier micro-step left in .grad
    p1.grad, p2.grad = g1.to(dev).clone(), g1.to(dev).clone()
    hh = nn8.fused_fc_relu2_nn(x3, p1, inplace=True)
    y = nn8.c_proj(hh, p2, True)
    y.backward(dy.view(3, 128, d).to(dev))
    yo, dxo, dw1o, dw2o = O.mlp_forward_backward(x, w1, w2, dy)
    assert y.shape == (3, 128, d) and rel_l2(y.reshape(M, d), yo) < 2e-3
    assert rel_l2(x3.grad.reshape(M, d), dxo) < 2e-2
    assert rel_l2(p1.grad, g1.float() + dw1o.float()) < 2e-2 and rel_l2(p2.grad, g1.float() + dw2o.float()) < 2e-2
    assert rel_l2(p1.grad.float() - g1.to(dev).float(), dw1o) < 5e-2       # the row-5 product itself, not hidden by g1
    assert api.nki_gemm_fp8.active(True) and not api.nki_gemm_fp8.active(False)


def test_band_attention_through_the_reference_calls(api, dev):
    """nki_causal_attention(..., nw) and nki_rope_attention(..., nw) (R2:4925 fused_rope_attention_band) against the
    oracle's composition with the band mask (K/nki_attn_bandpro.py:1654), forward and gradients."""
    from oracle import attention as O
    g = _g(16)
    B, H, T, D, nw = 1, 2, 512, 128, 2
    qkv = torch.randn(B, T, 3 * H * D, generator=g).bfloat16()
    cos, sin = O.rope_tables(T, D)
    qd = qkv.to(dev).requires_grad_(True)
    y = api.nki_rope_attention(qd, cos.to(dev), sin.to(dev), H, nw=nw)
    gy = torch.randn(B, T, H, D, generator=g).bfloat16()
    y.backward(gy.to(dev))
    q, k, v = (t.view(B, T, H, D) for t in qkv.split(H * D, dim=-1))
    qn, rq, iq = O.rope_norm(q, cos, sin)
    kn, rk, ik = O.rope_norm(k, cos, sin)
    q4, k4, v4 = qn.permute(0, 2, 1, 3), kn.permute(0, 2, 1, 3), v.permute(0, 2, 1, 3)
    scale = 1.0 / math.sqrt(D)
    yo, lo = O.forward(q4, k4, v4, scale, band_tiles=nw)
    assert y.shape == (B, T, H, D) and rel_l2(y, yo) < BF16_TOL
    dq4, dk4, dv4 = O.backward(q4, k4, v4, yo, gy, lo, scale, band_tiles=nw)
    dq = O.rope_norm_backward(dq4.permute(0, 2, 1, 3), rq, iq, cos, sin)
    dk = O.rope_norm_backward(dk4.permute(0, 2, 1, 3), rk, ik, cos, sin)
    want = torch.cat([t.reshape(B, T, H * D) for t in (dq, dk, dv4.permute(0, 2, 1, 3))], dim=-1)
    assert rel_l2(qd.grad, want) < 2 * BF16_TOL
    q64 = torch.randn(1, 2, 512, 64, generator=g).bfloat16().to(dev)
    a = api.nki_causal_attention(q64, q64, q64, nw=4)
    b = api.nki_causal_attention(q64, q64, q64)
    assert torch.equal(a, b)                                                     # a band as wide as the sequence


class _Lin:
    def __init__(self, w):
        self.weight = w


class _SharedMlp:
    def __init__(self, wf, wp):
        self.c_fc, self.c_proj = _Lin(wf), _Lin(wp)


class _MoeModule:
    """The attributes of the reference's MoeMLP (round2/source/train.py:10818-10875) that moe_mlp reads."""

    def __init__(self, router, w_fc, w_proj, topk, cap, e8, shared):
        self.router, self.w_fc, self.w_proj, self.topk, self.cap, self.e8, self.shared = router, w_fc, w_proj, topk, cap, e8, shared


@pytest.mark.parametrize("e8", [True, False])
def test_moe_mlp_module_mirror(api, dev, e8):
    """train_api.moe_mlp as MoeMLP.forward / forward_e8 (round2/source/train.py:10941-11067): the routed output against the
    oracle layer with the same per-sequence capacity on the kernel's selections (fp8 experts 2e-2, bf16 experts 5e-3), the
    shared half added to it, the statistics vector (kept share, lb, z, load shares) against the oracle's tables and terms,
    and gradients reaching the router, the experts and the shared half."""
    from oracle import moe as O
    from trainium_frontier_them_bones_amd import ops
    B, T, d, H, E, topk, cap = 4, 256, 256, 512, 8, 2, 48
    g = torch.Generator().manual_seed(17)
    x = torch.randn(B, T, d, generator=g).bfloat16()
    router = torch.randn(E, d, generator=g) * 0.5
    wf = (torch.randn(E, H, d, generator=g) * 0.05).bfloat16()
    wp = (torch.randn(E, d, H, generator=g) * 0.05).bfloat16()
    sf = (torch.randn(2 * H, d, generator=g) * 0.05).bfloat16()
    sp = (torch.randn(d, 2 * H, generator=g) * 0.05).bfloat16()
    xd = x.to(dev).requires_grad_(True)
    rd, wfd, wpd = (t.to(dev).requires_grad_(True) for t in (router, wf, wp))
    sfd, spd = sf.to(dev).requires_grad_(True), sp.to(dev).requires_grad_(True)
    alpha, beta, gamma = 0.01, 0.001, 0.02
    bare = _MoeModule(rd, wfd, wpd, topk, cap, e8, None)
    full = _MoeModule(rd, wfd, wpd, topk, cap, e8, _SharedMlp(sfd, spd))
    routed = api.moe_mlp(bare, xd)
    out, aux, stats = api.moe_mlp(full, xd, want_stats=True, aux_weights=(alpha, beta, gamma))
    # the kernel's selections, then the oracle's layer on them
    p, idx, _, logits = ops.moe_route(x.to(dev).reshape(-1, d), router.to(dev).contiguous(), topk, None, want_logits=True)
    ic = idx.cpu().long()
    xo, ro, wfo, wpo = (t.clone().requires_grad_(True) for t in (x, router, wf, wp))
    oo, _ = O.moe_forward(xo, ro, wfo, wpo, topk, None, fp8=e8, capacity=cap, idx=ic)
    tol = 2e-2 if e8 else 5e-3
    assert rel_l2(routed, oo) < tol
    shared_out = api.mlp_fused8(full.shared, xd) if e8 else api.relu_squared(xd.detach() @ sfd.detach().t()) @ spd.detach().t()
    assert rel_l2(out, routed.detach().float() + shared_out.detach().float()) < 5e-3
    slot, _, _ = O.tables(ic, E, T, cap)
    lb, z, f, seq = O.aux_terms(p.cpu().double(), logits.cpu().double(), ic, topk, seq_len=T)
    assert stats.shape == (3 + E,)
    assert abs(stats[0].item() - float((slot >= 0).sum()) / (B * T * topk)) < 1e-6 and stats[0].item() < 1.0   # it does drop
    assert abs(stats[1].item() - lb.item()) < 1e-4 * lb.item() and abs(stats[2].item() - z.item()) < 1e-4 * z.item()
    assert rel_l2(stats[3:], f) < 1e-6
    assert abs(aux.item() - (alpha * lb + beta * z + gamma * seq).item()) < 1e-4 * abs(aux.item())
    (out.float().square().mean() + aux).backward()
    for t in (xd, rd, wfd, wpd, sfd, spd):
        assert t.grad is not None and bool(torch.isfinite(t.grad.float()).all()) and float(t.grad.float().abs().max()) > 0


def test_dense_bf16_fused_mlp_kernels_and_wrapper(dev):
    """mlp_fwd_kernel / mlp_bwd_kernel in the reference's call style ((x2, w_fc, w_proj, tb) -> (y, rT);
    (dy2, rT, w_fc, w_proj, tb, dw_mode) -> (dx, h, dpre), K/nki_mlp_fused.py:242, 290) against the oracle's restatement of
    the kernels' arithmetic, and mlp_fused(mlp, x) with its weight gradients against autograd of the kit's expression."""
    from oracle import mlp8 as O
    from trainium_frontier_them_bones_amd import train_api as T
    g = torch.Generator().manual_seed(5)
    M, d, F = 512, 256, 1024
    x = torch.randn(M, d, generator=g).bfloat16()
    wf = (0.05 * torch.randn(F, d, generator=g)).bfloat16()
    wp = (0.05 * torch.randn(d, F, generator=g)).bfloat16()
    dy = torch.randn(M, d, generator=g).bfloat16()
    assert T.mlp_fused_applies(x, F) and not T.mlp_fused_applies(x[:100], F)
    y, rT = T.mlp_fwd_kernel(x.to(dev), wf.to(dev), wp.to(dev), 512)
    yo, ro = O.forward_bf16(x, wf, wp)
    assert tuple(rT.shape) == (F, M)
    assert rel_l2(rT.t(), ro) < 2e-3 and rel_l2(y, yo) < 5e-3
    dx, h, dpre = T.mlp_bwd_kernel(dy.to(dev), rT, wf.to(dev), wp.to(dev), 512, 0)
    dxo, ho, dpo = O.backward_bf16(dy, rT.t().cpu(), wf, wp)
    assert torch.equal(h.cpu(), ho) and rel_l2(dpre, dpo) < 2e-3 and rel_l2(dx, dxo) < 5e-3
    dx1, hT, dpT = T.mlp_bwd_kernel(dy.to(dev), rT, wf.to(dev), wp.to(dev), 512, 1)
    assert torch.equal(dx1, dx) and torch.equal(hT, h.t()) and torch.equal(dpT, dpre.t())

    class M_:                                        # a module with the reference's attribute names
        pass
    mlp = M_()
    mlp.c_fc, mlp.c_proj = M_(), M_()
    mlp.c_fc.weight = wf.to(dev).requires_grad_(True)
    mlp.c_proj.weight = wp.to(dev).requires_grad_(True)
    xl = x.view(2, M // 2, d).to(dev).requires_grad_(True)
    out = T.mlp_fused(mlp, xl)
    out.backward(dy.view(2, M // 2, d).to(dev))
    xr, wfr, wpr = (t.clone().float().requires_grad_(True) for t in (x, wf, wp))
    ref = torch.nn.functional.linear(torch.relu(torch.nn.functional.linear(xr, wfr)).square(), wpr)
    ref.backward(dy.float())
    assert rel_l2(out.reshape(M, d), ref) < 5e-3 and rel_l2(xl.grad.reshape(M, d), xr.grad) < 1e-2
    assert rel_l2(mlp.c_fc.weight.grad, wfr.grad) < 1e-2 and rel_l2(mlp.c_proj.weight.grad, wpr.grad) < 1e-2
    with pytest.raises(Exception):
        T.mlp_fwd_kernel(x[:100].to(dev), wf.to(dev), wp.to(dev))     # 100 rows: not a shape the kernels take


def test_fused_gradient_norm_and_clip_factor(dev):
    """grad_norm_fused over a bf16 and an fp32 gradient buffer (lengths off every vector width): the norm against fp64, the
    clipping factor clamp(clip / (gnorm + 1e-6), max=1) (R1:1714), each buffer alone, and clip <= 0 giving 1."""
    from trainium_frontier_them_bones_amd import ops
    from trainium_frontier_them_bones_amd import train_api as T
    g = torch.Generator().manual_seed(9)
    for nb, nf in ((8 * 1000 + 8, 4 * 333 + 4), (1 << 22, 1 << 20), (8 * 77, 4 * 5)):
        gb = torch.randn(nb, generator=g).bfloat16()
        gf = torch.randn(nf, generator=g)
        want = math.sqrt(float(gb.double().pow(2).sum() + gf.double().pow(2).sum()))
        gn, sc = T.grad_norm_fused(gb.to(dev), gf.to(dev), 1.0)
        assert abs(gn.item() - want) < 1e-5 * want
        assert abs(sc.item() - min(1.0 / (want + 1e-6), 1.0)) < 1e-5
        out = ops.gradnorm(gb.to(dev), gf.to(dev), 0.0).cpu()
        assert abs(out[0].item() - float(gb.double().pow(2).sum())) < 1e-5 * out[0].item() and out[3].item() == 1.0
        only_b = ops.gradnorm(gb.to(dev), None, 1e9).cpu()
        assert abs(only_b[2].item() - math.sqrt(float(gb.double().pow(2).sum()))) < 1e-5 * only_b[2].item() and only_b[3].item() == 1.0
        only_f = ops.gradnorm(None, gf.to(dev), 0.5).cpu()
        assert abs(only_f[1].item() - float(gf.double().pow(2).sum())) < 1e-5 * only_f[1].item()


@pytest.mark.parametrize("shape", [(2, 128, 256), (4, 256, 768), (1, 512, 1024)])
def test_mix_tail_forward_and_backward(dev, shape):
    """mix_tail(x, xn_dead, lam) (R1:7308) against the oracle: s1 bit for bit, xn2 and inv to rounding, and the gradients of
    both outputs (gx, and dlam rounded to lam's dtype) through autograd; sequence starts read zeros and nothing crosses a
    sequence boundary (perturbing one sequence leaves the others' outputs and gradients unchanged)."""
    from oracle import norm as O
    from trainium_frontier_them_bones_amd import train_api as T
    B, Tn, C = shape
    g = torch.Generator().manual_seed(B + Tn + C)
    x = torch.randn(B, Tn, C, generator=g).bfloat16()
    lam = torch.tensor(0.37).bfloat16()
    gy = torch.randn(B, Tn, C, generator=g).bfloat16()
    ge = torch.randn(B, Tn, C, generator=g).bfloat16()
    xl = x.to(dev).requires_grad_(True)
    ll = lam.to(dev).requires_grad_(True)
    s1, y = T.mix_tail(xl, None, ll)
    so, yo, invo = O.mix_tail(x, lam.float())
    assert torch.equal(s1.cpu(), so) and rel_l2(y, yo) < 2e-3
    torch.autograd.backward([s1, y], [ge.to(dev), gy.to(dev)])
    gxo, dlo = O.mix_tail_backward(x, so, invo, lam.float(), gy, ge)
    assert rel_l2(xl.grad, gxo) < 3e-3
    assert ll.grad.dtype == torch.bfloat16 and abs(ll.grad.float().item() - float(dlo)) <= 2e-2 * abs(float(dlo)) + 0.5
    # only one of the two gradients given
    xl2 = x.to(dev).requires_grad_(True)
    s2, y2 = T.mix_tail(xl2, None, lam.to(dev))
    y2.backward(gy.to(dev))
    assert rel_l2(xl2.grad, O.mix_tail_backward(x, so, invo, lam.float(), gy, None)[0]) < 3e-3
    if B > 1:
        xp = x.clone()
        xp[0] += 1.0
        s3, y3 = T.mix_tail(xp.to(dev), None, lam.to(dev))
        assert torch.equal(s3[1:], s1[1:].detach()) and torch.equal(y3[1:], y[1:].detach())
