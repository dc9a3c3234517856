"""The torch.library registration of the kernel calls (the form of the reference's round2 sources, round2/source/train.py:4988-5036,
6858-6913): the ops against the autograd.Function wrappers they mirror, their fake implementations and schemas."""
import pytest
import torch

from helpers import rel_l2

pytestmark = pytest.mark.gpu


def _g(seed):
    return torch.Generator().manual_seed(seed)


def test_custom_ops_match_the_function_wrappers_and_pass_opcheck(dev):
    from trainium_frontier_them_bones_amd import autograd as A, library_ops, ops
    o = library_ops.register()
    assert library_ops.register() is o                                            # idempotent
    g = _g(3)
    # attention
    q, k, v = (torch.randn(1, 2, 256, 64, generator=g).bfloat16().to(dev).requires_grad_(True) for _ in range(3))
    do = torch.randn(1, 256, 2, 64, generator=g).bfloat16().to(dev)
    out, lse = torch.ops.tfb.attn_fwd(q, k, v, 0.125)
    out.backward(do)
    q2, k2, v2 = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    ref = A.CausalAttentionFn.apply(q2, k2, v2, 0.125)
    ref.backward(do)
    assert torch.equal(out, ref) and torch.equal(q.grad, q2.grad) and torch.equal(k.grad, k2.grad) and torch.equal(v.grad, v2.grad)
    assert not lse.requires_grad
    torch.library.opcheck(torch.ops.tfb.attn_fwd.default, (q.detach(), k.detach(), v.detach(), 0.125),
                          test_utils=("test_schema", "test_faketensor"))
    # fp8 MLP with pre-cast weights
    M, d, F = 256, 256, 512
    x = torch.randn(M, d, generator=g).bfloat16().to(dev).requires_grad_(True)
    wf = (0.05 * torch.randn(F, d, generator=g)).bfloat16().to(dev).requires_grad_(True)
    wp = (0.05 * torch.randn(d, F, generator=g)).bfloat16().to(dev).requires_grad_(True)
    sc = ops.mlp8_forward_scales(wf.detach(), wp.detach())
    w8 = torch.ops.tfb.mlp8_precast(wf.detach(), wp.detach(), sc)
    y, r = torch.ops.tfb.mlp8_fwd(x, wf, wp, sc, w8)
    gy = torch.randn(M, d, generator=g).bfloat16().to(dev)
    y.backward(gy)
    st = A.Mlp8State()
    st.refresh(wf.detach(), wp.detach())
    x2, wf2, wp2 = (t.detach().clone().requires_grad_(True) for t in (x, wf, wp))
    y2 = A.Mlp8Fn.apply(x2, wf2, wp2, st)
    y2.backward(gy)
    assert torch.equal(w8, st.w8) and torch.equal(y, y2) and torch.equal(x.grad, x2.grad)
    assert torch.equal(wf.grad, wf2.grad) and torch.equal(wp.grad, wp2.grad) and not r.requires_grad
    torch.library.opcheck(torch.ops.tfb.mlp8_fwd.default, (x.detach(), wf.detach(), wp.detach(), sc, w8),
                          test_utils=("test_schema", "test_faketensor"))
    torch.library.opcheck(torch.ops.tfb.mlp8_bwd.default, (gy, r, x.detach(), wf.detach(), wp.detach(), sc, w8),
                          test_utils=("test_schema", "test_faketensor"))
    # loss head on materialised logits, mean over the valid rows
    N, V = 256, 1024
    logits = torch.randn(N, V, generator=g).bfloat16().to(dev).requires_grad_(True)
    tg = torch.randint(0, V, (N,), generator=g)
    tg[::7] = -1
    valid = (tg >= 0).float()
    row_w = (valid / valid.sum()).to(dev)
    loss_rows, lz = torch.ops.tfb.loss_head_fwd(logits, tg.to(dev), row_w, 15.0)
    loss_rows.sum().backward()
    lf = logits.detach().float().cpu().requires_grad_(True)
    want = torch.nn.functional.cross_entropy(15.0 * torch.tanh(lf / 15.0), tg, ignore_index=-1)
    want.backward()
    assert abs(loss_rows.sum().item() - want.item()) < 1e-3 * want.item()
    assert rel_l2(logits.grad, lf.grad) < 5e-3
    torch.library.opcheck(torch.ops.tfb.loss_head_fwd.default, (logits.detach(), tg.to(dev), row_w, 15.0),
                          test_utils=("test_schema", "test_faketensor"))
