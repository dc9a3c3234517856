"""Pins of oracle/proj8.py (fp8 attention projections) without the reference: library routines and exact invariants."""
import torch

from helpers import fp8_table, rel_l2
from oracle import mlp8, proj8


def _g(seed):
    return torch.Generator().manual_seed(seed)


def test_scales_are_the_closed_form_powers_of_two():
    g = _g(1)
    w = (0.02 * torch.randn(384, 256, generator=g)).bfloat16()
    s, inv = proj8.weight_scale(w)
    amax = w.float().abs().amax()
    e = torch.floor(torch.log2(torch.tensor(240.0) / amax))
    assert s.item() == 2.0 ** e.item() and (s * inv).item() == 1.0 and (amax * s).item() <= 240.0 < (amax * s * 2).item()
    gs, ginv = proj8.grad_scale(torch.randn(64, 64, generator=g) * 1e-3)
    assert (gs * ginv).item() == 1.0


def test_casts_decode_through_the_bit_level_tables():
    g = _g(2)
    x = torch.randn(1024, generator=g) * 50
    for fmt, name in ((0, "e4m3fn"), (1, "e5m2")):
        dec = fp8_table(name)
        b = mlp8.fp8_bytes(x, fmt)
        assert torch.equal(dec[b.long()].float(), mlp8.fp8_round(x, fmt))


def test_forward_and_input_gradient_against_the_bf16_projection():
    g = _g(3)
    M, K, N = 512, 256, 384
    a = torch.randn(M, K, generator=g).bfloat16()
    w = (0.05 * torch.randn(N, K, generator=g)).bfloat16()
    s_w, _ = proj8.weight_scale(w)
    y = proj8.forward(a, w, proj8.X_SCALE, s_w)
    ref = proj8.reference_forward(a, w)
    assert rel_l2(y, ref) < 5e-2                     # two e4m3 roundings of 2^-4 relative step each
    a_s, _ = proj8.act_scale(a)
    assert rel_l2(proj8.forward(a, w, a_s, s_w), ref) < 5e-2
    gy = torch.randn(M, N, generator=g).bfloat16()
    af = a.float().requires_grad_(True)
    (af @ w.float().t()).backward(gy.float())
    s_g, _ = proj8.grad_scale(gy)
    assert rel_l2(proj8.backward_input(gy, w, s_g, s_w), af.grad) < 8e-2   # e5m2 gradient: 2^-3 relative step
    wf = w.float().requires_grad_(True)
    (a.float() @ wf.t()).backward(gy.float())
    assert rel_l2(proj8.weight_grad(gy, a), wf.grad) < 5e-3


def test_fp8_weight_gradient_against_autograd_and_the_byte_tables():
    from helpers import fp8_table
    g = _g(5)
    M, K, N = 512, 256, 384
    a = torch.randn(M, K, generator=g).bfloat16()
    gy = (1e-2 * torch.randn(M, N, generator=g)).bfloat16()
    s_g, _ = proj8.grad_scale(gy)
    dw = proj8.weight_grad_fp8(gy, a, s_g, proj8.X_SCALE)
    assert dw.shape == (N, K)
    assert rel_l2(dw, proj8.weight_grad(gy, a)) < 8e-2                    # e5m2 gradient x e4m3 activation
    g8 = fp8_table("e5m2")[mlp8.fp8_bytes(gy.float() * s_g, 1).long()]
    a8 = fp8_table("e4m3fn")[mlp8.fp8_bytes(a.float() * proj8.X_SCALE, 0).long()]
    assert rel_l2(dw, (g8.t() @ a8) / float(s_g * proj8.X_SCALE)) < 3e-3   # one bf16 rounding + fp32 summation
    s_a, _ = proj8.act_scale(a)
    dw2 = proj8.weight_grad_fp8(gy, a, s_g, s_a)
    assert rel_l2(dw2, proj8.weight_grad(gy, a)) < 8e-2
    # a gradient 16 times larger gets a scale 16 times smaller: identical bytes, the result exactly 16 times larger
    gy16 = (gy.float() * 16).bfloat16()
    assert torch.equal(proj8.weight_grad_fp8(gy16, a, proj8.grad_scale(gy16)[0], proj8.X_SCALE).float(), dw.float() * 16)


def test_forward_is_exactly_invariant_under_power_of_two_weight_rescaling():
    g = _g(4)
    a = torch.randn(256, 128, generator=g).bfloat16()
    w = (0.03 * torch.randn(128, 128, generator=g)).bfloat16()
    y1 = proj8.forward(a, w, proj8.X_SCALE, proj8.weight_scale(w)[0])
    w2 = (w.float() * 8).bfloat16()
    y2 = proj8.forward(a, w2, proj8.X_SCALE, proj8.weight_scale(w2)[0])
    assert torch.equal((y1.float() * 8).bfloat16(), y2)
