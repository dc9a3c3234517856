"""Pins of oracle/r1fp8.py (CPU)."""
import torch

from helpers import fp8_table, rel_l2, round_to_table
from oracle import r1fp8 as O


def test_casts_follow_the_byte_tables_and_the_clamp():
    g = torch.Generator().manual_seed(0)
    for fmt, name, scale in ((0, "e4m3fn", 4.0), (0, "e4m3fn", 1.0 / 128), (1, "e5m2", 2.0 ** 30)):
        table = fp8_table(name)
        span = O.clip_bound(scale, fmt) * 1.5                           # some values beyond the clamp
        x = ((torch.rand(4096, generator=g) * 2 - 1) * span).bfloat16()
        got = O.q(x, scale, fmt).double()
        b = O.clip_bound(scale, fmt)
        want = table[round_to_table(x.double().clamp(-b, b) * scale, table)]
        assert torch.equal(got, want)
        hi = O.E5M2_MAX if fmt else O.E4M3_MAX
        assert got.abs().max() <= hi                                     # the clamp keeps e4m3 inside the legacy 240
        # the bound's defining property: b * scale fits, the next bf16 above does not
        nb = torch.nextafter(torch.tensor(b, dtype=torch.bfloat16), torch.tensor(float("inf"), dtype=torch.bfloat16))
        assert b * scale <= hi < float(nb) * scale


def test_power_of_two_scales_are_exact_and_rows_track_the_unrounded_products():
    g = torch.Generator().manual_seed(1)
    M, d, F = 256, 128, 256
    x = torch.randn(M, d, generator=g).bfloat16()
    w1 = (0.7 * torch.randn(d, F, generator=g)).bfloat16()              # h = relu(x w1)^2 of the magnitude the 1 / 128 scale is for
    w2 = (0.05 * torch.randn(d, F, generator=g)).bfloat16()
    dy = (1e-7 * torch.randn(M, d, generator=g)).bfloat16()
    # scaling an operand by another power of two inside the format's range changes nothing but the exponent
    assert torch.equal(O.q(x, 4.0, 0), O.q((x.float() * 2).bfloat16(), 2.0, 0))
    y, dx, dw1, dw2 = O.mlp_forward_backward(x, w1, w2, dy)
    pre = x.double() @ w1.double()
    h = torch.relu(pre) ** 2
    assert rel_l2(y, h @ w2.double().t()) < 6e-2                         # e4m3 x e4m3: ~2.4 % per operand
    dh = dy.double() @ w2.double()
    dpre = 2 * torch.relu(pre) * dh
    assert rel_l2(dx, dpre @ w1.double().t()) < 1.2e-1                   # e5m2 gradients: ~6 % per operand, chained
    assert rel_l2(dw1, x.double().t() @ dpre) < 1.2e-1
    assert rel_l2(dw2, dy.double().t() @ h) < 1.2e-1
    # a transposed operand or a wrong row spec is far outside those budgets
    assert rel_l2(O.row_matmul(x, w1, 1), pre) < 4e-2
    assert O.ROW_SPEC[2]["trans_b"] and not O.ROW_SPEC[4]["trans_b"]
