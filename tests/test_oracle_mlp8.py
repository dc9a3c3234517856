"""Pins oracle/mlp8.py without the reference: closed forms, the fp8 format tables, invariants, autograd."""
import math

import pytest
import torch

from oracle import mlp8 as O
from helpers import fp8_table, rel_l2, round_to_table


def test_pow2_scale_matches_closed_form_brute_force():
    # every exponent in a wide window x several mantissas, against 2^floor(log2(limit / v)) clipped to the window
    for limit, (lo, hi) in ((240.0, O.EXP_W), (448.0, O.EXP_W), (28672.0, O.EXP_G), (57344.0, O.EXP_G)):
        vs, want = [], []
        for e in range(-60, 70):
            for mant in (1.0, 1.0 + 2 ** -20, 1.171875, 1.5, 1.875, 2.0 - 2 ** -20):
                v = mant * 2.0 ** e
                v32 = torch.tensor(v, dtype=torch.float32).item()
                if not math.isfinite(v32) or v32 <= 0:
                    continue
                k = math.floor(math.log2(limit / v32))
                # exact check of the boundary in float64 (log2 may be off by one at exact powers)
                while v32 * 2.0 ** (k + 1) <= limit:
                    k += 1
                while v32 * 2.0 ** k > limit:
                    k -= 1
                k = max(lo, min(hi, k))
                vs.append(v32)
                want.append(2.0 ** k)
        s, inv = O.pow2_floor_scale(torch.tensor(vs, dtype=torch.float32), limit, lo, hi)
        assert torch.equal(s.double(), torch.tensor(want, dtype=torch.float64))
        assert torch.equal(s * inv, torch.ones_like(s))
    s, inv = O.pow2_floor_scale(torch.zeros(1), 240.0, *O.EXP_W)
    assert s.item() == 2.0 ** O.EXP_W[1]          # v = 0 gives the top of the window


def test_pow4_scale_is_even_power_and_maximal():
    v = torch.logspace(-12, 6, 400, dtype=torch.float32)
    s, inv, c, ic = O.pow4_floor_scale(v, 240.0, *O.EXP_H)
    assert torch.equal(c * c, s) and torch.equal(s * inv, torch.ones_like(s)) and torch.equal(c * ic, torch.ones_like(s))
    e = torch.log2(c)
    assert torch.equal(e, e.round())
    inside = (e > O.EXP_H[0]) & (e < O.EXP_H[1])
    assert bool(((v * s <= 240.0) | (e == O.EXP_H[0])).all())
    assert bool((v[inside] * s[inside] * 4.0 > 240.0).all())  # the next power of four would overflow the limit


def test_fp8_round_matches_format_tables():
    # the oracle's cast (torch's) against a brute-force nearest-even rounding onto the decoded byte tables
    g = torch.Generator().manual_seed(1)
    for fmt, name, lim in ((0, "e4m3fn", 448.0), (1, "e5m2", 57344.0)):
        table = fp8_table(name)
        x = torch.cat([torch.randn(4000, generator=g) * s for s in (1e-3, 0.1, 1.0, 30.0, lim / 3)])
        x = x.clamp(-lim, lim).bfloat16().float()
        ties = (table[torch.isfinite(table)][:-1] + table[torch.isfinite(table)][1:]) / 2   # exact midpoints
        x = torch.cat([x, ties.float()[torch.isfinite(ties.float())]])
        got = O.fp8_bytes(x, fmt).long()
        want = round_to_table(x, table)
        same_value = table[got] == table[want]
        assert bool(same_value.all()), (x[~same_value][:5], table[got][~same_value][:5], table[want][~same_value][:5])


def test_e4m3_values_up_to_240_survive_bf16():
    table = fp8_table("e4m3fn")
    vals = table[torch.isfinite(table) & (table.abs() <= 240.0)]
    assert vals.numel() == 2 * 120 or vals.numel() > 200
    assert torch.equal(vals.float().bfloat16().double(), vals)


def _layer(seed, M=256, d=256, F=512):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, d, generator=g).bfloat16()
    wf = (0.02 * torch.randn(F, d, generator=g)).bfloat16()
    wp = (0.02 * torch.randn(d, F, generator=g)).bfloat16()
    dy = torch.randn(M, d, generator=g).bfloat16()
    return x, wf, wp, dy


def test_scale_rows_keep_every_cast_in_range():
    x, wf, wp, dy = _layer(0)
    x = (x.float() / x.float().pow(2).mean(-1, keepdim=True).sqrt()).bfloat16()   # unit-RMS rows, as the norm delivers
    row = O.forward_scales(wf, wp)
    c = O.COL
    assert (wf.float().abs().max() * row[c["s_wfc"]]).item() <= 240.0 < (wf.float().abs().max() * row[c["s_wfc"]] * 2).item()
    assert (wp.float().abs().max() * row[c["s_wproj"]]).item() <= 240.0
    assert row[c["dq_fc"]].item() == (row[c["i_wfc"]] / 4.0).item()
    y, r = O.forward(x, wf, wp, row)
    assert torch.isfinite(y.float()).all()
    rb = O.backward_scales(dy, row)
    assert (dy.float().abs().max() * rb[c["s_dy"]]).item() <= 57344.0 / 2
    dx, h, dpre = O.backward(dy, r, wf, wp, rb)
    assert (dpre.float().abs().max() * rb[c["s_dp"]]).item() <= 57344.0
    assert torch.isfinite(dx.float()).all()


def test_fp8_mlp_tracks_bf16_mlp_within_fp8_budget():
    x, wf, wp, dy = _layer(2)
    row = O.forward_scales(wf, wp)
    y8, r8 = O.forward(x, wf, wp, row)
    yb, rb = O.forward_bf16(x, wf, wp)
    assert torch.equal(yb, O.reference_forward(x, wf, wp)) or rel_l2(yb, O.reference_forward(x, wf, wp)) < 4e-3
    assert rel_l2(r8, rb) < 0.06 and rel_l2(y8, yb) < 0.12
    dx8, h8, dp8 = O.backward(dy, r8, wf, wp, O.backward_scales(dy, row))
    dxb, hb, dpb = O.backward_bf16(dy, rb, wf, wp)
    assert rel_l2(dp8, dpb) < 0.12 and rel_l2(dx8, dxb) < 0.15


def test_bf16_mlp_backward_is_autograd_of_reference_forward():
    x, wf, wp, dy = _layer(3, M=128, d=128, F=256)
    xf = x.double().requires_grad_(True)
    wff = wf.double().requires_grad_(True)
    wpf = wp.double().requires_grad_(True)
    y = torch.relu(xf @ wff.t()).square() @ wpf.t()
    y.backward(dy.double())
    _, r = O.forward_bf16(x, wf, wp)
    dx, h, dpre = O.backward_bf16(dy, r, wf, wp)
    dw_fc, dw_proj = O.weight_grads(dy, x, h, dpre)
    assert rel_l2(dx, xf.grad) < 1e-2 and rel_l2(dw_fc, wff.grad) < 1e-2 and rel_l2(dw_proj, wpf.grad) < 1e-2


def test_fp8_weight_grad_close_to_bf16_weight_grad():
    x, wf, wp, dy = _layer(4)
    s_g, _ = O.pow2_floor_scale(dy.float().abs().amax(), 57344.0 / 2, *O.EXP_G)
    out = O.fp8_weight_grad(dy, x, s_g, 4.0, 1.0 / (s_g * 4.0), 1, 0)
    ref = (dy.float().t() @ x.float()).bfloat16()
    assert rel_l2(out, ref) < 0.1


def _decode(bytes_u8, fmt):
    """fp8 bytes -> fp64 values through the format tables (decoded from the format definitions, not by torch's cast)."""
    from helpers import fp8_table
    return fp8_table("e5m2" if fmt == 1 else "e4m3fn")[bytes_u8.long()]


def test_fp8_weight_grads_independent_route_budget_and_invariance():
    x, wf, wp, dy = _layer(5, M=256, d=256, F=512)
    row = O.forward_scales(wf, wp)
    y, r = O.forward(x, wf, wp, row)
    rowb = O.backward_scales(dy, row)
    dx, h, dpre = O.backward(dy, r, wf, wp, rowb)
    dw_fc, dw_proj = O.weight_grads_fp8(x, dy, h, dpre, rowb)
    assert dw_fc.shape == wf.shape and dw_proj.shape == wp.shape and dw_fc.dtype == x.dtype
    # (1) independent route: the operand bytes decoded through the tables, one fp64 product, the inverse scales applied
    s_dp, s_h, s_dy = (float(rowb[O.COL[k]]) for k in ("s_dp", "s_h", "s_dy"))
    g8 = _decode(O.fp8_bytes(dpre.float() * s_dp, 1), 1)
    a8 = _decode(O.fp8_bytes(x.float() * 4.0, 0), 0)
    ref_fc = (g8.t() @ a8) / (s_dp * 4.0)
    hq = _decode(O.fp8_bytes(torch.clamp_max(h.float() * s_h, 240.0), 0), 0)
    d8 = _decode(O.fp8_bytes(dy.float() * s_dy, 1), 1)
    ref_pj = (d8.t() @ hq) / (s_dy * s_h)
    assert rel_l2(dw_fc, ref_fc) < 3e-3 and rel_l2(dw_proj, ref_pj) < 3e-3   # one bf16 rounding + fp32 summation
    # (2) the fp8 budget against the bf16 weight gradients (the reference quotes ~6 % mean relative)
    b_fc, b_pj = O.weight_grads(dy, x, h, dpre)
    assert rel_l2(dw_fc, b_fc) < 0.08 and rel_l2(dw_proj, b_pj) < 0.08
    # (3) a dropped or doubled scale factor, or swapped formats, would break these: exact power-of-two covariance
    dw2 = O.fp8_weight_grad(dpre * 4.0, x, s_dp / 4.0, 4.0, 1.0 / (s_dp * 4.0), 1, 0)
    assert torch.equal(dw2, dw_fc)
    dw3 = O.fp8_weight_grad(dpre, x, s_dp, 4.0, 2.0 / (s_dp * 4.0), 1, 0)
    assert torch.equal(dw3.float(), dw_fc.float() * 2.0)
    # (4) the clamp is on the g side only and only above the limit: a tiny limit changes dw_proj, a huge one does not
    same = O.weight_grads_fp8(x, dy, h, dpre, rowb, e4m3_limit=448.0)[1]
    assert torch.equal(same, dw_proj) or float((h.float() * s_h).max()) > 240.0
    small = O.weight_grads_fp8(x, dy, h, dpre, rowb, e4m3_limit=1.0)[1]
    assert not torch.equal(small, dw_proj)
