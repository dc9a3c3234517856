"""The oracle against vectors the REFERENCE's own torch emulations produced (tests/golden/ref_vectors.npz, written by
tests/golden/make_ref_vectors.py in the build container from round2/source/kernels/*.py): scale rows, the fp8 MLP's
forward / backward / weight gradients incl. a case that reaches the hidden clamp, attention forward / backward (full and
banded), the fp8 weight gradient, the residual-mix backward and the Newton-Schulz chain.

Power-of-two scales, casts and elementwise outputs must be equal bit for bit. Outputs that pass through a long fp32 sum
are also expected to be equal (same torch, one thread), but the assertion allows a summation-order difference: at most
0.5 % of the elements may differ, each by at most one unit in the last place of the output dtype. A misplaced clamp, a
rounding made at another point or a wrong descale moves far more elements than that (tests at the bottom show it)."""
import os

import numpy as np
import pytest
import torch

from oracle import attention as OA
from oracle import mlp8 as O8
from oracle import muon as OM
from oracle import norm as ON

HERE = os.path.dirname(os.path.abspath(__file__))
bf = torch.bfloat16


@pytest.fixture(scope="module")
def ref():
    z = np.load(os.path.join(HERE, "golden", "ref_vectors.npz"), allow_pickle=False)
    out = {}
    for k in z.files:
        a = z[k]
        if k.endswith(":bf16"):
            out[k[:-5]] = torch.from_numpy(a.view(np.int16).copy()).view(bf)
        else:
            out[k] = torch.from_numpy(np.array(a))
    return out


def close_ulp(got, want, frac=5e-3):
    """equal, or different in at most `frac` of the elements and there by one unit in the last place"""
    assert got.shape == want.shape and got.dtype == want.dtype
    if torch.equal(got, want):
        return True
    if got.dtype == bf:
        gi, wi = got.view(torch.int16).int(), want.view(torch.int16).int()
        d = (gi - wi).abs()
        # (a step across zero or a sign change is not one ulp in this integer view: never allowed)
        return bool((d <= 1).all()) and float((d != 0).float().mean()) <= frac
    d = (got.double() - want.double()).abs()
    tol = want.double().abs() * 2.0 ** -22 + 1e-30
    return bool((d <= tol).all())


def close_sum(got, want, frac=5e-3, rel=1e-4):
    """for outputs whose values may be small against their summands (weight gradients): a summation-order difference
    can then move an element by more than one ulp, so the bar is few differing elements and a tiny relative distance"""
    assert got.shape == want.shape and got.dtype == want.dtype
    diff = float((got != want).float().mean())
    dist = float((got.double() - want.double()).norm() / want.double().norm())
    return diff <= frac and dist <= rel


def test_scale_rows_equal_the_references(ref):
    rows = ref["scales.rows"]
    for i in range(rows.shape[0]):
        r0 = O8.forward_scales(ref["scales.%d.w_fc" % i], ref["scales.%d.w_proj" % i])
        r1 = O8.backward_scales(ref["scales.%d.dy" % i], r0)
        assert torch.equal(r0, rows[i, 0]), i
        assert torch.equal(r1, rows[i, 1]), i
    assert torch.equal(O8.forward_scales(ref["mlp8.w_fc"], ref["mlp8.w_proj"]), ref["mlp8.row"])
    assert torch.equal(O8.backward_scales(ref["mlp8.dy"], ref["mlp8.row"]), ref["mlp8.brow"])


@pytest.mark.parametrize("case", ["mlp8", "mlp8c"])
def test_fp8_mlp_equals_the_references_emulation(ref, case):
    w_fc, w_proj, dy, row, brow = ref["mlp8.w_fc"], ref["mlp8.w_proj"], ref["mlp8.dy"], ref["mlp8.row"], ref["mlp8.brow"]
    x = ref[case + ".x"]
    y, r = O8.forward(x, w_fc, w_proj, row)
    want_r = ref[case + ".rT"].t().contiguous()
    assert close_ulp(r, want_r) and close_ulp(y, ref[case + ".y"])
    dx, h, dpre = O8.backward(dy, want_r, w_fc, w_proj, brow)
    assert torch.equal(h, (want_r.float() * want_r.float()).to(bf))
    assert close_ulp(dpre, ref[case + ".dpre"]) and close_ulp(dx, ref[case + ".dx"])
    if case == "mlp8":
        assert torch.equal(h, ref["mlp8.h"])
        dw_fc, dw_proj = O8.weight_grads(dy, x, ref["mlp8.h"], ref["mlp8.dpre"])
        # (the reference multiplies in bf16 `mm`, the oracle in fp32 `@` + one rounding: the same sums in another order)
        assert close_sum(dw_fc, ref["mlp8.dw_fc"]) and close_sum(dw_proj, ref["mlp8.dw_proj"])
    else:
        # the case exists for the clamp: a good share of the hidden activations must sit above it
        rc = want_r.float() * row[O8.COL["c_h"]]
        assert float((rc > O8.H_CLAMP).float().mean()) > 0.02


def test_fp8_mlp_vectors_tell_a_misplaced_clamp_or_rounding_apart(ref):
    """The same vectors reject the plausible mistakes: r saved AFTER the clamp, the clamp applied to r^2 instead of r,
    h8 taken from the unrounded r c, and a backward that forgets the factor 2 carried by dq_dh2."""
    x, w_fc, w_proj, row = ref["mlp8c.x"], ref["mlp8.w_fc"], ref["mlp8.w_proj"], ref["mlp8.row"]
    C = O8.COL
    x8 = O8.fp8_round(x.float() * O8.X_SCALE, 0)
    a8 = O8.fp8_round(w_fc.float() * row[C["s_wfc"]], 0)
    b8 = O8.fp8_round(w_proj.float() * row[C["s_wproj"]], 0)
    pre = torch.clamp_min((x8 @ a8.t()) * row[C["dq_fc"]], 0.0)
    r = pre.to(bf)
    want_y, want_r = ref["mlp8c.y"], ref["mlp8c.rT"].t().contiguous()
    # (0) the restatement written out here is the emulation
    rc0 = torch.clamp_max(r.float() * row[C["c_h"]], O8.H_CLAMP).to(bf).float()
    assert close_ulp(((O8.fp8_round(rc0 * rc0, 0) @ b8.t()) * row[C["dq_proj"]]).to(bf), want_y)
    # (1) r saved after the clamp
    r_clamped = (torch.clamp_max(r.float() * row[C["c_h"]], O8.H_CLAMP) / row[C["c_h"]]).to(bf)
    assert not close_ulp(r_clamped, want_r)
    # (2) clamp on the square
    rc2 = torch.clamp_max((r.float() * row[C["c_h"]]) ** 2, O8.H_CLAMP)
    y2 = ((O8.fp8_round(rc2, 0) @ b8.t()) * row[C["dq_proj"]]).to(bf)
    assert not close_ulp(y2, want_y)
    # (3) no bf16 rounding of r (and of r c) before the square
    rc3 = torch.clamp_max(pre * row[C["c_h"]], O8.H_CLAMP)
    y3 = ((O8.fp8_round(rc3 * rc3, 0) @ b8.t()) * row[C["dq_proj"]]).to(bf)
    assert not close_ulp(y3, want_y)
    # (4) the factor 2 of d(r^2)
    brow = ref["mlp8.brow"].clone()
    brow[C["dq_dh2"]] *= 0.5
    _, _, dpre4 = O8.backward(ref["mlp8.dy"], want_r, w_fc, w_proj, brow)
    assert not close_ulp(dpre4, ref["mlp8c.dpre"])


def _split_heads(t3, B, T, H, D):
    return t3.view(B, T, H, D)


def test_attention_equals_the_references_emulation(ref):
    q, k, v, do3 = ref["attn.q"], ref["attn.k"], ref["attn.v"], ref["attn.do3"]
    B, H, T, D = q.shape
    shift = float(ref["attn.shift"])
    for tag, band in (("", None), ("b", 1)):
        o, lse = OA.forward(q, k, v, 0.125, shift=shift, band_tiles=band)
        o3 = ref["attn.o3" + tag]
        assert close_ulp(o.reshape(B, T, H * D), o3)
        # the reference keeps lse as [B H, 128, T / 128] with query g 128 + p at [p, g]
        lse_ref = ref["attn.lse3" + tag].transpose(1, 2).reshape(B, H, T)
        assert close_ulp(lse, lse_ref)
        dq, dk, dv = OA.backward(q, k, v, _split_heads(o3, B, T, H, D), _split_heads(do3, B, T, H, D), lse_ref, 0.125,
                                 band_tiles=band)
        assert close_ulp(dq, ref["attn.dq" + tag]) and close_ulp(dk, ref["attn.dk" + tag])
        assert close_ulp(dv.transpose(1, 2).reshape(B, T, H * D), ref["attn.dv3" + tag])
    # the row-maximum shift the HIP kernels use gives the same function; P is then rounded to bf16 at another magnitude,
    # so o agrees to the bf16 path's tolerance rather than bit for bit
    o_max, lse_max = OA.forward(q, k, v, 0.125)
    o_ref = ref["attn.o3"].float()
    assert float((o_max.reshape(B, T, H * D).float() - o_ref).norm() / o_ref.norm()) < 5e-3
    # (lse is the log of a sum of bf16-rounded P: rounding them at another magnitude moves it by up to ~2^-9)
    assert float((lse_max - ref["attn.lse3"].transpose(1, 2).reshape(B, H, T)).abs().max()) < 4e-3


def test_fp8_weight_gradient_equals_the_references_emulation(ref):
    g2, a2, h = ref["dw8.g2"], ref["dw8.a2"], ref["dw8.h"]
    s_g, s_a = 2.0 ** 20, 4.0
    out = O8.fp8_weight_grad(g2, a2, s_g, s_a, 1.0 / (s_g * s_a), 1, 0)
    assert close_ulp(out, ref["dw8.out_e5m2_e4m3"])
    out2 = O8.fp8_weight_grad(h, g2, 64.0, s_g, 1.0 / (64.0 * s_g), 0, 1, clamp_g=240.0)
    assert close_ulp(out2, ref["dw8.out_e4m3c_e5m2"])
    assert float((h.float() * 64.0 > 240.0).float().mean()) > 0.05           # the clamp is exercised
    assert not close_ulp(O8.fp8_weight_grad(h, g2, 64.0, s_g, 1.0 / (64.0 * s_g), 0, 1, clamp_g=448.0),
                         ref["dw8.out_e4m3c_e5m2"])


def test_resmix_backward_equals_the_references_emulation(ref):
    dx, dx0, da, db = ON.resmix_backward(ref["resmix.g"], ref["resmix.x"], ref["resmix.x0"], ref["resmix.a"][0],
                                         ref["resmix.b"][0])
    assert torch.equal(dx, ref["resmix.dx"]) and torch.equal(dx0, ref["resmix.dx0"])
    lam = ref["resmix.part"].sum(dim=0)              # the reference finishes its per-partition partials with one sum
    assert abs(float(da) - float(lam[0])) <= 1e-5 * abs(float(lam[0])) + 1e-4
    assert abs(float(db) - float(lam[1])) <= 1e-5 * abs(float(lam[1])) + 1e-4


def test_newton_schulz_equals_the_references_emulation(ref):
    assert np.array_equal(np.asarray(OM.NS_COEFFS, dtype=np.float64), ref["nsk.coeffs"].numpy())
    ga, gb = ref["nsk.ga"].float(), ref["nsk.gb"].float()
    ya, va = OM.ns5(ga, ref["nsk.d_a"])
    yb, vb = OM.ns5(gb, ref["nsk.d_b"])
    # the chain amplifies a one-ulp difference of the fp32 summation order, so here the bar is a relative distance
    for got, want in ((ya, ref["nsk.ya"]), (yb, ref["nsk.yb"])):
        assert got.shape == want.shape
        assert float((got.float() - want.float()).norm() / want.float().norm()) < 1e-2
    assert float((va - ref["nsk.va"]).norm() / ref["nsk.va"].norm()) < 1e-2
    assert float((vb - ref["nsk.vb"]).norm() / ref["nsk.vb"].norm()) < 1e-2
