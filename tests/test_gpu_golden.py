"""The HIP kernels, through the C-ABI, against vectors the REFERENCE's own torch emulations produced
(tests/golden/ref_vectors.npz; generator tests/golden/make_ref_vectors.py, run in the build container only).
Tolerances: power-of-two scales, fp8 operand bytes and elementwise outputs bit-exact; bf16 paths rel-L2 <= 5e-3;
fp8 paths <= 2e-2 (the saved activation and dpre, which see one GEMM only, <= 2e-3)."""
import os

import numpy as np
import pytest
import torch

from helpers import rel_l2

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
bf = torch.bfloat16
BF16_TOL, FP8_TOL = 5e-3, 2e-2


@pytest.fixture(scope="module")
def ops(dev):
    from trainium_frontier_them_bones_amd import ops as _ops
    return _ops


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


def test_scale_rows(ops, dev, ref):
    rows = ref["scales.rows"]
    pow2 = [0, 1, 2, 3, 4, 11, 12, 13, 14, 15]
    cases = [(ref["scales.%d.w_fc" % i], ref["scales.%d.w_proj" % i], ref["scales.%d.dy" % i], rows[i, 0], rows[i, 1])
             for i in range(rows.shape[0])]
    cases.append((ref["mlp8.w_fc"], ref["mlp8.w_proj"], ref["mlp8.dy"], ref["mlp8.row"], ref["mlp8.brow"]))
    for i, (wf, wp, dy, r0, r1) in enumerate(cases):
        print("scale row case %d" % i, flush=True)
        row = ops.mlp8_forward_scales(wf.to(dev), wp.to(dev), 240.0)
        assert torch.equal(row.cpu()[pow2], r0[pow2]), i                       # scales, descales and amax: exact
        assert torch.allclose(row.cpu()[9:11], r0[9:11], rtol=1e-5), i         # norms: fp32 summation order
        rowb = ops.mlp8_backward_scales(dy.to(dev), r0.to(dev))
        assert torch.equal(rowb.cpu()[5:9], r1[5:9]), i


@pytest.mark.parametrize("case", ["mlp8", "mlp8c"])
def test_fp8_mlp(ops, dev, ref, case):
    wf, wp, dy = ref["mlp8.w_fc"].to(dev), ref["mlp8.w_proj"].to(dev), ref["mlp8.dy"].to(dev)
    row, brow = ref["mlp8.row"].to(dev), ref["mlp8.brow"].to(dev)
    x = ref[case + ".x"].to(dev)
    w8 = ops.mlp8_precast(wf, wp, row)
    y, r = ops.mlp8_fwd(x, w8, row, wf.shape[0])
    want_r = ref[case + ".rT"].t().contiguous()
    assert rel_l2(r, want_r) < 2e-3 and rel_l2(y, ref[case + ".y"]) < FP8_TOL
    # the backward from the reference's own saved activation
    dx, h, dpre = ops.mlp8_bwd(dy, want_r.to(dev), w8, brow)
    assert torch.equal(h.cpu(), (want_r.float() * want_r.float()).to(bf))
    assert rel_l2(dpre, ref[case + ".dpre"]) < 2e-3 and rel_l2(dx, ref[case + ".dx"]) < FP8_TOL
    if case == "mlp8":
        assert rel_l2(ops.matmul(ref["mlp8.dpre"].to(dev), x, trans_a=True), ref["mlp8.dw_fc"]) < BF16_TOL
        assert rel_l2(ops.mlp_dw_proj(dy, want_r.to(dev)), ref["mlp8.dw_proj"]) < BF16_TOL
    else:
        # with a fifth of the activations on the clamp, the output still follows the reference's clamp placement: an
        # unclamped hidden activation would be off by far more than the fp8 tolerance
        rc = want_r.float() * ref["mlp8.row"][2]
        assert float((rc > 15.375).float().mean()) > 0.02


def test_attention(ops, dev, ref):
    q, k, v = (ref["attn." + n].to(dev) for n in ("q", "k", "v"))
    B, H, T, D = q.shape
    do = ref["attn.do3"].view(B, T, H, D).to(dev)
    for tag, band in (("", 0), ("b", 1)):
        print("attention vectors, band %d" % band, flush=True)
        o, lse = ops.attn_fwd(q, k, v, 0.125, band=band)
        assert rel_l2(o.reshape(B, T, H * D), ref["attn.o3" + tag]) < BF16_TOL
        lse_ref = ref["attn.lse3" + tag].transpose(1, 2).reshape(B, H, T)
        assert float((lse.cpu() - lse_ref).abs().max()) < 4e-3
        o_ref = ref["attn.o3" + tag].view(B, T, H, D).to(dev)
        dq, dk, dv = ops.attn_bwd(q, k, v, o_ref, do, lse_ref.contiguous().to(dev), 0.125, band=band)
        assert rel_l2(dq, ref["attn.dq" + tag]) < BF16_TOL and rel_l2(dk, ref["attn.dk" + tag]) < BF16_TOL
        assert rel_l2(dv.permute(0, 2, 1, 3).reshape(B, T, H * D), ref["attn.dv3" + tag]) < BF16_TOL


def test_fp8_weight_gradient(ops, dev, ref):
    g2, a2, h = ref["dw8.g2"].to(dev), ref["dw8.a2"].to(dev), ref["dw8.h"].to(dev)
    s_g, s_a = 2.0 ** 20, 4.0
    g8, a8 = ops.quant_fp8(g2, s_g, 1), ops.quant_fp8(a2, s_a, 0)
    out = ops.gemm_fp8_tn(g8, a8, 1, 0, imm=1.0 / (s_g * s_a))
    assert rel_l2(out, ref["dw8.out_e5m2_e4m3"]) < 1e-3                        # same bytes, fp32 sums in another order
    # the clamped e4m3 form: the clamp at 240 is applied to the scaled value before the cast
    h8 = ops.quant_fp8(torch.clamp_max(h.float() * 64.0, 240.0).to(bf), 1.0, 0)
    out2 = ops.gemm_fp8_tn(h8, g8, 0, 1, imm=1.0 / (64.0 * s_g))
    assert rel_l2(out2, ref["dw8.out_e4m3c_e5m2"]) < 1e-3


def test_resmix_backward(ops, dev, ref):
    ab = torch.stack([ref["resmix.a"][0].float(), ref["resmix.b"][0].float()]).to(dev)
    dx, dx0, dab = ops.resmix_bwd(ref["resmix.g"].to(dev), ref["resmix.x"].to(dev), ref["resmix.x0"].to(dev), ab)
    assert torch.equal(dx.cpu(), ref["resmix.dx"]) and torch.equal(dx0.cpu(), ref["resmix.dx0"])
    lam = ref["resmix.part"].sum(dim=0)
    assert abs(dab[0].item() - lam[0].item()) < 1e-4 * abs(lam[0].item()) + 1e-3
    assert abs(dab[1].item() - lam[1].item()) < 1e-4 * abs(lam[1].item()) + 1e-3


def test_newton_schulz(ops, dev, ref):
    for s in ("a", "b"):
        g = ref["nsk.g" + s].float().to(dev)
        y, v = ops.ns5(g, ref["nsk.d_" + s].to(dev))
        assert rel_l2(y, ref["nsk.y" + s]) < FP8_TOL       # the chain amplifies one-ulp flips: the stated 2e-2 bar
        assert rel_l2(v, ref["nsk.v" + s]) < FP8_TOL
