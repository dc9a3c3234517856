"""Pins of oracle/muon.py (CPU): the restatement of the reference's Newton-Schulz kernel arithmetic against the kit's own
expression in fp64, the SVD polar factor, the singular-value band and the tall / wide symmetry."""
import torch

from helpers import rel_l2
from oracle import muon as O


def _stack(K, r, c, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(K, r, c, generator=g) * 0.02


def test_restatement_tracks_the_kits_expression_in_fp64():
    for shape in ((2, 384, 128), (2, 128, 384), (1, 256, 256)):
        g = _stack(*shape, seed=1)
        d = O.muon_denominator(g)
        y, _ = O.ns5(g, d)
        x0 = torch.stack([O.x0_of(g[j], d.reshape(-1)[j]) for j in range(g.shape[0])])
        want = O.kit_ns(x0.double())
        # five iterations in bf16 with three roundings each: inside the bf16 band of the exact iteration
        assert rel_l2(y, want) < 2e-2, shape
        # a dropped term or a wrong coefficient moves the result by far more than that
        bad = O.kit_ns(x0.double(), O.NS_COEFFS[1:] + O.NS_COEFFS[:1])
        assert rel_l2(y, bad) > 0.1


def test_result_approximates_the_polar_factor():
    g = _stack(1, 512, 128, seed=2)
    d = O.muon_denominator(g)
    y, v = O.ns5(g, d)
    x0 = O.x0_of(g[0], d.reshape(-1)[0]).double()
    u, s, vh = torch.linalg.svd(x0, full_matrices=False)
    polar = u @ vh
    # Polar Express maps every singular value into a band around 1 (it does not converge to exactly 1 in five steps)
    sv = torch.linalg.svdvals(y[0].double())
    assert sv.min() > 0.6 and sv.max() < 1.3
    # same singular vectors as X0: y^T polar is close to a multiple of the identity's band, and the cosine is high
    cos = (y[0].double() * polar).sum() / (y[0].double().norm() * polar.norm())
    assert cos > 0.97
    assert rel_l2(v[0], y[0].float().square().sum(-1)) < 1e-6


def test_wide_is_the_transpose_of_tall():
    g = _stack(2, 128, 384, seed=3)
    d = O.muon_denominator(g)
    yw, vw = O.ns5(g, d)
    yt, vt = O.ns5(g.transpose(1, 2).contiguous(), d)
    assert torch.equal(yw, yt.transpose(1, 2)) and torch.equal(vw, vt)
    assert vw.shape == (2, 384)


def test_denominator_and_x0_rounding_points():
    g = _stack(1, 128, 128, seed=4)
    d = O.muon_denominator(g)
    assert d.dtype == torch.bfloat16 and d.shape == (1, 1, 1)
    want = (g[0].bfloat16().float() * (1.0 / d.float().reshape(()))).bfloat16()
    assert torch.equal(O.x0_of(g[0], d.reshape(-1)[0]), want)
    # spectral norm of X0 is below 1 (Frobenius-normalised with a 1 % margin): the iteration's domain
    assert torch.linalg.svdvals(O.x0_of(g[0], d.reshape(-1)[0]).double()).max() < 1.0


def test_sensitivity_to_the_order_of_the_fp32_sums():
    """The same rounding points with the matmuls accumulated in fp64 instead of fp32: the five-iteration results differ by
    several 1e-3 (one-ulp bf16 flips amplified by the chain). This is the floor of any implementation that does not
    reproduce the accumulation order, and the reason the GPU test holds the chained result to 2e-2."""
    g = _stack(1, 768, 256, seed=5)
    d = O.muon_denominator(g)
    x0 = O.x0_of(g[0], d.reshape(-1)[0])
    x = x0
    for a, b, c in O.NS_COEFFS:
        xf = x.float()
        gm = O._sym_upper((xf.double().T @ xf.double()).float().to(torch.bfloat16)).float()
        bm = O._sym_upper((((gm.double().T @ gm.double()).float() * c) + (gm * b)).to(torch.bfloat16))
        x = (((xf.double() @ bm.double()).float() * 1.0) + (xf * a)).to(torch.bfloat16)
    s = rel_l2(O.ns_tall(x0), x)
    assert 5e-4 < s < 1.5e-2
