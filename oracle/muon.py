"""CPU restatement of the reference's Newton-Schulz ("Polar Express") kernel arithmetic. TEST INFRASTRUCTURE ONLY: the
product path never imports this module.

Follows round2/source/kernels/nki_nsk.py: emulate_nsk (:452-468) and _ns_tall (:426-449) for the rounding points
(X0 = bf16(bf16(g) * fp32(1 / d)); G rounded once to bf16 from its fp32 accumulator; B = bf16(fp32(G^2 c) + fp32(b G));
X' = bf16(fp32(X B) + fp32(a X)); row sums of squares in fp32 from the bf16 X5), with the accumulation over the row tiles
written as one fp32 matmul (the order of an fp32 sum is not part of the contract: the reference itself calls its kernel
"the kit's within the bf16 band, not bitwise", :55-57). The kernel's mirror fill of G and B (_sym_fill_t, :415) is the
identity on an exactly symmetric matrix; here G and B are symmetrised the same way, from their upper triangles.

Pins (tests/test_oracle_muon.py): the kit's own expression of the loop (reference_ns, :471-481) evaluated in fp64; the
polar factor U V^T of X0 from torch.linalg.svd (what the iteration approximates); singular values of X5 inside the
Polar Express band; tall / wide transposition symmetry.
"""
import torch

NS_COEFFS = (
    (8.156554524902461, -22.48329292557795, 15.878769915207462),
    (4.042929935166739, -2.808917465908714, 0.5000178451051316),
    (3.8916678022926607, -2.772484153217685, 0.5060648178503393),
    (3.285753657755655, -2.3681294933425376, 0.46449024233003106),
    (2.3465413258596377, -1.7097828382687081, 0.42323551169305323),
)


def _sym_upper(t):
    """The matrix with its lower triangle replaced by the mirror of its upper one."""
    u = torch.triu(t)
    return u + torch.triu(t, 1).transpose(0, 1)


def ns_tall(x0, coeffs=NS_COEFFS):
    """Five iterations on one tall bf16 matrix [M, N] (nki_nsk.py:426 _ns_tall)."""
    x = x0
    for a, b, c in coeffs:
        xf = x.float()
        g = _sym_upper((xf.transpose(0, 1) @ xf).to(torch.bfloat16))
        gf = g.float()
        g2 = gf.transpose(0, 1) @ gf
        bm = _sym_upper(((g2 * c) + (gf * b)).to(torch.bfloat16))
        xb = xf @ bm.float()
        x = ((xb * 1.0) + (xf * a)).to(torch.bfloat16)
    return x


def x0_of(g, d):
    """bf16(bf16(g) * fp32(1 / d)) (nki_nsk.py:460)."""
    return (g.to(torch.bfloat16).float() * (1.0 / d.float())).to(torch.bfloat16)


def ns5(g, d, coeffs=NS_COEFFS):
    """(y bf16 [K, r, c], v fp32 [K, max(r, c)]) from a stack g fp32 [K, r, c] and its denominators d [K]
    (nki_nsk.py:452 emulate_nsk: the tall stack as it is, the wide one through its transposes)."""
    ys, vs = [], []
    dd = d.reshape(-1)
    for j in range(g.shape[0]):
        x0 = x0_of(g[j], dd[j])
        wide = x0.shape[0] < x0.shape[1]
        x5 = ns_tall(x0.transpose(0, 1).contiguous() if wide else x0, coeffs)
        vs.append(x5.float().square().sum(dim=-1))
        ys.append(x5.transpose(0, 1) if wide else x5)
    return torch.stack(ys), torch.stack(vs)


def kit_ns(x, coeffs=NS_COEFFS):
    """The kit's own loop on [K, r, c] in x's dtype (nki_nsk.py:471 reference_ns)."""
    if x.shape[-2] > x.shape[-1]:
        for a, b, c in coeffs:
            xtx = x.mT @ x
            x = a * x + x @ (b * xtx + c * (xtx @ xtx))
    else:
        for a, b, c in coeffs:
            xxt = x @ x.mT
            x = a * x + (b * xxt + c * (xxt @ xxt)) @ x
    return x


def muon_denominator(g):
    """d = bf16(bf16(||bf16(g)||) * 1.01 + 1e-6) per matrix (nki_nsk.py:7-9, torch's own bf16 expression of the kit)."""
    x = g.to(torch.bfloat16)
    return x.norm(dim=(-2, -1), keepdim=True) * 1.01 + 1e-6
