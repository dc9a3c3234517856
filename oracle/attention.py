"""Causal attention oracle (bf16 in, fp32 accumulate) and RoPE.

Restates K/nki_attn_bandpro.py:1510-1551 (the forward / backward kernels' arithmetic: P rounded to the input
dtype before every product, row sum over the rounded values, dS rounded, dQ/dK scaled in fp32 then rounded),
its band mask :1654-1658, and the eager expression the kernels replace, SDPA(q, k, v, is_causal, scale)
transposed to [B, T, H, D] (R1:7476-7487, 8099-8125). RoPE is the half-split rotation R1:4188-4193 with the
tables of R1:8951-8962 (inv_freq = base^(-2i/D), cos/sin rounded to bf16).

The reference subtracts a fixed shift inside exp; a row maximum is used here (shift = "max") unless a number is
passed. Both give the same P up to fp32 rounding because softmax is shift-invariant.

Pinned by (tests/test_oracle_attention.py): torch SDPA in fp64 for forward and autograd gradients, a brute-force
per-row softmax loop at T = 128, row sums of P = 1, causality (future tokens do not change the past), dV with
dO = 1 equals column sums of P, RoPE norm preservation and its inverse being the transpose rotation.
"""
import math

import torch


def mask(T, band_tiles=None, device=None):
    """[q, k] True where attended: k <= q, and with a band only the last `band_tiles` 128-key tiles."""
    i = torch.arange(T, device=device)
    m = i[None, :] <= i[:, None]
    if band_tiles is not None:
        m = m & (i[None, :] // 128 > i[:, None] // 128 - band_tiles)
    return m


def forward(q4, k4, v4, scale=None, shift="max", band_tiles=None):
    """q4, k4, v4 [B, H, T, D] -> (o [B, T, H, D] in the input dtype, lse [B, H, T] fp32)."""
    B, H, T, D = q4.shape
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    dt = q4.dtype
    s = torch.matmul(q4.float(), k4.float().transpose(-1, -2)) * scale         # [B, H, q, k]
    keep = mask(T, band_tiles, q4.device)
    s = s.masked_fill(~keep, float("-inf"))
    c = s.amax(dim=-1, keepdim=True) if shift == "max" else torch.full_like(s[..., :1], float(shift))
    e = torch.exp(s - c).to(dt).float()                                        # rounded once, masked entries are 0
    den = e.sum(dim=-1, keepdim=True)
    o = (torch.matmul(e, v4.float()) * (1.0 / den)).to(dt)
    lse = (torch.log(den) + c).squeeze(-1)
    return o.transpose(1, 2).contiguous(), lse


def backward(q4, k4, v4, o, do, lse, scale=None, band_tiles=None):
    """o, do [B, T, H, D]; returns (dq, dk, dv) as [B, H, T, D] in the input dtype."""
    B, H, T, D = q4.shape
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    dt = q4.dtype
    qf, kf, vf = q4.float(), k4.float(), v4.float()
    of = o.transpose(1, 2).float()
    gf = do.transpose(1, 2).float()
    s = torch.matmul(qf, kf.transpose(-1, -2)) * scale
    p = torch.exp(s - lse[..., None]).to(dt).float()
    p = p * mask(T, band_tiles, q4.device).to(p.dtype)
    dp = torch.matmul(gf, vf.transpose(-1, -2))
    dsum = (gf * of).sum(dim=-1, keepdim=True)
    ds = ((dp - dsum) * p).to(dt).float()
    dv = torch.matmul(p.transpose(-1, -2), gf).to(dt)
    dk = (scale * torch.matmul(ds.transpose(-1, -2), qf)).to(dt)
    dq = (scale * torch.matmul(ds, kf)).to(dt)
    return dq, dk, dv


def sdpa_reference(q4, k4, v4, scale=None, dtype=torch.float64):
    """The library routine: SDPA in `dtype`, transposed to [B, T, H, D]."""
    y = torch.nn.functional.scaled_dot_product_attention(q4.to(dtype), k4.to(dtype), v4.to(dtype), is_causal=True,
                                                         scale=scale)
    return y.transpose(1, 2)


def rope_tables(T, D, base=10000.0, dtype=torch.bfloat16):
    """(cos, sin) [T, D/2] in `dtype`."""
    inv_freq = 1.0 / (base ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    ang = torch.outer(torch.arange(T, dtype=torch.float32), inv_freq)
    return ang.cos().to(dtype), ang.sin().to(dtype)


def rope(x, cos, sin):
    """Half-split rotation of x [B, T, H, D] with tables [T, D/2]: y1 = x1 c + x2 s, y2 = -x1 s + x2 c; fp32 math,
    one rounding."""
    D = x.shape[-1]
    c = cos.float()[None, :, None, :]
    s = sin.float()[None, :, None, :]
    x1, x2 = x.float()[..., : D // 2], x.float()[..., D // 2:]
    return torch.cat((x1 * c + x2 * s, x2 * c - x1 * s), dim=-1).to(x.dtype)


def rope_backward(gy, cos, sin):
    """The transpose rotation: g1 = gy1 c - gy2 s, g2 = gy2 c + gy1 s."""
    D = gy.shape[-1]
    c = cos.float()[None, :, None, :]
    s = sin.float()[None, :, None, :]
    g1, g2 = gy.float()[..., : D // 2], gy.float()[..., D // 2:]
    return torch.cat((g1 * c - g2 * s, g2 * c + g1 * s), dim=-1).to(gy.dtype)


QK_NORM_EPS = 2.0 ** -23


def rope_norm(x, cos, sin, eps=QK_NORM_EPS):
    """(y, r, inv): r = rope(x) rounded to x's dtype, inv = rsqrt(mean_D(r^2) + eps) fp32 [..., 1], y = (r inv) rounded:
    the rotation followed by the parameter-free per-head RMSNorm, norm(apply_rotary_emb(x, cos, sin)) of
    round1/source/train.py:4184-4196 (kernel :4308; eps :4172), before its transpose(1, 2). x [B, T, H, D]."""
    r = rope(x, cos, sin)
    rf = r.float()
    inv = torch.rsqrt(rf.pow(2).mean(-1, keepdim=True) + eps)
    return (rf * inv).to(x.dtype), r, inv


def rope_norm_backward(g, r, inv, cos, sin):
    """Gradient of rope_norm's input (round1/source/train.py:4353-4381): u = g - r inv^2 (g . r) / D, gr = (u inv)
    rounded to g's dtype, then the transposed rotation."""
    gf, rf = g.float(), r.float()
    D = g.shape[-1]
    coef = inv * inv * (gf * rf).sum(-1, keepdim=True) / D
    gr = ((gf - rf * coef) * inv).to(g.dtype)
    return rope_backward(gr, cos, sin)

