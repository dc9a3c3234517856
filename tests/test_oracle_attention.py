"""Pins oracle/attention.py: torch SDPA (library routine) in fp64, a brute-force softmax loop, invariants."""
import math

import torch

from oracle import attention as O
from helpers import rel_l2


def _qkv(seed, B=2, H=2, T=256, D=64, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(B, H, T, D, generator=g).to(dtype) for _ in range(3)]


def test_forward_matches_sdpa_fp64():
    q, k, v = _qkv(0)
    o, lse = O.forward(q, k, v)
    ref = O.sdpa_reference(q, k, v)
    assert rel_l2(o, ref) < 5e-3
    s = (q.double() @ k.double().transpose(-1, -2)) / math.sqrt(64)
    s = s.masked_fill(~O.mask(256), float("-inf"))
    assert rel_l2(lse, torch.logsumexp(s, -1)) < 1e-3   # the sum runs over bf16-rounded exponentials


def test_forward_brute_force_rows():
    q, k, v = _qkv(1, B=1, H=1, T=128, D=64, dtype=torch.float32)
    o, _ = O.forward(q, k, v, scale=0.125)
    out = torch.zeros(128, 64, dtype=torch.float64)
    for i in range(128):
        w = [math.exp(0.125 * float(q[0, 0, i].double() @ k[0, 0, j].double())) for j in range(i + 1)]
        z = sum(w)
        for j in range(i + 1):
            out[i] += (w[j] / z) * v[0, 0, j].double()
    assert rel_l2(o[0, :, 0, :], out) < 1e-5


def test_fixed_shift_equals_running_max():
    q, k, v = _qkv(2, T=128)
    q = torch.nn.functional.normalize(q.float(), dim=-1).bfloat16()   # the reference's fixed shift assumes bounded scores
    k = torch.nn.functional.normalize(k.float(), dim=-1).bfloat16()
    o1, l1 = O.forward(q, k, v, scale=1.0, shift="max")
    o2, l2 = O.forward(q, k, v, scale=1.0, shift=1.0)
    assert rel_l2(o1, o2) < 5e-3 and rel_l2(l1, l2) < 1e-3


def test_backward_matches_autograd_fp64():
    q, k, v = _qkv(3, T=128)
    g = torch.Generator().manual_seed(9)
    do = torch.randn(2, 128, 2, 64, generator=g).bfloat16()
    o, lse = O.forward(q, k, v)
    dq, dk, dv = O.backward(q, k, v, o, do, lse)
    qd, kd, vd = (t.double().requires_grad_(True) for t in (q, k, v))
    O.sdpa_reference(qd, kd, vd).backward(do.double())
    assert rel_l2(dq, qd.grad) < 1e-2 and rel_l2(dk, kd.grad) < 1e-2 and rel_l2(dv, vd.grad) < 1e-2


def test_causality_and_dv_column_sums():
    q, k, v = _qkv(4, B=1, H=1, T=128, dtype=torch.float32)
    o1, lse = O.forward(q, k, v)
    k2, v2 = k.clone(), v.clone()
    k2[..., 100:, :] += 3.0
    v2[..., 100:, :] -= 2.0
    o2, _ = O.forward(q, k2, v2)
    assert torch.equal(o1[:, :100], o2[:, :100])          # the past does not see the future
    do = torch.ones(1, 128, 1, 64)
    _, _, dv = O.backward(q, k, v, o1, do, lse)
    s = (q @ k.transpose(-1, -2)) / 8.0
    p = torch.softmax(s.masked_fill(~O.mask(128), float("-inf")), -1)
    assert rel_l2(dv[0, 0, :, 0], p[0, 0].sum(0)) < 1e-5   # dV with dO = 1: column sums of P
    assert torch.allclose(p.sum(-1), torch.ones(1, 1, 128), atol=1e-6)


def test_band_mask_keeps_last_tiles():
    m = O.mask(512, band_tiles=2)
    assert bool(m[300, 300]) and bool(m[300, 129]) and bool(m[300, 128]) and not bool(m[300, 127]) and not bool(m[300, 301])
    assert torch.equal(O.mask(256, band_tiles=2), O.mask(256))


def test_rope_is_a_rotation():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 64, 3, 64, generator=g)
    cos, sin = O.rope_tables(64, 64, dtype=torch.float32)
    y = O.rope(x, cos, sin)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), rtol=1e-5)           # norm preserving
    assert torch.allclose(O.rope_backward(y, cos, sin), x, atol=1e-5)           # the transpose is the inverse
    assert torch.equal(y[:, 0], x[:, 0])                                        # position 0 is the identity
    # relative-position property: <rope(q)_m, rope(k)_n> depends only on m - n
    q = torch.randn(1, 1, 1, 64, generator=g).expand(1, 64, 1, 64).contiguous()
    kk = torch.randn(1, 1, 1, 64, generator=g).expand(1, 64, 1, 64).contiguous()
    rq, rk = O.rope(q, cos, sin)[0, :, 0], O.rope(kk, cos, sin)[0, :, 0]
    d = rq @ rk.t()
    assert torch.allclose(d[10, 7], d[40, 37], atol=1e-4) and torch.allclose(d[5, 9], d[25, 29], atol=1e-4)
    xr = x.clone().requires_grad_(True)
    O.rope(xr, cos, sin).backward(y)
    assert torch.allclose(xr.grad, O.rope_backward(y, cos, sin), atol=1e-6)


def test_rope_norm_is_library_rms_norm_of_the_rotation_and_autograd():
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(6)
    B, T, H, D = 2, 64, 3, 64
    x = torch.randn(B, T, H, D, generator=g).bfloat16()
    cos, sin = O.rope_tables(T, D)
    y, r, inv = O.rope_norm(x, cos, sin)
    assert torch.equal(r, O.rope(x, cos, sin))
    # the library routine on the rounded rotation (fp32 in, the oracle's eps), one rounding
    assert torch.equal(y, F.rms_norm(r.float(), (D,), eps=O.QK_NORM_EPS).to(x.dtype))
    assert torch.allclose(y.float().pow(2).mean(-1), torch.ones(B, T, H), atol=2e-2)   # unit RMS per head
    assert torch.allclose(inv.squeeze(-1), 1.0 / r.float().pow(2).mean(-1).sqrt(), rtol=1e-5)
    # gradient: autograd of rms_norm(rope(x)) in fp64 (no intermediate roundings there)
    gy = torch.randn(B, T, H, D, generator=g).bfloat16()
    xd = x.double().requires_grad_(True)
    c, s = cos.double()[None, :, None, :], sin.double()[None, :, None, :]
    x1, x2 = xd[..., : D // 2], xd[..., D // 2:]
    rd = torch.cat((x1 * c + x2 * s, x2 * c - x1 * s), dim=-1)
    F.rms_norm(rd, (D,), eps=O.QK_NORM_EPS).backward(gy.double())
    dx = O.rope_norm_backward(gy, r, inv, cos, sin)
    assert rel_l2(dx, xd.grad) < 6e-3                                                   # bf16 roundings of r, gr, dx
    # the norm's Jacobian annihilates the radial direction: a gradient along y itself gives (almost) nothing
    dx_rad = O.rope_norm_backward(y, r, inv, cos, sin)
    assert float(dx_rad.float().abs().max()) < 2e-2 * float(dx.float().abs().max())
    # scale invariance: rope_norm(4 x) == rope_norm(x) bit for bit (powers of two commute with every rounding)
    assert torch.equal(O.rope_norm((x.float() * 4).bfloat16(), cos, sin, eps=O.QK_NORM_EPS * 16)[0], y)
