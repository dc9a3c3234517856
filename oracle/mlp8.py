"""fp8 fused MLP oracle (up-projection -> ReLU^2 -> down-projection, e4m3 forward / e5m2 gradients,
per-tensor power-of-two scales).

Restates K/nki_mlp_fused8.py: constants :97-114, the greedy power-of-two / power-of-four scale searches
:742-779, forward_scales :782-800, backward_scales :803-813, the fp8 rounding q8 :821-825,
emulate8_forward :828-839, emulate8_backward :842-858, the bf16 kernels' arithmetic :684-703, the weight
gradients :706-711, and K/nki_dw8.py:323-333 (fp8 weight gradient). R1's off-device form of the same MLP is
plain bf16 relu(x @ w)^2 (R1:2128-2133), which is `reference_forward` here.

Pinned by (tests/test_oracle_mlp8.py): the scale search against the closed form 2^floor(log2(limit / v))
clipped to the exponent window by brute force over exponents and mantissas; s * (1/s) == 1; every e4m3 value up
to 240 surviving a bf16 round trip; the fp8 cast against an independent bit-level rounding routine; the fp8
MLP against the bf16 MLP within the fp8 error budget; weight gradients against torch.autograd of the bf16 form; the
fp8 weight gradients against an independent route (operands decoded byte by byte through the format tables, one
fp64 matmul), against the bf16 weight gradients within the fp8 budget, and by exact invariance under power-of-two
rescaling of the operands.
"""
import torch

E4M3_LIMIT_REF = 240.0     # the reference's fp8 format tops out at 240; OCP e4m3fn at 448
E4M3_LIMIT_OCP = 448.0
E5M2_LIMIT = 57344.0
X_SCALE = 4.0
H_CLAMP = 15.375
H_BOUND = 1.3
DY_HEADROOM = 2.0
DP_BOUND = 36.16
EXP_W = (-24, 40)
EXP_H = (-16, 8)
EXP_G = (-40, 60)

COLS = ("s_wfc", "dq_fc", "c_h", "s_wproj", "dq_proj", "s_dy", "dq_dh2", "s_dp", "dq_dx", "rho2", "kappa2", "i_wfc",
        "i_wproj", "s_h", "amax_wfc", "amax_wproj")
COL = {n: i for i, n in enumerate(COLS)}
NSC = len(COLS)


def pow2_floor_scale(v, limit, e_lo, e_hi):
    """(s, 1/s) with s = 2^e, e the largest integer in [e_lo, e_hi] such that v * s <= limit, found with the
    reference's bitwise search (only comparisons and exact power-of-two products). v >= 0 fp32 tensor."""
    v = v.float()
    s = torch.full_like(v, 2.0 ** e_lo)
    r = torch.full_like(v, 2.0 ** (-e_lo))
    room = e_hi - e_lo
    step = 64
    while step >= 1:
        if step <= room:
            trial = s * (2.0 ** step)
            take = (v * trial <= limit) & (trial <= 2.0 ** e_hi)
            s = torch.where(take, trial, s)
            r = torch.where(take, r * (2.0 ** -step), r)
        step //= 2
    return s, r


def pow4_floor_scale(v, limit, e_lo, e_hi):
    """(s, 1/s, c, 1/c) with s = 4^e (c = 2^e), e the largest integer in [e_lo, e_hi] with v * s <= limit."""
    v = v.float()
    s = torch.full_like(v, 4.0 ** e_lo)
    r = torch.full_like(v, 4.0 ** (-e_lo))
    c = torch.full_like(v, 2.0 ** e_lo)
    rc = torch.full_like(v, 2.0 ** (-e_lo))
    room = e_hi - e_lo
    step = 32
    while step >= 1:
        if step <= room:
            trial = s * (4.0 ** step)
            take = (v * trial <= limit) & (trial <= 4.0 ** e_hi)
            s = torch.where(take, trial, s)
            r = torch.where(take, r * (4.0 ** -step), r)
            c = torch.where(take, c * (2.0 ** step), c)
            rc = torch.where(take, rc * (2.0 ** -step), rc)
        step //= 2
    return s, r, c, rc


def forward_scales(w_fc, w_proj, e4m3_limit=E4M3_LIMIT_REF, x_scale=X_SCALE):
    """The layer's 16-float scale row from its weights (w_fc [F, d], w_proj [d, F]) as bf16 values."""
    a = w_fc.detach().to(torch.bfloat16).float()
    b = w_proj.detach().to(torch.bfloat16).float()
    amax_a, amax_b = a.abs().amax(), b.abs().amax()
    s_a, i_a = pow2_floor_scale(amax_a, e4m3_limit, *EXP_W)
    s_b, i_b = pow2_floor_scale(amax_b, e4m3_limit, *EXP_W)
    rho2 = (a * a).sum(dim=1).amax()       # largest squared row norm of w_fc
    kappa2 = (b * b).sum(dim=0).amax()     # largest squared column norm of w_proj
    s_h, i_h, c_h, _ = pow4_floor_scale(rho2 * (H_BOUND * w_fc.shape[1]), e4m3_limit, *EXP_H)
    z = torch.zeros_like(amax_a)
    return torch.stack([s_a, i_a * (1.0 / x_scale), c_h, s_b, i_h * i_b, z, z, z, z, rho2, kappa2, i_a, i_b, s_h,
                        amax_a, amax_b])


def backward_scales(dy2, row, amax=None):
    """The backward call's row: the forward row with s_dy, dq_dh2, s_dp, dq_dx filled from this call's dy (from a given
    amax instead when the caller holds only part of the rows the scales are taken over)."""
    amax = dy2.detach().abs().amax().float() if amax is None else torch.as_tensor(amax, dtype=torch.float32)
    s_dy, i_dy = pow2_floor_scale(amax, E5M2_LIMIT / DY_HEADROOM, *EXP_G)
    bound = torch.sqrt(row[COL["rho2"]] * row[COL["kappa2"]]) * amax * (DP_BOUND * dy2.shape[1])
    s_dp, i_dp = pow2_floor_scale(bound, E5M2_LIMIT, *EXP_G)
    out = row.clone()
    out[COL["s_dy"]] = s_dy
    out[COL["dq_dh2"]] = i_dy * row[COL["i_wproj"]] * 2.0
    out[COL["s_dp"]] = s_dp
    out[COL["dq_dx"]] = i_dp * row[COL["i_wfc"]]
    return out


def fp8_round(t, fmt):
    """fp32 values of t rounded (nearest even) to e4m3 (fmt 0) or e5m2 (fmt 1)."""
    return t.float().to(torch.float8_e5m2 if fmt == 1 else torch.float8_e4m3fn).float()


def fp8_bytes(t, fmt):
    return t.float().to(torch.float8_e5m2 if fmt == 1 else torch.float8_e4m3fn).view(torch.uint8)


def forward(x2, w_fc, w_proj, row, x_scale=X_SCALE):
    """(y [M, d], r [M, F]) in x2's dtype: the fp8 forward with the kernel's rounding points. r is what the
    backward needs (the reference saves its transpose)."""
    dt = x2.dtype
    x8 = fp8_round(x2.float() * x_scale, 0)
    a8 = fp8_round(w_fc.float() * row[COL["s_wfc"]], 0)
    r = torch.clamp_min((x8 @ a8.t()) * row[COL["dq_fc"]], 0.0).to(dt)
    rc = torch.clamp_max(r.float() * row[COL["c_h"]], H_CLAMP).to(dt)
    h8 = fp8_round(rc.float() * rc.float(), 0)
    b8 = fp8_round(w_proj.float() * row[COL["s_wproj"]], 0)
    y = ((h8 @ b8.t()) * row[COL["dq_proj"]]).to(dt)
    return y, r


def backward(dy2, r, w_fc, w_proj, row):
    """(dx [M, d], h [M, F], dpre [M, F]) in dy2's dtype: the fp8 backward; row from backward_scales."""
    dt = dy2.dtype
    g8 = fp8_round(dy2.float() * row[COL["s_dy"]], 1)
    b8 = fp8_round(w_proj.float() * row[COL["s_wproj"]], 0)
    rf = r.float()
    dpre = (((g8 @ b8) * row[COL["dq_dh2"]]) * rf).to(dt)
    h = (rf * rf).to(dt)
    p8 = fp8_round(dpre.float() * row[COL["s_dp"]], 1)
    a8 = fp8_round(w_fc.float() * row[COL["s_wfc"]], 0)
    dx = ((p8 @ a8) * row[COL["dq_dx"]]).to(dt)
    return dx, h, dpre


def weight_grads(dy2, x2, h, dpre):
    """(dw_fc [F, d], dw_proj [d, F]): the bf16 weight gradients from the backward's bf16 h and dpre."""
    dw_fc = (dpre.float().t() @ x2.float()).to(x2.dtype)
    dw_proj = (dy2.float().t() @ h.float()).to(x2.dtype)
    return dw_fc, dw_proj


def forward_bf16(x2, w_fc, w_proj):
    """The bf16 fused MLP's arithmetic (K/nki_mlp_fused.py:684-691): (y, r)."""
    dt = x2.dtype
    r = torch.relu(x2.float() @ w_fc.float().t()).to(dt)
    h = (r.float() * r.float()).to(dt)
    return (h.float() @ w_proj.float().t()).to(dt), r


def backward_bf16(dy2, r, w_fc, w_proj):
    """(dx, h, dpre) of the bf16 fused MLP (K/nki_mlp_fused.py:694-703)."""
    dt = dy2.dtype
    rf = r.float()
    dpre = (((dy2.float() @ w_proj.float()) * 2.0) * rf).to(dt)
    h = (rf * rf).to(dt)
    dx = (dpre.float() @ w_fc.float()).to(dt)
    return dx, h, dpre


def reference_forward(x2, w_fc, w_proj):
    """The plain expression both rounds fall back to off-device: c_proj(relu(c_fc(x))^2) in bf16."""
    F = torch.nn.functional
    return F.linear(torch.relu(F.linear(x2, w_fc)).square(), w_proj)


def fp8_weight_grad(g2, a2, s_g, s_a, dq, fmt_g, fmt_a, clamp_g=None):
    """K/nki_dw8.py:323: out [O, D] = dtype((fp8(g2 s_g)^T @ fp8(a2 s_a)) dq)."""
    g = g2.float() * s_g
    if clamp_g is not None:
        g = torch.clamp_max(g, clamp_g)
    return ((fp8_round(g, fmt_g).t() @ fp8_round(a2.float() * s_a, fmt_a)) * dq).to(g2.dtype)


def weight_grads_fp8(x2, dy2, h, dpre, row, x_scale=X_SCALE, e4m3_limit=E4M3_LIMIT_REF):
    """(dw_fc [F, d], dw_proj [d, F]) in fp8 (round2/source/train.py:8209-8229 mlp8_weight_grads under its fp8
    weight-gradient switch): dw_fc = dpre^T x with dpre e5m2 at s_dp (the bytes the backward's second GEMM
    multiplies) and x e4m3 at x_scale (the forward's), dw_proj = (h^T dy)^T with h e4m3 at s_h clamped at the format's
    limit and dy e5m2 at s_dy; descales are the exact inverse powers of two. row = the backward row."""
    s_dp, s_h, s_dy = row[COL["s_dp"]], row[COL["s_h"]], row[COL["s_dy"]]
    dw_fc = fp8_weight_grad(dpre, x2, s_dp, x_scale, 1.0 / (s_dp * x_scale), 1, 0)
    dw_pt = fp8_weight_grad(h, dy2, s_h, s_dy, 1.0 / (s_h * s_dy), 0, 1, clamp_g=e4m3_limit)
    return dw_fc, dw_pt.t().contiguous()

