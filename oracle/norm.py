"""RMSNorm / residual-block oracle.

Restates R1:5165-5168 (eager block head: x_new = l1*x + l2*x0, norm(x_new)), R1:5594 (rmsnorm_fast),
R1:6106-6159 (head_skip / tail_norm2 / final_norm eager forms), R2:8805-8825 (nf_norm_rows and its
backward: upcast, rs = rsqrt(mean(x^2) + eps), one rounding per output; G = inv * (g - x * (g.x) * inv^2 / C)).
The optional per-channel weight and eps are configuration 1 of BASELINE.json's generalisation (reference: no weight, eps 2^-23).

Pinned by: torch.nn.functional.rms_norm (forward), torch.autograd on an fp64 restatement (backward),
the invariant that J^T(g) is orthogonal to x when weight is None.
"""
import torch

RMS_EPS = float(2.0 ** -23)


def rmsnorm(x, weight=None, eps=RMS_EPS):
    """(y, inv): y = dtype(x32 * rs * w32), inv = rs [rows] fp32."""
    xf = x.float()
    rs = torch.rsqrt(xf.square().mean(dim=-1, keepdim=True) + eps)
    y = xf * rs
    if weight is not None:
        y = y * weight.float()
    return y.to(x.dtype), rs.reshape(-1)


def rmsnorm_backward(gy, x, inv, weight=None):
    """(dx, dw): dx in x.dtype, dw fp32 [C] (None without weight). fp32 math, one rounding."""
    C = x.shape[-1]
    g = gy.float().reshape(-1, C)
    xf = x.float().reshape(-1, C)
    rs = inv.float().reshape(-1, 1)
    dw = None
    if weight is not None:
        dw = (g * xf * rs).sum(dim=0)
        g = g * weight.float()
    dot = (g * xf).sum(dim=-1, keepdim=True)
    dx = rs * (g - xf * (dot * rs * rs / C))
    return dx.reshape(x.shape), dw


def add_rmsnorm(x, res, weight=None, eps=RMS_EPS):
    """tail_norm2 / final_norm: s = dtype(x + res); (s, norm(s), inv)."""
    s = (x.float() + res.float()).to(x.dtype)
    y, inv = rmsnorm(s, weight, eps)
    return s, y, inv


def add_rmsnorm_backward(gs, gy, s, inv, weight=None):
    """Gradient wrt s (= wrt x = wrt res): gs + J^T(gy), rounded once; and dw."""
    dx, dw = rmsnorm_backward(gy, s, inv, weight)
    if gs is not None:
        dx = dx + gs.float()
    return dx.to(s.dtype), dw


def block_head(x, x0, l1, l2, skip=None, l3=None, eps=RMS_EPS):
    """x_new = dtype(l1*(x [+ l3*skip]) + l2*x0) in fp32 from fp32 gains (the skip joins the stream BEFORE the block
    head: round1/source/train.py:5644-5647 eager form, kernel 5743-5744); x_norm = norm(x_new); inv."""
    s = x.float()
    if skip is not None:
        s = s + l3.float() * skip.float()
    v = l1.float() * s + l2.float() * x0.float()
    x_new = v.to(x.dtype)
    x_norm, inv = rmsnorm(x_new, None, eps)
    return x_new, x_norm, inv


def block_head_backward(g_new, g_norm, x, x0, x_new, inv, l1, l2, skip=None, l3=None):
    """(dx, dx0, dskip, dl1, dl2, dl3) with G = g_new + J^T(g_norm): dx = l1 G, dx0 = l2 G, dskip = l1 l3 G; gain
    grads fp32 sums G.(x + l3 skip), G.x0, l1 G.skip (round1/source/train.py:5794-5795)."""
    jt, _ = rmsnorm_backward(g_norm, x_new, inv, None)
    G = jt if g_new is None else jt + g_new.float()
    dt = x.dtype
    dx = (l1.float() * G).to(dt)
    dx0 = (l2.float() * G).to(dt)
    dl2 = (G * x0.float()).sum()
    if skip is None:
        return dx, dx0, None, (G * x.float()).sum(), dl2, None
    gs = (G * skip.float()).sum()
    return dx, dx0, (l1.float() * l3.float() * G).to(dt), (G * x.float()).sum() + l3.float() * gs, dl2, l1.float() * gs


def relu2(x):
    """R1:663 relu_squared: relu(x)^2 computed in fp32, one rounding."""
    r = torch.relu(x.float())
    return (r * r).to(x.dtype)


def relu2_backward(x, gy):
    """R1:597: gy * 2 * relu(x), one rounding."""
    return (gy.float() * 2.0 * torch.relu(x.float())).to(x.dtype)


def relu2_backward_from_h(h, dh):
    """R1:625-631: dtype(dtype(sqrt(4 h)) * dh): the gradient from the saved output h = relu(x)^2."""
    root = torch.sqrt(4.0 * h.float()).to(h.dtype)
    return (root.float() * dh.float()).to(h.dtype)


def resmix_backward(g, x, x0, a, b):
    """K/nki_resmix.py:148-162: x_new = a*x + b*x0 backward in one pass: dx = g*a, dx0 = g*b (gains rounded to
    the stream dtype as the eager chain does), gain grads = fp32 sums of the dtype-rounded products."""
    dt = g.dtype
    ad, bd = a.to(dt), b.to(dt)
    dx = g * ad
    dx0 = g * bd
    da = (g * x).float().sum()
    db = (g * x0).float().sum()
    return dx, dx0, da, db


def shift1(x):
    """[B, T, C]: token t reads token t - 1 of its sequence, token 0 zeros (round1/source/train.py:300)."""
    return torch.cat([torch.zeros_like(x[:, :1]), x[:, :-1]], dim=1)


def mix_tail(x, lam, eps=2.0 ** -23):
    """(s1, xn2, inv) for x [B, T, C] bf16: s1 = bf16(x + bf16(lam shift1(x))), xn2 = RMSNorm(s1) without weight
    (round1/source/train.py:7098 docstring; the unfused chain :7275-7278)."""
    dt = x.dtype
    mix = (float(lam) * shift1(x).float()).to(dt)
    s1 = (x.float() + mix.float()).to(dt)
    sf = s1.float()
    inv = torch.rsqrt((sf * sf).mean(dim=-1) + eps)
    return s1, (sf * inv[..., None]).to(dt), inv


def mix_tail_backward(x, s1, inv, lam, gy, ge):
    """(gx, dlam fp32): g = bf16(ge + inv (gy - s1 (gy . s1) inv^2 / C)) (the tail norm's backward, one rounding),
    gx[t] = bf16(g[t] + bf16(lam g[t + 1])) (zero past a sequence's end), dlam = the fp32 sum of the bf16 products
    bf16(g shift1(x)) (round1/source/train.py:7041 _g_rows, :7146 docstring)."""
    dt = x.dtype
    C = x.shape[-1]
    sf = s1.float()
    g = torch.zeros_like(sf)
    if gy is not None:
        gyf = gy.float()
        dot = (gyf * sf).sum(dim=-1, keepdim=True)
        iv = inv[..., None]
        g = iv * (gyf - sf * (dot * iv * iv * (1.0 / C)))
    if ge is not None:
        g = g + ge.float()
    g = g.to(dt)
    nxt = torch.cat([g[:, 1:], torch.zeros_like(g[:, :1])], dim=1)
    gx = (g.float() + (float(lam) * nxt.float()).to(dt).float()).to(dt)
    dlam = (g.float() * shift1(x).float()).to(dt).float().sum()
    return gx, dlam
