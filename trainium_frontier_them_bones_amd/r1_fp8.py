"""The fp8 MLP recipe of the reference's round1 sources: six GEMM "rows" with FIXED power-of-two scales, in the reference's call style
(round1/source/train.py: nki_gemm_fp8 1780-2265 = row 1, nki_gemm_fp8_nn 2269-4140 = rows 2-6).

    row 1  c_fc forward    x [M, d] @ W1 [d, F]        x e4m3 @ 4        W1 e4m3 @ 64      (1758-1759)
    row 2  c_proj forward  h [M, F] @ W2^T, W2 [d, F]  h e4m3 @ 1/128    W2 e4m3 @ 16      (ROW_SPEC, 2300)
    row 3  c_fc dX         dpre [M, F] @ W1^T          dpre e5m2 @ 2^30  W1 e4m3 @ 128
    row 4  c_proj dX       dy [M, d] @ W2              dy e5m2 @ 2^30    W2 e4m3 @ 16
    row 5  c_fc dW         x^T @ dpre -> [d, F]        x e4m3 @ 16       dpre e5m2 @ 2^30
    row 6  c_proj dW       dy^T @ h -> [d, F]          dy e5m2 @ 2^30    h e4m3 @ 1/128

Every operand is clamped in the unscaled bf16 domain at the largest bf16 b with b * scale <= the format's maximum
(240 for the reference chip's e4m3, 57344 for e5m2: clip_bound, 2272), multiplied by its scale (exact), rounded once
to fp8; products are exact in fp32, accumulation is fp32, the result is descaled by the exact 1 / (s_a s_b) and
rounded once to bf16. W1 is LinearT [in, out], W2 is [out, in] (2169, 3728). inplace=True sums the weight gradient into
an existing w.grad and returns None for it (3718-3723, 4050-4055). The fp8 copies of a weight are made once per
optimizer step: begin_step() starts a new step (2059, 3247).
"""
import math

import torch

from . import ops
from ._lib import TfbError

bf16 = torch.bfloat16
E4M3_MAX, E5M2_MAX = 240.0, 57344.0
A_SCALE, W_SCALE = 4.0, 64.0                       # row 1
H_SCALE, G_SCALE = 0.0078125, 1073741824.0         # 1 / 128, 2^30
W_SCALE_FC, W_SCALE_PROJ, A_SCALE_DW = 128.0, 16.0, 16.0
ROW_SPEC = {
    1: dict(afmt=0, ascale=A_SCALE, wscale=W_SCALE, trans_b=False),
    2: dict(afmt=0, ascale=H_SCALE, wscale=W_SCALE_PROJ, trans_b=True),
    3: dict(afmt=1, ascale=G_SCALE, wscale=W_SCALE_FC, trans_b=True),
    4: dict(afmt=1, ascale=G_SCALE, wscale=W_SCALE_PROJ, trans_b=False),
    5: dict(afmt=0, ascale=A_SCALE_DW, bfmt=1, bscale=G_SCALE),
    6: dict(afmt=1, ascale=G_SCALE, bfmt=0, bscale=H_SCALE),
}
_FMT = {0: ops.FMT_E4M3, 1: ops.FMT_E5M2}


def clip_bound(scale, fmt=0):
    """The largest bf16 b with b * scale <= the format's maximum finite value (round1/source/train.py:2272)."""
    hi = E5M2_MAX if fmt == 1 else E4M3_MAX
    b = torch.tensor(hi / scale, dtype=torch.float32).to(bf16)
    for _ in range(4):
        if float(b) * scale <= hi:
            break
        b = torch.nextafter(b, torch.tensor(0.0, dtype=bf16))
    return float(b)


def quantise(a2d, scale, fmt):
    """fp8(clamp(a, -b, b) * scale) bytes of a bf16 matrix."""
    b = clip_bound(scale, fmt)
    return ops.quant_fp8(a2d.clamp(-b, b).contiguous(), float(scale), _FMT[fmt])


_EPOCH = [0]
_WCACHE = {}


def begin_step():
    """Once per optimizer step: the cached fp8 copies of the weights are made again on their next use (2059, 3247)."""
    _EPOCH[0] += 1
    _WCACHE.clear()


def active(training):
    """The fp8 rows run in training (the reference's evaluation mode keeps bf16, 2043, 3206)."""
    return bool(training)


def quantised_weight(w, scale, transposed):
    """e4m3(clamp(w) * scale) bytes of a weight in its own layout or transposed, cached for the step and invalidated
    when the parameter is written (keys: step epoch, data_ptr, _version: 2065-2103, 3265)."""
    key = (_EPOCH[0], w.data_ptr(), w._version, float(scale))
    hit = _WCACHE.get(key)
    if hit is None:
        b = clip_bound(scale, 0)
        s = torch.tensor([float(scale)], dtype=torch.float32, device=w.device)
        hit = _WCACHE[key] = ops.precast8(w.detach().clamp(-b, b).contiguous(), s)
    return hit[1] if transposed else hit[0]


def _usable(*ts):
    return all(t.is_cuda and t.dtype == bf16 and t.dim() == 2 for t in ts)


def row_matmul(a2d, w, row, key=None):
    """a2d @ (w.T if the row's trans_b else w) for rows 1-4 in fp8 (3412). Shapes the kernels do not take raise."""
    sp = ROW_SPEC[row]
    a8 = quantise(a2d.contiguous(), sp["ascale"], sp["afmt"])
    # the GEMM wants the weight as [N][K]: its own layout when the row multiplies by w.T, transposed otherwise
    w8 = quantised_weight(w if key is None else key, sp["wscale"], transposed=not sp["trans_b"])
    return ops.gemm_fp8(a8, w8, _FMT[sp["afmt"]], None, None, 1.0 / (sp["ascale"] * sp["wscale"]))


def dw_matmul(a2d, b2d, row, key=None):
    """a2d^T @ b2d [Ka, N] for rows 5 / 6 in fp8, or None = "not done, run your own line" when the operands are not the
    kernel's (3486-3493: not bf16 device matrices, or a shape it does not take)."""
    if row not in (5, 6) or not _usable(a2d, b2d) or a2d.shape[0] != b2d.shape[0]:
        return None
    sp = ROW_SPEC[row]
    a8 = quantise(a2d.contiguous(), sp["ascale"], sp["afmt"])
    b8 = quantise(b2d.contiguous(), sp["bscale"], sp["bfmt"])
    try:
        return ops.gemm_fp8_tn(a8, b8, _FMT[sp["afmt"]], _FMT[sp["bfmt"]], None, None, 1.0 / (sp["ascale"] * sp["bscale"]))
    except TfbError as e:
        if e.status == 1:
            return None
        raise


def _grad_into(w, dw, inplace):
    """The reference's weight-gradient convention: summed into an existing w.grad (None returned) or returned."""
    if inplace and w.grad is not None:
        w.grad.add_(dw.to(w.grad.dtype))
        return None
    return dw


class FcRelu2NNFn(torch.autograd.Function):
    """h = relu(x @ W1)^2: row 1 forward, ReLU^2 backward on the saved bf16 pre, row 3 dX, row 5 dW (4019-4095)."""

    @staticmethod
    def forward(ctx, x2d, w, inplace):
        pre = row_matmul(x2d, w, 1)
        ctx.save_for_backward(x2d, w, pre)
        ctx.inplace = bool(inplace)
        return ops.relu2(pre)

    @staticmethod
    def backward(ctx, dh):
        x2d, w, pre = ctx.saved_tensors
        dpre = ops.relu2_bwd(pre, dh.contiguous())
        dx = row_matmul(dpre, w, 3)
        dw = dw_matmul(x2d, dpre, 5)
        if dw is None:
            dw = ops.matmul(x2d, dpre, trans_a=True)
        return dx, _grad_into(w, dw, ctx.inplace), None


class ProjFn(torch.autograd.Function):
    """y = h @ W2^T: row 2 forward, row 4 dX, row 6 dW (3666-3726)."""

    @staticmethod
    def forward(ctx, h2d, w, inplace):
        ctx.save_for_backward(h2d, w)
        ctx.inplace = bool(inplace)
        return row_matmul(h2d, w, 2)

    @staticmethod
    def backward(ctx, dy):
        h2d, w = ctx.saved_tensors
        dy2d = dy.contiguous()
        dh = row_matmul(dy2d, w, 4)
        dw = dw_matmul(dy2d, h2d, 6)
        if dw is None:
            dw = ops.matmul(dy2d, h2d, trans_a=True)
        return dh, _grad_into(w, dw, ctx.inplace), None


def fused_fc_relu2_nn(x, w, inplace=False):
    """relu(x @ w)^2 for any leading shape, w [in, out] (4097; the same call as nki_gemm_fp8.fused_fc_relu2_fp8, 2169)."""
    x2d = x.reshape(-1, x.shape[-1]).contiguous()
    return FcRelu2NNFn.apply(x2d, w, inplace).view(*x.shape[:-1], w.shape[1])


fused_fc_relu2_fp8 = fused_fc_relu2_nn


def c_proj(x, w, inplace):
    """x @ w^T for any leading shape, w [out, in] (3728)."""
    x2d = x.reshape(-1, x.shape[-1]).contiguous()
    return ProjFn.apply(x2d, w, inplace).view(*x.shape[:-1], w.shape[0])


class _Namespace:
    """The reference uses its modules as namespaces (nki_gemm_fp8.begin_step(), nki_gemm_fp8_nn.c_proj(...))."""

    def __init__(self, **kw):
        self.__dict__.update(kw)


nki_gemm_fp8 = _Namespace(begin_step=begin_step, active=active, fused_fc_relu2_fp8=fused_fc_relu2_fp8,
                          quantised_weight=quantised_weight, clip_bound=clip_bound, A_SCALE=A_SCALE, W_SCALE=W_SCALE)
nki_gemm_fp8_nn = _Namespace(begin_step=begin_step, active=active, c_proj=c_proj, fused_fc_relu2_nn=fused_fc_relu2_nn,
                             row_matmul=row_matmul, dw_matmul=dw_matmul, clip_bound=clip_bound, ROW_SPEC=ROW_SPEC)
