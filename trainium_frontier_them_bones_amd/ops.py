"""Functional layer over the C-ABI: torch tensors in, torch tensors out, one HIP launch (or a
short fixed sequence of launches) per call on torch's current stream. No autograd here (see
autograd.py) and no fallbacks: every function requires CUDA(ROCm) tensors and the built
library. torch supplies device memory and the stream; all arithmetic is in the HIP kernels.
"""
import torch

from . import _lib

bf16 = torch.bfloat16


def _p(t):
    return None if t is None else t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _chk(t, dtype=bf16):
    if t is None:
        return
    if not t.is_cuda:
        raise RuntimeError("tfb ops need device tensors (the HIP kernels are the only implementation)")
    if t.dtype != dtype:
        raise TypeError("expected %s, got %s" % (dtype, t.dtype))
    if not t.is_contiguous():
        raise RuntimeError("tensor must be contiguous")


# ------------------------------------------------------------------------------------------ GEMM
_WS = {}


def _workspace(device, nbytes=256 << 20):
    """One fp32 split-K workspace per (device, stream), allocated on first use: launches on different streams would
    otherwise race on the same partial sums."""
    key = (device, torch.cuda.current_stream(device).cuda_stream)
    ws = _WS.get(key)
    if ws is None or ws.numel() * 4 < nbytes:
        ws = torch.empty(nbytes // 4, dtype=torch.float32, device=device)
        _WS[key] = ws
    return ws


def matmul(a, b, trans_a=False, trans_b=False, out=None, accumulate=False, out_dtype=bf16, alpha=None):
    """op(a) @ op(b) with fp32 accumulation. a is [M,K] (or [K,M] with trans_a), b is [K,N] (or [N,K] with
    trans_b). `out` (bf16 or fp32) may be given; accumulate=True adds into it (one rounding). alpha: a 1-element fp32
    device tensor the product is multiplied by before that rounding (no host read-back)."""
    _chk(a), _chk(b), _chk(alpha, torch.float32)
    if alpha is not None and alpha.numel() != 1:
        raise ValueError("alpha is one fp32 element")
    M, K = (a.shape[1], a.shape[0]) if trans_a else (a.shape[0], a.shape[1])
    Kb, N = (b.shape[1], b.shape[0]) if trans_b else (b.shape[0], b.shape[1])
    if K != Kb:
        raise ValueError("inner dimensions differ: %d vs %d" % (K, Kb))
    if out is None:
        if accumulate:
            raise ValueError("accumulate needs out")
        out = torch.empty(M, N, dtype=out_dtype, device=a.device)
    else:
        _chk(out, out.dtype)
        if out.dtype not in (bf16, torch.float32) or tuple(out.shape) != (M, N):
            raise ValueError("bad out")
    ws = _workspace(a.device)
    if alpha is None:
        _lib.call("tfb_gemm_bf16", _p(a), _p(b), _p(out), M, N, K, int(trans_a), int(trans_b),
                  int(out.dtype == torch.float32), int(accumulate), _p(ws), ws.numel() * 4, _stream())
    else:
        _lib.call("tfb_gemm_bf16_scaled", _p(a), _p(b), _p(out), M, N, K, int(trans_a), int(trans_b),
                  int(out.dtype == torch.float32), int(accumulate), _p(ws), ws.numel() * 4, _p(alpha), _stream())
    return out


def matmul_res(a, b, res, trans_b=False):
    """bf16(res + bf16(a @ op(b))): a projection with the residual add that follows it made in the GEMM's store (equal to
    matmul followed by a bf16 add, bit for bit). a [M,K]; b [K,N] or, with trans_b, [N,K]; res [M,N]."""
    _chk(a), _chk(b), _chk(res)
    M, K = a.shape
    Kb, N = (b.shape[1], b.shape[0]) if trans_b else (b.shape[0], b.shape[1])
    if K != Kb or tuple(res.shape) != (M, N):
        raise ValueError("shapes differ")
    out = torch.empty(M, N, dtype=bf16, device=a.device)
    _lib.call("tfb_gemm_bf16_res", _p(a), _p(b), _p(res), _p(out), M, N, K, int(trans_b), _stream())
    return out


def qkv_rope(x2, w, cos, sin, T, rot_cols):
    """rope(x2 @ w^T): the fused attention projection [M, N] with the rotary embedding of its first rot_cols columns
    (heads of 64) applied in the GEMM epilogue; row m is token m % T."""
    _chk(x2), _chk(w), _chk(cos), _chk(sin)
    M, K = x2.shape
    N = w.shape[0]
    out = torch.empty(M, N, dtype=bf16, device=x2.device)
    _lib.call("tfb_qkv_rope_fwd", _p(x2), _p(w), _p(cos), _p(sin), _p(out), M, N, K, T, rot_cols, _stream())
    return out


# ------------------------------------------------------------------------------------------ norms
def rmsnorm_fwd(x, weight=None, eps=2.0 ** -23, res=None):
    """y = RMSNorm(s) * weight with s = x (res None) or bf16(x + res). Returns (s, y, inv[rows] fp32)."""
    _chk(x), _chk(res), _chk(weight)
    C = x.shape[-1]
    rows = x.numel() // C
    y = torch.empty_like(x)
    s = torch.empty_like(x) if res is not None else x
    inv = torch.empty(rows, dtype=torch.float32, device=x.device)
    _lib.call("tfb_rmsnorm_fwd", _p(x), _p(res), _p(weight), _p(s) if res is not None else None, _p(y), _p(inv),
              rows, C, float(eps), _stream())
    return s, y, inv


def rmsnorm_fwd_q(x, weight=None, eps=2.0 ** -23, res=None, y8_scale=4.0, want_y=True):
    """rmsnorm_fwd that also returns y8 = e4m3(bf16(y) * y8_scale) bytes, the operand cast of the fp8 GEMM that consumes y
    (equal to quant_fp8(y, y8_scale), bit for bit). Returns (s, y, inv, y8); want_y False: the bf16 rows are not written and
    y is None (for a consumer that reads only the bytes)."""
    _chk(x), _chk(res), _chk(weight)
    C = x.shape[-1]
    rows = x.numel() // C
    y = torch.empty_like(x) if want_y else None
    s = torch.empty_like(x) if res is not None else x
    inv = torch.empty(rows, dtype=torch.float32, device=x.device)
    y8 = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    _lib.call("tfb_rmsnorm_fwd_q", _p(x), _p(res), _p(weight), _p(s) if res is not None else None, _p(y), _p(inv), _p(y8),
              float(y8_scale), rows, C, float(eps), _stream())
    return s, y, inv, y8


def rmsnorm_bwd(gy, s, inv, weight=None, gs=None, dw=None, accumulate=False, part=None, want_amax=False):
    """dx = gs + J^T(gy) for y = RMSNorm(s) * weight. Returns (dx, dw fp32 [C] or None); a given dw is written, or
    added into with accumulate=True. With `part` (fp32 [tfb_norm_bwd_blocks(rows), C]) the weight gradient is left there
    as partial sums for norm_dw_finish and None is returned for it. want_amax: a third value, fp32 [tfb_norm_bwd_blocks(rows)]
    whose maximum is amax(dx) (per-workgroup partials, for mlp8_backward_scales(..., amax_part=))."""
    _chk(gy), _chk(s), _chk(weight), _chk(gs), _chk(inv, torch.float32)
    C = s.shape[-1]
    rows = s.numel() // C
    dx = torch.empty_like(s)
    acc = 0
    am = torch.empty(_lib.lib().tfb_norm_bwd_blocks(rows), dtype=torch.float32, device=s.device) if want_amax else None

    def call(part_, dw_, acc_):
        if want_amax:
            _lib.call("tfb_rmsnorm_bwd_amax", _p(gy), _p(gs), _p(s), _p(weight), _p(inv), _p(dx), _p(part_), _p(dw_), acc_, _p(am),
                      rows, C, _stream())
        else:
            _lib.call("tfb_rmsnorm_bwd", _p(gy), _p(gs), _p(s), _p(weight), _p(inv), _p(dx), _p(part_), _p(dw_), acc_, rows, C,
                      _stream())

    if weight is not None and part is not None:
        _chk(part, torch.float32)
        call(part, None, 0)
        return (dx, None, am) if want_amax else (dx, None)
    if weight is not None:
        nb = _lib.lib().tfb_norm_bwd_blocks(rows)
        part = torch.empty(nb, C, dtype=torch.float32, device=s.device)
        if dw is None:
            dw = torch.empty(C, dtype=torch.float32, device=s.device)
        else:
            _chk(dw, torch.float32)
            acc = int(accumulate)
    call(part, dw, acc)
    return (dx, dw, am) if want_amax else (dx, dw)


def norm_bwd_blocks(rows):
    return int(_lib.lib().tfb_norm_bwd_blocks(rows))


def norm_dw_finish(parts, dw, rows, accumulate=False):
    """dw [count, C] fp32 (+)= the weight gradients whose partial sums rmsnorm_bwd(part=parts[i]) left in parts
    [count, blocks, C]: one launch for all of them."""
    _chk(parts, torch.float32), _chk(dw, torch.float32)
    count, nb, C = parts.shape
    if tuple(dw.shape) != (count, C) or nb != norm_bwd_blocks(rows):
        raise ValueError("parts [count, blocks, C], dw [count, C]")
    _lib.call("tfb_norm_dw_finish", _p(parts), _p(dw), count, nb * C, C, int(accumulate), rows, C, _stream())
    return dw


def block_head_fwd(x, x0, gains, skip=None, eps=2.0 ** -23):
    """x_new = l1*x + l2*x0 (+ l3*skip), x_norm = RMSNorm(x_new). gains: fp32 device tensor [3]."""
    _chk(x), _chk(x0), _chk(skip), _chk(gains, torch.float32)
    C = x.shape[-1]
    rows = x.numel() // C
    x_new = torch.empty_like(x)
    x_norm = torch.empty_like(x)
    inv = torch.empty(rows, dtype=torch.float32, device=x.device)
    _lib.call("tfb_block_head_fwd", _p(x), _p(x0), _p(skip), _p(gains), _p(x_new), _p(x_norm), _p(inv), rows, C,
              float(eps), _stream())
    return x_new, x_norm, inv


def block_head_bwd(g_new, g_norm, x, x0, x_new, inv, gains, skip=None):
    """Returns (dx, dx0, dskip or None, dgains fp32 [4] = sum G.x, G.x0, G.skip, 0)."""
    _chk(g_new), _chk(g_norm), _chk(x), _chk(x0), _chk(skip), _chk(x_new)
    C = x.shape[-1]
    rows = x.numel() // C
    dx = torch.empty_like(x)
    dx0 = torch.empty_like(x)
    dskip = torch.empty_like(x) if skip is not None else None
    nb = _lib.lib().tfb_norm_bwd_blocks(rows)
    part = torch.empty(nb, 4, dtype=torch.float32, device=x.device)
    dg = torch.empty(4, dtype=torch.float32, device=x.device)
    _lib.call("tfb_block_head_bwd", _p(g_new), _p(g_norm), _p(x), _p(x0), _p(skip), _p(x_new), _p(inv), _p(gains),
              _p(dx), _p(dx0), _p(dskip), _p(part), _p(dg), rows, C, _stream())
    return dx, dx0, dskip, dg


# ------------------------------------------------------------------------------------------ fp8 MLP
NSC = 16
FMT_E4M3, FMT_E5M2 = 0, 1
fp8_dtypes = (torch.float8_e4m3fn, torch.float8_e5m2)


def _scratch(device, nfloats):
    return torch.empty(nfloats, dtype=torch.float32, device=device)


def _scale_arg(x_scale):
    """(float, device pointer) for an activation scale given as a python float or as a 1-element fp32 device tensor."""
    if isinstance(x_scale, torch.Tensor):
        _chk(x_scale, torch.float32)
        if x_scale.numel() != 1:
            raise ValueError("a device activation scale is one fp32 element")
        return 0.0, _p(x_scale)
    return float(x_scale), None


def mlp8_forward_scales(w_fc, w_proj, e4m3_limit=240.0, x_scale=4.0):
    """The layer's fp32 [16] scale row, computed on the device from the bf16 weights (w_fc [F,d], w_proj [d,F]).
    x_scale: python float (the reference's constant 4) or a 1-element fp32 device tensor (no host synchronisation)."""
    _chk(w_fc), _chk(w_proj)
    F, d = w_fc.shape
    if tuple(w_proj.shape) != (d, F):
        raise ValueError("w_proj must be [d, F]")
    row = torch.empty(NSC, dtype=torch.float32, device=w_fc.device)
    scr = _scratch(w_fc.device, _lib.lib().tfb_mlp8_scale_scratch_floats(F))
    xf, xd = _scale_arg(x_scale)
    _lib.call("tfb_mlp8_forward_scales", _p(w_fc), _p(w_proj), _p(row), _p(scr), F, d, float(e4m3_limit), xf, xd, _stream())
    return row


def mlp8_refresh_layers(w_fc0, w_proj0, layer_stride, layers, e4m3_limit=240.0, x_scale=4.0, rows=None, w8=None):
    """Scale rows [layers, 16] and e4m3 packs [layers, 4, F*d] of `layers` MLPs whose weights share one flat buffer:
    layer i's w_fc [F, d] starts layer_stride elements after layer i-1's (w_fc0, w_proj0: layer 0's), likewise w_proj.
    Six launches whatever the layer count; rows / w8 may be given to be overwritten."""
    _chk(w_fc0), _chk(w_proj0)
    F, d = w_fc0.shape
    if tuple(w_proj0.shape) != (d, F):
        raise ValueError("w_proj must be [d, F]")
    dev = w_fc0.device
    if rows is None:
        rows = torch.empty(layers, NSC, dtype=torch.float32, device=dev)
    if w8 is None:
        w8 = torch.empty(layers, 4, F * d, dtype=torch.uint8, device=dev)
    _chk(rows, torch.float32), _chk(w8, torch.uint8)
    scr = _scratch(dev, layers * _lib.lib().tfb_mlp8_scale_scratch_floats(F))
    _lib.call("tfb_mlp8_refresh_layers", _p(w_fc0), _p(w_proj0), int(layer_stride), int(layers), _p(rows), _p(w8), _p(scr),
              F, d, float(e4m3_limit), float(x_scale), _stream())
    return rows, w8


def mlp8_backward_scales(dy2, row, amax_part=None):
    """The backward call's scale row from amax(dy2), or from amax_part (fp32 partials whose maximum is that amax, as
    rmsnorm_bwd(want_amax=True) leaves them for the dx it wrote) without reading dy2."""
    _chk(dy2), _chk(row, torch.float32), _chk(amax_part, torch.float32)
    M, d = dy2.shape
    out = torch.empty(NSC, dtype=torch.float32, device=dy2.device)
    if amax_part is not None:
        _lib.call("tfb_mlp8_backward_scales_part", _p(amax_part), amax_part.numel(), _p(row), _p(out), d, _stream())
        return out
    scr = _scratch(dy2.device, 4096)
    _lib.call("tfb_mlp8_backward_scales", _p(dy2), _p(row), _p(out), _p(scr), M, d, _stream())
    return out


def amax_scale(x, limit, e_lo, e_hi):
    """fp32 [3] = (s, 1/s, amax): s the largest power of two in [2^e_lo, 2^e_hi] with amax(x) * s <= limit."""
    _chk(x)
    out = torch.empty(3, dtype=torch.float32, device=x.device)
    scr = _scratch(x.device, 4096)
    _lib.call("tfb_amax_scale", _p(x), x.numel(), float(limit), int(e_lo), int(e_hi), _p(out), _p(scr), _stream())
    return out


def quant_fp8(x, scale, fmt=FMT_E4M3):
    """uint8-carried fp8 of x * scale; scale a python float or a 1-element fp32 device tensor (no host sync)."""
    _chk(x)
    out = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    if isinstance(scale, torch.Tensor):
        _chk(scale, torch.float32)
        _lib.call("tfb_quant_fp8", _p(x), _p(scale), 0.0, fmt, _p(out), x.numel(), _stream())
    else:
        _lib.call("tfb_quant_fp8", _p(x), None, float(scale), fmt, _p(out), x.numel(), _stream())
    return out


def precast8(w, scale):
    """(w8 [R,C], w8T [C,R]) uint8: e4m3(w * scale) in both byte layouts; scale a 1-element fp32 device tensor."""
    _chk(w), _chk(scale, torch.float32)
    R, C = w.shape
    w8 = torch.empty(R, C, dtype=torch.uint8, device=w.device)
    w8t = torch.empty(C, R, dtype=torch.uint8, device=w.device)
    _lib.call("tfb_precast8", _p(w), _p(scale), _p(w8), _p(w8t), R, C, _stream())
    return w8, w8t


def gemm_fp8(a8, b8, fmt_a=FMT_E4M3, dq_a=None, dq_b=None, dq=1.0):
    """bf16 [M,N] = (a8 [M,K] @ b8 [N,K]^T) * dq * dq_a * dq_b; a8 e4m3 or e5m2 bytes, b8 e4m3 bytes; dq_a, dq_b
    1-element fp32 device tensors (or None)."""
    _chk(a8, torch.uint8), _chk(b8, torch.uint8), _chk(dq_a, torch.float32), _chk(dq_b, torch.float32)
    M, K = a8.shape
    N = b8.shape[0]
    if b8.shape[1] != K:
        raise ValueError("inner dimensions differ")
    out = torch.empty(M, N, dtype=bf16, device=a8.device)
    _lib.call("tfb_gemm_fp8", _p(a8), int(fmt_a), _p(b8), _p(dq_a), _p(dq_b), float(dq), _p(out), M, N, K, _stream())
    return out


def gemm_fp8_res(a8, b8, res, dq_a=None, dq_b=None, dq=1.0):
    """bf16(res + bf16((a8 [M,K] @ b8 [N,K]^T) * dq * dq_a * dq_b)): gemm_fp8 (e4m3 activations) with the residual add
    in the store, equal to gemm_fp8 followed by a bf16 add bit for bit."""
    _chk(a8, torch.uint8), _chk(b8, torch.uint8), _chk(dq_a, torch.float32), _chk(dq_b, torch.float32), _chk(res)
    M, K = a8.shape
    N = b8.shape[0]
    if b8.shape[1] != K or tuple(res.shape) != (M, N):
        raise ValueError("shapes differ")
    out = torch.empty(M, N, dtype=bf16, device=a8.device)
    _lib.call("tfb_gemm_fp8_res", _p(a8), _p(b8), _p(dq_a), _p(dq_b), float(dq), _p(res), _p(out), M, N, K, _stream())
    return out


def gemm_fp8_tn(g8, a8, fmt_g=FMT_E5M2, fmt_a=FMT_E4M3, s_g=None, s_a=None, imm=1.0, out=None, accumulate=False,
                out_dtype=bf16):
    """[O,D] (+)= (g8 [M,O]^T @ a8 [M,D]) * imm / (s_g s_a): a weight gradient in fp8 (dw8_grad,
    round2/source/train.py:8185). s_g, s_a: 1-element fp32 device tensors (the scales the bytes were cast at) or None."""
    _chk(g8, torch.uint8), _chk(a8, torch.uint8), _chk(s_g, torch.float32), _chk(s_a, torch.float32)
    M, O = g8.shape
    D = a8.shape[1]
    if a8.shape[0] != M:
        raise ValueError("token counts differ")
    if out is None:
        if accumulate:
            raise ValueError("accumulate needs out")
        out = torch.empty(O, D, dtype=out_dtype, device=g8.device)
    else:
        _chk(out, out.dtype)
        if out.dtype not in (bf16, torch.float32) or tuple(out.shape) != (O, D):
            raise ValueError("bad out")
    ws = _workspace(g8.device)
    _lib.call("tfb_gemm_fp8_tn", _p(g8), int(fmt_g), _p(a8), int(fmt_a), _p(s_g), _p(s_a), float(imm), _p(out), M, O, D,
              int(out.dtype == torch.float32), int(accumulate), _p(ws), ws.numel() * 4, _stream())
    return out


def mlp8_precast(w_fc, w_proj, row):
    """uint8 [4, F*d]: w_fc and w_proj cast once to e4m3 at the row's scales, each in both byte layouts."""
    _chk(w_fc), _chk(w_proj), _chk(row, torch.float32)
    F, d = w_fc.shape
    w8 = torch.empty(4, F * d, dtype=torch.uint8, device=w_fc.device)
    _lib.call("tfb_mlp8_precast", _p(w_fc), _p(w_proj), _p(row), _p(w8), F, d, _stream())
    return w8


def mlp8_fwd(x2, w8, row, F, x_scale=4.0, want_x8=False, x8=None, res=None):
    """y [M,d], r [M,F] (bf16): the fp8 forward. x_scale: python float (the reference's constant 4) or a device scalar.
    want_x8 also returns x8 = e4m3(x x_scale) [M,d] bytes (the fp8 weight gradient's operand). A given x8 (from
    rmsnorm_fwd_q) is used instead of casting x2; with res [M,d], y = bf16(res + bf16(MLP(x))) (the block's residual add
    made in the second GEMM's store)."""
    _chk(x2), _chk(w8, torch.uint8), _chk(row, torch.float32), _chk(x8, torch.uint8), _chk(res)
    if x2 is None and x8 is None:
        raise ValueError("give x2 or its bytes x8")
    M, d = x2.shape if x2 is not None else x8.shape      # x2 may be left out when its bytes are given
    dev = w8.device
    if x8 is None:
        x8 = quant_fp8(x2, x_scale, FMT_E4M3)
    elif tuple(x8.shape) != (M, d):
        raise ValueError("x8 shape")
    y = torch.empty(M, d, dtype=bf16, device=dev)
    r = torch.empty(M, F, dtype=bf16, device=dev)
    h8 = torch.empty(M, F, dtype=torch.uint8, device=dev)
    if res is None:
        _lib.call("tfb_mlp8_fwd", _p(x8), _p(w8), _p(row), _p(y), _p(r), _p(h8), M, d, F, _stream())
    else:
        if tuple(res.shape) != (M, d):
            raise ValueError("res shape")
        _lib.call("tfb_mlp8_fwd_res", _p(x8), _p(w8), _p(row), _p(res), _p(y), _p(r), _p(h8), M, d, F, _stream())
    return (y, r, x8) if want_x8 else (y, r)


def mlp8_bwd(dy2, r, w8, row, want_h=True):
    """dx [M,d], h [M,F] (or None), dpre [M,F]: the fp8 backward; row = this call's backward row."""
    _chk(dy2), _chk(r), _chk(w8, torch.uint8), _chk(row, torch.float32)
    M, d = dy2.shape
    F = r.shape[1]
    dy8 = quant_fp8(dy2, row[5:6], FMT_E5M2)
    dx = torch.empty(M, d, dtype=bf16, device=dy2.device)
    dpre = torch.empty(M, F, dtype=bf16, device=dy2.device)
    h = torch.empty(M, F, dtype=bf16, device=dy2.device) if want_h else None
    dp8 = torch.empty(M, F, dtype=torch.uint8, device=dy2.device)
    _lib.call("tfb_mlp8_bwd", _p(dy8), _p(r), _p(w8), _p(row), _p(dx), _p(h), _p(dpre), _p(dp8), M, d, F, _stream())
    return dx, h, dpre


def mlp8_bwd_q(dy2, r, w8, row, e4m3_limit=240.0, want_dpre=True):
    """The fp8 backward keeping the byte tensors of the fp8 weight gradients: (dx [M,d], dpre [M,F] (None without
    want_dpre: the fp8 weight gradients read only its bytes), dp8 [M,F] e5m2 bytes, hq8 [M,F] = e4m3(min(bf16(r^2) s_h,
    e4m3_limit)) bytes, dy8 [M,d] e5m2 bytes)."""
    _chk(dy2), _chk(r), _chk(w8, torch.uint8), _chk(row, torch.float32)
    M, d = dy2.shape
    F = r.shape[1]
    dy8 = quant_fp8(dy2, row[5:6], FMT_E5M2)
    dx = torch.empty(M, d, dtype=bf16, device=dy2.device)
    dpre = torch.empty(M, F, dtype=bf16, device=dy2.device) if want_dpre else None
    dp8 = torch.empty(M, F, dtype=torch.uint8, device=dy2.device)
    hq8 = torch.empty(M, F, dtype=torch.uint8, device=dy2.device)
    _lib.call("tfb_mlp8_bwd_q", _p(dy8), _p(r), _p(w8), _p(row), _p(dx), None, _p(dpre), _p(dp8), _p(hq8), float(e4m3_limit),
              M, d, F, _stream())
    return dx, dpre, dp8, hq8, dy8


def mlp8_dw8(x8, dp8, hq8, dy8, row, x_scale=4.0, dw_fc=None, dw_proj=None, accumulate=False, out_dtype=bf16):
    """(dw_fc [F,d], dw_proj [d,F]) (+)= the fp8 weight gradients from the forward's x8 and the backward's dp8, hq8, dy8
    (mlp8_weight_grads under the fp8 weight-gradient switch, round2/source/train.py:8209)."""
    for t in (x8, dp8, hq8, dy8):
        _chk(t, torch.uint8)
    _chk(row, torch.float32)
    M, d = x8.shape
    F = dp8.shape[1]
    if tuple(hq8.shape) != (M, F) or tuple(dy8.shape) != (M, d):
        raise ValueError("operand shapes")
    if (dw_fc is None) != (dw_proj is None):
        raise ValueError("give both outputs or neither")
    if dw_fc is None:
        if accumulate:
            raise ValueError("accumulate needs the outputs")
        dw_fc = torch.empty(F, d, dtype=out_dtype, device=x8.device)
        dw_proj = torch.empty(d, F, dtype=out_dtype, device=x8.device)
    else:
        _chk(dw_fc, dw_fc.dtype), _chk(dw_proj, dw_proj.dtype)
        if dw_fc.dtype != dw_proj.dtype or dw_fc.dtype not in (bf16, torch.float32):
            raise ValueError("bad outputs")
        if tuple(dw_fc.shape) != (F, d) or tuple(dw_proj.shape) != (d, F):
            raise ValueError("bad output shapes")
    ws = _workspace(x8.device)
    xf, xd = _scale_arg(x_scale)
    _lib.call("tfb_mlp8_dw8", _p(x8), _p(dp8), _p(hq8), _p(dy8), _p(row), xf, _p(dw_fc), _p(dw_proj), M, d, F,
              int(dw_fc.dtype == torch.float32), int(accumulate), _p(ws), ws.numel() * 4, xd, _stream())
    return dw_fc, dw_proj


def mlp_dw_proj(dy2, r, out=None, accumulate=False, out_dtype=bf16):
    """dw_proj [d,F] (+)= dy^T @ bf16(r^2) without materialising h."""
    _chk(dy2), _chk(r)
    M, d = dy2.shape
    F = r.shape[1]
    if out is None:
        out = torch.empty(d, F, dtype=out_dtype, device=dy2.device)
    ws = _workspace(dy2.device)
    _lib.call("tfb_mlp_dw_proj", _p(dy2), _p(r), _p(out), M, d, F, int(out.dtype == torch.float32), int(accumulate), _p(ws),
              ws.numel() * 4, _stream())
    return out


# ------------------------------------------------------------------------------------------ attention
import ctypes as _ct

_L3 = _ct.c_long * 3


def _bht(t, layout):
    """(batch, head, token) element strides of a 4-D tensor given as "bhtd" or "bthd" (head dim contiguous)."""
    if t.stride(3) != 1:
        raise RuntimeError("head dimension must be contiguous")
    if layout == "bhtd":
        return _L3(t.stride(0), t.stride(1), t.stride(2))
    return _L3(t.stride(0), t.stride(2), t.stride(1))


def _attn_chk(t):
    if not t.is_cuda or t.dtype != bf16:
        raise TypeError("attention takes bf16 device tensors")


def _attn_bwd_chk(q, k, v, o, do, lse, dq, dk, dv, layout, out_layout):
    """Host checks of an attention backward call: a tensor of the wrong shape, or a log-sum-exp that is not fp32
    [B, H, T] contiguous, would be an out-of-bounds access on the device (the entry point sees only pointers and strides)."""
    for t in (q, k, v, o, do, dq, dk, dv):
        _attn_chk(t)
        if t.dim() != 4:
            raise ValueError("attention tensors are 4-D")
    B, H, T, D = q.shape if layout == "bhtd" else (q.shape[0], q.shape[2], q.shape[1], q.shape[3])
    if T % 128 or D not in (64, 128):
        raise ValueError("attention takes T % 128 == 0 and D 64 or 128")
    inp = (B, H, T, D) if layout == "bhtd" else (B, T, H, D)
    outp = (B, H, T, D) if out_layout == "bhtd" else (B, T, H, D)
    if tuple(k.shape) != inp or tuple(v.shape) != inp or tuple(q.shape) != inp:
        raise ValueError("q, k, v shapes differ")
    if tuple(o.shape) != (B, T, H, D) or tuple(do.shape) != (B, T, H, D):
        raise ValueError("o and do are [B, T, H, D]")
    for t in (dq, dk, dv):
        if tuple(t.shape) != outp:
            raise ValueError("dq, dk, dv shapes do not match out_layout")
    if not lse.is_cuda or lse.dtype != torch.float32 or not lse.is_contiguous() or lse.numel() != B * H * T:
        raise ValueError("lse is fp32 [B, H, T] contiguous")
    return B, H, T, D


def attn_fwd(q, k, v, scale, layout="bhtd", band=0):
    """q, k, v: 4-D views [B,H,T,D] ("bhtd") or [B,T,H,D] ("bthd"), arbitrary batch/head/token strides.
    Returns o [B,T,H,D] contiguous and lse [B,H,T] fp32. band = nw > 0: the reference's tile band (a query of 128-token
    tile i sees the keys k <= q of tiles i - nw + 1 .. i; K/nki_attn_bandpro.py:1654); 0: all keys k <= q."""
    for t in (q, k, v):
        _attn_chk(t)
    if layout == "bhtd":
        B, H, T, D = q.shape
    else:
        B, T, H, D = q.shape
    o = torch.empty(B, T, H, D, dtype=bf16, device=q.device)
    lse = torch.empty(B, H, T, dtype=torch.float32, device=q.device)
    if band:
        _lib.call("tfb_attn_fwd_band", _p(q), _bht(q, layout), _p(k), _bht(k, layout), _p(v), _bht(v, layout), _p(o),
                  _bht(o, "bthd"), _p(lse), B, H, T, D, float(scale), int(band), _stream())
    else:
        _lib.call("tfb_attn_fwd", _p(q), _bht(q, layout), _p(k), _bht(k, layout), _p(v), _bht(v, layout), _p(o),
                  _bht(o, "bthd"), _p(lse), B, H, T, D, float(scale), _stream())
    return o, lse


def attn_bwd(q, k, v, o, do, lse, scale, layout="bhtd", dq=None, dk=None, dv=None, out_layout="bhtd", rope=None, band=0):
    """Gradients of attn_fwd. o, do are [B,T,H,D]. dq/dk/dv may be given as (strided) views with `out_layout`;
    otherwise dq, dk are allocated [B,H,T,D] and dv [B,T,H,D] (returned as a [B,H,T,D] view), as the reference returns.
    rope = (cos, sin) (bf16 [T, D/2]): dq and dk come back with the inverse rotation applied (D = 64)."""
    _attn_chk(q)
    if q.dim() != 4:
        raise ValueError("attention tensors are 4-D")
    if layout == "bhtd":
        B, H, T, D = q.shape
    else:
        B, T, H, D = q.shape
    if dq is None:
        dq = torch.empty(B, H, T, D, dtype=bf16, device=q.device)
        dk = torch.empty(B, H, T, D, dtype=bf16, device=q.device)
        dv = torch.empty(B, T, H, D, dtype=bf16, device=q.device).permute(0, 2, 1, 3)
        out_layout = "bhtd"
    _attn_bwd_chk(q, k, v, o, do, lse, dq, dk, dv, layout, out_layout)
    delta = torch.empty(2, B, H, T, dtype=torch.float32, device=q.device)
    cos, sin = rope if rope is not None else (None, None)
    _chk(cos), _chk(sin)
    ptrs = (_p(q), _bht(q, layout), _p(k), _bht(k, layout), _p(v), _bht(v, layout), _p(o), _bht(o, "bthd"), _p(do),
            _bht(do, "bthd"), _p(dq), _bht(dq, out_layout), _p(dk), _bht(dk, out_layout), _p(dv), _bht(dv, out_layout), _p(lse),
            _p(delta))
    if band:
        _lib.call("tfb_attn_bwd_band", *ptrs, _p(cos), _p(sin), B, H, T, D, float(scale), int(band), _stream())
    elif rope is not None:
        _lib.call("tfb_attn_bwd_rope", *ptrs, _p(cos), _p(sin), B, H, T, D, float(scale), _stream())
    else:
        _lib.call("tfb_attn_bwd", *ptrs, B, H, T, D, float(scale), _stream())
    return dq, dk, dv


def attn_bwd_static_max_rows():
    """The largest B * H * T attn_bwd_static takes (the size of the library's static scratch array)."""
    return int(_lib.lib().tfb_attn_bwd_static_max_rows())


def attn_bwd_static(q, k, v, o, do, lse, scale, dq, dk, dv, layout="bhtd", out_layout="bhtd"):
    """attn_bwd into caller-provided dq, dk, dv through the entry point that allocates nothing: its row-statistic scratch
    is a static device array inside the library (B * H * T <= tfb_attn_bwd_static_max_rows(); TfbError status 4 beyond).
    Calls that overlap on one GPU share that array and race; this wrapper creates no tensor either. The FIRST call on a
    device looks up the array's address: make one call eagerly before capturing this one into a HIP graph."""
    B, H, T, D = _attn_bwd_chk(q, k, v, o, do, lse, dq, dk, dv, layout, out_layout)
    _lib.call("tfb_attn_bwd_static", _p(q), _bht(q, layout), _p(k), _bht(k, layout), _p(v), _bht(v, layout), _p(o),
              _bht(o, "bthd"), _p(do), _bht(do, "bthd"), _p(dq), _bht(dq, out_layout), _p(dk), _bht(dk, out_layout), _p(dv),
              _bht(dv, out_layout), _p(lse), B, H, T, D, float(scale), _stream())
    return dq, dk, dv


# ------------------------------------------------------------------------------------------ elementwise
def relu2(x):
    _chk(x)
    out = torch.empty_like(x)
    _lib.call("tfb_relu2", _p(x), None, _p(out), x.numel(), 0, _stream())
    return out


def relu2_bwd(x, gy):
    _chk(x), _chk(gy)
    out = torch.empty_like(x)
    _lib.call("tfb_relu2", _p(x), _p(gy), _p(out), x.numel(), 1, _stream())
    return out


def relu2_bwd_from_h(h, dh):
    _chk(h), _chk(dh)
    out = torch.empty_like(h)
    _lib.call("tfb_relu2", _p(h), _p(dh), _p(out), h.numel(), 2, _stream())
    return out


def rope_(x, cos, sin, T, nheads, D, inverse=False, out=None):
    """Rotate the first nheads*D columns of each row of x ([rows, row_stride] view, contiguous rows) in place
    (or into `out`). cos, sin: bf16 [T, D/2]; row r is token r % T."""
    _chk(cos), _chk(sin)
    if not x.is_cuda or x.dtype != bf16 or x.stride(-1) != 1:
        raise TypeError("rope_ takes a bf16 device tensor with contiguous rows")
    x2 = x.reshape(-1, x.shape[-1]) if x.is_contiguous() else x
    rows, stride = x2.shape[0], x2.stride(0)
    o = x2 if out is None else out
    _lib.call("tfb_rope", _p(x2), _p(cos), _p(sin), _p(o), rows, T, nheads, D, stride, o.stride(0), int(inverse), _stream())
    return x if out is None else out


def _rows2d(x):
    if not x.is_cuda or x.dtype != bf16 or x.stride(-1) != 1:
        raise TypeError("expected a bf16 device tensor with contiguous rows")
    return x.reshape(-1, x.shape[-1]) if x.is_contiguous() else x


def rope_norm_fwd(x, cos, sin, T, nheads, D, eps=2.0 ** -23, want_r=True):
    """RoPE then parameter-free RMSNorm of each of the first `nheads` heads (D columns each) of every row of x
    ([rows, row_stride] view). Returns (y [rows, nheads*D] normalised, r [rows, nheads*D] rotated or None,
    inv [rows, nheads] fp32)."""
    _chk(cos), _chk(sin)
    x2 = _rows2d(x)
    rows = x2.shape[0]
    y = torch.empty(rows, nheads * D, dtype=bf16, device=x.device)
    r = torch.empty(rows, nheads * D, dtype=bf16, device=x.device) if want_r else None
    inv = torch.empty(rows, nheads, dtype=torch.float32, device=x.device)
    _lib.call("tfb_rope_norm_fwd", _p(x2), _p(cos), _p(sin), _p(r), _p(y), _p(inv), rows, T, nheads, D, x2.stride(0),
              nheads * D, nheads * D, float(eps), _stream())
    return y, r, inv


def rope_norm_bwd(g, r, inv, cos, sin, T, nheads, D, out=None):
    """The gradient of rope_norm_fwd's input from g (gradient of y; [rows, row_stride] view), the saved r and inv; written
    into `out` ([rows, row_stride] view) or a fresh [rows, nheads*D] tensor."""
    _chk(cos), _chk(sin), _chk(r), _chk(inv, torch.float32)
    g2 = _rows2d(g)
    rows = g2.shape[0]
    o = torch.empty(rows, nheads * D, dtype=bf16, device=g.device) if out is None else _rows2d(out)
    _lib.call("tfb_rope_norm_bwd", _p(g2), _p(r), _p(inv), _p(cos), _p(sin), _p(o), rows, T, nheads, D, g2.stride(0),
              r.stride(0), o.stride(0), _stream())
    return o if out is None else out


def resmix_bwd(g, x, x0, ab):
    """dx = g*a, dx0 = g*b, dab = (sum g*x, sum g*x0) for x_new = a*x + b*x0; ab: fp32 device [2]."""
    _chk(g), _chk(x), _chk(x0), _chk(ab, torch.float32)
    dx, dx0 = torch.empty_like(g), torch.empty_like(g)
    nb = _lib.lib().tfb_resmix_bwd_blocks(g.numel())
    part = torch.empty(2 * nb, dtype=torch.float32, device=g.device)
    dab = torch.empty(2, dtype=torch.float32, device=g.device)
    _lib.call("tfb_resmix_bwd", _p(g), _p(x), _p(x0), _p(ab), _p(dx), _p(dx0), _p(part), _p(dab), g.numel(), _stream())
    return dx, dx0, dab


def embedding_fwd(idx, weight):
    """weight rows gathered by idx; an id outside [0, V) gives a zero row (and receives no gradient in embedding_bwd)."""
    _chk(weight)
    if idx.dtype not in (torch.int64, torch.int32) or not idx.is_cuda:
        raise TypeError("idx must be an int32/int64 device tensor")
    idx = idx.contiguous()
    C = weight.shape[1]
    out = torch.empty(*idx.shape, C, dtype=bf16, device=weight.device)
    _lib.call("tfb_embedding_fwd", _p(idx), int(idx.dtype == torch.int64), _p(weight), _p(out), idx.numel(), C,
              weight.shape[0], _stream())
    return out


def embedding_bwd(idx, dy, dw, grouped=True):
    """dw (fp32 [V, C]) += scatter of dy rows by idx. grouped: rows sorted by token on the device and summed per token
    (deterministic order inside a token's run); False: one fp32 atomic add per element (the plain entry point)."""
    _chk(dy), _chk(dw, torch.float32)
    idx = idx.contiguous()
    n, V = idx.numel(), dw.shape[0]
    if not grouped:
        _lib.call("tfb_embedding_bwd", _p(idx), int(idx.dtype == torch.int64), _p(dy), _p(dw), n, dy.shape[-1], V,
                  _stream())
        return dw
    scr = _scratch(dw.device, _lib.lib().tfb_embedding_bwd_scratch_ints(n, V))  # 4-byte elements, used as int32
    _lib.call("tfb_embedding_bwd_grouped", _p(idx), int(idx.dtype == torch.int64), _p(dy), _p(dw), n, dy.shape[-1], V,
              _p(scr), _stream())
    return dw


def fill_f32_(t, val=0.0):
    _chk(t, torch.float32)
    _lib.call("tfb_fill_f32", _p(t), float(val), t.numel(), _stream())
    return t


def adamw_(p, g, m, v, step, lr, beta1, beta2, eps, weight_decay, p_bf16=None):
    """One in-place AdamW update of the fp32 master p (and its optional bf16 copy) from g (fp32 or bf16)."""
    _chk(p, torch.float32), _chk(m, torch.float32), _chk(v, torch.float32), _chk(g, g.dtype), _chk(p_bf16)
    if g.dtype not in (torch.float32, bf16):
        raise TypeError("grad must be fp32 or bf16")
    bias1 = 1.0 - beta1 ** step
    bias2 = 1.0 - beta2 ** step
    _lib.call("tfb_adamw", _p(p), _p(g), int(g.dtype == torch.float32), _p(m), _p(v), _p(p_bf16), p.numel(), float(lr),
              float(weight_decay), float(1.0 - beta1), float(1.0 - beta2), float(eps), float(bias1), float(bias2), _stream())


# ------------------------------------------------------------------------------------------ loss head
def _tg(targets):
    if targets.dtype not in (torch.int64, torch.int32) or not targets.is_cuda:
        raise TypeError("targets must be an int32/int64 device tensor")
    return targets.contiguous()


def loss_fwd(logits2, targets, softcap=15.0, row_w=None):
    """Row losses (already multiplied by row_w) and lse, from bf16 logits [N, V]; targets < 0 are ignored."""
    _chk(logits2), _chk(row_w, torch.float32)
    tg = _tg(targets)
    N, V = logits2.shape
    loss = torch.empty(N, dtype=torch.float32, device=logits2.device)
    lse = torch.empty(N, dtype=torch.float32, device=logits2.device)
    _lib.call("tfb_loss_fwd", _p(logits2), _p(tg), int(tg.dtype == torch.int64), _p(row_w), _p(loss), _p(lse), N, V,
              float(softcap or 0.0), _stream())
    return loss, lse


def loss_bwd(logits2, targets, lse, grow, softcap=15.0, inplace=False):
    """dlogits bf16 [N, V]; grow fp32 [N] = d(total)/d(row loss) * row weight."""
    _chk(logits2), _chk(lse, torch.float32), _chk(grow, torch.float32)
    tg = _tg(targets)
    N, V = logits2.shape
    out = logits2 if inplace else torch.empty_like(logits2)
    _lib.call("tfb_loss_bwd", _p(logits2), _p(tg), int(tg.dtype == torch.int64), _p(lse), _p(grow), _p(out), N, V,
              float(softcap or 0.0), _stream())
    return out


def loss_row_weights(targets, reduction="mean", V=None):
    """fp32 [N] weights of the row losses in the reduced loss: valid / max(1, count of valid) for "mean", valid for "sum";
    a row is valid when 0 <= t < V (the rows the loss kernels give a loss to; V None: when t >= 0)."""
    tg = _tg(targets)
    w = torch.empty(tg.numel(), dtype=torch.float32, device=tg.device)
    _lib.call("tfb_loss_row_weights", _p(tg), int(tg.dtype == torch.int64), _p(w), tg.numel(), int(reduction == "mean"),
              int(V or 0), _stream())
    return w


LOSS_FWD_BWD_MAX_V = 65536


def loss_fwd_bwd(logits2, targets, row_w=None, softcap=15.0):
    """(loss rows fp32 [N], lse fp32 [N]) as loss_fwd gives them, and logits2 OVERWRITTEN by the gradient of sum(rows):
    row_w (softmax - onehot) (1 - tanh^2), what loss_bwd gives for grow = row_w. One pass over the logits; V <= 65536."""
    _chk(logits2), _chk(row_w, torch.float32)
    tg = _tg(targets)
    N, V = logits2.shape
    loss = torch.empty(N, dtype=torch.float32, device=logits2.device)
    lse = torch.empty(N, dtype=torch.float32, device=logits2.device)
    _lib.call("tfb_loss_fwd_bwd", _p(logits2), _p(tg), int(tg.dtype == torch.int64), _p(row_w), _p(loss), _p(lse), N, V,
              float(softcap or 0.0), _stream())
    return loss, lse


def loss_multi_fwd(logits2, targets, row_w, softcap=15.0, eps=0.0):
    """Row losses sum_k row_w[k] (lse - (1 - eps) s_{t_k} - eps mean_v s_v) and lse; targets [K, N] (int64 / int32, < 0 =
    weight 0), row_w fp32 [K, N]."""
    _chk(logits2), _chk(row_w, torch.float32)
    tg = _tg(targets)
    K, N = tg.shape
    V = logits2.shape[1]
    if tuple(row_w.shape) != (K, N) or logits2.shape[0] != N:
        raise ValueError("targets [K, N], row_w [K, N], logits [N, V]")
    loss = torch.empty(N, dtype=torch.float32, device=logits2.device)
    lse = torch.empty(N, dtype=torch.float32, device=logits2.device)
    _lib.call("tfb_loss_multi_fwd", _p(logits2), _p(tg), int(tg.dtype == torch.int64), _p(row_w), K, float(eps), _p(loss),
              _p(lse), N, V, float(softcap or 0.0), _stream())
    return loss, lse


def loss_multi_bwd(logits2, targets, row_w, lse, g, softcap=15.0, eps=0.0, inplace=False):
    """dlogits bf16 [N, V] of loss_multi_fwd; g fp32 [N] = d(total)/d(row loss)."""
    _chk(logits2), _chk(row_w, torch.float32), _chk(lse, torch.float32), _chk(g, torch.float32)
    tg = _tg(targets)
    K, N = tg.shape
    V = logits2.shape[1]
    out = logits2 if inplace else torch.empty_like(logits2)
    _lib.call("tfb_loss_multi_bwd", _p(logits2), _p(tg), int(tg.dtype == torch.int64), _p(row_w), K, float(eps), _p(lse),
              _p(g), _p(out), N, V, float(softcap or 0.0), _stream())
    return out


def lmhead_fwd(x2, W, targets, softcap=None, row_w=None):
    """logits = x2 @ W^T (W [V, d]) with the row log-sum-exp fused into the GEMM epilogue.
    Returns (logits bf16 [N, V], loss rows fp32 [N], lse fp32 [N])."""
    _chk(x2), _chk(W), _chk(row_w, torch.float32)
    tg = _tg(targets)
    N, d = x2.shape
    V = W.shape[0]
    logits = torch.empty(N, V, dtype=bf16, device=x2.device)
    part = torch.empty(N, V // 64, 2, dtype=torch.float32, device=x2.device)
    loss = torch.empty(N, dtype=torch.float32, device=x2.device)
    lse = torch.empty(N, dtype=torch.float32, device=x2.device)
    _lib.call("tfb_lmhead_fwd", _p(x2), _p(W), _p(tg), int(tg.dtype == torch.int64), _p(row_w), _p(logits), _p(part), _p(loss),
              _p(lse), N, d, V, float(softcap or 0.0), _stream())
    return logits, loss, lse


# ------------------------------------------------------------------------------------------ mixture of experts
def moe_max_rows(N, E, topk):
    return _lib.lib().tfb_moe_max_rows(N, E, topk)


def moe_route(h2, wr, topk, bias=None, want_logits=False):
    """(p fp32 [N,E], idx int32 [N,topk], gate fp32 [N,topk], logits or None) from h2 bf16 [N,d], wr fp32 [E,d]."""
    _chk(h2), _chk(wr, torch.float32), _chk(bias, torch.float32)
    N, d = h2.shape
    E = wr.shape[0]
    dev = h2.device
    p = torch.empty(N, E, dtype=torch.float32, device=dev)
    idx = torch.empty(N, topk, dtype=torch.int32, device=dev)
    gate = torch.empty(N, topk, dtype=torch.float32, device=dev)
    logits = torch.empty(N, E, dtype=torch.float32, device=dev) if want_logits else None
    _lib.call("tfb_moe_route", _p(h2), _p(wr), _p(bias), _p(logits), _p(p), _p(idx), _p(gate), N, d, E, topk, _stream())
    return p, idx, gate, logits


def moe_tables(idx, E, seq_len=None, capacity=None):
    """Slot tables for the ragged layout: dict(cnt, seg, tile_expert, slot, tok, ksel, rmax). Dropless by default; with
    seq_len and capacity the reference's per-sequence capacity (round2/source/train.py:10555-10634): each sequence keeps its
    first `capacity` assignments per expert, the rest get slot -1; the dict then also holds cnt_all (every assignment)."""
    _chk(idx, torch.int32)
    N, topk = idx.shape
    dev = idx.device
    rmax = moe_max_rows(N, E, topk)
    i32 = dict(dtype=torch.int32, device=dev)
    t = {"cnt": torch.empty(E, **i32), "seg": torch.empty(E + 1, **i32), "tile_expert": torch.empty(rmax // 128, **i32),
         "slot": torch.empty(N, topk, **i32), "tok": torch.empty(rmax, **i32), "ksel": torch.empty(rmax, **i32), "rmax": rmax}
    nw = (N + 63) // 64
    if capacity is None:
        scratch = torch.empty(nw * E, **i32)
        _lib.call("tfb_moe_tables", _p(idx), _p(t["cnt"]), _p(t["seg"]), _p(t["tile_expert"]), _p(t["slot"]), _p(t["tok"]),
                  _p(t["ksel"]), _p(scratch), N, E, topk, rmax, _stream())
        return t
    if seq_len is None:
        raise ValueError("a capacity is counted per sequence: seq_len is needed")
    t["cnt_all"] = torch.empty(E, **i32)
    t["capacity"] = int(capacity)
    scratch = torch.empty(2 * nw * E, **i32)
    _lib.call("tfb_moe_tables_cap", _p(idx), _p(t["cnt"]), _p(t["cnt_all"]), _p(t["seg"]), _p(t["tile_expert"]), _p(t["slot"]),
              _p(t["tok"]), _p(t["ksel"]), _p(scratch), N, int(seq_len), int(capacity), E, topk, rmax, _stream())
    return t


def moe_gather(h2, tab, x_scale=4.0, want_xs=True):
    """(xs bf16 [rmax,d], xs8 uint8 [rmax,d]); x_scale None: no fp8 copy (xs8 is None); want_xs False: no bf16 copy (xs is
    None: fp8 experts whose weight gradients are in fp8 too never read it)."""
    _chk(h2)
    d = h2.shape[1]
    rmax = tab["rmax"]
    xs = torch.empty(rmax, d, dtype=bf16, device=h2.device) if want_xs or x_scale is None else None
    if x_scale is None:
        _lib.call("tfb_moe_gather", _p(h2), _p(tab["tok"]), None, 1.0, _p(xs), None, rmax, d, _stream())
        return xs, None
    xs8 = torch.empty(rmax, d, dtype=torch.uint8, device=h2.device)
    if isinstance(x_scale, torch.Tensor):
        _lib.call("tfb_moe_gather", _p(h2), _p(tab["tok"]), _p(x_scale), 0.0, _p(xs), _p(xs8), rmax, d, _stream())
    else:
        _lib.call("tfb_moe_gather", _p(h2), _p(tab["tok"]), None, float(x_scale), _p(xs), _p(xs8), rmax, d, _stream())
    return xs, xs8


def moe_mlp8_fwd(xs8, w8, rows, tab, F):
    """Grouped fp8 expert MLP forward: (ys bf16 [rmax,d], r bf16 [rmax,F]). w8 uint8 [E,4,F*d], rows fp32 [E,16]."""
    _chk(xs8, torch.uint8), _chk(w8, torch.uint8), _chk(rows, torch.float32)
    rmax, d = xs8.shape
    ys = torch.empty(rmax, d, dtype=bf16, device=xs8.device)
    r = torch.empty(rmax, F, dtype=bf16, device=xs8.device)
    h8 = torch.empty(rmax, F, dtype=torch.uint8, device=xs8.device)
    _lib.call("tfb_moe_mlp8_fwd", _p(xs8), _p(w8), _p(rows), _p(tab["tile_expert"]), _p(ys), _p(r), _p(h8), rmax, d, F, _stream())
    return ys, r


def moe_mlp_fwd(xs, w_fc, w_proj, tab):
    """Grouped bf16 expert MLP forward: (ys bf16 [rmax,d], r bf16 [rmax,F] = relu(pre), h bf16 [rmax,F] = r^2).
    w_fc bf16 [E,F,d], w_proj bf16 [E,d,F]."""
    _chk(xs), _chk(w_fc), _chk(w_proj)
    rmax, d = xs.shape
    E, F, _ = w_fc.shape
    if tuple(w_fc.shape) != (E, F, d) or tuple(w_proj.shape) != (E, d, F):
        raise ValueError("moe_mlp_fwd: w_fc [E,F,d] and w_proj [E,d,F] expected")
    ys = torch.empty(rmax, d, dtype=bf16, device=xs.device)
    r = torch.empty(rmax, F, dtype=bf16, device=xs.device)
    h = torch.empty(rmax, F, dtype=bf16, device=xs.device)
    _lib.call("tfb_moe_mlp_fwd", _p(xs), _p(w_fc), _p(w_proj), _p(tab["tile_expert"]), _p(ys), _p(r), _p(h), rmax, d, F, _stream())
    return ys, r, h


def moe_mlp_bwd(dys, r, w_fc, w_proj, tab):
    """Grouped bf16 expert MLP backward: (dxs bf16 [rmax,d], dpre bf16 [rmax,F])."""
    _chk(dys), _chk(r), _chk(w_fc), _chk(w_proj)
    rmax, d = dys.shape
    F = r.shape[1]
    dxs = torch.empty(rmax, d, dtype=bf16, device=dys.device)
    dpre = torch.empty(rmax, F, dtype=bf16, device=dys.device)
    _lib.call("tfb_moe_mlp_bwd", _p(dys), _p(r), _p(w_fc), _p(w_proj), _p(tab["tile_expert"]), _p(dxs), _p(dpre), rmax, d, F, _stream())
    return dxs, dpre


def moe_backward_scales(dys, rows, tab):
    _chk(dys), _chk(rows, torch.float32)
    E = rows.shape[0]
    out = torch.empty_like(rows)
    scratch = torch.empty(E, dtype=torch.int32, device=dys.device)
    _lib.call("tfb_moe_backward_scales", _p(dys), _p(tab["tile_expert"]), _p(rows), _p(out), _p(scratch), dys.shape[0],
              dys.shape[1], E, _stream())
    return out


def moe_backward_scales_rowmax(rowmax, rows, tab, d):
    """moe_backward_scales from the row maxima moe_combine_bwd(..., want_rowmax=True) left: the same rows, no pass over dys."""
    _chk(rowmax, torch.float32), _chk(rows, torch.float32)
    E = rows.shape[0]
    out = torch.empty_like(rows)
    _lib.call("tfb_moe_backward_scales_rowmax", _p(rowmax), _p(tab["seg"]), _p(rows), _p(out), d, E, _stream())
    return out


def moe_quant(x, rows, col, fmt, tab):
    _chk(x), _chk(rows, torch.float32)
    out = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    _lib.call("tfb_moe_quant", _p(x), _p(tab["tile_expert"]), _p(rows), col, fmt, _p(out), x.shape[0], x.shape[1], _stream())
    return out


def moe_mlp8_bwd(dys, r, w8, rows_bwd, tab):
    """(dxs bf16 [rmax,d], dpre bf16 [rmax,F]) from dys; rows_bwd from moe_backward_scales."""
    _chk(dys), _chk(r)
    rmax, d = dys.shape
    F = r.shape[1]
    dy8 = moe_quant(dys, rows_bwd, 5, FMT_E5M2, tab)
    dxs = torch.empty(rmax, d, dtype=bf16, device=dys.device)
    dpre = torch.empty(rmax, F, dtype=bf16, device=dys.device)
    dp8 = torch.empty(rmax, F, dtype=torch.uint8, device=dys.device)
    _lib.call("tfb_moe_mlp8_bwd", _p(dy8), _p(r), _p(w8), _p(rows_bwd), _p(tab["tile_expert"]), _p(dxs), _p(dpre), _p(dp8), rmax, d,
              F, _stream())
    return dxs, dpre


def moe_mlp8_bwd_q(dys, r, w8, rows_bwd, tab, hq_limit):
    """The grouped fp8 backward for the fp8 weight gradients: (dxs bf16 [rmax,d], dp8 e5m2 [rmax,F], hq8 e4m3 [rmax,F],
    dy8 e5m2 [rmax,d]); no bf16 dpre is written."""
    _chk(dys), _chk(r)
    rmax, d = dys.shape
    F = r.shape[1]
    dy8 = moe_quant(dys, rows_bwd, 5, FMT_E5M2, tab)
    dxs = torch.empty(rmax, d, dtype=bf16, device=dys.device)
    dp8 = torch.empty(rmax, F, dtype=torch.uint8, device=dys.device)
    hq8 = torch.empty(rmax, F, dtype=torch.uint8, device=dys.device)
    _lib.call("tfb_moe_mlp8_bwd_q", _p(dy8), _p(r), _p(w8), _p(rows_bwd), _p(tab["tile_expert"]), _p(dxs), None, _p(dp8), _p(hq8),
              float(hq_limit), rmax, d, F, _stream())
    return dxs, dp8, hq8, dy8


def moe_dw8(xs8, dp8, hq8, dy8, rows_bwd, x_scale, tab, E, dw_fc=None, dw_proj=None, accumulate=False, out_dtype=bf16):
    """(dw_fc [E,F,d], dw_proj [E,d,F]) in fp8 over each expert's row segment, from the bytes the other GEMMs multiplied."""
    _chk(xs8, torch.uint8), _chk(dp8, torch.uint8), _chk(hq8, torch.uint8), _chk(dy8, torch.uint8), _chk(rows_bwd, torch.float32)
    d, F = xs8.shape[1], dp8.shape[1]
    if dw_fc is None:
        dw_fc = torch.empty(E, F, d, dtype=out_dtype, device=xs8.device)
        dw_proj = torch.empty(E, d, F, dtype=out_dtype, device=xs8.device)
    _lib.call("tfb_moe_dw8", _p(xs8), _p(dp8), _p(hq8), _p(dy8), _p(rows_bwd), float(x_scale), _p(tab["seg"]), _p(dw_fc), _p(dw_proj),
              E, d, F, int(dw_fc.dtype == torch.float32), int(accumulate), _stream())
    return dw_fc, dw_proj


def moe_dw(dpre, xs, dys, r, tab, E, dw_fc=None, dw_proj=None, accumulate=False, out_dtype=bf16):
    """(dw_fc [E,F,d], dw_proj [E,d,F]) over each expert's row segment."""
    d, F = xs.shape[1], r.shape[1]
    if dw_fc is None:
        dw_fc = torch.empty(E, F, d, dtype=out_dtype, device=xs.device)
        dw_proj = torch.empty(E, d, F, dtype=out_dtype, device=xs.device)
    _lib.call("tfb_moe_dw", _p(dpre), _p(xs), _p(dys), _p(r), _p(tab["seg"]), _p(dw_fc), _p(dw_proj), E, d, F,
              int(dw_fc.dtype == torch.float32), int(accumulate), _stream())
    return dw_fc, dw_proj


def moe_combine(ys, tab, gate, N):
    _chk(ys), _chk(gate, torch.float32)
    d = ys.shape[1]
    out = torch.empty(N, d, dtype=bf16, device=ys.device)
    _lib.call("tfb_moe_combine", _p(ys), _p(tab["slot"]), _p(gate), _p(out), N, d, gate.shape[1], _stream())
    return out


def moe_combine_bwd(dout, ys, tab, gate, want_rowmax=False):
    """(dys, dgate), and with want_rowmax the fp32 [rmax] maxima of |dys| per row for moe_backward_scales_rowmax."""
    _chk(dout), _chk(ys), _chk(gate, torch.float32)
    rmax, d = ys.shape
    dys = torch.empty_like(ys)
    # the kernel writes the gate gradient of every assignment that holds a row; a skipped one's is zero
    dgate = torch.zeros_like(gate) if "capacity" in tab else torch.empty_like(gate)
    if want_rowmax:
        rowmax = torch.empty(rmax, dtype=torch.float32, device=ys.device)
        _lib.call("tfb_moe_combine_bwd_rowmax", _p(dout), _p(ys), _p(tab["tok"]), _p(tab["ksel"]), _p(gate), _p(dys), _p(dgate),
                  _p(rowmax), rmax, d, gate.shape[1], _stream())
        return dys, dgate, rowmax
    _lib.call("tfb_moe_combine_bwd", _p(dout), _p(ys), _p(tab["tok"]), _p(tab["ksel"]), _p(gate), _p(dys), _p(dgate), rmax, d,
              gate.shape[1], _stream())
    return dys, dgate


def moe_route_bwd(dgate, p, idx, dxs, tab, h2, wr, dwr=None, accumulate=False, aux=None):
    """(dh bf16 [N,d], dwr fp32 [E,d], dlogits fp32 [N,E]). aux = (terms, lse, gaux, alpha, beta): the gradient gaux
    (1-element fp32 device tensor) of the weighted auxiliary terms alpha lb + beta z of moe_aux_fwd is folded into dlogits;
    aux = (terms, lse, gaux, alpha, beta, fs, gamma, seq_len) adds the per-sequence term gamma seq of moe_aux_seq_fwd."""
    N, d = h2.shape
    E = wr.shape[0]
    dlogits = torch.empty(N, E, dtype=torch.float32, device=h2.device)
    dh = torch.empty_like(h2)
    if dwr is None:
        dwr = torch.empty(E, d, dtype=torch.float32, device=h2.device)
        accumulate = False
    scr = _scratch(h2.device, 64 * E * d)
    if aux is None:
        _lib.call("tfb_moe_route_bwd", _p(dgate), _p(p), _p(idx), _p(dxs), _p(tab["slot"]), _p(h2), _p(wr), _p(dlogits), _p(dh),
                  _p(dwr), int(accumulate), _p(scr), N, d, E, idx.shape[1], _stream())
    elif len(aux) == 8:
        terms, lse, gaux, alpha, beta, fs, gamma, seq_len = aux
        _chk(terms, torch.float32), _chk(lse, torch.float32), _chk(gaux, torch.float32), _chk(fs, torch.float32)
        if N % int(seq_len) or tuple(fs.shape) != (N // int(seq_len), E):
            raise ValueError("moe_route_bwd: fs must be [N / seq_len, E]")
        _lib.call("tfb_moe_route_bwd_aux_seq", _p(dgate), _p(p), _p(idx), _p(dxs), _p(tab["slot"]), _p(h2), _p(wr), _p(dlogits),
                  _p(dh), _p(dwr), int(accumulate), _p(scr), _p(terms), _p(lse), _p(gaux), float(alpha), float(beta), _p(fs),
                  float(gamma), int(seq_len), N, d, E, idx.shape[1], _stream())
    else:
        terms, lse, gaux, alpha, beta = aux
        _chk(terms, torch.float32), _chk(lse, torch.float32), _chk(gaux, torch.float32)
        _lib.call("tfb_moe_route_bwd_aux", _p(dgate), _p(p), _p(idx), _p(dxs), _p(tab["slot"]), _p(h2), _p(wr), _p(dlogits),
                  _p(dh), _p(dwr), int(accumulate), _p(scr), _p(terms), _p(lse), _p(gaux), float(alpha), float(beta), N, d, E,
                  idx.shape[1], _stream())
    return dh, dwr, dlogits


def moe_aux_fwd(p, logits, tab, topk):
    """(terms fp32 [2 + E] = (lb, z, f_e), lse fp32 [N]): the router's load-balance term E sum_e f_e P_e, its z term
    mean(logsumexp(logits)^2) and the experts' load shares (round2/source/train.py:10779 moe_aux_terms)."""
    _chk(p, torch.float32), _chk(logits, torch.float32)
    N, E = p.shape
    terms = torch.empty(2 + E, dtype=torch.float32, device=p.device)
    lse = torch.empty(N, dtype=torch.float32, device=p.device)
    scr = torch.empty(64 * 17, dtype=torch.float32, device=p.device)
    _lib.call("tfb_moe_aux_fwd", _p(p), _p(logits), _p(tab.get("cnt_all", tab["cnt"])), _p(terms), _p(lse), _p(scr), N, E, topk, _stream())
    return terms, lse


def moe_aux_seq_fwd(p, idx, seq_len, topk):
    """(term fp32 [1], fs fp32 [N / seq_len, E]): the per-sequence balance term of moe_aux_terms
    (round2/source/train.py:10789-10792) = mean over sequences of E sum_e fs ps, and the sequences' load shares."""
    _chk(p, torch.float32), _chk(idx, torch.int32)
    N, E = p.shape
    T = int(seq_len)
    if T <= 0 or N % T:
        raise ValueError("moe_aux_seq_fwd: %d tokens are not whole sequences of %d" % (N, T))
    fs = torch.empty(N // T, E, dtype=torch.float32, device=p.device)
    term = torch.empty(1, dtype=torch.float32, device=p.device)
    scr = torch.empty(N // T, dtype=torch.float32, device=p.device)
    _lib.call("tfb_moe_aux_seq_fwd", _p(p), _p(idx), _p(fs), _p(term), _p(scr), N, T, E, topk, _stream())
    return term, fs


# ------------------------------------------------------------------------------------------ Muon Newton-Schulz
# the kit's POLAR_EXPRESS_COEFFS as the reference's kernel module holds them (round2/source/kernels/nki_nsk.py:82-88)
NS_COEFFS = (
    (8.156554524902461, -22.48329292557795, 15.878769915207462),
    (4.042929935166739, -2.808917465908714, 0.5000178451051316),
    (3.8916678022926607, -2.772484153217685, 0.5060648178503393),
    (3.285753657755655, -2.3681294933425376, 0.46449024233003106),
    (2.3465413258596377, -1.7097828382687081, 0.42323551169305323),
)
_NS_WS = {}


def ns5(g, d, coeffs=NS_COEFFS):
    """Five Newton-Schulz iterations on a stack g fp32 [K, r, c] (tall r >= c, or wide: handled as the transposes) from
    X0 = bf16(bf16(g) / d), d [K] (any float dtype; the reciprocal is taken in fp32 as the reference's sc_tile does).
    Returns (y bf16 [K, r, c], v fp32 [K, max(r, c)] = the sums of y^2 along the short side)."""
    import ctypes
    _chk(g, torch.float32)
    K, r, c = g.shape
    wide = r < c
    M, N = (c, r) if wide else (r, c)
    inv = (1.0 / d.reshape(-1).float()).contiguous()
    if inv.numel() != K:
        raise ValueError("one denominator per matrix")
    _chk(inv, torch.float32)
    need = _lib.lib().tfb_ns5_workspace_bytes(K, M, N)
    # one workspace per (device, stream), grown to the largest stack seen (never one per shape)
    key = (g.device, torch.cuda.current_stream(g.device).cuda_stream)
    ws = _NS_WS.get(key)
    if ws is None or ws.numel() < need:
        ws = _NS_WS[key] = torch.empty(max(need, 256), dtype=torch.uint8, device=g.device)
    y = torch.empty(K, r, c, dtype=bf16, device=g.device)
    v = torch.empty(K, M, dtype=torch.float32, device=g.device)
    co = (ctypes.c_float * 15)(*[float(x) for t in coeffs for x in t])
    _lib.call("tfb_ns5", _p(g), _p(inv), co, _p(y), _p(v), K, M, N, int(wide), _p(ws), ws.numel(), _stream())
    return y, v


# ------------------------------------------------------------------------------------------ dense bf16 fused MLP
def mlp_fwd(x2, w_fc, w_proj):
    """(y [M,d], r [M,F]) bf16: y = bf16(bf16(r r) @ w_proj^T), r = bf16(relu(x2 @ w_fc^T)); w_fc [F,d], w_proj [d,F]
    (K/nki_mlp_fused.py:242). r is token-major (the reference's rT is r.t())."""
    _chk(x2), _chk(w_fc), _chk(w_proj)
    M, d = x2.shape
    F = w_fc.shape[0]
    if tuple(w_fc.shape) != (F, d) or tuple(w_proj.shape) != (d, F):
        raise ValueError("w_fc is [F, d], w_proj is [d, F]")
    y = torch.empty(M, d, dtype=bf16, device=x2.device)
    r = torch.empty(M, F, dtype=bf16, device=x2.device)
    h = torch.empty(M, F, dtype=bf16, device=x2.device)
    _lib.call("tfb_mlp_fwd", _p(x2), _p(w_fc), _p(w_proj), _p(y), _p(r), _p(h), M, d, F, _stream())
    return y, r


def mlp_bwd(dy2, r, w_fc, w_proj, want_h=True):
    """(dx [M,d], h [M,F] or None, dpre [M,F]) bf16: dpre = bf16(((dy2 @ w_proj) 2) r), h = bf16(r r), dx = bf16(dpre @ w_fc)
    (K/nki_mlp_fused.py:290 with dw_mode 0)."""
    _chk(dy2), _chk(r), _chk(w_fc), _chk(w_proj)
    M, d = dy2.shape
    F = w_fc.shape[0]
    if tuple(r.shape) != (M, F) or tuple(w_fc.shape) != (F, d) or tuple(w_proj.shape) != (d, F):
        raise ValueError("shapes differ")
    dx = torch.empty(M, d, dtype=bf16, device=dy2.device)
    dpre = torch.empty(M, F, dtype=bf16, device=dy2.device)
    h = torch.empty(M, F, dtype=bf16, device=dy2.device) if want_h else None
    _lib.call("tfb_mlp_bwd", _p(dy2), _p(r), _p(w_fc), _p(w_proj), _p(dx), _p(h), _p(dpre), M, d, F, _stream())
    return dx, h, dpre


# ------------------------------------------------------------------------------------------ gradient norm
def gradnorm(g_bf16=None, g_f32=None, clip=0.0):
    """fp32 [4] on the device: (sum of squares of g_bf16, of g_f32, the norm of both together, the clipping factor
    min(clip / (norm + 1e-6), 1), 1 when clip <= 0). Either buffer may be None (R1:1480, 1634)."""
    _chk(g_bf16), _chk(g_f32, torch.float32)
    ref = g_bf16 if g_bf16 is not None else g_f32
    if ref is None:
        raise ValueError("give at least one gradient buffer")
    out = torch.empty(4, dtype=torch.float32, device=ref.device)
    scr = _scratch(ref.device, int(_lib.lib().tfb_gradnorm_scratch_floats()))
    _lib.call("tfb_gradnorm", _p(g_bf16), 0 if g_bf16 is None else g_bf16.numel(), _p(g_f32),
              0 if g_f32 is None else g_f32.numel(), float(clip), _p(scr), _p(out), _stream())
    return out


# ------------------------------------------------------------------------------------------ mixer tail
def mix_tail_fwd(x2, lam, T, eps=2.0 ** -23):
    """(s1, xn2, inv): s1 = bf16(x2 + bf16(lam shift1(x2))) with shift1 inside sequences of T rows, xn2 = RMSNorm(s1);
    lam a 1-element fp32 device tensor (R1:7097)."""
    _chk(x2), _chk(lam, torch.float32)
    rows, C = x2.shape
    s1, xn2 = torch.empty_like(x2), torch.empty_like(x2)
    inv = torch.empty(rows, dtype=torch.float32, device=x2.device)
    _lib.call("tfb_mix_tail_fwd", _p(x2), _p(lam), _p(s1), _p(xn2), _p(inv), rows, C, int(T), float(eps), _stream())
    return s1, xn2, inv


def mix_tail_bwd(s1, inv, x2, lam, T, gy=None, ge=None):
    """(gx bf16 [rows,C], dlam fp32 [1]) from the gradients gy of xn2 and ge of s1 (either may be None) (R1:7145)."""
    _chk(s1), _chk(x2), _chk(gy), _chk(ge), _chk(inv, torch.float32), _chk(lam, torch.float32)
    if gy is None and ge is None:
        raise ValueError("give gy or ge")
    rows, C = s1.shape
    gx = torch.empty_like(s1)
    part = _scratch(s1.device, int(_lib.lib().tfb_norm_bwd_blocks(rows)))
    dlam = torch.empty(1, dtype=torch.float32, device=s1.device)
    _lib.call("tfb_mix_tail_bwd", _p(s1), _p(gy), _p(ge), _p(inv), _p(x2), _p(lam), _p(gx), _p(part), _p(dlam), rows, C, int(T),
              _stream())
    return gx, dlam
