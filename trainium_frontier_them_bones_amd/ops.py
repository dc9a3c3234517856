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
    """One fp32 split-K workspace per device, allocated on first use."""
    ws = _WS.get(device)
    if ws is None or ws.numel() * 4 < nbytes:
        ws = torch.empty(nbytes // 4, dtype=torch.float32, device=device)
        _WS[device] = ws
    return ws


def matmul(a, b, trans_a=False, trans_b=False, out=None, accumulate=False, out_dtype=bf16):
    """op(a) @ op(b) with fp32 accumulation. a is [M,K] (or [K,M] with trans_a), b is [K,N] (or [N,K] with
    trans_b). `out` (bf16 or fp32) may be given; accumulate=True adds into it (one rounding)."""
    _chk(a), _chk(b)
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
    _lib.call("tfb_gemm_bf16", _p(a), _p(b), _p(out), M, N, K, int(trans_a), int(trans_b),
              int(out.dtype == torch.float32), int(accumulate), _p(ws), ws.numel() * 4, _stream())
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


def rmsnorm_bwd(gy, s, inv, weight=None, gs=None, dw=None):
    """dx = gs + J^T(gy) for y = RMSNorm(s) * weight. Returns (dx, dw fp32 [C] or None); dw given => accumulated into."""
    _chk(gy), _chk(s), _chk(weight), _chk(gs), _chk(inv, torch.float32)
    C = s.shape[-1]
    rows = s.numel() // C
    dx = torch.empty_like(s)
    part = None
    acc = 0
    if weight is not None:
        nb = _lib.lib().tfb_norm_bwd_blocks(rows)
        part = torch.empty(nb, C, dtype=torch.float32, device=s.device)
        if dw is None:
            dw = torch.empty(C, dtype=torch.float32, device=s.device)
        else:
            _chk(dw, torch.float32)
            acc = 1
    _lib.call("tfb_rmsnorm_bwd", _p(gy), _p(gs), _p(s), _p(weight), _p(inv), _p(dx), _p(part), _p(dw), acc, rows, C,
              _stream())
    return dx, dw


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


def mlp8_forward_scales(w_fc, w_proj, e4m3_limit=240.0, x_scale=4.0):
    """The layer's fp32 [16] scale row, computed on the device from the bf16 weights (w_fc [F,d], w_proj [d,F])."""
    _chk(w_fc), _chk(w_proj)
    F, d = w_fc.shape
    if tuple(w_proj.shape) != (d, F):
        raise ValueError("w_proj must be [d, F]")
    row = torch.empty(NSC, dtype=torch.float32, device=w_fc.device)
    scr = _scratch(w_fc.device, _lib.lib().tfb_mlp8_scale_scratch_floats(F))
    _lib.call("tfb_mlp8_forward_scales", _p(w_fc), _p(w_proj), _p(row), _p(scr), F, d, float(e4m3_limit), float(x_scale),
              _stream())
    return row


def mlp8_backward_scales(dy2, row):
    _chk(dy2), _chk(row, torch.float32)
    M, d = dy2.shape
    out = torch.empty(NSC, dtype=torch.float32, device=dy2.device)
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


def mlp8_precast(w_fc, w_proj, row):
    """uint8 [4, F*d]: w_fc and w_proj cast once to e4m3 at the row's scales, each in both byte layouts."""
    _chk(w_fc), _chk(w_proj), _chk(row, torch.float32)
    F, d = w_fc.shape
    w8 = torch.empty(4, F * d, dtype=torch.uint8, device=w_fc.device)
    _lib.call("tfb_mlp8_precast", _p(w_fc), _p(w_proj), _p(row), _p(w8), F, d, _stream())
    return w8


def mlp8_fwd(x2, w8, row, F, x_scale=4.0):
    """y [M,d], r [M,F] (bf16): the fp8 forward. x_scale: python float (the reference's constant 4) or a device scalar."""
    _chk(x2), _chk(w8, torch.uint8), _chk(row, torch.float32)
    M, d = x2.shape
    x8 = quant_fp8(x2, x_scale, FMT_E4M3)
    y = torch.empty(M, d, dtype=bf16, device=x2.device)
    r = torch.empty(M, F, dtype=bf16, device=x2.device)
    h8 = torch.empty(M, F, dtype=torch.uint8, device=x2.device)
    _lib.call("tfb_mlp8_fwd", _p(x8), _p(w8), _p(row), _p(y), _p(r), _p(h8), M, d, F, _stream())
    return y, r


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
