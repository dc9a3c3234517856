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
