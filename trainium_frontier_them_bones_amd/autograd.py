"""torch.autograd.Function wrappers around the HIP ops: the same role the reference's `*Fn` classes play
(round1/source/train.py NkiAttnFn 8016, FcRelu2NNFn 4062, _ProjFn 3666, the loss head's LossHeadFn, Head2Fn 6599,
_LinearGemm / _LmHeadDwSplit 8419-8711). Weight gradients follow the reference's in-place convention
(round1/source/train.py:8463-8472): when a weight carries a `grad_buf` tensor the gradient GEMM accumulates into it
and autograd gets None for that weight; otherwise the gradient is returned as usual.
"""
import math

import torch

from . import ops

bf16 = torch.bfloat16


def _accumulate_into(w):
    """(buffer, accumulate flag) for a weight with an in-place gradient buffer, else (None, False)."""
    buf = getattr(w, "grad_buf", None)
    if buf is None:
        return None, False
    fresh = getattr(w, "grad_fresh", True)
    w.grad_fresh = False
    return buf, not fresh


def _tail_grads(ctx, gy):
    """Gradients of the optional trailing (x8, res) inputs of Linear8Fn / Mlp8Fn: none for the bytes, the output's
    gradient itself for the residual (the add's other operand)."""
    return (None, gy) if ctx.has_res else (None, None)


class RMSNormFn(torch.autograd.Function):
    """y = RMSNorm(x) * weight (weight optional)."""

    @staticmethod
    def forward(ctx, x, weight, eps):
        x = x.contiguous()
        _, y, inv = ops.rmsnorm_fwd(x, weight, eps)
        ctx.save_for_backward(x, inv, weight)
        return y

    @staticmethod
    def backward(ctx, gy):
        x, inv, weight = ctx.saved_tensors
        part = getattr(weight, "dw_part", None)
        if part is not None:   # the weight gradient is finished later, with the other norms', by ops.norm_dw_finish
            return ops.rmsnorm_bwd(gy.contiguous(), x, inv, weight, None, part=part)[0], None, None
        buf, acc = (None, False) if weight is None else _accumulate_into(weight)
        dx, dw = ops.rmsnorm_bwd(gy.contiguous(), x, inv, weight, None, buf, acc)
        if weight is None or buf is not None:
            return dx, None, None
        return dx, dw.to(weight.dtype), None


AMAX_HINT = "_tfb_amax_part"   # attribute on a gradient tensor: fp32 partials whose maximum is the tensor's amax
USE_AMAX_HINT = True           # False: consumers ignore the attribute and read the tensor for its amax


def _attach_amax(t, am):
    """Hang the amax partials of t's present contents on t, with t's version counter: an in-place update of t afterwards
    (autograd may add a second incoming gradient into it) makes the partials void."""
    setattr(t, AMAX_HINT, (am, t._version))
    return t


def _amax_hint(g, g2):
    """The amax partials the producer of gradient g attached to it, when g2 (the rows the caller will use) is g's own memory
    and g has not been written to since."""
    hint = getattr(g, AMAX_HINT, None) if USE_AMAX_HINT else None
    if hint is None:
        return None
    am, version = hint
    return am if (g._version == version and g2.data_ptr() == g.data_ptr() and g2.numel() == g.numel()) else None


_NAN = {}


def _nan_placeholder(like):
    """A tensor of like's shape and dtype without storage of its own: one NaN element (made once per device and dtype), expanded."""
    key = (like.device, like.dtype)
    if key not in _NAN:
        _NAN[key] = torch.full((1,), float("nan"), dtype=like.dtype, device=like.device)
    return _NAN[key].expand(like.shape)


class RMSNormPassFn(torch.autograd.Function):
    """(x, y[, y8]) = (x, RMSNorm(x) * weight[, e4m3(y * y8_scale)]) for a residual stream whose adds are made in the
    stores of the projections (LinearFn / Linear8Fn / Mlp8Fn with `res`): x is handed through so that the stream's
    gradient and the norm's meet in ONE backward launch (dx = g_x + J^T g_y), as in AddRMSNormFn. y8 is the operand cast
    of the fp8 GEMM that consumes y, made in the norm's pass (the norm prologue of round2/source/kernels/nki_mlp_nr8.py:1032
    and nki_attn_nr8.py:929)."""

    @staticmethod
    def forward(ctx, x, weight, eps, y8_scale=None, bytes_only=False):
        """bytes_only (with y8_scale): the consumer reads y8 alone (Mlp8Fn with its weight gradients in fp8 too), so the bf16
        rows of y are not written; the y handed back is then a placeholder of y's shape without storage of its own (one NaN
        element, expanded), there only to carry the gradient edge: whoever reads it gets NaN, not stale memory."""
        x = x.contiguous()
        ctx.set_materialize_grads(False)      # no zero tensor for the byte output's (or an unused output's) gradient
        if y8_scale is None:
            if bytes_only:
                raise ValueError("bytes_only needs y8_scale")
            _, y, inv = ops.rmsnorm_fwd(x, weight, eps)
            outs = (x, y)
        else:
            _, y, inv, y8 = ops.rmsnorm_fwd_q(x, weight, eps, None, float(y8_scale), want_y=not bytes_only)
            if y is None:
                y = _nan_placeholder(x)
            ctx.mark_non_differentiable(y8)
            outs = (x, y, y8)
        ctx.save_for_backward(x, inv, weight)
        return outs

    @staticmethod
    def backward(ctx, gs, gy, g8=None):
        x, inv, weight = ctx.saved_tensors
        gs = None if gs is None else gs.contiguous()
        if gy is None:
            return gs, None, None, None, None
        # the gradient handed upstream carries its amax partials (attribute AMAX_HINT): an fp8 MLP whose backward receives
        # this very tensor as its dy takes its scales from them instead of reading it once more
        part = getattr(weight, "dw_part", None)
        if part is not None:
            dx, _, am = ops.rmsnorm_bwd(gy.contiguous(), x, inv, weight, gs, part=part, want_amax=True)
            _attach_amax(dx, am)
            return dx, None, None, None, None
        buf, acc = (None, False) if weight is None else _accumulate_into(weight)
        dx, dw, am = ops.rmsnorm_bwd(gy.contiguous(), x, inv, weight, gs, buf, acc, want_amax=True)
        _attach_amax(dx, am)
        gw = dw.to(weight.dtype) if (weight is not None and buf is None) else None
        return dx, gw, None, None, None


class AddRMSNormFn(torch.autograd.Function):
    """(s, y) = (x + res, RMSNorm(x + res) * weight): the residual add fused in front of the norm
    (round1/source/train.py:6117 tail_norm2, 6826 final_norm)."""

    @staticmethod
    def forward(ctx, x, res, weight, eps):
        s, y, inv = ops.rmsnorm_fwd(x.contiguous(), weight, eps, res=res.contiguous())
        ctx.save_for_backward(s, inv, weight)
        return s, y

    @staticmethod
    def backward(ctx, gs, gy):
        s, inv, weight = ctx.saved_tensors
        part = getattr(weight, "dw_part", None)
        if part is not None and gy is not None:
            dx = ops.rmsnorm_bwd(gy.contiguous(), s, inv, weight, None if gs is None else gs.contiguous(), part=part)[0]
            return dx, dx, None, None
        if gy is None:
            return gs, gs, None, None
        buf, acc = (None, False) if weight is None else _accumulate_into(weight)   # (only once the buffer is surely written)
        dx, dw = ops.rmsnorm_bwd(gy.contiguous(), s, inv, weight, None if gs is None else gs.contiguous(), buf, acc)
        gw = dw.to(weight.dtype) if (weight is not None and buf is None) else None
        return dx, dx, gw, None


class BlockHeadFn(torch.autograd.Function):
    """(x_new, x_norm) = (l1 x + l2 x0 [+ l3 skip], RMSNorm(x_new)); gains are (1,) fp32 tensors."""

    @staticmethod
    def forward(ctx, x, x0, l1, l2, skip, l3, eps):
        gains = torch.cat([l1.reshape(1).float(), l2.reshape(1).float(),
                           (l3.reshape(1).float() if skip is not None else torch.zeros_like(l1.reshape(1).float()))])
        x, x0 = x.contiguous(), x0.contiguous()
        skip = None if skip is None else skip.contiguous()
        x_new, x_norm, inv = ops.block_head_fwd(x, x0, gains, skip, eps)
        ctx.save_for_backward(x, x0, skip, x_new, inv, gains)
        ctx.has_skip = skip is not None
        return x_new, x_norm

    @staticmethod
    def backward(ctx, g_new, g_norm):
        x, x0, skip, x_new, inv, gains = ctx.saved_tensors
        if g_norm is None:
            g_norm = torch.zeros_like(x)
        dx, dx0, dskip, dg = ops.block_head_bwd(None if g_new is None else g_new.contiguous(), g_norm.contiguous(), x, x0, x_new,
                                                inv, gains, skip)
        return dx, dx0, dg[0:1], dg[1:2], dskip, (dg[2:3] if ctx.has_skip else None), None


class LinearFn(torch.autograd.Function):
    """y = x @ w^T with w [out, in] (nn.Linear layout); dW accumulates into w.grad_buf when present."""

    @staticmethod
    def forward(ctx, x, w, res=None):
        x2 = x.reshape(-1, x.shape[-1]).contiguous()
        if res is None:
            y = ops.matmul(x2, w, trans_b=True)
        else:   # bf16(res + bf16(x @ w^T)): the residual add made in the GEMM's store (nki_attn_nr8.py:1003)
            y = ops.matmul_res(x2, w, res.reshape(-1, w.shape[0]).contiguous(), trans_b=True)
        ctx.save_for_backward(x2, w)
        ctx.xshape, ctx.has_res = x.shape, res is not None
        return y.view(*x.shape[:-1], w.shape[0])

    @staticmethod
    def backward(ctx, gy):
        x2, w = ctx.saved_tensors
        g2 = gy.reshape(-1, gy.shape[-1]).contiguous()
        dx = ops.matmul(g2, w).view(ctx.xshape)
        buf, acc = _accumulate_into(w)
        if buf is not None:
            ops.matmul(g2, x2, trans_a=True, out=buf, accumulate=acc)
            dw = None
        else:
            dw = ops.matmul(g2, x2, trans_a=True)
        return (dx, dw, gy) if ctx.has_res else (dx, dw)


class CausalAttentionFn(torch.autograd.Function):
    """nki_causal_attention(q, k, v, scale): q, k, v [B, H, T, D] -> [B, T, H, D] (round1/source/train.py:8069)."""

    @staticmethod
    def forward(ctx, q, k, v, scale, band=0):
        """band = nw > 0: the reference's tile band (K/nki_attn_bandpro.py:1654): keys of the last nw 128-token tiles."""
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        o, lse = ops.attn_fwd(q, k, v, scale, "bhtd", band)
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.scale, ctx.band = scale, band
        return o

    @staticmethod
    def backward(ctx, go):
        q, k, v, o, lse = ctx.saved_tensors
        # gradients in the inputs' own (contiguous [B, H, T, D]) layout: autograd then keeps them as they are instead of
        # copying a permuted dv into that layout (34 us of the 0.72 ms that B16 H12 T2048 D64 takes forward + backward)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        ops.attn_bwd(q, k, v, o, go.contiguous(), lse, ctx.scale, "bhtd", dq, dk, dv, "bhtd", band=ctx.band)
        return dq, dk, dv, None, None


class RopeAttentionFn(torch.autograd.Function):
    """Attention straight from the fused projection output qkv [B, T, 3C]: RoPE of the q and k thirds into a buffer of its
    own (the input is left untouched: whoever produced or saved it still holds the values it made), causal attention
    reading q, k from that buffer and v from qkv through strides, one dqkv [B, T, 3C] back (the call shape of
    nki_rope_attention, round1/source/train.py:8197, without its QK-norm)."""

    @staticmethod
    def forward(ctx, qkv, cos, sin, n_head, scale):
        B, T, C3 = qkv.shape
        C = C3 // 3
        D = C // n_head
        qkv = qkv.contiguous()
        rot = torch.empty(B, T, 2 * C, dtype=qkv.dtype, device=qkv.device)
        ops.rope_(qkv.view(B * T, C3), cos, sin, T, 2 * n_head, D, out=rot.view(B * T, 2 * C))
        q, k = (t.view(B, T, n_head, D) for t in rot.split(C, dim=-1))
        v = qkv[..., 2 * C:].view(B, T, n_head, D)
        o, lse = ops.attn_fwd(q, k, v, scale, "bthd")
        ctx.save_for_backward(qkv, rot, o, lse, cos, sin)
        ctx.n_head, ctx.scale = n_head, scale
        return o.view(B, T, C)

    @staticmethod
    def backward(ctx, go):
        qkv, rot, o, lse, cos, sin = ctx.saved_tensors
        B, T, C3 = qkv.shape
        C = C3 // 3
        H = ctx.n_head
        D = C // H
        q, k = (t.view(B, T, H, D) for t in rot.split(C, dim=-1))
        v = qkv[..., 2 * C:].view(B, T, H, D)
        dqkv = torch.empty_like(qkv)
        dq, dk, dv = (t.view(B, T, H, D) for t in dqkv.split(C, dim=-1))
        if D == 64:  # the inverse rotation of dq, dk rides the backward kernels' stores
            ops.attn_bwd(q, k, v, o, go.contiguous().view(B, T, H, D), lse, ctx.scale, "bthd", dq, dk, dv, "bthd", rope=(cos, sin))
        else:
            ops.attn_bwd(q, k, v, o, go.contiguous().view(B, T, H, D), lse, ctx.scale, "bthd", dq, dk, dv, "bthd")
            ops.rope_(dqkv.view(B * T, C3), cos, sin, T, 2 * H, D, inverse=True)
        return dqkv, None, None, None, None


class RopeNormFn(torch.autograd.Function):
    """norm(apply_rotary_emb(x, cos, sin)) for x [B, T, H, D]: RoPE then the parameter-free per-head RMSNorm
    (round1/source/train.py:4411 RopeNormFn; rope_norm 4447 returns this transposed to [B, H, T, D])."""

    @staticmethod
    def forward(ctx, x, cos, sin, eps):
        B, T, H, D = x.shape
        x = x.contiguous()
        y, r, inv = ops.rope_norm_fwd(x.view(B * T, H * D), cos, sin, T, H, D, eps)
        ctx.save_for_backward(r, inv, cos, sin)
        ctx.dims = (B, T, H, D)
        return y.view(B, T, H, D)

    @staticmethod
    def backward(ctx, gy):
        r, inv, cos, sin = ctx.saved_tensors
        B, T, H, D = ctx.dims
        dx = ops.rope_norm_bwd(gy.contiguous().view(B * T, H * D), r, inv, cos, sin, T, H, D)
        return dx.view(B, T, H, D), None, None, None


class RopeNormAttentionFn(torch.autograd.Function):
    """nki_rope_attention(qkv, cos, sin, n_head, scale) (round1/source/train.py:8197, NkiRopeAttnFn 8135): causal
    SDPA(QKnorm(RoPE(q)), QKnorm(RoPE(k)), v) straight from the fused projection output qkv [B, T, 3C], one dqkv
    [B, T, 3C] back. The input is not modified: the normalised q and k go to a fresh buffer, v is read in place through
    strides; saved for backward: qkv's v third, the rotated q, k (r5), their inverse RMS (inv3), o, lse."""

    @staticmethod
    def forward(ctx, qkv, cos, sin, n_head, scale, eps, band=0):
        """band = nw > 0: the tile-band form (round2/source/train.py:4925 fused_rope_attention_band)."""
        B, T, C3 = qkv.shape
        C = C3 // 3
        D = C // n_head
        qkv = qkv.contiguous()
        qk, r, inv = ops.rope_norm_fwd(qkv.view(B * T, C3), cos, sin, T, 2 * n_head, D, eps)
        q, k = (t.view(B, T, n_head, D) for t in qk.view(B, T, 2 * C).split(C, dim=-1))
        v = qkv[..., 2 * C:].view(B, T, n_head, D)
        o, lse = ops.attn_fwd(q, k, v, scale, "bthd", band)
        ctx.save_for_backward(qkv, qk, r, inv, o, lse, cos, sin)
        ctx.n_head, ctx.scale, ctx.band = n_head, scale, band
        return o.view(B, T, C)

    @staticmethod
    def backward(ctx, go):
        qkv, qk, r, inv, o, lse, cos, sin = ctx.saved_tensors
        B, T, C3 = qkv.shape
        C = C3 // 3
        H = ctx.n_head
        D = C // H
        q, k = (t.view(B, T, H, D) for t in qk.view(B, T, 2 * C).split(C, dim=-1))
        v = qkv[..., 2 * C:].view(B, T, H, D)
        dqkv = torch.empty_like(qkv)
        dq, dk, dv = (t.view(B, T, H, D) for t in dqkv.split(C, dim=-1))
        ops.attn_bwd(q, k, v, o, go.contiguous().view(B, T, H, D), lse, ctx.scale, "bthd", dq, dk, dv, "bthd", band=ctx.band)
        g2 = dqkv.view(B * T, C3)
        ops.rope_norm_bwd(g2, r, inv, cos, sin, T, 2 * H, D, out=g2)   # in place on the q and k thirds
        return dqkv, None, None, None, None, None, None


class QkvRopeAttentionFn(torch.autograd.Function):
    """Attention block core in one autograd node: qkv = rope(x @ w_qkv^T) (rotation in the projection's epilogue), causal
    attention on the thirds, and in backward the inverse rotation inside the attention kernels' stores followed by the
    projection's dX and dW (accumulated into w_qkv.grad_buf when present). Head dimension 64."""

    @staticmethod
    def forward(ctx, x, w_qkv, cos, sin, n_head, scale):
        B, T, Cin = x.shape
        C3 = w_qkv.shape[0]
        C = C3 // 3
        D = C // n_head
        x2 = x.reshape(B * T, Cin).contiguous()
        qkv = ops.qkv_rope(x2, w_qkv, cos, sin, T, 2 * C).view(B, T, C3)
        q, k, v = (t.view(B, T, n_head, D) for t in qkv.split(C, dim=-1))
        o, lse = ops.attn_fwd(q, k, v, scale, "bthd")
        ctx.save_for_backward(x2, w_qkv, qkv, o, lse, cos, sin)
        ctx.n_head, ctx.scale, ctx.xshape = n_head, scale, x.shape
        return o.view(B, T, C)

    @staticmethod
    def backward(ctx, go):
        x2, w, qkv, o, lse, cos, sin = ctx.saved_tensors
        B, T, C3 = qkv.shape
        C = C3 // 3
        H = ctx.n_head
        D = C // H
        q, k, v = (t.view(B, T, H, D) for t in qkv.split(C, dim=-1))
        dqkv = torch.empty_like(qkv)
        dq, dk, dv = (t.view(B, T, H, D) for t in dqkv.split(C, dim=-1))
        ops.attn_bwd(q, k, v, o, go.contiguous().view(B, T, H, D), lse, ctx.scale, "bthd", dq, dk, dv, "bthd", rope=(cos, sin))
        g2 = dqkv.view(B * T, C3)
        dx = ops.matmul(g2, w).view(ctx.xshape)
        buf, acc = _accumulate_into(w)
        if buf is not None:
            ops.matmul(g2, x2, trans_a=True, out=buf, accumulate=acc)
            return dx, None, None, None, None, None
        return dx, ops.matmul(g2, x2, trans_a=True), None, None, None, None


class Linear8State:
    """Per-weight fp8 state of a projection, refreshed once per optimizer step: the weight's power-of-two scale
    (s, 1/s, amax on the device) and its e4m3 bytes in both layouts (forward_scales / precast_ref,
    round2/source/kernels/nki_attn_tt8g.py:700, 795)."""

    def __init__(self, limit=240.0, dw_fp8=False):
        self.limit = limit
        self.dw_fp8 = dw_fp8   # the weight gradient in fp8 too (attn8_weight_grad, round2/source/train.py:8232)
        self.sc = None
        self.w8 = self.w8t = None

    def refresh(self, w):
        self.sc = ops.amax_scale(w.detach(), self.limit, -24, 40)
        self.w8, self.w8t = ops.precast8(w.detach(), self.sc[0:1])


class Linear8Fn(torch.autograd.Function):
    """y = x @ w^T with the forward in e4m3 x e4m3 and the input gradient in e5m2 x e4m3 (per-tensor power-of-two
    scales, fp32 accumulation, one bf16 rounding); the weight gradient in bf16, or with state.dw_fp8 in fp8 from the
    gradient's e5m2 bytes and the forward's e4m3 activation bytes (round2/source/train.py:8232 attn8_weight_grad);
    either is accumulated into w.grad_buf when present. x_scale: the reference's constant (4 for an RMSNorm output) or
    None for the per-tensor amax scale of x. The arithmetic of emulate_fwd / emulate_bwd (nki_attn_tt8g.py:745-757)."""

    @staticmethod
    def forward(ctx, x, w, state, x_scale, x8=None, res=None):
        """x8: the bytes e4m3(x * x_scale) when the norm that made x already cast them (RMSNormPassFn); res: a residual
        added in the GEMM's store, bf16(res + bf16(x @ w^T)) (nki_attn_nr8.py:1003)."""
        x2 = x.reshape(-1, x.shape[-1]).contiguous()
        r2 = None if res is None else res.reshape(-1, w.shape[0]).contiguous()
        if x_scale is None:
            sx = ops.amax_scale(x2, state.limit, -24, 40)
            x8 = ops.quant_fp8(x2, sx[0:1], ops.FMT_E4M3)
            dq_a, dq = sx[1:2], 1.0
            ctx.sx, ctx.sx_imm = sx[0:1], 1.0
        else:
            x8 = ops.quant_fp8(x2, float(x_scale), ops.FMT_E4M3) if x8 is None else x8.reshape(x2.shape)
            dq_a, dq = None, 1.0 / float(x_scale)
            ctx.sx, ctx.sx_imm = None, 1.0 / float(x_scale)
        if r2 is None:
            y = ops.gemm_fp8(x8, state.w8, ops.FMT_E4M3, dq_a, state.sc[1:2], dq)
        else:
            y = ops.gemm_fp8_res(x8, state.w8, r2, dq_a, state.sc[1:2], dq)
        ctx.save_for_backward(x8 if state.dw_fp8 else x2, w)
        ctx.state, ctx.xshape, ctx.nin = state, x.shape, 4 + (x8 is not None) + (res is not None)
        ctx.has_res = res is not None
        return y.view(*x.shape[:-1], w.shape[0])

    @staticmethod
    def backward(ctx, gy):
        xa, w = ctx.saved_tensors
        st = ctx.state
        g2 = gy.reshape(-1, gy.shape[-1]).contiguous()
        sg = ops.amax_scale(g2, 57344.0 / 2.0, -40, 60)
        g8 = ops.quant_fp8(g2, sg[0:1], ops.FMT_E5M2)
        dx = ops.gemm_fp8(g8, st.w8t, ops.FMT_E5M2, sg[1:2], st.sc[1:2]).view(ctx.xshape)
        buf, acc = _accumulate_into(w)
        if st.dw_fp8:
            dw = ops.gemm_fp8_tn(g8, xa, ops.FMT_E5M2, ops.FMT_E4M3, sg[0:1], ctx.sx, ctx.sx_imm, out=buf, accumulate=acc)
        else:
            dw = ops.matmul(g2, xa, trans_a=True, out=buf, accumulate=acc)
        return (dx, (None if buf is not None else dw), None, None) + _tail_grads(ctx, gy)


class Mlp8State:
    """Per-layer fp8 state refreshed once per optimizer step: the scale row and the e4m3 weight pack
    (round2/source/train.py:6617 fp8_refresh_weights, 7003 mlp8_scales_into, 7267 mlp8_precast_into)."""

    def __init__(self, e4m3_limit=240.0, x_scale=4.0, dw_fp8=False):
        self.e4m3_limit, self.x_scale = e4m3_limit, x_scale
        self.dw_fp8 = dw_fp8   # weight gradients in fp8 too (round2/source/train.py:8209 under its switch 9k; R1 DW_ROWS)
        self.row = None
        self.w8 = None

    def refresh(self, w_fc, w_proj):
        self.row = ops.mlp8_forward_scales(w_fc.detach(), w_proj.detach(), self.e4m3_limit, self.x_scale)
        self.w8 = ops.mlp8_precast(w_fc.detach(), w_proj.detach(), self.row)


class Mlp8Fn(torch.autograd.Function):
    """y = c_proj(relu(c_fc(x))^2) with the four activation GEMMs in fp8 and the weight gradients in bf16
    (K/nki_mlp_fused8.py:706 weight_grads) or, with state.dw_fp8, in fp8 from the bytes the other GEMMs multiplied
    (round2/source/train.py:8209 mlp8_weight_grads)."""

    @staticmethod
    def forward(ctx, x, w_fc, w_proj, state, x8=None, res=None):
        """x8: the bytes e4m3(x * state.x_scale) when the norm that made x already cast them (RMSNormPassFn); res: the
        block's residual, added in the second GEMM's store: y = bf16(res + bf16(MLP(x))) (nki_mlp_nr8.py:1032)."""
        rows2 = (x.numel() // x.shape[-1], x.shape[-1])
        x8 = None if x8 is None else x8.reshape(rows2)
        r2 = None if res is None else res.reshape(rows2).contiguous()
        # with the bytes given and the weight gradients in fp8 nothing reads x itself (it may be a storage-less placeholder)
        x2 = None if (x8 is not None and state.dw_fp8) else x.reshape(rows2).contiguous()
        if state.dw_fp8:
            y, r, x8 = ops.mlp8_fwd(x2, state.w8, state.row, w_fc.shape[0], state.x_scale, want_x8=True, x8=x8, res=r2)
            ctx.save_for_backward(x8, r, w_fc, w_proj)
        else:
            y, r = ops.mlp8_fwd(x2, state.w8, state.row, w_fc.shape[0], state.x_scale, x8=x8, res=r2)
            ctx.save_for_backward(x2, r, w_fc, w_proj)
        ctx.state = state
        ctx.xshape, ctx.has_res = x.shape, res is not None
        return y.view(x.shape)

    @staticmethod
    def backward(ctx, gy):
        x2, r, w_fc, w_proj = ctx.saved_tensors
        st = ctx.state
        g2 = gy.reshape(-1, gy.shape[-1]).contiguous()
        rowb = ops.mlp8_backward_scales(g2, st.row, _amax_hint(gy, g2))
        if st.dw_fp8:
            dx, _, dp8, hq8, dy8 = ops.mlp8_bwd_q(g2, r, st.w8, rowb, st.e4m3_limit, want_dpre=False)
            (bf, af), (bp, ap) = _accumulate_into(w_fc), _accumulate_into(w_proj)
            if (bf is None) != (bp is None) or af != ap:
                raise RuntimeError("the fp8 weight gradients write both MLP weights' gradient buffers in one call")
            if bf is not None:
                ops.mlp8_dw8(x2, dp8, hq8, dy8, rowb, st.x_scale, dw_fc=bf, dw_proj=bp, accumulate=af)
                return (dx.view(ctx.xshape), None, None, None) + _tail_grads(ctx, gy)
            dw_fc, dw_proj = ops.mlp8_dw8(x2, dp8, hq8, dy8, rowb, st.x_scale)
            return (dx.view(ctx.xshape), dw_fc, dw_proj, None) + _tail_grads(ctx, gy)
        dx, _, dpre = ops.mlp8_bwd(g2, r, st.w8, rowb, want_h=False)
        buf, acc = _accumulate_into(w_fc)
        if buf is not None:
            ops.matmul(dpre, x2, trans_a=True, out=buf, accumulate=acc)
            dw_fc = None
        else:
            dw_fc = ops.matmul(dpre, x2, trans_a=True)
        buf, acc = _accumulate_into(w_proj)
        if buf is not None:
            ops.mlp_dw_proj(g2, r, out=buf, accumulate=acc)
            dw_proj = None
        else:
            dw_proj = ops.mlp_dw_proj(g2, r)
        return (dx.view(ctx.xshape), dw_fc, dw_proj, None) + _tail_grads(ctx, gy)


class NrMlpFn(torch.autograd.Function):
    """x_out = x1 + MLP(rms_norm(x1)) for a dense block on rows x1 [M, d] (round2/source/train.py:9168 NrMlp): the norm
    (parameter-free, eps 2^-23) also writes the MLP's e4m3 operand, the residual add is made in the second GEMM's store,
    and in the backward the norm's backward and the residual gradient's add are one launch (gx = g + J^T dxn)."""

    @staticmethod
    def forward(ctx, x2, w_fc, w_proj, state, eps=2.0 ** -23):
        x2 = x2.contiguous()
        # (with the weight gradients in fp8 too nothing reads the norm's bf16 rows: only its e4m3 bytes are written)
        _, xn, inv, x8 = ops.rmsnorm_fwd_q(x2, None, eps, None, state.x_scale, want_y=not state.dw_fp8)
        xo, r = ops.mlp8_fwd(xn, state.w8, state.row, w_fc.shape[0], state.x_scale, x8=x8, res=x2)
        ctx.save_for_backward(x2, x8 if state.dw_fp8 else xn, inv, r, w_fc, w_proj)
        ctx.state = state
        return xo

    @staticmethod
    def backward(ctx, g):
        x2, xa, inv, r, w_fc, w_proj = ctx.saved_tensors
        st = ctx.state
        g_in, g = g, g.contiguous()
        rowb = ops.mlp8_backward_scales(g, st.row, _amax_hint(g_in, g))
        if st.dw_fp8:
            dxn, _, dp8, hq8, dy8 = ops.mlp8_bwd_q(g, r, st.w8, rowb, st.e4m3_limit, want_dpre=False)
            dw_fc, dw_proj = ops.mlp8_dw8(xa, dp8, hq8, dy8, rowb, st.x_scale)
        else:
            dxn, _, dpre = ops.mlp8_bwd(g, r, st.w8, rowb, want_h=False)
            dw_fc = ops.matmul(dpre, xa, trans_a=True)
            dw_proj = ops.mlp_dw_proj(g, r)
        gx, _, am = ops.rmsnorm_bwd(dxn, x2, inv, None, g, want_amax=True)
        _attach_amax(gx, am)      # for the block before this one, whose backward receives gx as its dy
        return gx, dw_fc, dw_proj, None, None


LM_HEAD_ONE_PASS = True   # False: LmHeadLossFn always takes the GEMM with the lse epilogue and the separate loss backward


class LmHeadLossFn(torch.autograd.Function):
    """loss = reduce(CE(softcap(x @ W^T), targets)). When a gradient is wanted the forward is the plain LM-head GEMM followed
    by ONE pass over the logits that writes lse and the row losses and leaves, in place of the logits, their gradient for an
    upstream gradient of one; the backward is the two gradient GEMMs, each multiplying its product by the upstream scalar
    (a device value) before its rounding. The logits thus make one trip to HBM each way, and nothing recomputes an
    exponential. Without a gradient (or beyond the one-pass kernel's vocabulary limit) the GEMM with the log-sum-exp in its
    epilogue runs instead, and a backward from there writes dlogits in place of the logits first."""

    _caller_grad_mode = True

    @classmethod
    def apply(cls, *args):
        # inside forward() the grad mode is always off, and needs_input_grad is True for parameters under torch.no_grad()
        # as well: the caller's mode is noted here, so that evaluation takes the cheaper forward
        cls._caller_grad_mode = torch.is_grad_enabled()
        return super().apply(*args)

    @staticmethod
    def forward(ctx, x, W, targets, softcap, reduction):
        x2 = x.reshape(-1, x.shape[-1]).contiguous()
        tg = targets.reshape(-1)
        w = ops.loss_row_weights(tg, reduction, W.shape[0])
        ctx.softcap = softcap
        ctx.xshape = x.shape
        ctx.one_pass = (LM_HEAD_ONE_PASS and LmHeadLossFn._caller_grad_mode
                        and (ctx.needs_input_grad[0] or ctx.needs_input_grad[1])
                        and W.shape[0] <= ops.LOSS_FWD_BWD_MAX_V)
        if ctx.one_pass:
            dl = ops.matmul(x2, W, trans_b=True)
            rows, _ = ops.loss_fwd_bwd(dl, tg, w, softcap)
            ctx.save_for_backward(x2, W, dl)
            return rows.sum()
        logits, rows, lse = ops.lmhead_fwd(x2, W, tg, softcap, w)
        ctx.save_for_backward(x2, W, tg, logits, lse, w)
        return rows.sum()

    @staticmethod
    def backward(ctx, g):
        if ctx.one_pass:
            x2, W, dl = ctx.saved_tensors
            alpha = g.detach().to(torch.float32).reshape(1)
        else:
            x2, W, tg, logits, lse, w = ctx.saved_tensors
            if getattr(ctx, "logits_consumed", False):
                raise RuntimeError("LmHeadLossFn: second backward through the same node (retain_graph): the saved logits "
                                   "were overwritten by their gradient in the first one")
            ctx.logits_consumed = True
            grow = (w * g.to(torch.float32)).contiguous()
            dl = ops.loss_bwd(logits, tg, lse, grow, ctx.softcap, inplace=True)
            alpha = None
        dx = ops.matmul(dl, W, alpha=alpha).view(ctx.xshape)
        buf, acc = _accumulate_into(W)
        if buf is not None:
            ops.matmul(dl, x2, trans_a=True, out=buf, accumulate=acc, alpha=alpha)
            return dx, None, None, None, None
        return dx, ops.matmul(dl, x2, trans_a=True, alpha=alpha), None, None, None


class FusedLossFn(torch.autograd.Function):
    """fused_loss(logits, targets, reduction, softcap) rows on materialised logits (round1/source/train.py:4691)."""

    @staticmethod
    def forward(ctx, logits2, targets, softcap):
        rows, lse = ops.loss_fwd(logits2, targets, softcap)
        ctx.save_for_backward(logits2, targets, lse)
        ctx.softcap = softcap
        return rows

    @staticmethod
    def backward(ctx, grows):
        logits2, targets, lse = ctx.saved_tensors
        return ops.loss_bwd(logits2, targets, lse, grows.contiguous().float(), ctx.softcap), None, None


class FusedLossMultiFn(torch.autograd.Function):
    """rows [N] = sum_k rw[k] (lse - (1 - eps) s_{t_k} - eps mean_v s_v) on materialised logits: several targets per row
    (round1/source/train.py:4870 LossMultiFn) and / or label smoothing (round2/source/train.py:6344 ChunkedLossHeadLS)."""

    @staticmethod
    def forward(ctx, logits2, tg, rw, softcap, eps):
        rows, lse = ops.loss_multi_fwd(logits2, tg, rw, softcap, eps)
        ctx.save_for_backward(logits2, tg, rw, lse)
        ctx.softcap, ctx.eps = softcap, eps
        return rows

    @staticmethod
    def backward(ctx, grows):
        logits2, tg, rw, lse = ctx.saved_tensors
        return ops.loss_multi_bwd(logits2, tg, rw, lse, grows.contiguous().float(), ctx.softcap, ctx.eps), None, None, None, None


class EmbeddingFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, idx, weight):
        ctx.save_for_backward(idx, weight)
        return ops.embedding_fwd(idx, weight)

    @staticmethod
    def backward(ctx, gy):
        idx, weight = ctx.saved_tensors
        buf, acc = _accumulate_into(weight)
        if buf is not None:
            if not acc:
                ops.fill_f32_(buf, 0.0)
            ops.embedding_bwd(idx, gy.contiguous(), buf)
            return None, None
        dw = ops.fill_f32_(torch.empty(weight.shape, dtype=torch.float32, device=weight.device), 0.0)
        ops.embedding_bwd(idx, gy.contiguous(), dw)
        return None, dw.to(weight.dtype)


class Relu2Fn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        x = x.contiguous()
        ctx.save_for_backward(x)
        return ops.relu2(x)

    @staticmethod
    def backward(ctx, gy):
        (x,) = ctx.saved_tensors
        return ops.relu2_bwd(x, gy.contiguous())


def default_scale(D):
    return 1.0 / math.sqrt(D)


class Moe8State:
    """Per-layer fp8 state of the experts, refreshed once per optimizer step: a scale row and an e4m3 weight pack per
    expert (the reference's exp8_sc [E,128,16] / exp8_w8 buffers, round2/source/train.py:10900-10935)."""

    def __init__(self, e4m3_limit=240.0, x_scale=4.0, dw_fp8=False):
        """dw_fp8: the experts' weight gradients in fp8 as well, from the bytes the other four GEMMs multiplied (the
        reference's fp8 weight-gradient switch, round2/source/train.py:8209-8229, inside each expert's backward)."""
        self.e4m3_limit, self.x_scale, self.dw_fp8 = e4m3_limit, x_scale, dw_fp8
        self.rows = None
        self.w8 = None

    def refresh(self, w_fc, w_proj):
        E, F, d = w_fc.shape
        wf, wp = w_fc.detach(), w_proj.detach()
        if wf.is_contiguous() and wp.is_contiguous():      # the experts as E layers of one flat buffer: four launches
            self.rows, self.w8 = ops.mlp8_refresh_layers(wf[0], wp[0], F * d, E, self.e4m3_limit, self.x_scale)
            return
        rows = [ops.mlp8_forward_scales(wf[e], wp[e], self.e4m3_limit, self.x_scale) for e in range(E)]
        self.rows = torch.stack(rows).contiguous()
        self.w8 = torch.stack([ops.mlp8_precast(wf[e], wp[e], rows[e]) for e in range(E)]).contiguous()


class MoeMlp8Fn(torch.autograd.Function):
    """The routed half of MoeMLP.forward_e8 (round2/source/train.py:11003-11067) with every expert on this GPU:
    router -> top-k -> dropless dispatch -> grouped fp8 expert MLPs -> gated combine. h [.., d] bf16, router fp32 [E, d],
    w_fc [E, F, d], w_proj [E, d, F] bf16; router_bias fp32 [E] or None (added to the logits).
    state None: the experts run in bf16 (MoeMLP.forward with moe_experts_local, round2/source/train.py:10941-11001, 10716:
    the kit's expression per expert, d and F multiples of 128)."""

    @staticmethod
    def forward(ctx, h, router, w_fc, w_proj, state, topk, router_bias, aux_weights=None, capacity=None, info=None):
        """aux_weights = (alpha, beta): also returns (aux, stats) with aux = alpha lb + beta z, the router's weighted
        load-balance and z terms (round2/source/train.py:10779 moe_aux_terms; differentiable, its gradient joins the
        router's in the backward), and stats fp32 [2 + E] = (lb, z, the experts' load shares f_e).
        aux_weights = (alpha, beta, gamma) adds gamma times the per-sequence balance term (the reference's R2_MOE_AUX_SEQ,
        10789-10792), the sequences being the rows of h [b, t, d].
        info: a dict that receives "kept" = the share of the assignments that hold a row (1 without a capacity), the first
        entry of the reference layer's statistics vector."""
        h2 = h.reshape(-1, h.shape[-1]).contiguous()
        E, F, d = w_fc.shape
        wr = router.detach().float().contiguous()
        p, idx, gate, logits = ops.moe_route(h2, wr, topk, router_bias, want_logits=aux_weights is not None)
        # capacity: the reference's per-sequence count (round2/source/train.py:10555): each row of h [b, t, d] keeps its first
        # `capacity` assignments per expert; None keeps everything
        tab = ops.moe_tables(idx, E) if capacity is None else ops.moe_tables(idx, E, h.shape[-2], capacity)
        if state is not None:
            xs, xs8 = ops.moe_gather(h2, tab, state.x_scale, want_xs=not state.dw_fp8)
            ys, r = ops.moe_mlp8_fwd(xs8, state.w8, state.rows, tab, F)
        else:
            xs, _ = ops.moe_gather(h2, tab, None)
            ys, r, _h = ops.moe_mlp_fwd(xs, w_fc.detach().to(bf16).contiguous(), w_proj.detach().to(bf16).contiguous(), tab)
        out = ops.moe_combine(ys, tab, gate, h2.shape[0])
        if info is not None:
            info["kept"] = tab["cnt"].sum().float() / float(h2.shape[0] * topk)
        ctx.tab, ctx.state, ctx.hshape, ctx.aux_weights = tab, state, h.shape, aux_weights
        ctx.xs8 = xs8 if state is not None and state.dw_fp8 else None    # the fp8 weight gradient's operand (not an input of any op)
        if aux_weights is None:
            ctx.save_for_backward(h2, wr, p, idx, gate, xs, ys, r, router, w_fc, w_proj)
            return out.view(h.shape)
        terms, lse = ops.moe_aux_fwd(p, logits, tab, topk)
        aux = float(aux_weights[0]) * terms[0] + float(aux_weights[1]) * terms[1]
        if len(aux_weights) > 2 and float(aux_weights[2]) != 0.0:
            if h.dim() < 3:
                raise ValueError("MoeMlp8Fn: the per-sequence balance term needs h [b, t, d]")
            seq_term, fs = ops.moe_aux_seq_fwd(p, idx, h.shape[-2], topk)
            aux = aux + float(aux_weights[2]) * seq_term[0]
            ctx.seq_len = h.shape[-2]
            ctx.save_for_backward(h2, wr, p, idx, gate, xs, ys, r, router, w_fc, w_proj, terms, lse, fs)
        else:
            ctx.seq_len = None
            ctx.save_for_backward(h2, wr, p, idx, gate, xs, ys, r, router, w_fc, w_proj, terms, lse)
        ctx.mark_non_differentiable(terms)
        return out.view(h.shape), aux, terms

    @staticmethod
    def backward(ctx, gout, gaux=None, _gterms=None):
        if ctx.aux_weights is None:
            h2, wr, p, idx, gate, xs, ys, r, router, w_fc, w_proj = ctx.saved_tensors
            aux = None
        else:
            h2, wr, p, idx, gate, xs, ys, r, router, w_fc, w_proj, terms, lse = ctx.saved_tensors[:13]
            ga = torch.zeros(1, dtype=torch.float32, device=h2.device) if gaux is None else gaux.reshape(1).float().contiguous()
            aux = (terms, lse, ga, ctx.aux_weights[0], ctx.aux_weights[1])
            if ctx.seq_len is not None:
                aux = aux + (ctx.saved_tensors[13], ctx.aux_weights[2], ctx.seq_len)
        tab, st = ctx.tab, ctx.state
        E = w_fc.shape[0]
        if gout is None:
            gout = torch.zeros(ctx.hshape, dtype=h2.dtype, device=h2.device)
        g2 = gout.reshape(-1, gout.shape[-1]).contiguous()
        dw8 = st is not None and st.dw_fp8
        if st is not None:   # the experts' amax(dys) rides the kernel that writes dys
            dys, dgate, rowmax = ops.moe_combine_bwd(g2, ys, tab, gate, want_rowmax=True)
            rows_b = ops.moe_backward_scales_rowmax(rowmax, st.rows, tab, dys.shape[1])
        else:
            dys, dgate = ops.moe_combine_bwd(g2, ys, tab, gate)
        if dw8:
            dxs, dp8, hq8, dy8 = ops.moe_mlp8_bwd_q(dys, r, st.w8, rows_b, tab, st.e4m3_limit)
        elif st is not None:
            dxs, dpre = ops.moe_mlp8_bwd(dys, r, st.w8, rows_b, tab)
        else:
            dxs, dpre = ops.moe_mlp_bwd(dys, r, w_fc.detach().to(bf16).contiguous(), w_proj.detach().to(bf16).contiguous(), tab)
        # one grouped launch writes both gradients: both weights carry a gradient buffer (in the same state) or neither
        # does; the "fresh" flags are only touched on the branch that really writes the buffers
        if (getattr(w_fc, "grad_buf", None) is None) != (getattr(w_proj, "grad_buf", None) is None):
            raise RuntimeError("MoeMlp8Fn: give both expert weights a grad_buf, or neither")
        if getattr(w_fc, "grad_buf", None) is not None:
            (bf, accf), (bp, accp) = _accumulate_into(w_fc), _accumulate_into(w_proj)
            if accf != accp:
                raise RuntimeError("MoeMlp8Fn: the two expert weights' gradient buffers are in different states")
            if dw8:
                ops.moe_dw8(ctx.xs8, dp8, hq8, dy8, rows_b, st.x_scale, tab, E, bf, bp, accumulate=accf)
            else:
                ops.moe_dw(dpre, xs, dys, r, tab, E, bf, bp, accumulate=accf)
            dw_fc = dw_proj = None
        elif dw8:
            dw_fc, dw_proj = ops.moe_dw8(ctx.xs8, dp8, hq8, dy8, rows_b, st.x_scale, tab, E)
        else:
            dw_fc, dw_proj = ops.moe_dw(dpre, xs, dys, r, tab, E)
        br, accr = _accumulate_into(router)
        dh, dwr, _ = ops.moe_route_bwd(dgate, p, idx, dxs, tab, h2, wr, br, accr, aux=aux)
        return (dh.view(ctx.hshape), (None if br is not None else dwr.to(router.dtype)), dw_fc, dw_proj, None, None, None, None,
                None, None)


class MlpFusedFn(torch.autograd.Function):
    """The dense bf16 fused MLP: y = c_proj(relu(c_fc(x))^2) on [M, d] rows with the fused kernels' rounding points; saves
    x2 and r only; dW accumulates into the weights' grad_buf when present (round2/source/kernels/nki_mlp_fused.py:408
    EmulatedFusedMlp; kernels :242, :290)."""

    @staticmethod
    def forward(ctx, x2, w_fc, w_proj):
        x2 = x2.contiguous()
        y, r = ops.mlp_fwd(x2, w_fc, w_proj)
        ctx.save_for_backward(x2, r, w_fc, w_proj)
        return y

    @staticmethod
    def backward(ctx, dy):
        x2, r, w_fc, w_proj = ctx.saved_tensors
        dy = dy.contiguous()
        dx, h, dpre = ops.mlp_bwd(dy, r, w_fc, w_proj)
        grads = []
        for w, a, b in ((w_fc, dpre, x2), (w_proj, dy, h)):     # dw_fc = dpre^T x, dw_proj = dy^T h
            buf, acc = _accumulate_into(w)
            if buf is not None:
                ops.matmul(a, b, trans_a=True, out=buf, accumulate=acc)
                grads.append(None)
            else:
                grads.append(ops.matmul(a, b, trans_a=True))
        return dx, grads[0], grads[1]


class MixTailFn(torch.autograd.Function):
    """(s1, xn2) = (x + lam shift1(x), RMSNorm(s1)) on the [N, C] stream, sequences of T rows; gradients (gx, dlam)
    (round1/source/train.py:7330 MixTailFn)."""

    @staticmethod
    def forward(ctx, x2, lam, T):
        ctx.set_materialize_grads(False)
        x2 = x2.contiguous()
        lam32 = lam.detach().reshape(1).to(torch.float32)
        s1, xn2, inv = ops.mix_tail_fwd(x2, lam32, T)
        ctx.save_for_backward(x2, s1, inv, lam32)
        ctx.T, ctx.lam_meta = T, (lam.shape, lam.dtype)
        return s1, xn2

    @staticmethod
    def backward(ctx, ge, gy):
        x2, s1, inv, lam32 = ctx.saved_tensors
        if ge is None and gy is None:
            return None, None, None
        gx, dlam = ops.mix_tail_bwd(s1, inv, x2, lam32, ctx.T, None if gy is None else gy.contiguous(),
                                    None if ge is None else ge.contiguous())
        shape, dtype = ctx.lam_meta
        return gx, dlam.to(dtype).reshape(shape), None
