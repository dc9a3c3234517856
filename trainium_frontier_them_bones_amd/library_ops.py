"""torch.library registration of the kernel calls, in the form of the reference's round2 sources: `torch.library.custom_op(name,
mutates_args=())` + `register_fake` (the op's own output allocations) + `register_autograd` with a `setup_context` that
marks the auxiliary outputs non-differentiable and switches gradient materialisation off
(round2/source/train.py:4988-5036 s2attn::*, 6858-6913 s2mlp8::*, 7127-7160 s2mlp8l::*, 6145-6156 s2b::loss_head_*).
The ops allocate and return fresh outputs and mutate nothing, so they can be traced.

Registered (namespace `tfb`):
  tfb::attn_fwd(q, k, v, scale) -> (o [B,T,H,D], lse [B,H,T])          tfb::attn_bwd(q, k, v, o, do, lse, scale) -> (dq, dk, dv)
  tfb::mlp8_precast(w_fc, w_proj, sc) -> w8 [4, F d]                    (s2mlp8l::precast)
  tfb::mlp8_fwd(x2, w_fc, w_proj, sc, w8) -> (y [M,d], rT [F,M])        (s2mlp8l::fwd; rT is the reference's shape, here the
                                                                         transposed VIEW of the token-major r [M,F] the kernels keep)
  tfb::mlp8_bwd(dy2, rT, x2, w_fc, w_proj, sc, w8) -> (dx, dw_fc, dw_proj)  (s2mlp8l::bwd)
  tfb::loss_head_fwd(logits, targets, row_w, softcap) -> (loss_rows, lz)    tfb::loss_head_bwd(logits, targets, lz, g, softcap) -> dlogits
`register()` is idempotent and returns the dict of op callables.
"""
import torch

from . import ops

_OPS = {}


def register():
    if _OPS:
        return _OPS
    op = torch.library.custom_op

    # ---------------------------------------------------------------- attention (R2:4988 form, R1:8016 NkiAttnFn arithmetic)
    @op("tfb::attn_fwd", mutates_args=())
    def attn_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float) -> tuple[torch.Tensor, torch.Tensor]:
        return ops.attn_fwd(q.contiguous(), k.contiguous(), v.contiguous(), scale, "bhtd")

    @op("tfb::attn_bwd", mutates_args=())
    def attn_bwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, o: torch.Tensor, do: torch.Tensor, lse: torch.Tensor,
                 scale: float) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        dq, dk, dv = ops.attn_bwd(q.contiguous(), k.contiguous(), v.contiguous(), o, do.contiguous(), lse, scale, "bhtd")
        return dq, dk, dv.contiguous()

    @torch.library.register_fake("tfb::attn_fwd")
    def _(q, k, v, scale):
        B, H, T, D = q.shape
        return q.new_empty(B, T, H, D), q.new_empty(B, H, T, dtype=torch.float32)

    @torch.library.register_fake("tfb::attn_bwd")
    def _(q, k, v, o, do, lse, scale):
        return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)

    def attn_setup(ctx, inputs, output):
        q, k, v, scale = inputs
        o, lse = output
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.scale = scale
        ctx.mark_non_differentiable(lse)
        ctx.set_materialize_grads(False)

    def attn_backward(ctx, d_o, _d_lse):
        q, k, v, o, lse = ctx.saved_tensors
        dq, dk, dv = attn_bwd(q, k, v, o, d_o.contiguous(), lse, ctx.scale)
        return dq, dk, dv, None

    torch.library.register_autograd("tfb::attn_fwd", attn_backward, setup_context=attn_setup)

    # ---------------------------------------------------------------- fp8 MLP with pre-cast weights (R2:7127-7160)
    @op("tfb::mlp8_precast", mutates_args=())
    def mlp8_precast(w_fc: torch.Tensor, w_proj: torch.Tensor, sc: torch.Tensor) -> torch.Tensor:
        return ops.mlp8_precast(w_fc.contiguous(), w_proj.contiguous(), sc)

    @op("tfb::mlp8_fwd", mutates_args=())
    def mlp8_fwd(x2: torch.Tensor, w_fc: torch.Tensor, w_proj: torch.Tensor, sc: torch.Tensor,
                 w8: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        y, r = ops.mlp8_fwd(x2.contiguous(), w8, sc, w_fc.shape[0])
        return y, r.t()   # [F, M] as the reference's op returns it (round2/source/train.py:6858); no copy

    @op("tfb::mlp8_bwd", mutates_args=())
    def mlp8_bwd(dy2: torch.Tensor, rT: torch.Tensor, x2: torch.Tensor, w_fc: torch.Tensor, w_proj: torch.Tensor,
                 sc: torch.Tensor, w8: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        dy2 = dy2.contiguous()
        r = rT.t().contiguous()                    # token-major [M, F]: free for the view mlp8_fwd returned
        sc_b = ops.mlp8_backward_scales(dy2, sc)   # this call's dy amax and the dpre bound, on the device
        dx, _, dpre = ops.mlp8_bwd(dy2, r, w8, sc_b, want_h=False)
        return dx, ops.matmul(dpre, x2.contiguous(), trans_a=True), ops.mlp_dw_proj(dy2, r)

    @torch.library.register_fake("tfb::mlp8_precast")
    def _(w_fc, w_proj, sc):
        return w_fc.new_empty(4, w_fc.numel(), dtype=torch.uint8)

    @torch.library.register_fake("tfb::mlp8_fwd")
    def _(x2, w_fc, w_proj, sc, w8):
        return torch.empty_like(x2), x2.new_empty(x2.shape[0], w_fc.shape[0]).t()

    @torch.library.register_fake("tfb::mlp8_bwd")
    def _(dy2, rT, x2, w_fc, w_proj, sc, w8):
        return torch.empty_like(dy2), torch.empty_like(w_fc), torch.empty_like(w_proj)

    def mlp_setup(ctx, inputs, output):
        x2, w_fc, w_proj, sc, w8 = inputs
        _y, rT = output
        ctx.save_for_backward(x2, rT, w_fc, w_proj, sc, w8)
        ctx.mark_non_differentiable(rT)
        ctx.set_materialize_grads(False)

    def mlp_backward(ctx, dy2, _d_r):
        x2, rT, w_fc, w_proj, sc, w8 = ctx.saved_tensors
        dx, dw_fc, dw_proj = mlp8_bwd(dy2, rT, x2, w_fc, w_proj, sc, w8)
        return dx, dw_fc, dw_proj, None, None

    torch.library.register_autograd("tfb::mlp8_fwd", mlp_backward, setup_context=mlp_setup)

    # ---------------------------------------------------------------- loss head on materialised logits (R2:6145-6156)
    @op("tfb::loss_head_fwd", mutates_args=())
    def loss_head_fwd(logits: torch.Tensor, targets: torch.Tensor, row_w: torch.Tensor,
                      softcap: float) -> tuple[torch.Tensor, torch.Tensor]:
        return ops.loss_fwd(logits.contiguous(), targets, softcap, row_w)

    @op("tfb::loss_head_bwd", mutates_args=())
    def loss_head_bwd(logits: torch.Tensor, targets: torch.Tensor, lz: torch.Tensor, g: torch.Tensor,
                      softcap: float) -> torch.Tensor:
        return ops.loss_bwd(logits.contiguous(), targets, lz, g.contiguous(), softcap)

    @torch.library.register_fake("tfb::loss_head_fwd")
    def _(logits, targets, row_w, softcap):
        n = logits.shape[0]
        return logits.new_empty(n, dtype=torch.float32), logits.new_empty(n, dtype=torch.float32)

    @torch.library.register_fake("tfb::loss_head_bwd")
    def _(logits, targets, lz, g, softcap):
        return torch.empty_like(logits)

    def loss_setup(ctx, inputs, output):
        logits, targets, row_w, softcap = inputs
        _loss, lz = output
        ctx.save_for_backward(logits, targets, row_w, lz)
        ctx.softcap = softcap
        ctx.mark_non_differentiable(lz)
        ctx.set_materialize_grads(False)

    def loss_backward(ctx, d_loss, _d_lz):
        logits, targets, row_w, lz = ctx.saved_tensors
        g = (d_loss.float() * row_w).contiguous()   # d(total) / d(row loss) times the row weight the forward applied
        return loss_head_bwd(logits, targets, lz, g, ctx.softcap), None, None, None

    torch.library.register_autograd("tfb::loss_head_fwd", loss_backward, setup_context=loss_setup)

    _OPS.update(attn_fwd=attn_fwd, attn_bwd=attn_bwd, mlp8_precast=mlp8_precast, mlp8_fwd=mlp8_fwd, mlp8_bwd=mlp8_bwd,
                loss_head_fwd=loss_head_fwd, loss_head_bwd=loss_head_bwd)
    return _OPS
