"""The benchmark model in plain PyTorch on the CPU: the path the reference takes off-device (eager expressions and
the kernels' torch emulations behind autograd Functions), restated for the full-step configuration of BASELINE.json (12 layers, d 768,
12 heads of 64, fp8 squared-ReLU MLP 3072, weighted RMSNorm pre-norm, RoPE, untied head, vocab 32768).

Follows the reference's Block / GPT forward order (R1:8826-8867, 9163-9228; R2:11094-11123, 11612-11709): norm ->
fused QKV projection -> RoPE -> causal attention -> output projection -> residual -> norm -> MLP -> residual; final
norm -> lm_head -> cross-entropy; bf16 activations with fp32 accumulation in every matmul, one rounding per op.
The fp8 MLP and the attention use the emulations' rounding points (oracle.mlp8, oracle.attention) through
autograd Functions, as EmulatedFusedMlp8 (K/nki_mlp_fused8.py:861-888) and the EMULATE route of the attention
wrapper (K/nki_attn_bandpro.py:1763-1768) do.

Pinned by: each building block's own pins, plus tests/test_oracle_model.py (the bf16-MLP variant of this model against a
straight nn.functional fp32 transformer within bf16 tolerance; loss at zero-initialised head = ln V).
"""
import math

import torch
import torch.nn.functional as F

from . import attention as oattn
from . import loss as oloss
from . import mlp8 as omlp
from . import norm as onorm
from . import optim as ooptim

bf16 = torch.bfloat16


class _Mlp8(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x2, w_fc, w_proj, row, x_scale, dw_fp8_limit=None):
        y, r = omlp.forward(x2, w_fc, w_proj, row, x_scale)
        ctx.save_for_backward(x2, r, w_fc, w_proj, row)
        ctx.x_scale, ctx.dw_fp8_limit = x_scale, dw_fp8_limit
        return y

    @staticmethod
    def backward(ctx, dy):
        x2, r, w_fc, w_proj, row = ctx.saved_tensors
        dy = dy.contiguous()
        rowb = omlp.backward_scales(dy, row)
        dx, h, dpre = omlp.backward(dy, r, w_fc, w_proj, rowb)
        if ctx.dw_fp8_limit is None:
            dw_fc, dw_proj = omlp.weight_grads(dy, x2, h, dpre)
        else:   # both weight gradients in fp8 too (round2/source/train.py:8209 under its fp8 weight-gradient switch)
            dw_fc, dw_proj = omlp.weight_grads_fp8(x2, dy, h, dpre, rowb, ctx.x_scale, ctx.dw_fp8_limit)
        return dx, dw_fc, dw_proj, None, None, None


class _Attention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q4, k4, v4, scale):
        o, lse = oattn.forward(q4, k4, v4, scale)
        ctx.save_for_backward(q4, k4, v4, o, lse)
        ctx.scale = scale
        return o

    @staticmethod
    def backward(ctx, do):
        q4, k4, v4, o, lse = ctx.saved_tensors
        dq, dk, dv = oattn.backward(q4, k4, v4, o, do, lse, ctx.scale)
        return dq, dk, dv, None


class _RMSNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w, eps):
        y, inv = onorm.rmsnorm(x, w, eps)
        ctx.save_for_backward(x, inv, w)
        return y

    @staticmethod
    def backward(ctx, gy):
        x, inv, w = ctx.saved_tensors
        dx, dw = onorm.rmsnorm_backward(gy, x, inv, w)
        return dx.to(x.dtype), dw.to(w.dtype), None


class _Rope(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, cos, sin):
        ctx.save_for_backward(cos, sin)
        return oattn.rope(x, cos, sin)

    @staticmethod
    def backward(ctx, g):
        cos, sin = ctx.saved_tensors
        return oattn.rope_backward(g, cos, sin), None, None


class _Loss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits2, targets, softcap):
        rows, lse = oloss.loss_rows(logits2, targets, softcap)
        w = oloss.row_weights(targets, "mean", logits2.shape[-1])
        ctx.save_for_backward(logits2, targets, lse, w)
        ctx.softcap = softcap
        return (rows * w).sum()

    @staticmethod
    def backward(ctx, g):
        logits2, targets, lse, w = ctx.saved_tensors
        return oloss.loss_backward(logits2, targets, lse, w * g, ctx.softcap), None, None


class OracleGPT:
    """params: dict name -> bf16 CPU tensor (the same names and values as the HIP model's init_values)."""

    def __init__(self, cfg, params, fp8=True):
        self.cfg = cfg
        self.fp8 = fp8
        self.p = {k: v.clone().float().to(bf16).requires_grad_(True) for k, v in params.items()}
        self.master = {k: v.clone().float() for k, v in params.items()}
        self.m = {k: torch.zeros_like(v, dtype=torch.float32) for k, v in params.items()}
        self.v = {k: torch.zeros_like(v, dtype=torch.float32) for k, v in params.items()}
        self.cos, self.sin = oattn.rope_tables(cfg.seq_len, cfg.head_dim, cfg.rope_base)
        self.step_count = 0
        self.refresh_fp8()

    def refresh_fp8(self):
        self.rows = [omlp.forward_scales(self.p["w_fc.%d" % i].detach(), self.p["w_proj.%d" % i].detach(),
                                         self.cfg.e4m3_limit, self.cfg.x_scale) for i in range(self.cfg.n_layer)]

    def mlp(self, h, i):
        w_fc, w_proj = self.p["w_fc.%d" % i], self.p["w_proj.%d" % i]
        h2 = h.reshape(-1, h.shape[-1])
        if self.fp8:
            y = _Mlp8.apply(h2, w_fc, w_proj, self.rows[i], self.cfg.x_scale,
                            self.cfg.e4m3_limit if getattr(self.cfg, "fp8_mlp_dw", False) else None)
        else:
            y = F.linear(torch.relu(F.linear(h2, w_fc)).square(), w_proj)
        return y.view(h.shape)

    def block(self, i, x):
        """One pre-norm block on the residual stream x [B, T, d]: x + attention(norm1(x)), then + MLP(norm2(.))."""
        return self.mlp_half(i, self.attention_half(i, x))

    def mlp_half(self, i, x):
        h = _RMSNorm.apply(x, self.p["norm2.%d" % i], self.cfg.norm_eps)
        return x + self.mlp(h, i)

    def attention_half(self, i, x):
        cfg, p = self.cfg, self.p
        B, T, _ = x.shape
        H, D = cfg.n_head, cfg.head_dim
        cos, sin = self.cos[:T], self.sin[:T]
        h = _RMSNorm.apply(x, p["norm1.%d" % i], cfg.norm_eps)
        qkv = F.linear(h, p["w_qkv.%d" % i])
        q, k, v = (t.reshape(B, T, H, D) for t in qkv.split(cfg.d_model, dim=-1))
        q, k = _Rope.apply(q, cos, sin), _Rope.apply(k, cos, sin)
        o = _Attention.apply(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), 1.0 / math.sqrt(D))
        att = F.linear(o.reshape(B, T, cfg.d_model), p["w_o.%d" % i])
        return x + att

    def forward(self, idx, targets):
        cfg, p = self.cfg, self.p
        x = F.embedding(idx, p["wte"])
        for i in range(cfg.n_layer):
            x = self.block(i, x)
        h = _RMSNorm.apply(x, p["norm_f"], cfg.norm_eps)
        logits = F.linear(h, p["lm_head"])
        return _Loss.apply(logits.reshape(-1, cfg.vocab), targets.reshape(-1), cfg.softcap or None)

    def train_step(self, idx, targets, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1):
        for t in self.p.values():
            t.grad = None
        loss = self.forward(idx, targets)
        loss.backward()
        self.step_count += 1
        with torch.no_grad():
            for name, t in self.p.items():
                if t.grad is None:
                    continue
                wd = weight_decay if (t.dim() == 2 and name != "wte") else 0.0
                ooptim.adamw_step(self.master[name], t.grad, self.m[name], self.v[name], self.step_count, lr, betas[0],
                                  betas[1], eps, wd)
                t.copy_(self.master[name].to(bf16))
        self.refresh_fp8()
        return loss.detach()
