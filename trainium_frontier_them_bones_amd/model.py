"""Decoder-only transformer training step on the HIP kernels: the caller side of the hot path.

The reference's model is GPT / Block / CausalSelfAttention / MLP (round1/source/train.py:8713-9237,
round2/source/train.py:10136-11750) driven by `loss = model(x, y); loss.backward(); optimizer.step()`
(round1/source/train.py:10328-10367). This module is that loop for the benchmark configuration: pre-norm blocks
(weighted RMSNorm, fused QKV projection, RoPE, causal attention, output projection, residual add fused with the
next norm, fp8 squared-ReLU MLP), untied LM head with the fused loss, AdamW on fp32 masters with bf16 working
weights. Every tensor op is one of the library's kernels; torch provides memory, streams and the autograd tape.
"""
import math
from dataclasses import dataclass

import torch

from . import autograd as A
from . import ops

bf16 = torch.bfloat16


@dataclass
class GPTConfig:
    n_layer: int = 12
    d_model: int = 768
    n_head: int = 12
    d_ff: int = 3072
    vocab: int = 32768
    seq_len: int = 2048
    rope_base: float = 10000.0
    norm_eps: float = 1e-6
    softcap: float = 0.0          # 0 = no logit softcap (the reference model uses 15)
    init_std: float = 0.02
    e4m3_limit: float = 240.0     # fp8 scale search limit (240 = the reference's rows, 448 = OCP maximum)
    x_scale: float = 4.0          # constant activation scale of the fp8 MLP input (a unit-RMS norm output)
    fp8_attn_proj: bool = False   # QKV and output projections in fp8 (e4m3 forward, e5m2 dX, bf16 dW); off in configuration 4 of BASELINE.json
    fp8_attn_dw: bool = False     # with fp8_attn_proj: their weight gradients in fp8 as well (R2_DW8_SET=qkv,proj)
    fp8_mlp_dw: bool = True       # the MLP's two weight gradients in fp8 as well: all six MLP GEMMs in fp8, as the reference's final recipe (round1/source/train.py:2226-2233 DW_ROWS '5,6'; round2/source/train.py:8209)
    fuse_residual: bool = True    # residual adds in the projections' stores, fp8 operand casts in the norms (same values)

    @property
    def head_dim(self):
        return self.d_model // self.n_head


def rope_tables(T, D, base, device):
    """cos, sin bf16 [T, D/2] (round1/source/train.py:8951-8962)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    ang = torch.outer(torch.arange(T, dtype=torch.float32), inv_freq)
    return ang.cos().to(bf16).to(device), ang.sin().to(bf16).to(device)


class FlatParams:
    """Parameters of one AdamW group as views into flat buffers: bf16 working copy, fp32 master, fp32 moments and a
    gradient buffer (bf16 for matrices, fp32 for the rest), so the optimizer is one launch per group."""

    def __init__(self, shapes, grad_dtype, device):
        self.names = list(shapes)
        self.shapes = shapes
        sizes = [int(math.prod(s)) for s in shapes.values()]
        pad = [(-n) % 8 for n in sizes]
        self.offsets = {}
        off = 0
        for name, n, p in zip(self.names, sizes, pad):
            self.offsets[name] = (off, n)
            off += n + p
        self.numel = off
        self.w = torch.zeros(off, dtype=bf16, device=device)
        self.master = torch.zeros(off, dtype=torch.float32, device=device)
        self.m = torch.zeros(off, dtype=torch.float32, device=device)
        self.v = torch.zeros(off, dtype=torch.float32, device=device)
        self.grad = torch.zeros(off, dtype=grad_dtype, device=device)
        self.params = {}
        for name in self.names:
            o, n = self.offsets[name]
            p = self.w[o:o + n].view(shapes[name]).requires_grad_(True)
            p.grad_buf = self.grad[o:o + n].view(shapes[name])
            p.grad_fresh = True
            self.params[name] = p

    def load(self, name, value):
        o, n = self.offsets[name]
        self.master[o:o + n].copy_(value.reshape(-1).float())
        self.w[o:o + n].copy_(value.reshape(-1).to(bf16))

    def mark_fresh(self):
        for p in self.params.values():
            p.grad_fresh = True


class GPT:
    def __init__(self, cfg: GPTConfig, device, seed=0):
        self.cfg = cfg
        self.device = device
        d, F, V, L = cfg.d_model, cfg.d_ff, cfg.vocab, cfg.n_layer
        mats, others = {}, {}
        others["wte"] = (V, d)
        for i in range(L):
            others["norm1.%d" % i] = (d,)
            mats["w_qkv.%d" % i] = (3 * d, d)
            mats["w_o.%d" % i] = (d, d)
            others["norm2.%d" % i] = (d,)
            mats["w_fc.%d" % i] = (F, d)
            mats["w_proj.%d" % i] = (d, F)
        others["norm_f"] = (d,)
        mats["lm_head"] = (V, d)
        self.mats = FlatParams(mats, bf16, device)
        self.others = FlatParams(others, torch.float32, device)
        self.p = {}
        self.p.update(self.mats.params)
        self.p.update(self.others.params)
        self.mlp_state = [A.Mlp8State(cfg.e4m3_limit, cfg.x_scale, cfg.fp8_mlp_dw) for _ in range(L)]
        self.qkv_state = [A.Linear8State(cfg.e4m3_limit, cfg.fp8_attn_dw) for _ in range(L)] if cfg.fp8_attn_proj else None
        self.wo_state = [A.Linear8State(cfg.e4m3_limit, cfg.fp8_attn_dw) for _ in range(L)] if cfg.fp8_attn_proj else None
        self.cos, self.sin = rope_tables(cfg.seq_len, cfg.head_dim, cfg.rope_base, device)
        # The 2 L + 1 norm weights sit side by side in the flat fp32 buffer: their gradients are left as per-workgroup
        # partial sums by every norm backward and finished by ONE launch after the backward pass (norm_rows fixes the
        # partial buffer's shape on first use).
        self.norm_names = [n for n in self.others.names if n.startswith("norm")]
        o0 = self.others.offsets[self.norm_names[0]][0]
        assert all(self.others.offsets[n] == (o0 + i * d, d) for i, n in enumerate(self.norm_names))
        self.norm_grads = self.others.grad[o0:o0 + len(self.norm_names) * d].view(len(self.norm_names), d)
        self.norm_parts, self.norm_rows, self.norm_fresh = None, 0, True
        self.step_count = 0
        # a list here makes the fused forward keep the residual stream after the embedding and after every residual add
        # (with its gradient after the backward pass): [x0, x0 + attention, block 0's output, ...]; tests compare the
        # two halves of every block on their own inputs
        self.trace = None
        self.init_weights(seed)

    def init_weights(self, seed):
        """N(0, init_std) for every matrix and the embedding, ones for the norm weights; generated on the CPU so that
        the oracle model can be given identical values."""
        g = torch.Generator().manual_seed(seed)
        self.init_values = {}
        for grp in (self.mats, self.others):
            for name in grp.names:
                shape = grp.shapes[name]
                if name.startswith("norm"):
                    val = torch.ones(shape)
                else:
                    val = torch.randn(shape, generator=g) * self.cfg.init_std
                val = val.to(bf16)
                self.init_values[name] = val
                grp.load(name, val.to(self.device))
        self.refresh_fp8()

    def refresh_fp8(self):
        """Per-optimizer-step refresh of each layer's fp8 scale row and e4m3 weight pack."""
        L = self.cfg.n_layer
        o_fc = [self.mats.offsets["w_fc.%d" % i][0] for i in range(L)]
        o_pj = [self.mats.offsets["w_proj.%d" % i][0] for i in range(L)]
        stride = o_fc[1] - o_fc[0] if L > 1 else 0
        if all(o_fc[i] - o_fc[0] == i * stride and o_pj[i] - o_pj[0] == i * stride for i in range(L)):
            # the layers' weights sit one stride apart in the flat buffer: one batched refresh (four launches)
            st0 = self.mlp_state[0]
            self._mlp_rows, self._mlp_w8 = ops.mlp8_refresh_layers(
                self.p["w_fc.0"].detach(), self.p["w_proj.0"].detach(), stride, L, st0.e4m3_limit, st0.x_scale,
                getattr(self, "_mlp_rows", None), getattr(self, "_mlp_w8", None))
            for i, st in enumerate(self.mlp_state):
                st.row, st.w8 = self._mlp_rows[i], self._mlp_w8[i]
        else:
            for i, st in enumerate(self.mlp_state):
                st.refresh(self.p["w_fc.%d" % i], self.p["w_proj.%d" % i])
        if self.qkv_state is not None:
            for i in range(self.cfg.n_layer):
                self.qkv_state[i].refresh(self.p["w_qkv.%d" % i])
                self.wo_state[i].refresh(self.p["w_o.%d" % i])

    def _norm_partials(self, rows):
        if self.norm_rows != rows:
            nb = ops.norm_bwd_blocks(rows)
            self.norm_parts = torch.empty(len(self.norm_names), nb, self.cfg.d_model, dtype=torch.float32, device=self.device)
            self.norm_rows = rows
            for i, n in enumerate(self.norm_names):
                self.p[n].dw_part = self.norm_parts[i]

    def finish_norm_grads(self):
        """The norm weights' gradients from the partial sums of this backward pass (added to what earlier micro-steps
        left when the gradients are not fresh)."""
        ops.norm_dw_finish(self.norm_parts, self.norm_grads, self.norm_rows, accumulate=not self.norm_fresh)
        self.norm_fresh = False

    def forward(self, idx, targets):
        cfg, p = self.cfg, self.p
        B, T = idx.shape
        self._norm_partials(B * T)
        scale = 1.0 / math.sqrt(cfg.head_dim)
        x = A.EmbeddingFn.apply(idx, p["wte"])
        if cfg.fuse_residual:
            return self._forward_fused(x, targets, T, scale)
        h = A.RMSNormFn.apply(x, p["norm1.0"], cfg.norm_eps)
        for i in range(cfg.n_layer):
            if cfg.fp8_attn_proj:    # h is an RMSNorm output (constant scale 4); the attention output takes its amax scale
                qkv = A.Linear8Fn.apply(h, p["w_qkv.%d" % i], self.qkv_state[i], cfg.x_scale)
                att = A.RopeAttentionFn.apply(qkv, self.cos[:T], self.sin[:T], cfg.n_head, scale)
                att = A.Linear8Fn.apply(att, p["w_o.%d" % i], self.wo_state[i], None)
            else:
                if cfg.head_dim == 64:   # rotation fused into the projection's epilogue and the backward kernels' stores
                    att = A.QkvRopeAttentionFn.apply(h, p["w_qkv.%d" % i], self.cos[:T], self.sin[:T], cfg.n_head, scale)
                else:
                    qkv = A.LinearFn.apply(h, p["w_qkv.%d" % i])
                    att = A.RopeAttentionFn.apply(qkv, self.cos[:T], self.sin[:T], cfg.n_head, scale)
                att = A.LinearFn.apply(att, p["w_o.%d" % i])
            x, h = A.AddRMSNormFn.apply(x, att, p["norm2.%d" % i], cfg.norm_eps)
            m = A.Mlp8Fn.apply(h, p["w_fc.%d" % i], p["w_proj.%d" % i], self.mlp_state[i])
            nw = p["norm1.%d" % (i + 1)] if i + 1 < cfg.n_layer else p["norm_f"]
            x, h = A.AddRMSNormFn.apply(x, m, nw, cfg.norm_eps)
        return A.LmHeadLossFn.apply(h, p["lm_head"], targets, cfg.softcap, "mean")

    def _forward_fused(self, x, targets, T, scale):
        """The same network with the residual adds made in the stores of the output projection and of the MLP's second
        GEMM, and the MLP's (with fp8 attention projections also the QKV projection's) fp8 operand cast made by the norm
        that precedes it (round2/source/kernels/nki_attn_nr8.py, nki_mlp_nr8.py): bit-identical activations, two
        elementwise passes per layer fewer."""
        cfg, p = self.cfg, self.p
        q8 = cfg.x_scale if cfg.fp8_attn_proj else None

        def keep(t):
            if self.trace is not None:
                t.retain_grad()
                self.trace.append(t)
        keep(x)
        x, h, *h8 = A.RMSNormPassFn.apply(x, p["norm1.0"], cfg.norm_eps, q8)
        for i in range(cfg.n_layer):
            if cfg.fp8_attn_proj:
                qkv = A.Linear8Fn.apply(h, p["w_qkv.%d" % i], self.qkv_state[i], cfg.x_scale, h8[0])
                att = A.RopeAttentionFn.apply(qkv, self.cos[:T], self.sin[:T], cfg.n_head, scale)
                x = A.Linear8Fn.apply(att, p["w_o.%d" % i], self.wo_state[i], None, None, x)
            else:
                if cfg.head_dim == 64:
                    att = A.QkvRopeAttentionFn.apply(h, p["w_qkv.%d" % i], self.cos[:T], self.sin[:T], cfg.n_head, scale)
                else:
                    qkv = A.LinearFn.apply(h, p["w_qkv.%d" % i])
                    att = A.RopeAttentionFn.apply(qkv, self.cos[:T], self.sin[:T], cfg.n_head, scale)
                x = A.LinearFn.apply(att, p["w_o.%d" % i], x)
            keep(x)
            # (with the weight gradients in fp8 too the MLP reads only the norm's bytes: its bf16 rows are not written)
            x, h, h8m = A.RMSNormPassFn.apply(x, p["norm2.%d" % i], cfg.norm_eps, cfg.x_scale, self.mlp_state[i].dw_fp8)
            x = A.Mlp8Fn.apply(h, p["w_fc.%d" % i], p["w_proj.%d" % i], self.mlp_state[i], h8m, x)
            keep(x)
            nw = p["norm1.%d" % (i + 1)] if i + 1 < cfg.n_layer else p["norm_f"]
            x, h, *h8 = A.RMSNormPassFn.apply(x, nw, cfg.norm_eps, q8 if i + 1 < cfg.n_layer else None)
        return A.LmHeadLossFn.apply(h, p["lm_head"], targets, cfg.softcap, "mean")

    def zero_grad(self):
        self.mats.mark_fresh()
        self.others.mark_fresh()
        self.norm_fresh = True

    def backward(self, loss):
        loss.backward()
        self.finish_norm_grads()

    def optimizer_step(self, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1):
        self.step_count += 1
        for grp, wd in ((self.mats, weight_decay), (self.others, 0.0)):
            ops.adamw_(grp.master, grp.grad, grp.m, grp.v, self.step_count, lr, betas[0], betas[1], eps, wd, grp.w)
        self.refresh_fp8()
        self.zero_grad()

    def train_step(self, idx, targets, **opt):
        """One fwd + bwd + AdamW step; returns the loss tensor (no host sync)."""
        loss = self.forward(idx, targets)
        self.backward(loss)
        self.optimizer_step(**opt)
        return loss

    def num_params(self):
        return sum(int(math.prod(s)) for grp in (self.mats, self.others) for s in grp.shapes.values())


def zipf_tokens(B, T, vocab, s=1.1, seed=0):
    """B sequences of T+1 token ids drawn Zipfian (p_r ~ r^-s) on the CPU: (inputs [B,T], next-token targets [B,T])."""
    g = torch.Generator().manual_seed(seed)
    ranks = torch.arange(1, vocab + 1, dtype=torch.float64)
    prob = ranks.pow(-s)
    prob = prob / prob.sum()
    tok = torch.multinomial(prob.float(), B * (T + 1), replacement=True, generator=g).view(B, T + 1)
    return tok[:, :-1].contiguous(), tok[:, 1:].contiguous()
