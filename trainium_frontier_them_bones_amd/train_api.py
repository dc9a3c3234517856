"""The reference training loop's call signatures on the HIP kernels.

Every function here has the name, argument order, argument meaning and result layout of the wrapper the reference's
`train.py` calls (round1/source/train.py, cited as R1; round2/source/train.py, R2), so a call site switches over by
changing its import. Differences that a caller can see, all of them in the error behaviour:
  * there is no eager fallback: on a CPU tensor, a dtype other than bf16 or a shape the kernels do not take the call
    raises (`TypeError` / `_lib.TfbError`), which is R2's policy (R2:6947 "a shape the kernels do not take ... raises");
  * the three wrappers whose contract is "None = not done, run your own line" (`nki_rope_attention` R1:8197,
    `fused_loss_multi` R1:4908, `dw_matmul` R1:3486) return None exactly when the library answers "shape not taken".
Inputs are never modified; outputs are fresh tensors, except `inplace=True` weight gradients, which are accumulated into
`w.grad` (R1:8463-8472) and answered with a None gradient.
"""
import math

import torch

from . import autograd as A
from . import ops
from ._lib import TfbError

bf16 = torch.bfloat16
LOGIT_SOFTCAP = 15.0          # R1:81
RMS_EPS = 2.0 ** -23          # R1:5153, 4172
_SHAPE = 1                    # the library's "shape not taken" status


def _none_if_shape(fn, *args):
    try:
        return fn(*args)
    except TfbError as err:
        if err.status == _SHAPE:
            return None
        raise


# ------------------------------------------------------------------------------------------ attention (R1:8069-8210)
def nki_causal_attention(q, k, v, scale=None, nw=None):
    """Causal SDPA(q, k, v) for [B, H, T, D] inputs, returned as [B, T, H, D] (R1:8069). nw (the reference's band
    kernels' last argument, K/nki_attn_bandpro.py:1654; R2:4925 fused_rope_attention_band): a query of 128-token tile i
    sees the keys k <= q of tiles i - nw + 1 .. i only."""
    sc = float(scale) if scale is not None else 1.0 / math.sqrt(q.shape[-1])
    return A.CausalAttentionFn.apply(q, k, v, sc, int(nw) if nw else 0)


nki_attn_fn = nki_causal_attention   # R1:8207


def rope_norm(x, cos, sin):
    """norm(apply_rotary_emb(x, cos, sin)).transpose(1, 2): x [B, T, H, D] -> [B, H, T, D] (R1:4447). cos, sin hold
    T x D/2 values (any leading singleton shape, as the reference's [1, T, 1, D/2] buffers)."""
    B, T, H, D = x.shape
    c, s = _tables_2d(cos, sin, T, D // 2)
    return A.RopeNormFn.apply(x, c, s, RMS_EPS).transpose(1, 2)


def _tables_2d(cos, sin, T, half):
    c = cos.reshape(-1, half)[:T].to(bf16).contiguous()
    s = sin.reshape(-1, half)[:T].to(bf16).contiguous()
    if c.shape[0] != T:
        raise ValueError("rotary tables shorter than the sequence")
    return c, s


def nki_rope_attention(qkv, cos, sin, n_head, scale=None, nw=None):
    """y [B, T, H, D] = causal SDPA(QKnorm(RoPE(q)), QKnorm(RoPE(k)), v) straight from the fused projection output qkv
    [B, T, 3C]; None when the fused path does not apply (R1:8197). nw: the tile band of the reference's windowed layers
    (R2:4925 fused_rope_attention_band; kernels' last argument)."""
    if qkv.dim() != 3 or qkv.shape[-1] % (3 * n_head):
        return None
    B, T, C3 = qkv.shape
    D = C3 // 3 // n_head
    if D not in (64, 128):
        return None
    sc = float(scale) if scale is not None else 1.0 / math.sqrt(D)
    c, s = _tables_2d(cos, sin, T, D // 2)
    y = _none_if_shape(A.RopeNormAttentionFn.apply, qkv, c, s, n_head, sc, RMS_EPS, int(nw) if nw else 0)
    return None if y is None else y.view(B, T, n_head, D)


# ------------------------------------------------------------------------------------------ loss head (R1:4691, 4908; R2:6364)
def fused_loss(logits, targets, reduction="mean", softcap=LOGIT_SOFTCAP):
    """The static cross-entropy chain on the raw lm_head output (R1:4691): softcap * tanh(logits / softcap), log-softmax,
    ignore_index -1; reduction "mean" (over the targets not ignored), "sum" or "none" (rows in targets' shape)."""
    V = logits.shape[-1]
    x2 = logits.reshape(-1, V).contiguous()
    t = targets.reshape(-1)
    rows = A.FusedLossFn.apply(x2, t, softcap)
    if reduction == "none":
        return rows.view(targets.shape)
    if reduction == "sum":
        return rows.sum()
    if reduction != "mean":
        raise ValueError("reduction must be 'mean', 'sum' or 'none'")
    return rows.sum() / ((t >= 0) & (t < V)).sum().clamp_min(1).to(rows.dtype)   # the rows the kernel gives a loss to


def fused_loss_multi(logits, tg, rw, softcap=LOGIT_SOFTCAP, ref=None):
    """0-dim fp32 sum_i sum_k rw[k, i] nll(logits_i, tg[k, i]) through one kernel pair, or None when the kernels do not
    take the call (R1:4908). tg [K, N] integer targets, rw [K, N] weights; `ref` (the reference's self-check input) is
    accepted and unused."""
    V = logits.shape[-1]
    K, N = tg.shape
    if logits.numel() != N * V or not (1 <= K <= 8):
        return None
    rows = _none_if_shape(A.FusedLossMultiFn.apply, logits.reshape(N, V).contiguous(), tg.contiguous(),
                          rw.float().contiguous(), softcap, 0.0)
    return None if rows is None else rows.sum()


def chunked_loss_mean(logits, targets, smooth=False, tok_w=None, eps=0.0):
    """F.cross_entropy(softcap * tanh(logits.float() / softcap), targets, ignore_index=-1, reduction="mean") through the
    kernels (R2:6364): the mean and the ignored targets are row weights, `tok_w` (per-target weights) multiplies them,
    `smooth` selects the label-smoothed pair with the reference's R2_LABEL_SMOOTH passed here as `eps`."""
    b, t, v = logits.shape
    n = b * t
    y = targets.reshape(n)
    w = ops.loss_row_weights(y, "mean", v)
    if tok_w is not None:
        w = w * tok_w.reshape(n).to(torch.float32)
    x2 = logits.reshape(n, v).contiguous()
    rows = A.FusedLossMultiFn.apply(x2, y.view(1, n).contiguous(), w.view(1, n).contiguous(), LOGIT_SOFTCAP,
                                    float(eps) if smooth else 0.0)
    return rows.sum()


# ------------------------------------------------------------------------------------------ norm / residual blocks (R1:5578-6834)
def _gain(l, like):
    return l if torch.is_tensor(l) else torch.tensor([float(l)], dtype=torch.float32, device=like.device)


def block_head(x, x0, l1, l2):
    """(l1*x + l2*x0, norm(l1*x + l2*x0)) (R1:5578); l1, l2 one-element tensors (the model's learnable gains)."""
    C = x.shape[-1]
    x_new, x_norm = A.BlockHeadFn.apply(x.reshape(-1, C), x0.reshape(-1, C), _gain(l1, x), _gain(l2, x), None, None, RMS_EPS)
    return x_new.view(x.shape), x_norm.view(x.shape)


def head_skip(x, x0, skip, l1, l2, l3):
    """Block head with the U-net skip folded in: head(x + l3*skip, x0) = (l1*(x + l3*skip) + l2*x0, its norm) (R1:6106,
    eager form 5644-5647). skip None = the plain block head."""
    if skip is None:
        return block_head(x, x0, l1, l2)
    C = x.shape[-1]
    x_new, x_norm = A.BlockHeadFn.apply(x.reshape(-1, C), x0.reshape(-1, C), _gain(l1, x), _gain(l2, x),
                                        skip.reshape(-1, C), _gain(l3, x), RMS_EPS)
    return x_new.view(x.shape), x_norm.view(x.shape)


SELF_SKIP = object()   # head2's marker: the skip is the block's own (materialised) input (R1: mblk_SELF_SKIP)


def head2(x, x0, skip, l1, l2, l3, emit=False, key=None):
    """Block head whose input may be the previous block's (s1, mlp_out) pair (R1:6778): x_in = s1 + mlp_out (or x itself),
    then head_skip(x_in, x0, skip, l1, l2, l3) with skip None | tensor | SELF_SKIP (= x_in). Returns (x_new, x_norm,
    x_in when emit else None, x0). The pair's add is one bf16 pass in front of the block-head kernel (the reference's own
    composition when its folded kernel does not apply, R1:6803-6807); `key` (its gain-gradient bookkeeping) is unused."""
    x_t = x[0] + x[1] if isinstance(x, (tuple, list)) else x
    sk = x_t if skip is SELF_SKIP else skip
    x_new, x_norm = head_skip(x_t, x0, sk, l1, l2, l3)
    return x_new, x_norm, (x_t if emit else None), x0


def rmsnorm_fast(x):
    """F.rms_norm(x, (C,)) (R1:5594)."""
    C = x.shape[-1]
    return A.RMSNormFn.apply(x.reshape(-1, C), None, RMS_EPS).view(x.shape)


def tail_norm2(x_new, attn_out):
    """(x_new + attn_out, norm(x_new + attn_out)) (R1:6117)."""
    C = x_new.shape[-1]
    s1, y = A.AddRMSNormFn.apply(x_new.reshape(-1, C), attn_out.reshape(-1, C), None, RMS_EPS)
    return s1.view(x_new.shape), y.view(x_new.shape)


def final_norm(s1, mo):
    """norm(s1 + mo): the last block's residual add and the final RMSNorm (R1:6826)."""
    C = s1.shape[-1]
    _, y = A.AddRMSNormFn.apply(s1.reshape(-1, C), mo.reshape(-1, C), None, RMS_EPS)
    return y.view(s1.shape)


def relu_squared(x):
    """relu(x)**2 (R1:4161)."""
    return A.Relu2Fn.apply(x)


# ------------------------------------------------------------------------------------------ GEMM glue (R1:1137, 1231, 8407)
def nki_matmul(a, b, trans_a=False, trans_b=False):
    """out = op(a) @ op(b), fp32 accumulation, one rounding (R1:1137). No autograd, as in the reference (its callers are
    autograd Functions)."""
    return ops.matmul(a.contiguous(), b.contiguous(), trans_a=trans_a, trans_b=trans_b)


class _LinearTFn(torch.autograd.Function):
    """y = x @ w with w [in, out] (the reference's LinearT layout, R1:8419-8711)."""

    @staticmethod
    def forward(ctx, x2, w, inplace):
        ctx.save_for_backward(x2, w)
        ctx.inplace = inplace
        return ops.matmul(x2, w)

    @staticmethod
    def backward(ctx, gy):
        x2, w = ctx.saved_tensors
        g2 = gy.contiguous()
        dx = ops.matmul(g2, w, trans_b=True)
        if ctx.inplace and w.grad is not None and w.grad.dtype in (bf16, torch.float32) and w.grad.is_contiguous():
            ops.matmul(x2, g2, trans_a=True, out=w.grad, accumulate=True)     # R1:8463-8472: summed in the GEMM's output stage
            return dx, None, None
        return dx, ops.matmul(x2, g2, trans_a=True), None


def fused_fc_relu2(x, w, inplace=False):
    """relu(x @ w)^2 for any leading shape, w [in, out]; with inplace=True the c_fc dW goes straight into w.grad when it
    exists (R1:1231)."""
    K = x.shape[-1]
    h = A.Relu2Fn.apply(_LinearTFn.apply(x.reshape(-1, K).contiguous(), w, inplace))
    return h.view(*x.shape[:-1], w.shape[1])


def dw_matmul(a2d, b2d, row=None, key=None):
    """a2d^T @ b2d [Ka, N] from two token-major matrices, or None when the kernels do not take the shape (R1:3486: the
    weight-gradient GEMM; `row` and `key` select the reference's fp8 scale row and plan cache and are unused here)."""
    return _none_if_shape(lambda: ops.matmul(a2d.contiguous(), b2d.contiguous(), trans_a=True))


def embedding_fwd(idx, weight, out_dtype, shadow=None):
    """wte(idx).to(out_dtype) with the kernels' backward (R1:8407). `shadow` (the table already in out_dtype) is used for
    the forward gather when given."""
    if out_dtype != bf16:
        raise TypeError("the embedding kernels produce bf16")
    if shadow is not None:
        return _EmbeddingShadowFn.apply(idx, weight, shadow)
    return A.EmbeddingFn.apply(idx, weight if weight.dtype == bf16 else weight.to(bf16))


class _EmbeddingShadowFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, idx, weight, shadow):
        ctx.save_for_backward(idx, weight)
        return ops.embedding_fwd(idx, shadow)

    @staticmethod
    def backward(ctx, gy):
        idx, weight = ctx.saved_tensors
        dw = ops.fill_f32_(torch.empty(weight.shape, dtype=torch.float32, device=weight.device), 0.0)
        ops.embedding_bwd(idx, gy.contiguous(), dw)
        return None, dw.to(weight.dtype), None


# ------------------------------------------------------------------------------------------ fp8 fused MLP (R2:6617, 6947)
def fp8_refresh_weights(model, quantise_fn=None, *, e4m3_limit=240.0, x_scale=4.0, dw_fp8=False):
    """Once per optimizer step: every MLP's scale row and e4m3 weight bytes (R2:6617 fp8_refresh_weights(model,
    quantise_fn=None); the reference keeps them on the module as mlp8_sc / mlp8_w8, here as mlp.tfb_mlp8). `model` is
    the reference's model (its MLPs are model.transformer.h[i].mlp) or any iterable of modules with c_fc / c_proj.
    quantise_fn, when given, replaces the library's refresh and is called as the reference calls its own
    (R2:6638: quantise(c_proj weights, c_fc weights, destinations, destinations)), the destinations being the MLPs'
    Mlp8State objects."""
    blocks = getattr(getattr(model, "transformer", None), "h", None)
    mlps = [blk.mlp for blk in blocks] if blocks is not None else list(model)
    states = []
    for mlp in mlps:
        st = getattr(mlp, "tfb_mlp8", None)
        if st is None:
            st = mlp.tfb_mlp8 = A.Mlp8State(e4m3_limit, x_scale, dw_fp8)
        states.append(st)
    if quantise_fn is not None:
        quantise_fn([m.c_proj.weight for m in mlps], [m.c_fc.weight for m in mlps], states, states)
        return
    for mlp, st in zip(mlps, states):
        st.refresh(mlp.c_fc.weight.detach().to(bf16), mlp.c_proj.weight.detach().to(bf16))


def mlp_fused8(mlp, x):
    """MLP.forward on [b, t, n_embd] with the four activation GEMMs in fp8 (R2:6947): c_proj(relu(c_fc(x))^2), weights
    mlp.c_fc.weight [F, d] and mlp.c_proj.weight [d, F]; rows are padded with zeros to a multiple of 128 (a zero row
    touches no other row). The scale row and weight bytes come from fp8_refresh_weights (made here on first use)."""
    if getattr(mlp, "tfb_mlp8", None) is None or mlp.tfb_mlp8.row is None:
        fp8_refresh_weights([mlp])
    b, t, c = x.shape
    x2 = x.reshape(b * t, c)
    m = x2.shape[0]
    pad = (-m) % 128
    if pad:
        x2 = torch.nn.functional.pad(x2, (0, 0, 0, pad))
    w_fc = mlp.c_fc.weight if mlp.c_fc.weight.dtype == bf16 else mlp.c_fc.weight.to(bf16)
    w_proj = mlp.c_proj.weight if mlp.c_proj.weight.dtype == bf16 else mlp.c_proj.weight.to(bf16)
    y = A.Mlp8Fn.apply(x2, w_fc, w_proj, mlp.tfb_mlp8)
    if pad:
        y = y[:m]
    return y.reshape(b, t, c)


def moe_refresh_weights(moe, *, e4m3_limit=240.0, x_scale=4.0):
    """Once per optimizer step for a MoE block with fp8 experts: every expert's scale row and e4m3 weight bytes (what
    fp8_refresh_weights writes into MoeMLP.exp8_sc, R2:10862-10872), kept as moe.tfb_moe8."""
    st = getattr(moe, "tfb_moe8", None)
    if st is None:
        st = moe.tfb_moe8 = A.Moe8State(e4m3_limit, x_scale)
    st.refresh(moe.w_fc.detach().to(bf16), moe.w_proj.detach().to(bf16))
    return st


def moe_mlp(moe, x, want_stats=False, aux_weights=(0.0, 0.0, 0.0)):
    """MoeMLP.forward / forward_e8 (R2:10941-11067) with every expert on this GPU: x [b, t, d] bf16 -> the block's MLP output
    (routed experts, plus the shared half when the module has one); with want_stats also the weighted auxiliary sum
    aux_weights = (R2_MOE_AUX, R2_MOE_ZLOSS, R2_MOE_AUX_SEQ) . (lb, z, seq) and the statistics vector [3 + E] = (kept share
    of the assignments, lb, z, the experts' load shares), as the reference returns them. `moe` is the reference's module:
    router [E, d], w_fc [E, H, d], w_proj [E, d, H], topk, cap (per-sequence capacity; None or absent: dropless), e8 (fp8
    experts; their scales come from moe_refresh_weights, made here on first use), shared (a module with c_fc / c_proj, or
    None: run as mlp_fused8 when the experts are fp8, else as c_proj(relu_squared(c_fc(x))))."""
    if x.dim() != 3:
        raise ValueError("moe_mlp takes x [b, t, d]")
    e8 = bool(getattr(moe, "e8", False))
    st = None
    if e8:
        st = getattr(moe, "tfb_moe8", None)
        if st is None or st.rows is None:
            st = moe_refresh_weights(moe)
    cap = getattr(moe, "cap", None)
    info = {}
    args = (x, moe.router, moe.w_fc, moe.w_proj, st, int(moe.topk), None)
    if want_stats:
        out, aux, terms = A.MoeMlp8Fn.apply(*args, tuple(float(w) for w in aux_weights), cap, info)
    else:
        out = A.MoeMlp8Fn.apply(*args, None, cap, info)
    shared = getattr(moe, "shared", None)
    if shared is not None:
        if e8:
            out = out + mlp_fused8(shared, x)
        else:
            wf, wp = shared.c_fc.weight, shared.c_proj.weight
            out = out + A.LinearFn.apply(relu_squared(A.LinearFn.apply(x, wf if wf.dtype == bf16 else wf.to(bf16))),
                                         wp if wp.dtype == bf16 else wp.to(bf16))
    if not want_stats:
        return out
    stats = torch.cat([info["kept"].reshape(1), terms]).detach()
    return out, aux, stats


def nr_mlp(mlp, x1):
    """x1 + MLP(rms_norm(x1)) on [b, t, n_embd] with the norm and the residual add folded into the fp8 MLP's two calls
    (R2:9202 nr_mlp / 9168 NrMlp; kernels K/nki_mlp_nr8.py:1032): the norm's pass also writes the e4m3 operand, the add
    is made in the second GEMM's store, the backward's norm gradient and residual add are one launch. Rows are padded
    with zeros to a multiple of 128 (a zero row normalises to zero and adds zero)."""
    if getattr(mlp, "tfb_mlp8", None) is None or mlp.tfb_mlp8.row is None:
        fp8_refresh_weights([mlp])
    b, t, c = x1.shape
    x2 = x1.reshape(b * t, c)
    if x2.dtype != bf16:
        raise RuntimeError("the folded MLP takes bf16 rows, not %s" % x2.dtype)
    m = x2.shape[0]
    pad = (-m) % 128
    if pad:
        x2 = torch.nn.functional.pad(x2, (0, 0, 0, pad))
    w_fc = mlp.c_fc.weight if mlp.c_fc.weight.dtype == bf16 else mlp.c_fc.weight.to(bf16)
    w_proj = mlp.c_proj.weight if mlp.c_proj.weight.dtype == bf16 else mlp.c_proj.weight.to(bf16)
    xo = A.NrMlpFn.apply(x2, w_fc, w_proj, mlp.tfb_mlp8)
    if pad:
        xo = xo[:m]
    return xo.reshape(b, t, c)


def proj_residual(x, w, res):
    """res + x @ w^T with the add made in the GEMM's store (the bf16 form of _proj8_fwd_ra_kernel,
    K/nki_attn_nr8.py:1003; R2:9293 NrAttnOut): w [out, in], any leading shape, rows a multiple of 128."""
    return A.LinearFn.apply(x, w, res)


def shapes_apply8(m, d, f, tb=None):
    """The shapes the fp8 MLP kernels take (K/nki_mlp_fused8.py:666 shapes_apply8): M a multiple of 128, d and F multiples
    of 256. tb, the reference's token-block knob, has no counterpart here and is ignored."""
    return m > 0 and m % 128 == 0 and d > 0 and d % 256 == 0 and f > 0 and f % 256 == 0


def sc_tile(row):
    """[128, 16] fp32: the scale row down every partition, the form the reference's kernels take (K/nki_mlp_fused8.py:816).
    The entry points here read the 16-float row itself (`sc_tile(row)[0]`)."""
    return row.float().reshape(1, 16).expand(128, 16).contiguous()


def forward_scales(w_fc, w_proj):
    """The forward's 16-column scale row from the two weights (K/nki_mlp_fused8.py:782)."""
    return ops.mlp8_forward_scales(w_fc, w_proj)


def backward_scales(dy2, row):
    """The backward call's row: the forward row with this call's gradient scales filled in (K/nki_mlp_fused8.py:803)."""
    return ops.mlp8_backward_scales(dy2, row)


def dw8_grad(g2, a2, s_g, i_g, s_a, i_a, fg, fa):
    """One weight gradient g2^T a2 [O, D] in fp8 (R2:8185): the g side cast at s_g into format fg, the a side at s_a into
    fa (0 = e4m3, 1 = e5m2, 2 = e4m3 with g * s_g clamped at 240 first), the descale i_g * i_a. The scales are
    one-element fp32 device tensors and powers of two; i_g, i_a are their exact inverses, which the kernel forms itself.
    One side must be e5m2 and the other e4m3 (the two pairings the reference registers, R2:8156)."""
    f8 = {0: ops.FMT_E4M3, 1: ops.FMT_E5M2, 2: ops.FMT_E4M3}
    sg, sa = s_g.reshape(1).float(), s_a.reshape(1).float()
    if fg == 2:   # clamp(g s_g, 240) = s_g clamp(g, 240 / s_g): exact, s_g is a power of two
        g2 = torch.minimum(g2, (240.0 / sg).to(g2.dtype))
    g8 = ops.quant_fp8(g2.contiguous(), sg, f8[fg])
    a8 = ops.quant_fp8(a2.contiguous(), sa, f8[fa])
    return ops.gemm_fp8_tn(g8, a8, f8[fg], f8[fa], sg, sa)


# ------------------------------------------------------------------------------------------ Muon Newton-Schulz (K/nki_nsk.py)
def nsk(ga, gb, d_a, d_b, coeffs=ops.NS_COEFFS):
    """(ya, yb, va, vb) = the five Polar Express iterations of both stacks of a Muon step (K/nki_nsk.py:370 _nsk_kernel,
    arithmetic :452 emulate_nsk): ga fp32 [K, M, N] tall, gb fp32 [K2, N, M] wide, after the optimizer's two lerps; d_a, d_b
    the matrices' denominators bf16(bf16(||bf16(g)||) * 1.01 + 1e-6) ([K] or [K, 1, 1], any float dtype; the reciprocal is
    taken in fp32 as sc_tile does, :406). ya, yb bf16 in the inputs' layouts; va [K, M], vb [K2, M] fp32 = the sums of x^2
    along the N-long side (the caller divides by N). An empty stack is skipped, as in the reference."""
    def one(g, d):
        if g.shape[0] == 0:
            return (torch.empty(g.shape, dtype=bf16, device=g.device),
                    torch.empty(0, max(g.shape[1], g.shape[2]), dtype=torch.float32, device=g.device))
        return ops.ns5(g.contiguous(), d)
    ya, va = one(ga, d_a)
    yb, vb = one(gb, d_b)
    return ya, yb, va, vb


# ------------------------------------------------------------------------------------------ fused AdamW step (R1:1573)
@torch.no_grad()
def adamw_fused_step(opt) -> bool:
    """One AdamW step of every parameter group of `opt` (a torch.optim.AdamW-shaped object: param_groups with lr, betas,
    eps, weight_decay; state with step, exp_avg, exp_avg_sq) through the fused kernel, in place (R1:1573
    adamw_fused_step; update rule R1:9670-9677: p *= 1 - lr wd; m.lerp_(g, 1 - b1); v.lerp_(g^2, 1 - b2);
    p -= lr (m / bias1) / (sqrt(v / bias2) + eps)). Returns True when the groups were updated (the caller skips its own
    step), False - with nothing touched - when a parameter is not the kernel's layout (fp32 device parameter, contiguous
    fp32 or bf16 gradient of its shape): the reference's "not done, run your own line" convention."""
    todo = []
    for g in opt.param_groups:
        if g.get("amsgrad") or g.get("maximize"):
            return False
        for p in g["params"]:
            if p.grad is None:
                continue
            gr = p.grad
            if (not p.is_cuda or p.dtype != torch.float32 or not p.is_contiguous() or not gr.is_contiguous()
                    or gr.shape != p.shape or gr.dtype not in (torch.float32, bf16) or p.numel() == 0
                    or p.data_ptr() % 16 or gr.data_ptr() % (16 if gr.dtype == torch.float32 else 8)):
                return False
            st = opt.state.get(p, {})
            for key in ("exp_avg", "exp_avg_sq"):
                t = st.get(key)
                if t is not None and (t.dtype != torch.float32 or t.device != p.device or t.shape != p.shape
                                      or not t.is_contiguous() or t.data_ptr() % 16):
                    return False
            todo.append((g, p))
    # every (group, parameter) has passed: nothing below can refuse, so the optimizer is never left half-stepped
    for g, p in todo:
        st = opt.state[p]
        if len(st) == 0:
            st["step"] = torch.zeros((), dtype=torch.float32)
            st["exp_avg"] = torch.zeros_like(p)
            st["exp_avg_sq"] = torch.zeros_like(p)
        n = int(st["step"]) + 1
        b1, b2 = g["betas"]
        ops.adamw_(p, p.grad, st["exp_avg"], st["exp_avg_sq"], n, float(g["lr"]), b1, b2, g["eps"], g["weight_decay"])
        # the kernel wrote p behind autograd's back: bump its version as the reference does after its raw kernel write
        # (R1 optk_adamw_fused_step), so caches keyed on p._version (the per-step fp8 weight cache) see the update
        torch.autograd.graph.increment_version(p)
        if torch.is_tensor(st["step"]):
            st["step"] += 1
        else:
            st["step"] = n
    return True


# ------------------------------------------------------------------------------------------ R1 fp8 MLP rows (R1:1780-4140)
from .r1_fp8 import nki_gemm_fp8, nki_gemm_fp8_nn  # noqa: E402  (namespaces, as the reference uses its modules)


# ------------------------------------------------------------------------------------------ dense bf16 fused MLP (R2:6782; K/nki_mlp_fused.py)
def mlp_fused_applies(x2, f):
    """The shapes the dense fused MLP kernels take: token rows, model width and hidden width multiples of 128
    (K/nki_mlp_fused.py:364 shapes_apply)."""
    return x2.dim() == 2 and x2.shape[0] > 0 and x2.shape[0] % 128 == 0 and x2.shape[1] % 128 == 0 and f % 128 == 0


def mlp_fwd_kernel(x2, w_fc, w_proj, tb=None):
    """(y [M, d], rT [F, M]) as _mlp_fwd_kernel returns them (K/nki_mlp_fused.py:242); rT is a transposed view of the
    token-major r the backward reads. `tb` (the reference's token-block size) is accepted and unused."""
    y, r = ops.mlp_fwd(x2.contiguous(), w_fc.contiguous(), w_proj.contiguous())
    return y, r.t()


def mlp_bwd_kernel(dy2, rT, w_fc, w_proj, tb=None, dw_mode=0):
    """(dx, h, dpre) as _mlp_bwd_kernel returns them (K/nki_mlp_fused.py:290): token-major [M, F] for dw_mode 0, their
    transposes [F, M] for dw_mode 1."""
    r = rT.t()
    dx, h, dpre = ops.mlp_bwd(dy2.contiguous(), r if r.is_contiguous() else r.contiguous(), w_fc.contiguous(), w_proj.contiguous())
    if dw_mode == 1:
        return dx, h.t().contiguous(), dpre.t().contiguous()
    return dx, h, dpre


def mlp_fused(mlp, x):
    """MLP.forward on [b, t, n_embd] through the dense bf16 fused kernels (R2:6782): `mlp` has c_fc.weight [F, d] and
    c_proj.weight [d, F]. Raises TfbError for a shape the kernels do not take (the round-2 policy)."""
    b, t, c = x.shape
    x2 = x.reshape(b * t, c).contiguous()
    w_fc = mlp.c_fc.weight.to(dtype=x.dtype)
    w_proj = mlp.c_proj.weight.to(dtype=x.dtype)
    return A.MlpFusedFn.apply(x2, w_fc, w_proj).view(b, t, c)


# ------------------------------------------------------------------------------------------ gradient norm (R1:1480, 1634)
def grad_norm_fused(g_bf16=None, g_f32=None, clip=0.0):
    """(gnorm, scale) as 0-dim device tensors: the global gradient norm over the two flat gradient buffers in one kernel
    pair, and the clipping factor clamp(clip / (gnorm + 1e-6), max=1) the caller multiplies the gradients by (1 for
    clip <= 0), as reduce_fused computes them (R1:1634-1720). Nothing is read back by the host."""
    out = ops.gradnorm(g_bf16, g_f32, clip)
    return out[2], out[3]


# ------------------------------------------------------------------------------------------ mixer tail (R1:7308)
def shift1(x):
    """Token t of every sequence reads token t - 1; token 0 reads zeros (R1:300)."""
    return torch.cat([torch.zeros_like(x[:, :1]), x[:, :-1]], dim=1)


def mix_tail(x, xn_dead, lam):
    """(s1, xn2) = (x + lam * shift1(x), RMSNorm(s1)) for a [B, T, C] stream in one launch each way (R1:7308). xn_dead (the
    head's unused x_norm) is accepted for the reference's signature and not read."""
    B, T, C = x.shape
    s1, y = A.MixTailFn.apply(x.reshape(B * T, C), lam, T)
    return s1.view(B, T, C), y.view(B, T, C)
