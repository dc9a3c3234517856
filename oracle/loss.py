"""Loss-head oracle: softcap + log-softmax + cross-entropy on the raw LM-head output, and the composition
final RMSNorm -> LM-head GEMM -> loss that configuration 1 of BASELINE.json times.

Restates R1:4481-4495 (eager loss rows: logits.float(), softcap * tanh(logits / softcap), log_softmax, one-hot
pick), the gradient stated in the R1 loss-head docstring (R1:4466: d x = g (softmax - onehot) (1 - tanh^2)),
R2:6364-6391 / 11688-11703 (mean over valid rows with ignore_index -1 as row weights valid / sum(valid)), and
the LM head in front of it (R1:8668 `y = x2d @ W`, R1:9191-9212). The reference never fuses the GEMM with the
loss; its oracle is this composition, with the logits rounded to bf16 between the two.

Pinned by (tests/test_oracle_norm_loss.py): torch.nn.functional.cross_entropy on the softcapped fp32 logits,
torch.autograd for the gradient, loss at uniform logits = ln V, sum_v dlogits / (1 - tanh^2) = 0 per row; the
several-target / label-smoothed rows by F.cross_entropy(..., label_smoothing=eps) and by a weighted sum of single-target
F.cross_entropy calls, their gradient by torch.autograd in fp64.
"""
import torch
import torch.nn.functional as F


def softcap_logits(x, softcap):
    xf = x.float()
    if softcap:
        return softcap * torch.tanh(xf / softcap)
    return xf


def loss_rows(logits2, targets, softcap=15.0):
    """(rows fp32 [N], lse fp32 [N]); rows whose target lies outside [0, V) (the reference's ignore_index -1; an id
    beyond the vocabulary is treated the same way) give 0."""
    s = softcap_logits(logits2, softcap)
    lse = torch.logsumexp(s, dim=-1)
    t = targets.reshape(-1).long()
    valid = (t >= 0) & (t < s.shape[-1])
    picked = s.gather(1, t.clamp(0, s.shape[-1] - 1)[:, None]).squeeze(1)
    return torch.where(valid, lse - picked, torch.zeros_like(lse)), lse


def row_weights(targets, reduction="mean", V=None):
    """valid / sum(valid) for "mean", valid for "sum"; a row is valid when 0 <= t < V (V None: when t >= 0): the rows
    loss_rows gives a loss to."""
    t = targets.reshape(-1)
    valid = ((t >= 0) if V is None else ((t >= 0) & (t < V))).float()
    return valid / valid.sum().clamp_min(1.0) if reduction == "mean" else valid


def fused_loss(logits, targets, reduction="mean", softcap=15.0):
    V = logits.shape[-1]
    rows, _ = loss_rows(logits.reshape(-1, V), targets, softcap)
    if reduction == "none":
        return rows.view_as(targets)
    return (rows * row_weights(targets, reduction, V)).sum()


def loss_backward(logits2, targets, lse, grow, softcap=15.0):
    """dlogits in logits' dtype; grow [N] fp32 (upstream gradient times row weight)."""
    xf = logits2.float()
    t = targets.reshape(-1).long()
    valid = ((t >= 0) & (t < xf.shape[-1])).float()
    onehot = F.one_hot(t.clamp(0, xf.shape[-1] - 1), xf.shape[-1]).float()
    if softcap:
        th = torch.tanh(xf / softcap)
        p = torch.exp(softcap * th - lse[:, None])
        d = (p - onehot) * (1.0 - th * th)
    else:
        d = torch.exp(xf - lse[:, None]) - onehot
    return (d * (grow * valid)[:, None]).to(logits2.dtype)


def lmhead_loss(x, norm_w, W, targets, eps=1e-6, softcap=None):
    """Config 1 forward: mean loss from hidden states x [N, d] (bf16), norm weight [d], head weight W [V, d]."""
    from . import norm as _n
    xn, inv = _n.rmsnorm(x, norm_w, eps)
    logits = (xn.float() @ W.float().t()).to(x.dtype)
    return fused_loss(logits, targets, "mean", softcap), (xn, inv, logits)


def lmhead_loss_backward(x, norm_w, W, targets, saved, eps=1e-6, softcap=None, gloss=1.0):
    """(dx bf16 [N, d], dnorm_w fp32 [d], dW bf16 [V, d]) for the mean loss."""
    from . import norm as _n
    xn, inv, logits = saved
    _, lse = loss_rows(logits, targets, softcap)
    grow = row_weights(targets, "mean", logits.shape[-1]) * gloss
    dl = loss_backward(logits, targets, lse, grow, softcap)
    dxn = (dl.float() @ W.float()).to(x.dtype)
    dW = (dl.float().t() @ xn.float()).to(x.dtype)
    dx, dw = _n.rmsnorm_backward(dxn, x, inv, norm_w)
    return dx.to(x.dtype), dw, dW


def loss_multi_rows(logits2, tg, rw, softcap=15.0, eps=0.0):
    """(rows fp32 [N], lse fp32 [N]): rows = sum_k rw[k] (lse - (1 - eps) s_{t_k} - eps mean_v s_v), tg [K, N] (a target
    < 0 counts with weight 0), rw fp32 [K, N]. eps = 0: the multi-target rows sum_k rw_k nll_k of round1/source/train.py
    :4860-4868 (kernel :4725); K = 1, eps > 0: the label-smoothed row of round2/source/train.py:5697-5760
    (tgt_coef = -(1 - eps) c on tanh, mean_coef = -eps c / V on sum_v tanh)."""
    s = softcap_logits(logits2, softcap)
    lse = torch.logsumexp(s, dim=-1)
    mean_s = s.mean(dim=-1)
    rows = torch.zeros_like(lse)
    for k in range(tg.shape[0]):
        t = tg[k].reshape(-1).long()
        valid = (t >= 0).float()
        picked = s.gather(1, t.clamp_min(0)[:, None]).squeeze(1)
        rows = rows + rw[k].float() * valid * (lse - (1.0 - eps) * picked - eps * mean_s)
    return rows, lse


def loss_multi_backward(logits2, tg, rw, lse, g, softcap=15.0, eps=0.0):
    """dlogits = g (1 - tanh^2) (W softmax - (1 - eps) sum_k rw_k onehot_k - W eps / V), W = sum_k rw_k over the valid
    targets (round1/source/train.py:4778 docstring; round2/source/train.py:5762-5766 comment)."""
    xf = logits2.float()
    V = xf.shape[-1]
    hot = torch.zeros_like(xf)
    W = torch.zeros(xf.shape[0])
    for k in range(tg.shape[0]):
        t = tg[k].reshape(-1).long()
        w = rw[k].float() * (t >= 0).float()
        hot.scatter_add_(1, t.clamp_min(0)[:, None], w[:, None])
        W = W + w
    if softcap:
        th = torch.tanh(xf / softcap)
        p = torch.exp(softcap * th - lse[:, None])
        chain = 1.0 - th * th
    else:
        p = torch.exp(xf - lse[:, None])
        chain = 1.0
    d = (W[:, None] * p - (1.0 - eps) * hot - (W * eps / V)[:, None]) * chain
    return (d * g[:, None]).to(logits2.dtype)

