"""Mixture-of-experts oracle: router, top-k, dropless dispatch, per-expert fp8 MLPs, gated combine.

Restates R2:10505-10553 (moe_tournament: first maximum, ties low; moe_route: fp32 softmax of the router logits, top-2
gates renormalised v1 / (v1 + v2), top-1 gate = the probability), R2:10961 (logits = F.linear(h.float(), router.float())),
R2:10652-10688 (dispatch / combine as gathers), R2:10753-10776 (moe_experts8_local: one fp8 MLP per expert with the expert's
own scale row, rows padded with zeros to a multiple of 128) and R2:10990-10992 (out = g1.to(dt) * y1 + g2.to(dt) * y2 in the
activations' dtype). The reference places assignments in per-sequence capacity slots and drops the overflow; with a capacity
that drops nothing its output is this function, because a zero padding row yields a zero output row and touches no other
row (R2:10735-10737). Gradients come from torch.autograd over these expressions with the fp8 MLP's own backward
(oracle.mlp8), as EmulatedFusedMlp8 does.

Pinned by (tests/test_oracle_moe.py): torch.topk for the selections, gates summing to one, a brute-force per-token loop
with the bf16 expert MLP, permutation equivariance over tokens, and the reference's capacity layout computed with a cumsum
giving the same output when nothing is dropped; the auxiliary terms by their closed forms (uniform router, one-hot router),
fp64 autograd and, for the per-sequence term, its reduction to the global term on one sequence and a token loop; the capacity's keep rule by a plain loop over each sequence's tokens, and the
reference's [E][b][cap] buffer with its zero row for skipped assignments giving the same output bit for bit when it drops.
"""
import torch
import torch.nn.functional as F

from . import mlp8 as omlp


def route(h2, router, topk, bias=None):
    """(p [N, E] fp32, idx [N, k] int64, gate [N, k] fp32, logits)."""
    logits = F.linear(h2.float(), router.float())
    if bias is not None:
        logits = logits + bias.float()
    p = torch.softmax(logits, dim=-1)
    idx, gate = select(p, topk)
    return p, idx, gate, logits


def select(p, topk):
    """(idx [N, k] int64, gate [N, k] fp32) from probabilities p [N, E]: the reference's tournament
    (round2/source/train.py:10505 moe_tournament: the largest value wins, exact ties go to the LOWER expert index),
    the second choice the same over the rest, gates renormalised over the two (the probability itself at k = 1)."""
    i1 = torch.argmax(p, dim=-1)                      # first maximum: ties go to the lower index
    v1 = p.gather(1, i1[:, None]).squeeze(1)
    if topk == 1:
        return i1[:, None], v1[:, None]
    masked = p.masked_fill(F.one_hot(i1, p.shape[1]).bool(), -1.0)
    i2 = torch.argmax(masked, dim=-1)
    v2 = p.gather(1, i2[:, None]).squeeze(1)
    den = v1 + v2
    return torch.stack([i1, i2], 1), torch.stack([v1 / den, v2 / den], 1)


def tables(idx, E, seq_len=None, capacity=None):
    """Ragged layout: expert e's assignments contiguous in token order, segments padded to 128 rows.
    Returns (slot [N, k] int64, tok [R] int64 (-1 padding), seg [E+1]).
    With seq_len and capacity, the reference's keep rule (round2/source/train.py:10555 moe_positions, :10600 keep = pos < cap):
    an assignment's position is the number of assignments to its expert at earlier tokens of the same sequence, both choices
    counted; positions at or beyond the capacity are skipped (slot -1) and hold no row."""
    N, k = idx.shape
    flat_e = idx.reshape(-1)
    onehot = F.one_hot(flat_e, E).reshape(N, k, E).sum(1)             # assignments per token per expert (0/1)
    if capacity is None:
        keep = torch.ones(N, k, dtype=torch.bool)
    else:
        oh3 = onehot.reshape(N // seq_len, seq_len, E)
        excl = (torch.cumsum(oh3, 1) - oh3).reshape(N, E)             # earlier tokens of the same sequence
        keep = excl.gather(1, idx) < capacity
    kept = torch.zeros(N, E, dtype=torch.long)
    kept.scatter_add_(1, idx, keep.long())                            # kept assignments per token per expert (0/1)
    cnt = kept.sum(0)
    pad = (cnt + 127) // 128 * 128
    seg = torch.zeros(E + 1, dtype=torch.long)
    seg[1:] = torch.cumsum(pad, 0)
    before = torch.cumsum(kept, 0) - kept                             # kept ones from earlier tokens
    pos = before.gather(1, idx)
    slot = torch.where(keep, seg[idx] + pos, torch.full_like(pos, -1))
    tok = torch.full((int(seg[-1]),), -1, dtype=torch.long)
    for j in range(k):
        kj = keep[:, j]
        tok[slot[kj, j]] = torch.arange(N)[kj]
    return slot, tok, seg


class _ExpertMlp8(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x2, w_fc, w_proj, row, x_scale, dy_amax=None, dw_fp8=False, e4m3_limit=240.0):
        y, r = omlp.forward(x2, w_fc, w_proj, row, x_scale)
        ctx.save_for_backward(x2, r, w_fc, w_proj, row)
        ctx.dy_amax, ctx.dw_fp8, ctx.x_scale, ctx.e4m3_limit = dy_amax, dw_fp8, x_scale, e4m3_limit
        return y

    @staticmethod
    def backward(ctx, dy):
        x2, r, w_fc, w_proj, row = ctx.saved_tensors
        dy = dy.contiguous()
        # the expert's backward scales come from the amax of ITS rows of dy; a caller that runs only a slice of those
        # rows passes the amax over all of them (dy_amax), so the slice is rounded exactly as inside the whole layer
        row_b = omlp.backward_scales(dy, row, ctx.dy_amax)
        dx, h, dpre = omlp.backward(dy, r, w_fc, w_proj, row_b)
        if ctx.dw_fp8:   # the fp8 weight-gradient switch (round2/source/train.py:8209-8229) inside the expert's backward
            dw_fc, dw_proj = omlp.weight_grads_fp8(x2, dy, h, dpre, row_b, ctx.x_scale, ctx.e4m3_limit)
        else:
            dw_fc, dw_proj = omlp.weight_grads(dy, x2, h, dpre)
        return dx, dw_fc, dw_proj, None, None, None, None, None


def moe_forward(h, router, w_fc, w_proj, topk, bias=None, fp8=True, e4m3_limit=240.0, x_scale=4.0, dys_amax=None,
                capacity=None, idx=None, dw_fp8=False):
    """h [.., d] bf16; router [E, d]; w_fc [E, F, d]; w_proj [E, d, F]. Differentiable (autograd) in h, router, weights.
    fp8 False: the experts in bf16, the kit's expression per expert (round2/source/train.py:10716 moe_experts_local).
    dys_amax (optional, fp32 [E]): per-expert amax of the expert outputs' gradients to take the backward scales from,
    for a call that holds only some of the layer's tokens. idx (optional, [N, k]): selections to use instead of the
    oracle's own (a checker passes the kernel's, so that a near-tie cannot route a token differently); the gates are
    still this function's, from its own probabilities at those experts."""
    d = h.shape[-1]
    h2 = h.reshape(-1, d)
    E = w_fc.shape[0]
    p, idx_own, gate, _ = route(h2, router, topk, bias)
    if idx is None:
        idx = idx_own
    else:
        v = p.gather(1, idx)
        gate = v / v.sum(1, keepdim=True) if topk == 2 else v
    slot, tok, seg = tables(idx, E) if capacity is None else tables(idx, E, h.shape[-2], capacity)
    pad = torch.cat([h2, h2.new_zeros(1, d)], 0)
    xs = pad.index_select(0, torch.where(tok >= 0, tok, torch.full_like(tok, h2.shape[0])))
    outs = []
    for e in range(E):
        xe = xs[seg[e]:seg[e + 1]]
        if xe.shape[0] == 0:
            continue
        if fp8:
            row = omlp.forward_scales(w_fc[e].detach(), w_proj[e].detach(), e4m3_limit, x_scale)
            outs.append(_ExpertMlp8.apply(xe, w_fc[e], w_proj[e], row, x_scale,
                                          None if dys_amax is None else dys_amax[e], dw_fp8, e4m3_limit))
        else:
            outs.append(F.linear(torch.relu(F.linear(xe, w_fc[e])).square(), w_proj[e]))
    ys = torch.cat(outs, 0)
    dt = ys.dtype
    ysp = torch.cat([ys, ys.new_zeros(1, ys.shape[1])], 0)            # a skipped assignment reads the zero row
    sl = torch.where(slot >= 0, slot, torch.full_like(slot, ys.shape[0]))
    out = gate[:, 0].to(dt).unsqueeze(-1) * ysp.index_select(0, sl[:, 0])
    if topk == 2:
        out = out + gate[:, 1].to(dt).unsqueeze(-1) * ysp.index_select(0, sl[:, 1])
    return out.reshape(h.shape), {"p": p, "idx": idx, "gate": gate, "slot": slot, "tok": tok, "seg": seg}


def aux_terms(p, logits, idx, topk, seq_len=None):
    """(lb, z, f): the Switch load-balance term E sum_e f_e P_e (f_e the share of the k N assignments that chose e, no
    gradient; P_e the mean router probability) and the router z term mean(logsumexp(logits)^2)
    (round2/source/train.py:10779-10788 moe_aux_terms). With seq_len (the tokens are whole sequences of that length) a
    fourth value: the per-sequence balance term, the mean over sequences of E sum_e fs_e ps_e with the shares and mean
    probabilities taken inside each sequence (10789-10792, the reference's R2_MOE_AUX_SEQ)."""
    N, E = p.shape
    mall = torch.zeros(N, E, dtype=p.dtype)
    mall.scatter_add_(1, idx.long(), torch.ones(idx.shape, dtype=p.dtype))
    f = mall.mean(0) / topk
    lb = E * (f * p.mean(0)).sum()
    z = torch.logsumexp(logits, dim=-1).square().mean()
    if seq_len is None:
        return lb, z, f
    fs = mall.reshape(N // seq_len, seq_len, E).mean(1) / topk
    ps = p.reshape(N // seq_len, seq_len, E).mean(1)
    return lb, z, f, (E * (fs * ps).sum(-1)).mean()
