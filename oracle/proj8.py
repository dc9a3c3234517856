"""fp8 attention projections oracle (QKV and output projection: e4m3 forward, e5m2 input gradient, power-of-two
per-tensor scales, pre-cast weights). TEST INFRASTRUCTURE: imported by tests/ only.

Restates K/nki_attn_tt8g.py: constants :51-57, the greedy power-of-two scale search `_pow2_le` :670-685 (the same
search as the MLP's, oracle/mlp8.py pow2_floor_scale), the weight scale of forward_scales :700-719 (amax of the bf16
weight, limit 240, exponent window (-24, 40)), the gradient scale of backward_tile :728-735 (amax x s <= 57344 / 2,
window (-40, 60)), the fp8 rounding q8 :738-742, emulate_fwd :745-750, emulate_bwd :753-757, reference_fwd :760. The
activation scale is the reference's constant 4 for RMSNorm outputs, or (this build's option for inputs without such a
bound, e.g. the attention output) the per-tensor amax scale found by the same search.

Pinned by (tests/test_oracle_proj8.py): the scale search is the one pinned in tests/test_oracle_mlp8.py (brute force
against 2^floor(log2(limit / v))); the casts against the bit-level fp8 tables; forward and input gradient against the
bf16 projection F.linear and its autograd within the fp8 error budget; exact invariance of the forward under
power-of-two rescaling of the weight (the scale search absorbs it); the fp8 weight gradient against autograd's within
the e5m2 budget and against an fp64 product of the operands decoded through the byte tables.
"""
import torch

from . import mlp8

E4M3_MAX = 240.0
E5M2_MAX = 57344.0
X_SCALE = 4.0
G_HEADROOM = 2.0
E_W = (-24, 40)
E_G = (-40, 60)


def weight_scale(w, limit=E4M3_MAX):
    """(s_w, 1/s_w) from the exact amax of the bf16 weight (nki_attn_tt8g.py:706-709)."""
    return mlp8.pow2_floor_scale(w.detach().bfloat16().float().abs().amax(), limit, *E_W)


def act_scale(x, limit=E4M3_MAX):
    """(s, 1/s) from the exact amax of an activation tensor: the per-tensor amax scale."""
    return mlp8.pow2_floor_scale(x.detach().float().abs().amax(), limit, *E_W)


def grad_scale(g):
    """(s_g, 1/s_g): amax(g) x s_g <= 57344 / 2 (nki_attn_tt8g.py:731-733)."""
    return mlp8.pow2_floor_scale(g.detach().float().abs().amax(), E5M2_MAX / G_HEADROOM, *E_G)


def forward(a2, w, s_a, s_w):
    """bf16((e4m3(a2 s_a) @ e4m3(w s_w)^T) / (s_a s_w)) (emulate_fwd :745-750); w [N, K]."""
    a8 = mlp8.fp8_round(a2.float() * s_a, 0)
    w8 = mlp8.fp8_round(w.float() * s_w, 0)
    return ((a8 @ w8.t()) * ((1.0 / s_a) * (1.0 / s_w))).to(a2.dtype)


def backward_input(g2, w, s_g, s_w):
    """dx [M, K] = bf16((e5m2(g2 s_g) @ e4m3(w s_w)) / (s_g s_w)) (emulate_bwd :753-757)."""
    g8 = mlp8.fp8_round(g2.float() * s_g, 1)
    w8 = mlp8.fp8_round(w.float() * s_w, 0)
    return ((g8 @ w8) * ((1.0 / s_g) * (1.0 / s_w))).to(g2.dtype)


def weight_grad(g2, a2):
    """dw [N, K] = bf16(g2^T @ a2), fp32 accumulation (the bf16 weight gradient this build keeps for the projections)."""
    return (g2.float().t() @ a2.float()).to(a2.dtype)


def weight_grad_fp8(g2, a2, s_g, s_a):
    """dw [N, K] = bf16((e5m2(g2 s_g)^T @ e4m3(a2 s_a)) / (s_g s_a)): the projection's weight gradient in fp8
    (round2/source/train.py:8232 attn8_weight_grad -> dw8_grad 8185 -> nki_dw8.py:323 emulate_dw): the g side at the
    scale the input gradient was cast with, the a side at its forward's."""
    return mlp8.fp8_weight_grad(g2, a2, s_g, s_a, (1.0 / s_g) * (1.0 / s_a), 1, 0)


def reference_forward(a2, w):
    return torch.nn.functional.linear(a2, w)
