"""AdamW oracle: R1:9670-9677 (_adamw_update) == R2:13756-13766 (adamw_math_body): decay, two lerps, the update
divided by the two bias corrections separately, one subtraction. Not torch.optim.AdamW's operation order.

Pinned by (tests/test_oracle_norm_loss.py): agreement with torch.optim.AdamW to fp32 rounding over several steps, and the
closed form of the first step from zero state (update = lr * g / (|g| + eps), independent of beta)."""
import torch


def adamw_step(p, grad, exp_avg, exp_avg_sq, step, lr, beta1, beta2, eps, weight_decay):
    """In place on fp32 p, exp_avg, exp_avg_sq."""
    bias1 = 1.0 - beta1 ** step
    bias2 = 1.0 - beta2 ** step
    if weight_decay > 0:
        p.mul_(1 - lr * weight_decay)
    g = grad.float()
    exp_avg.lerp_(g, 1 - beta1)
    exp_avg_sq.lerp_(g.square(), 1 - beta2)
    update = exp_avg / bias1 / ((exp_avg_sq / bias2).sqrt() + eps)
    p.sub_(update * lr)
    return p
