"""CPU restatement of the fp8 MLP rows of the reference's round1 sources (fixed power-of-two scales). TEST INFRASTRUCTURE ONLY.

Follows round1/source/train.py: clip_bound 2272-2283, ROW_SPEC 2300, the constants 1758-1759 and 2234-2243, and the
arithmetic stated in the module text at 1746 ("out = (s_a A)^T (s_w W) / (s_a s_w), both operands rounded to e4m3 after
scaling, fp32 accumulation, one bf16 rounding"), with the reference chip's e4m3 maximum of 240 as the clamp.

Pins (tests/test_oracle_r1fp8.py): the casts against the byte tables decoded from the format definitions
(tests/golden/fp8_tables.json); the clamp bound's defining inequality; exactness of the power-of-two scaling; and the
rows against the plain fp64 products of the unrounded operands within the formats' rounding budgets.
"""
import torch

E4M3_MAX, E5M2_MAX = 240.0, 57344.0
ROW_SPEC = {
    1: dict(afmt=0, ascale=4.0, wscale=64.0, trans_b=False),
    2: dict(afmt=0, ascale=1.0 / 128, wscale=16.0, trans_b=True),
    3: dict(afmt=1, ascale=2.0 ** 30, wscale=128.0, trans_b=True),
    4: dict(afmt=1, ascale=2.0 ** 30, wscale=16.0, trans_b=False),
    5: dict(afmt=0, ascale=16.0, bfmt=1, bscale=2.0 ** 30),
    6: dict(afmt=1, ascale=2.0 ** 30, bfmt=0, bscale=1.0 / 128),
}
_DT = {0: torch.float8_e4m3fn, 1: torch.float8_e5m2}


def clip_bound(scale, fmt=0):
    hi = E5M2_MAX if fmt == 1 else E4M3_MAX
    b = torch.tensor(hi / scale, dtype=torch.float32).to(torch.bfloat16)
    for _ in range(4):
        if float(b) * scale <= hi:
            break
        b = torch.nextafter(b, torch.tensor(0.0, dtype=torch.bfloat16))
    return float(b)


def q(a, scale, fmt):
    """The fp8 value (as fp32) of clamp(a) * scale."""
    b = clip_bound(scale, fmt)
    return (a.clamp(-b, b).float() * scale).to(_DT[fmt]).float()


def row_matmul(a2d, w, row):
    sp = ROW_SPEC[row]
    qa, qw = q(a2d, sp["ascale"], sp["afmt"]), q(w, sp["wscale"], 0)
    acc = qa @ (qw.t() if sp["trans_b"] else qw)
    return (acc * (1.0 / (sp["ascale"] * sp["wscale"]))).to(torch.bfloat16)


def dw_matmul(a2d, b2d, row):
    sp = ROW_SPEC[row]
    qa, qb = q(a2d, sp["ascale"], sp["afmt"]), q(b2d, sp["bscale"], sp["bfmt"])
    return ((qa.t() @ qb) * (1.0 / (sp["ascale"] * sp["bscale"]))).to(torch.bfloat16)


def mlp_forward_backward(x, w1, w2, dy):
    """The six rows chained as the reference's FcRelu2NNFn / _ProjFn do: returns (y, dx, dw1, dw2)."""
    pre = row_matmul(x, w1, 1)
    h = (torch.relu(pre.float()) * pre.float()).to(torch.bfloat16)
    y = row_matmul(h, w2, 2)
    dh = row_matmul(dy, w2, 4)
    dpre = (2.0 * torch.relu(pre.float()) * dh.float()).to(torch.bfloat16)
    dx = row_matmul(dpre, w1, 3)
    return y, dx, dw_matmul(x, dpre, 5), dw_matmul(dy, h, 6)
