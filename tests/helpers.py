import json
import os

import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def rel_l2(a, b):
    a = a.detach().float().cpu()
    b = b.detach().float().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def fp8_table(name):
    with open(os.path.join(HERE, "golden", "fp8_tables.json")) as f:
        t = json.load(f)[name]
    return torch.tensor([float(v) if not isinstance(v, str) else float(v) for v in t], dtype=torch.float64)


def round_to_table(x, table):
    """Round-to-nearest-even of fp64 values x onto the finite values of an fp8 table (brute force over the 256 bytes):
    returns the chosen byte index. Ties go to the byte with an even mantissa (even byte value)."""
    finite = torch.isfinite(table)
    idx = torch.nonzero(finite).flatten()
    vals = table[idx]
    d = (x.double()[:, None] - vals[None, :]).abs()
    best = d.min(dim=1, keepdim=True).values
    cand = d == best
    # among candidates prefer even byte; for +-0 prefer the sign of x
    even = (idx % 2 == 0)[None, :]
    pick_even = cand & even
    use = torch.where(pick_even.any(dim=1, keepdim=True), pick_even, cand)
    neg = (torch.signbit(x.double()))[:, None]
    sign_ok = ((idx >= 128)[None, :] == neg)
    use2 = use & sign_ok
    use = torch.where(use2.any(dim=1, keepdim=True), use2, use)
    return idx[use.float().argmax(dim=1)]
