"""Pins oracle/moe.py: torch.topk, a brute-force per-token loop, invariants, and the reference's capacity layout."""
import torch
import torch.nn.functional as F

from oracle import moe as O
from helpers import rel_l2


def _layer(seed, N=384, d=128, Fd=256, E=8):
    g = torch.Generator().manual_seed(seed)
    h = torch.randn(N, d, generator=g).bfloat16()
    router = 0.5 * torch.randn(E, d, generator=g)
    wf = (0.05 * torch.randn(E, Fd, d, generator=g)).bfloat16()
    wp = (0.05 * torch.randn(E, d, Fd, generator=g)).bfloat16()
    return h, router, wf, wp


def test_route_matches_topk_and_gates_sum_to_one():
    h, router, _, _ = _layer(0)
    p, idx, gate, logits = O.route(h, router, 2)
    tv, ti = torch.topk(p, 2, dim=-1)
    assert torch.equal(idx, ti)
    assert torch.allclose(gate.sum(-1), torch.ones(h.shape[0]), atol=1e-6)
    assert torch.allclose(gate[:, 0], tv[:, 0] / tv.sum(-1))
    p1, idx1, gate1, _ = O.route(h, router, 1)
    assert torch.equal(idx1[:, 0], p.argmax(-1)) and torch.equal(gate1[:, 0], p.max(-1).values)
    tie = torch.zeros(4, 8)
    assert O.route(torch.zeros(4, 16).bfloat16(), torch.zeros(8, 16), 2)[1].tolist() == [[0, 1]] * 4    # ties go low
    bias = torch.zeros(8)
    bias[5] = 50.0
    assert bool((O.route(h, router, 2, bias)[1][:, 0] == 5).all())


def test_tables_are_a_stable_padded_partition():
    h, router, _, _ = _layer(1)
    _, idx, _, _ = O.route(h, router, 2)
    slot, tok, seg = O.tables(idx, 8)
    assert bool((seg % 128 == 0).all()) and int(seg[-1]) == tok.numel()
    assert int((tok >= 0).sum()) == idx.numel() and slot.unique().numel() == idx.numel()
    for e in range(8):
        rows = tok[seg[e]:seg[e + 1]]
        live = rows[rows >= 0]
        assert bool((live[1:] > live[:-1]).all())                       # token order inside an expert
        assert bool(((idx[live] == e).any(1)).all())
        assert bool((rows[live.numel():] == -1).all())                  # padding at the end of the segment


def test_forward_matches_brute_force_bf16_experts():
    h, router, wf, wp = _layer(2, N=128)
    out, aux = O.moe_forward(h, router, wf, wp, 2, fp8=False)
    ref = torch.zeros(128, 128)
    for n in range(128):
        acc = None
        for j in range(2):
            e = int(aux["idx"][n, j])
            y = F.linear(torch.relu(F.linear(h[n:n + 1], wf[e])).square(), wp[e])
            term = aux["gate"][n, j].to(torch.bfloat16) * y
            acc = term if acc is None else acc + term
        ref[n] = acc.float()
    assert rel_l2(out, ref) < 1e-2


def test_token_permutation_equivariance_and_fp8_budget():
    h, router, wf, wp = _layer(3)
    out, _ = O.moe_forward(h, router, wf, wp, 2)
    perm = torch.randperm(h.shape[0], generator=torch.Generator().manual_seed(1))
    out_p, _ = O.moe_forward(h[perm], router, wf, wp, 2)
    assert rel_l2(out_p, out[perm]) < 1e-6
    out16, _ = O.moe_forward(h, router, wf, wp, 2, fp8=False)
    assert rel_l2(out, out16) < 0.15


def test_reference_capacity_layout_gives_same_output_when_nothing_drops():
    """The reference's slots: [E][b][cap] with the position = earlier assignments to e in the same sequence (R2:10555-10600).
    With cap = t nothing is dropped and its gather/combine gives the dropless output."""
    h, router, wf, wp = _layer(4, N=256)
    b, t, E = 2, 128, 8
    _, idx, gate, _ = O.route(h, router, 2)
    mall = F.one_hot(idx, E).sum(1).reshape(b, t, E)
    excl = torch.cumsum(mall, 1) - mall
    cap = t
    row = torch.arange(b).repeat_interleave(t)
    pos = excl.reshape(b * t, E).gather(1, idx)
    slot = (idx * b + row[:, None]) * cap + pos
    xs = torch.zeros(E * b * cap, h.shape[1], dtype=h.dtype)
    for j in range(2):
        xs[slot[:, j]] = h
    ys = torch.stack([F.linear(torch.relu(F.linear(xs.reshape(E, b * cap, -1)[e], wf[e])).square(), wp[e]) for e in range(E)])
    ys = ys.reshape(E * b * cap, -1)
    out = gate[:, 0].bfloat16()[:, None] * ys[slot[:, 0]] + gate[:, 1].bfloat16()[:, None] * ys[slot[:, 1]]
    ref, _ = O.moe_forward(h, router, wf, wp, 2, fp8=False)
    assert torch.equal(out, ref)


def test_capacity_keep_rule_against_a_token_loop_and_the_reference_layout():
    """With a capacity that does drop: (1) the keep decisions equal a plain loop over each sequence's tokens (an assignment's
    position = assignments to its expert at EARLIER tokens of the sequence, both choices; keep while below cap, R2:10555-10600);
    (2) kept rows are dense per expert in token order; (3) the reference's [E][b][cap] slot buffer with its zero row for
    skipped assignments (R2:10600: slot = S) gives the oracle's output bit for bit."""
    h, router, wf, wp = _layer(6, N=256)
    b, t, E, cap = 2, 128, 8, 20
    _, idx, gate, _ = O.route(h, router, 2)
    slot, tok, seg = O.tables(idx, E, t, cap)
    keep_loop = torch.zeros(b * t, 2, dtype=torch.bool)
    for r in range(b):
        count = [0] * E
        for i in range(r * t, (r + 1) * t):
            for j in range(2):
                keep_loop[i, j] = count[int(idx[i, j])] < cap
            for j in range(2):
                count[int(idx[i, j])] += 1
    assert torch.equal(slot >= 0, keep_loop)
    assert int((~keep_loop).sum()) > 50 and int(keep_loop.sum()) > 50          # the case does drop, and does keep
    for e in range(E):
        want = [(i, j) for i in range(b * t) for j in range(2) if int(idx[i, j]) == e and keep_loop[i, j]]
        rows = tok[int(seg[e]):int(seg[e]) + len(want)]
        assert rows.tolist() == [i for i, _ in want]
        assert all(int(slot[i, j]) == int(seg[e]) + n for n, (i, j) in enumerate(want))
        assert (tok[int(seg[e]) + len(want):int(seg[e + 1])] == -1).all()
    # the reference's layout and zero row
    mall = F.one_hot(idx, E).sum(1).reshape(b, t, E)
    excl = (torch.cumsum(mall, 1) - mall).reshape(b * t, E)
    row = torch.arange(b).repeat_interleave(t)
    pos = excl.gather(1, idx)
    S = E * b * cap
    rslot = torch.where(pos < cap, (idx * b + row[:, None]) * cap + pos, torch.full_like(pos, S))
    xs = torch.zeros(S + 1, h.shape[1], dtype=h.dtype)
    for j in range(2):
        xs[rslot[:, j]] = h
    xs[S] = 0
    ys = torch.stack([F.linear(torch.relu(F.linear(xs[:S].reshape(E, b * cap, -1)[e], wf[e])).square(), wp[e]) for e in range(E)])
    ys = torch.cat([ys.reshape(S, -1), ys.new_zeros(1, ys.shape[-1])], 0)
    out = gate[:, 0].bfloat16()[:, None] * ys[rslot[:, 0]] + gate[:, 1].bfloat16()[:, None] * ys[rslot[:, 1]]
    ref, _ = O.moe_forward(h.reshape(b, t, -1), router, wf, wp, 2, fp8=False, capacity=cap)
    assert torch.equal(out, ref.reshape(b * t, -1))


def test_backward_is_consistent_with_plain_autograd():
    h, router, wf, wp = _layer(5, N=128)
    hs = [h.clone().requires_grad_(True) for _ in range(2)]
    rs = [router.clone().requires_grad_(True) for _ in range(2)]
    g = torch.randn(128, 128, generator=torch.Generator().manual_seed(2)).bfloat16()
    o8, _ = O.moe_forward(hs[0], rs[0], wf, wp, 2, fp8=True)
    o16, _ = O.moe_forward(hs[1], rs[1], wf, wp, 2, fp8=False)
    o8.backward(g)
    o16.backward(g)
    assert rel_l2(hs[0].grad, hs[1].grad) < 0.2 and rel_l2(rs[0].grad, rs[1].grad) < 0.2


def test_aux_terms_closed_forms_and_gradient():
    """The auxiliary router terms: a uniform router gives lb = 1 and z = log(E)^2 whatever the selections; all tokens on
    one expert with all probability there gives lb = E; the gradient of lb wrt the logits is the softmax Jacobian of
    E f / N (f constant), checked by fp64 autograd."""
    import math
    from oracle import moe as O
    N, E = 64, 8
    logits = torch.zeros(N, E, dtype=torch.float64)
    p = torch.softmax(logits, -1)
    idx = torch.stack([torch.arange(N) % E, (torch.arange(N) + 1) % E], 1)
    lb, z, f = O.aux_terms(p, logits, idx, 2)
    assert abs(lb.item() - 1.0) < 1e-12 and abs(z.item() - math.log(E) ** 2) < 1e-12 and abs(f.sum().item() - 1.0) < 1e-12
    logits = torch.full((N, E), -50.0, dtype=torch.float64)
    logits[:, 3] = 50.0
    lb, z, f = O.aux_terms(torch.softmax(logits, -1), logits, torch.full((N, 1), 3), 1)
    assert abs(lb.item() - E) < 1e-9 and abs(z.item() - 2500.0) < 1e-6 and f[3] == 1.0
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(N, E, generator=g, dtype=torch.float64, requires_grad=True)
    p = torch.softmax(logits, -1)
    idx = torch.topk(p, 2, dim=-1).indices
    lb, z, f = O.aux_terms(p, logits, idx, 2)
    (0.3 * lb + 0.7 * z).backward()
    pd = p.detach()
    dp = 0.3 * E * f / N
    want = pd * (dp - (pd * dp).sum(-1, keepdim=True)) + 0.7 * 2.0 / N * torch.logsumexp(logits.detach(), -1, keepdim=True) * pd
    assert torch.allclose(logits.grad, want, atol=1e-12)


def test_per_sequence_balance_term_special_cases_and_a_token_loop():
    """The per-sequence balance term (round2/source/train.py:10789-10792): with ONE sequence it is the global term lb;
    with identical sequences it equals each sequence's own lb; a sequence whose tokens all go, with all probability, to
    one expert contributes E, a uniform one 1, so two such sequences give (E + 1) / 2; and on random inputs it matches a
    plain loop over sequences, tokens and choices."""
    from oracle import moe as O
    g = torch.Generator().manual_seed(4)
    T, E = 32, 8
    logits = torch.randn(T, E, generator=g, dtype=torch.float64)
    p = torch.softmax(logits, -1)
    idx = torch.topk(p, 2, dim=-1).indices
    lb, z, f, seq = O.aux_terms(p, logits, idx, 2, seq_len=T)
    assert abs(seq.item() - lb.item()) < 1e-12                                   # one sequence: the global term
    lb3, _, _, seq3 = O.aux_terms(p.repeat(3, 1), logits.repeat(3, 1), idx.repeat(3, 1), 2, seq_len=T)
    assert abs(seq3.item() - lb.item()) < 1e-12 and abs(lb3.item() - lb.item()) < 1e-12
    hot = torch.full((T, E), -60.0, dtype=torch.float64)
    hot[:, 5] = 60.0
    flat = torch.zeros(T, E, dtype=torch.float64)
    lg = torch.cat([hot, flat])
    ix = torch.cat([torch.full((T, 1), 5), (torch.arange(T) % E).unsqueeze(1)])
    _, _, _, seq2 = O.aux_terms(torch.softmax(lg, -1), lg, ix, 1, seq_len=T)
    assert abs(seq2.item() - (E + 1) / 2) < 1e-9
    B = 5
    logits = torch.randn(B * T, E, generator=g, dtype=torch.float64) * 2
    p = torch.softmax(logits, -1)
    idx = torch.topk(p, 2, dim=-1).indices
    want = 0.0
    for b in range(B):
        cnt = [0] * E
        psum = [0.0] * E
        for t in range(T):
            n = b * T + t
            for k in range(2):
                cnt[int(idx[n, k])] += 1
            for e in range(E):
                psum[e] += float(p[n, e])
        want += E * sum((cnt[e] / (2 * T)) * (psum[e] / T) for e in range(E))
    _, _, _, seq = O.aux_terms(p, logits, idx, 2, seq_len=T)
    assert abs(seq.item() - want / B) < 1e-12

