"""MoE layer on the HIP kernels against the oracle (configuration 5 of BASELINE.json shapes in the last test)."""
import pytest
import torch

from helpers import rel_l2

pytestmark = pytest.mark.gpu


def _layer(seed, N, d, Fd, E, skew=0.0):
    g = torch.Generator().manual_seed(seed)
    h = torch.randn(N, d, generator=g).bfloat16()
    router = 0.02 * torch.randn(E, d, generator=g) * 8
    wf = (0.02 * torch.randn(E, Fd, d, generator=g)).bfloat16()
    wp = (0.02 * torch.randn(E, d, Fd, generator=g)).bfloat16()
    bias = torch.zeros(E)
    bias[:2] = skew
    return h, router, wf, wp, bias


@pytest.mark.parametrize("topk", [2, 1])
@pytest.mark.parametrize("skew", [0.0, 2.0])
def test_routing_tables_bit_exact(dev, topk, skew):
    from oracle import moe as O
    from trainium_frontier_them_bones_amd import ops
    h, router, _, _, bias = _layer(1, 2048 + 64, 256, 512, 8, skew)
    p, idx, gate, logits = ops.moe_route(h.to(dev), router.to(dev), topk, bias.to(dev), want_logits=True)
    po, io, go, lo = O.route(h, router, topk, bias)
    assert rel_l2(logits, lo) < 1e-5 and rel_l2(p, po) < 1e-5 and rel_l2(gate, go) < 1e-5
    agree = (idx.cpu().long() == io).all(1)
    assert agree.float().mean().item() > 0.999           # against torch's own logits a near-tie may pick differently ...
    # ... but the selection is index work: on the kernel's OWN probabilities the reference's rule (largest value, ties
    # to the lower index, gates renormalised over the two) must give the kernel's picks and gates bit for bit
    isel, gsel = O.select(p.cpu(), topk)
    assert torch.equal(idx.cpu().long(), isel) and torch.equal(gate.cpu(), gsel)
    assert rel_l2(p, torch.softmax(logits.cpu(), dim=-1)) < 1e-6
    tab = ops.moe_tables(idx, 8)
    slot, tok, seg = O.tables(idx.cpu().long(), 8)       # oracle tables from the kernel's own selections
    assert torch.equal(tab["seg"].cpu().long(), seg)
    assert torch.equal(tab["slot"].cpu().long(), slot)
    R = int(seg[-1])
    assert torch.equal(tab["tok"].cpu().long()[:R], tok)
    te = tab["tile_expert"].cpu()
    for e in range(8):
        assert bool((te[int(seg[e]) // 128:int(seg[e + 1]) // 128] == e).all())
    assert bool((te[R // 128:] == -1).all())


@pytest.mark.parametrize("topk", [2, 1])
def test_routing_exact_ties_go_to_the_lower_index(dev, topk):
    """Router rows 1 and 4 are equal, and so are rows 2 and 6: their logits and probabilities tie exactly on every token.
    The reference's tournament (round2/source/train.py:10505) gives a tie to the lower index, for the first choice and
    for the second."""
    from oracle import moe as O
    from trainium_frontier_them_bones_amd import ops
    h, router, _, _, _ = _layer(9, 1024, 256, 512, 8)
    router[4] = router[1]
    router[6] = router[2]
    p, idx, gate, logits = ops.moe_route(h.to(dev), router.to(dev), topk, None, want_logits=True)
    pc, ic = p.cpu(), idx.cpu().long()
    assert torch.equal(pc[:, 1], pc[:, 4]) and torch.equal(pc[:, 2], pc[:, 6])
    isel, gsel = O.select(pc, topk)
    assert torch.equal(ic, isel) and torch.equal(gate.cpu(), gsel)
    first = ic[:, 0]
    assert not bool(((first == 4) | (first == 6)).any())                  # the upper twin never wins the first place
    assert int(((first == 1) | (first == 2)).sum()) > 100                 # and the tie does decide many tokens
    if topk == 2:
        # where the lower twin won, its equal upper twin is the runner-up (nothing is larger than the maximum)
        assert bool((ic[first == 1, 1] == 4).all()) and bool((ic[first == 2, 1] == 6).all())
        # where the twins tie for second place, the lower one takes it
        assert not bool((((ic[:, 1] == 4) & (first != 1)) | ((ic[:, 1] == 6) & (first != 2))).any())
    # and against torch's argmax on torch's own logits (exact ties are exact there too)
    _, io, _, _ = O.route(h, router, topk)
    assert (ic == io).all(1).float().mean().item() > 0.999


@pytest.mark.parametrize("N,d,E", [(1003, 768, 5), (7, 64, 2), (4096, 1024, 8), (1000, 520, 11)])
@pytest.mark.parametrize("topk", [2, 1])
def test_routing_ragged_shapes(dev, N, d, E, topk):
    """Token counts that are not whole groups of eight, widths that leave lanes without columns (768, 520, 64) and expert
    counts below eight (and above, which take the one-token kernel): logits against the oracle, selections and gates by the
    reference's rule on the kernel's own probabilities, bit for bit."""
    from oracle import moe as O
    from trainium_frontier_them_bones_amd import ops
    h, router, _, _, _ = _layer(21, N, d, 64, E)
    bias = 0.1 * torch.randn(E, generator=torch.Generator().manual_seed(3))
    p, idx, gate, logits = ops.moe_route(h.to(dev), router.to(dev), topk, bias.to(dev), want_logits=True)
    po, _, _, lo = O.route(h, router, topk, bias)
    assert rel_l2(logits, lo) < 1e-5 and rel_l2(p, po) < 1e-5
    isel, gsel = O.select(p.cpu(), topk)
    assert torch.equal(idx.cpu().long(), isel) and torch.equal(gate.cpu(), gsel)
    assert rel_l2(p, torch.softmax(logits.cpu(), dim=-1)) < 1e-6
    p2, idx2, gate2, _ = ops.moe_route(h.to(dev), router.to(dev), topk, bias.to(dev))          # without the logits output
    assert torch.equal(p2, p) and torch.equal(idx2, idx) and torch.equal(gate2, gate)


@pytest.mark.parametrize("skew", [0.0, 2.0])
def test_backward_scales_from_the_combine_backward_row_maxima(dev, skew):
    """The experts' amax(dys) taken inside the combine backward (row maxima, then one maximum per segment) gives the scale
    rows of the separate pass over dys bit for bit, with a starved expert and padding rows in the buffer."""
    from trainium_frontier_them_bones_amd import autograd as A
    from trainium_frontier_them_bones_amd import ops
    N, d, Fd, E = 1000, 256, 512, 8
    h, router, wf, wp, bias = _layer(31, N, d, Fd, E, skew)
    bias[5] = -1e4
    hd, rd = h.to(dev), router.to(dev)
    st = A.Moe8State()
    st.refresh(wf.to(dev), wp.to(dev))
    _, idx, gate, _ = ops.moe_route(hd, rd, 2, bias.to(dev))
    tab = ops.moe_tables(idx, E)
    rmax = tab["tok"].shape[0]
    g = torch.Generator().manual_seed(7)
    ys = torch.randn(rmax, d, generator=g).bfloat16().to(dev)
    dout = (torch.randn(N, d, generator=g) * torch.logspace(-3, 2, N)[:, None]).bfloat16().to(dev)
    dys, dgate = ops.moe_combine_bwd(dout, ys, tab, gate)
    dys2, dgate2, rowmax = ops.moe_combine_bwd(dout, ys, tab, gate, want_rowmax=True)
    assert torch.equal(dys, dys2) and torch.equal(dgate, dgate2)
    assert torch.equal(rowmax, dys.float().abs().amax(1))
    rows_a = ops.moe_backward_scales(dys, st.rows, tab)
    rows_b = ops.moe_backward_scales_rowmax(rowmax, st.rows, tab, d)
    assert torch.equal(rows_a, rows_b)
    assert bool(torch.isfinite(rows_b).all()) and int(tab["cnt"][5]) == 0


@pytest.mark.parametrize("shape,topk,skew", [((1024, 256, 512, 8), 2, 0.0), ((1024, 256, 512, 4), 1, 0.0),
                                              ((2048, 512, 768, 8), 2, 2.0)])
def test_moe_layer_forward_backward(dev, shape, topk, skew):
    from oracle import moe as O
    from trainium_frontier_them_bones_amd import autograd as A
    N, d, Fd, E = shape
    h, router, wf, wp, bias = _layer(2, N, d, Fd, E, skew)
    hd = h.to(dev).requires_grad_(True)
    rd = router.to(dev).requires_grad_(True)
    wfd = wf.to(dev).requires_grad_(True)
    wpd = wp.to(dev).requires_grad_(True)
    st = A.Moe8State()
    st.refresh(wfd, wpd)
    out = A.MoeMlp8Fn.apply(hd, rd, wfd, wpd, st, topk, bias.to(dev) if skew else None)
    g = torch.randn(N, d, generator=torch.Generator().manual_seed(3)).bfloat16()
    out.backward(g.to(dev))
    ho, ro, wfo, wpo = (t.clone().requires_grad_(True) for t in (h, router, wf, wp))
    oo, aux = O.moe_forward(ho, ro, wfo, wpo, topk, bias if skew else None)
    oo.backward(g)
    assert rel_l2(out, oo) < 2e-2
    assert rel_l2(hd.grad, ho.grad) < 2e-2
    assert rel_l2(wfd.grad, wfo.grad) < 2e-2 and rel_l2(wpd.grad, wpo.grad) < 2e-2
    assert rel_l2(rd.grad, ro.grad) < 2e-2


@pytest.mark.parametrize("experts", ["fp8", "fp8 weight gradients too", "bf16"])
def test_moe_starved_expert_and_ragged_token_count(dev, experts):
    """One expert's router bias keeps every token away from it (empty segment, zero weight gradient, finite scales) and the
    token count is not a multiple of the 64-token counting groups; with the experts in fp8, with their weight gradients in
    fp8 as well, and in bf16."""
    from oracle import moe as O
    from trainium_frontier_them_bones_amd import autograd as A
    from trainium_frontier_them_bones_amd import ops
    N, d, Fd, E = 1000, 256, 512, 4
    h, router, wf, wp, bias = _layer(11, N, d, Fd, E)
    bias[2] = -1e4
    hd, rd, wfd, wpd = (t.to(dev).requires_grad_(True) for t in (h, router, wf, wp))
    st = None
    if experts != "bf16":
        st = A.Moe8State(dw_fp8=experts != "fp8")
        st.refresh(wfd, wpd)
    out = A.MoeMlp8Fn.apply(hd, rd, wfd, wpd, st, 2, bias.to(dev))
    g = torch.randn(N, d, generator=torch.Generator().manual_seed(5)).bfloat16()
    out.backward(g.to(dev))
    _, idx, _, _ = ops.moe_route(hd.detach(), rd.detach(), 2, bias.to(dev))
    tab = ops.moe_tables(idx, E)
    assert int(tab["cnt"][2]) == 0 and int(tab["cnt"].sum()) == 2 * N
    assert int(tab["seg"][3]) == int(tab["seg"][2])                              # an empty segment takes no rows
    ho, ro, wfo, wpo = (t.clone().requires_grad_(True) for t in (h, router, wf, wp))
    oo, _ = O.moe_forward(ho, ro, wfo, wpo, 2, bias, fp8=experts != "bf16", dw_fp8=experts == "fp8 weight gradients too")
    oo.backward(g)
    assert rel_l2(out, oo) < 2e-2 and rel_l2(hd.grad, ho.grad) < 2e-2 and rel_l2(rd.grad, ro.grad) < 2e-2
    assert float(wfd.grad[2].float().abs().max()) == 0.0 and float(wpd.grad[2].float().abs().max()) == 0.0
    keep = [0, 1, 3]
    assert rel_l2(wfd.grad[keep], wfo.grad[keep]) < 2e-2 and rel_l2(wpd.grad[keep], wpo.grad[keep]) < 2e-2
    for t in (out, hd.grad, rd.grad, wfd.grad, wpd.grad):
        assert bool(torch.isfinite(t.float()).all())


def test_moe_config5_full_size(dev):
    """16384 tokens, d 1024, 8 experts top-2, FFN 2816: balanced and skewed routing; a token slice against the oracle,
    exact equivariance under a token permutation, and load accounting."""
    from oracle import moe as O
    from trainium_frontier_them_bones_amd import autograd as A
    from trainium_frontier_them_bones_amd import ops
    N, d, Fd, E = 16384, 1024, 2816, 8
    for skew in (0.0, 2.0):
        h, router, wf, wp, bias = _layer(5, N, d, Fd, E, skew)
        hd, rd, wfd, wpd = (t.to(dev) for t in (h, router, wf, wp))
        st = A.Moe8State()
        st.refresh(wfd, wpd)
        b = bias.to(dev) if skew else None
        out = A.MoeMlp8Fn.apply(hd, rd, wfd, wpd, st, 2, b)
        p, idx, gate, _ = ops.moe_route(hd, rd, 2, b)
        tab = ops.moe_tables(idx, E)
        assert int(tab["cnt"].sum()) == 2 * N
        if skew:
            assert int(tab["cnt"][:2].min()) > 1.3 * int(tab["cnt"][2:].max())     # the biased experts are hot
        perm = torch.randperm(N, generator=torch.Generator().manual_seed(7)).to(dev)
        out_p = A.MoeMlp8Fn.apply(hd[perm].contiguous(), rd, wfd, wpd, st, 2, b)
        assert torch.equal(out_p, out[perm])
        # oracle on the tokens of one expert pair: run the oracle's experts on this slice with the layer's scale rows
        sl = slice(0, 512)
        oo, _ = O.moe_forward(h[sl], router, wf, wp, 2, bias if skew else None)
        assert rel_l2(out[sl], oo) < 2e-2


def test_moe_auxiliary_router_terms(dev):
    """moe_aux_terms (round2/source/train.py:10779): lb, z and the load shares against the oracle, and their gradient
    joining the router's: with the layer output's gradient zero the router and input gradients are those of the weighted
    auxiliary sum alone."""
    from oracle import moe as O
    from trainium_frontier_them_bones_amd import autograd as A
    N, d, Fd, E, topk = 2048, 256, 512, 8, 2
    h, router, wf, wp, bias = _layer(5, N, d, Fd, E, 1.0)
    hd, rd = h.to(dev).requires_grad_(True), router.to(dev).requires_grad_(True)
    wfd, wpd = wf.to(dev).requires_grad_(True), wp.to(dev).requires_grad_(True)
    st = A.Moe8State()
    st.refresh(wfd, wpd)
    alpha, beta = 0.01, 0.001
    out, aux, terms = A.MoeMlp8Fn.apply(hd, rd, wfd, wpd, st, topk, bias.to(dev), (alpha, beta))
    ho, ro = h.clone().float().requires_grad_(True), router.clone().float().requires_grad_(True)
    po, idxo, _, lo = O.route(ho, ro, topk, bias)
    lb, z, f = O.aux_terms(po, lo, idxo, topk)
    assert abs(terms[0].item() - lb.item()) < 1e-4 * abs(lb.item()) and abs(terms[1].item() - z.item()) < 1e-4 * abs(z.item())
    assert rel_l2(terms[2:], f) < 1e-3                                  # (a near-tie may select differently)
    assert abs(aux.item() - (alpha * lb + beta * z).item()) < 1e-4 * abs(aux.item())
    out0 = A.MoeMlp8Fn.apply(hd, rd, wfd, wpd, st, topk, bias.to(dev))
    assert torch.equal(out, out0)                                       # the layer's output does not depend on the switch
    (aux * 3.0).backward()
    (3.0 * (alpha * lb + beta * z)).backward()
    assert rel_l2(rd.grad, ro.grad) < 1e-2
    assert rel_l2(hd.grad, ho.grad) < 2e-2                              # one bf16 rounding of dh
    assert float(wfd.grad.abs().max()) == 0.0                           # no gradient reaches the experts through aux


@pytest.mark.parametrize("shape,topk,skew", [((1024, 256, 512, 8), 2, 0.0), ((1024, 256, 512, 4), 1, 0.0),
                                              ((2048, 512, 768, 8), 2, 2.0)])
def test_moe_layer_with_bf16_experts_forward_backward(dev, shape, topk, skew):
    """The experts in bf16 (MoeMLP.forward with moe_experts_local, round2/source/train.py:10716: the kit's expression per
    expert): layer output and every gradient against the oracle's bf16 layer fed the KERNEL'S selections (so that a near-tie
    of the router cannot move a token), to the bf16 bar 5e-3; the grouped expert MLP alone, on the kernel's own gathered
    rows, against the same expression expert by expert."""
    import torch.nn.functional as F
    from oracle import moe as O
    from trainium_frontier_them_bones_amd import autograd as A, ops
    N, d, Fd, E = shape
    h, router, wf, wp, bias = _layer(2, N, d, Fd, E, skew)
    hd, rd = h.to(dev).requires_grad_(True), router.to(dev).requires_grad_(True)
    wfd, wpd = wf.to(dev).requires_grad_(True), wp.to(dev).requires_grad_(True)
    b = bias.to(dev) if skew else None
    out = A.MoeMlp8Fn.apply(hd, rd, wfd, wpd, None, topk, b)
    g = torch.randn(N, d, generator=torch.Generator().manual_seed(3)).bfloat16()
    out.backward(g.to(dev))
    # the grouped MLP by itself: every expert's segment of the gathered rows through the eager bf16 expression
    p, idx, gate, _ = ops.moe_route(hd.detach(), rd.detach().float().contiguous(), topk, b, want_logits=True)
    tab = ops.moe_tables(idx, E)
    xs, none8 = ops.moe_gather(hd.detach(), tab, None)
    assert none8 is None
    ys, r, hh = ops.moe_mlp_fwd(xs, wfd.detach(), wpd.detach(), tab)
    seg = tab["seg"].cpu().tolist()
    for e in range(E):
        xe = xs[seg[e]:seg[e + 1]].cpu()
        pre = F.linear(xe, wf[e])
        assert torch.equal(r[seg[e]:seg[e + 1]].cpu(), torch.relu(pre)) or rel_l2(r[seg[e]:seg[e + 1]], torch.relu(pre)) < 3e-3
        assert rel_l2(ys[seg[e]:seg[e + 1]], F.linear(torch.relu(pre).square(), wp[e])) < 5e-3
    assert torch.equal(hh[:seg[-1]], (r * r)[:seg[-1]])                   # h = bf16(r^2) exactly (rows past the last segment are not written)
    ho, ro, wfo, wpo = (t.clone().requires_grad_(True) for t in (h, router, wf, wp))
    oo, _ = O.moe_forward(ho, ro, wfo, wpo, topk, bias if skew else None, fp8=False, idx=idx.cpu().long())
    oo.backward(g)
    assert rel_l2(out, oo) < 5e-3
    assert rel_l2(hd.grad, ho.grad) < 5e-3
    assert rel_l2(wfd.grad, wfo.grad) < 5e-3 and rel_l2(wpd.grad, wpo.grad) < 5e-3
    assert rel_l2(rd.grad, ro.grad) < 1e-2


@pytest.mark.parametrize("shape,topk,skew", [((1024, 256, 512, 8), 2, 0.0), ((2048, 512, 768, 8), 2, 2.0)])
def test_moe_layer_with_fp8_weight_gradients(dev, shape, topk, skew):
    """The experts' weight gradients in fp8 as well (round2/source/train.py:8209-8229 inside each expert's backward): same
    output and input / router gradients as with bf16 weight gradients (those GEMMs are untouched: bit-equal), the weight
    gradients against the oracle's fp8 form on the kernel's selections within the fp8 bar, and close to the bf16 ones."""
    from oracle import moe as O
    from trainium_frontier_them_bones_amd import autograd as A, ops
    N, d, Fd, E = shape
    h, router, wf, wp, bias = _layer(2, N, d, Fd, E, skew)
    b = bias.to(dev) if skew else None
    g = torch.randn(N, d, generator=torch.Generator().manual_seed(3)).bfloat16()
    res = {}
    for dw8 in (False, True):
        hd, rd = h.to(dev).requires_grad_(True), router.to(dev).requires_grad_(True)
        wfd, wpd = wf.to(dev).requires_grad_(True), wp.to(dev).requires_grad_(True)
        st = A.Moe8State(dw_fp8=dw8)
        st.refresh(wfd, wpd)
        out = A.MoeMlp8Fn.apply(hd, rd, wfd, wpd, st, topk, b)
        out.backward(g.to(dev))
        res[dw8] = (out.detach(), hd.grad, rd.grad, wfd.grad, wpd.grad)
    assert torch.equal(res[True][0], res[False][0]) and torch.equal(res[True][1], res[False][1])
    assert torch.equal(res[True][2], res[False][2])
    assert rel_l2(res[True][3], res[False][3]) < 6e-2 and rel_l2(res[True][4], res[False][4]) < 6e-2
    assert not torch.equal(res[True][3], res[False][3])                  # it is another arithmetic
    _, idx, _, _ = ops.moe_route(h.to(dev), router.to(dev).contiguous(), topk, b, want_logits=True)
    ho, ro, wfo, wpo = (t.clone().requires_grad_(True) for t in (h, router, wf, wp))
    oo, _ = O.moe_forward(ho, ro, wfo, wpo, topk, bias if skew else None, idx=idx.cpu().long(), dw_fp8=True)
    oo.backward(g)
    assert rel_l2(res[True][3], wfo.grad) < 2e-2 and rel_l2(res[True][4], wpo.grad) < 2e-2


@pytest.mark.parametrize("topk", [1, 2])
def test_moe_per_sequence_balance_term(dev, topk):
    """The per-sequence balance term of moe_aux_terms (round2/source/train.py:10789-10792): the kernel's term and the
    sequences' load shares against the oracle ON THE KERNEL'S OWN selections (shares bit-exact: they are counts over a
    power-of-two length), and through the autograd node: the weighted sum alpha lb + beta z + gamma seq and its gradient to
    the router and the input, with the layer's own output gradient zero."""
    from oracle import moe as O
    from trainium_frontier_them_bones_amd import autograd as A, ops
    B, T, d, Fd, E = 8, 256, 256, 512, 8
    h, router, wf, wp, bias = _layer(7, B * T, d, Fd, E, 1.5)
    hd, rd = h.to(dev).view(B, T, d).requires_grad_(True), router.to(dev).requires_grad_(True)
    wfd, wpd = wf.to(dev).requires_grad_(True), wp.to(dev).requires_grad_(True)
    p, idx, gate, logits = ops.moe_route(hd.detach().reshape(-1, d), rd.detach().float().contiguous(), topk, bias.to(dev), want_logits=True)
    term, fs = ops.moe_aux_seq_fwd(p, idx, T, topk)
    *_, seq_o = O.aux_terms(p.cpu().double(), logits.cpu().double(), idx.cpu(), topk, seq_len=T)
    mall = torch.zeros(B * T, E, dtype=torch.float64).scatter_add_(1, idx.cpu().long(), torch.ones(B * T, topk, dtype=torch.float64))
    assert torch.equal(fs.cpu().double(), mall.view(B, T, E).mean(1) / topk)
    assert abs(term.item() - seq_o.item()) < 1e-5 * abs(seq_o.item())
    st = A.Moe8State()
    st.refresh(wfd, wpd)
    alpha, beta, gamma = 0.01, 0.001, 0.02
    out, aux, terms = A.MoeMlp8Fn.apply(hd, rd, wfd, wpd, st, topk, bias.to(dev), (alpha, beta, gamma))
    out2, aux2, _ = A.MoeMlp8Fn.apply(hd, rd, wfd, wpd, st, topk, bias.to(dev), (alpha, beta))
    assert torch.equal(out, out2)
    assert abs((aux - aux2).item() - gamma * term.item()) < 1e-6 * abs(aux.item())
    (aux * 2.0).backward()
    ho, ro = h.clone().float().requires_grad_(True), router.clone().float().requires_grad_(True)
    po, _, _, lo = O.route(ho, ro, topk, bias)
    lb, z, f, seq = O.aux_terms(po, lo, idx.cpu(), topk, seq_len=T)      # the kernel's selections: a near-tie cannot differ
    (2.0 * (alpha * lb + beta * z + gamma * seq)).backward()
    assert rel_l2(rd.grad, ro.grad) < 1e-2
    assert rel_l2(hd.grad.view(-1, d), ho.grad) < 2e-2                  # one bf16 rounding of dh
    with pytest.raises(ValueError):
        ops.moe_aux_seq_fwd(p, idx, 384, topk)                          # 2048 tokens are not whole sequences of 384


@pytest.mark.parametrize("skew,dw_fp8", [(0.0, False), (2.0, False), (2.0, True)])
def test_moe_config5_full_size_backward(dev, skew, dw_fp8):
    """Configuration 5 at full size, forward AND backward (16384 tokens, d 1024, 8 experts top-2, FFN 2816; balanced and
    with +2.0 on two experts' logits), against the oracle on parts it finishes in seconds: (1) one expert's whole row
    segment (its activations, input gradient and BOTH weight gradients: the ragged token-contraction GEMMs over
    thousands of rows, in bf16 and, dw_fp8, in fp8 from the bytes the other GEMMs multiplied), (2) the input gradient of 512 tokens routed to the most frequent expert pair, through autograd
    of the oracle layer on those tokens with the backward scales taken from the full layer's per-expert amax."""
    from oracle import mlp8 as O8
    from oracle import moe as O
    from trainium_frontier_them_bones_amd import autograd as A
    from trainium_frontier_them_bones_amd import ops
    N, d, Fd, E = 16384, 1024, 2816, 8
    h, router, wf, wp, bias = _layer(5, N, d, Fd, E, skew)
    dout = torch.randn(N, d, generator=torch.Generator().manual_seed(6)).bfloat16()
    hd, rd, wfd, wpd = (t.to(dev).requires_grad_(True) for t in (h, router, wf, wp))
    st = A.Moe8State(dw_fp8=dw_fp8)
    st.refresh(wfd, wpd)
    b = bias.to(dev) if skew else None
    print("config 5 full size fwd+bwd, skew %.1f, fp8 weight gradients %s" % (skew, dw_fp8), flush=True)
    out = A.MoeMlp8Fn.apply(hd, rd, wfd, wpd, st, 2, b)
    out.backward(dout.to(dev))
    for t in (out, hd.grad, rd.grad, wfd.grad, wpd.grad):
        assert bool(torch.isfinite(t.float()).all())
    # the kernel's own routing (bit-checked against the reference's rule in the tests above) defines the segments
    p, idx, gate, _ = ops.moe_route(hd.detach(), rd.detach(), 2, b)
    idx, gate = idx.cpu().long(), gate.cpu()
    slot, tok, seg = O.tables(idx, E)
    ksel = torch.zeros_like(tok)
    for j in range(2):
        ksel[slot[:, j]] = j
    rows_all = torch.nonzero(tok >= 0).flatten()
    gate_rows = torch.zeros(tok.shape[0])
    gate_rows[rows_all] = gate[tok[rows_all], ksel[rows_all]]
    dys = (gate_rows.bfloat16()[:, None] * dout[tok.clamp_min(0)]) * (tok >= 0)[:, None]     # bf16(gate) * dout, bf16
    amax = torch.stack([dys[seg[e]:seg[e + 1]].float().abs().amax() for e in range(E)])
    # (1) the busiest expert's whole segment
    cnt = seg[1:] - seg[:-1]
    e = int(torch.argmax(cnt))
    rows = torch.arange(int(seg[e]), int(seg[e + 1]))
    rows = rows[tok[rows] >= 0]
    xe, ge = h[tok[rows]], dys[rows]
    row = O8.forward_scales(wf[e], wp[e])
    ye, re = O8.forward(xe, wf[e], wp[e], row)
    row_b = O8.backward_scales(ge, row, amax[e])
    dxe, he, dpe = O8.backward(ge, re, wf[e], wp[e], row_b)
    dwf, dwp = O8.weight_grads_fp8(xe, ge, he, dpe, row_b) if dw_fp8 else O8.weight_grads(ge, xe, he, dpe)
    assert rel_l2(wfd.grad[e], dwf) < 2e-2 and rel_l2(wpd.grad[e], dwp) < 2e-2
    assert rows.numel() > (3000 if not skew else 5000)                    # thousands of rows: the ragged long contraction
    # (2) 512 tokens of the most frequent (unordered) expert pair, input gradient through the whole layer's backward
    pair = torch.sort(idx, dim=1).values
    key = pair[:, 0] * E + pair[:, 1]
    best = int(torch.mode(key).values)
    _, io, _, _ = O.route(h, router, 2, bias if skew else None)
    same = (io == idx).all(1)                                             # (a near-tie on torch's own logits may differ)
    S = torch.nonzero((key == best) & same).flatten()[:512]
    assert S.numel() == 512
    ho, ro = h[S].clone().requires_grad_(True), router.clone().requires_grad_(True)
    oo, info = O.moe_forward(ho, ro, wf, wp, 2, bias if skew else None, dys_amax=amax)
    assert torch.equal(info["idx"], idx[S])                               # (torch's logits pick the same experts here)
    oo.backward(dout[S])
    assert rel_l2(out[S], oo) < 2e-2
    assert rel_l2(hd.grad[S], ho.grad) < 2e-2


@pytest.mark.parametrize("topk,skew,cap", [(2, 0.0, 100), (2, 2.0, 64), (1, 2.0, 40), (2, 0.0, 512)])
def test_capacity_tables_bit_exact(dev, topk, skew, cap):
    """The reference's per-sequence capacity (round2/source/train.py:10555-10600) is index work: on the kernel's own
    selections the oracle's keep rule must give the same slots (-1 for a skipped assignment), rows and segments bit for bit;
    a capacity nobody reaches (the last case) gives the dropless tables."""
    from oracle import moe as O
    from trainium_frontier_them_bones_amd import ops
    b, t, E = 4, 512, 8
    h, router, _, _, bias = _layer(21, b * t, 256, 512, E, skew)
    _, idx, _, _ = ops.moe_route(h.to(dev), router.to(dev), topk, bias.to(dev))
    tab = ops.moe_tables(idx, E, t, cap)
    slot, tok, seg = O.tables(idx.cpu().long(), E, t, cap)
    assert torch.equal(tab["slot"].cpu().long(), slot)
    assert torch.equal(tab["seg"].cpu().long(), seg)
    R = int(seg[-1])
    assert torch.equal(tab["tok"].cpu().long()[:R], tok) and bool((tab["tok"].cpu()[R:] == -1).all())
    kept = torch.bincount(idx.cpu().long()[slot >= 0], minlength=E)
    assert torch.equal(tab["cnt"].cpu().long(), kept)
    assert torch.equal(tab["cnt_all"].cpu().long(), torch.bincount(idx.cpu().long().reshape(-1), minlength=E))
    te = tab["tile_expert"].cpu()
    for e in range(E):
        assert bool((te[int(seg[e]) // 128:int(seg[e + 1]) // 128] == e).all())
    dropped = int((slot < 0).sum())
    if cap == 512:
        free = ops.moe_tables(idx, E)
        assert dropped == 0 and all(torch.equal(tab[k], free[k]) for k in ("slot", "seg", "tok", "cnt", "tile_expert"))
        live = free["tok"] >= 0                                                 # (ksel is only defined for rows that hold a token)
        assert torch.equal(tab["ksel"][live], free["ksel"][live])
    else:
        assert dropped > 100                                                    # the case does drop


def test_capacity_rejects_a_sequence_that_is_not_whole_wavefronts(dev):
    from trainium_frontier_them_bones_amd import ops
    from trainium_frontier_them_bones_amd._lib import TfbError
    idx = torch.zeros(200, 2, dtype=torch.int32, device=dev)
    idx[:, 1] = 1
    with pytest.raises(TfbError):
        ops.moe_tables(idx, 4, 100, 8)


@pytest.mark.parametrize("experts", ["fp8", "fp8 weight gradients too", "bf16"])
def test_moe_layer_with_capacity_forward_backward(dev, experts):
    """The whole routed layer (experts in fp8, with fp8 weight gradients, in bf16) with a capacity that drops about a sixth of the assignments, against the oracle's restatement
    of the reference's keep rule: output, input / router / expert-weight gradients, and the load shares of the auxiliary term
    (made of EVERY assignment, kept or not: round2/source/train.py:10786 takes them from the masks)."""
    from oracle import moe as O
    from trainium_frontier_them_bones_amd import autograd as A
    from trainium_frontier_them_bones_amd import ops
    b, t, d, Fd, E, topk, cap = 4, 512, 256, 512, 8, 2, 96
    h, router, wf, wp, bias = _layer(22, b * t, d, Fd, E, 2.0)
    h = h.reshape(b, t, d)
    hd, rd, wfd, wpd = (x.to(dev).requires_grad_(True) for x in (h, router, wf, wp))
    st = None
    if experts != "bf16":
        st = A.Moe8State(dw_fp8=experts != "fp8")
        st.refresh(wfd, wpd)
    out, aux, terms = A.MoeMlp8Fn.apply(hd, rd, wfd, wpd, st, topk, bias.to(dev), (0.01, 0.001), cap)
    g = torch.randn(b, t, d, generator=torch.Generator().manual_seed(3)).bfloat16()
    (out.float() * g.to(dev).float()).sum().add(aux).backward()
    ho, ro, wfo, wpo = (x.clone().requires_grad_(True) for x in (h, router, wf, wp))
    oo, info = O.moe_forward(ho, ro, wfo, wpo, topk, bias, capacity=cap, fp8=experts != "bf16",
                             dw_fp8=experts == "fp8 weight gradients too")
    # the comparison needs the two routers to agree on every pick (a different pick would move every later position of
    # its sequence); the kernel's picks are held to the reference's rule bit for bit in test_routing_tables_bit_exact
    _, idx, _, _ = ops.moe_route(hd.detach().reshape(-1, d), rd.detach(), topk, bias.to(dev))
    assert torch.equal(idx.cpu().long(), info["idx"]), "near-tie between the two routers: pick another seed"
    frac = float((info["slot"] < 0).float().mean())
    assert 0.05 < frac < 0.5
    p_o, logits_o = info["p"], torch.nn.functional.linear(ho.reshape(-1, d).float(), ro.float()) + bias
    lb, z, f = O.aux_terms(p_o, logits_o, info["idx"], topk)
    (oo.float() * g.float()).sum().add(0.01 * lb + 0.001 * z).backward()
    assert rel_l2(out, oo) < 2e-2
    assert rel_l2(terms[2:], f) < 1e-6 and abs(float(terms[0]) - float(lb.detach())) < 1e-4 * abs(float(lb.detach()))
    assert rel_l2(hd.grad, ho.grad) < 2e-2
    assert rel_l2(wfd.grad, wfo.grad) < 2e-2 and rel_l2(wpd.grad, wpo.grad) < 2e-2
    assert rel_l2(rd.grad, ro.grad) < 2e-2
    # a skipped assignment adds nothing: tokens whose BOTH picks were skipped come out exactly zero
    both = (info["slot"] < 0).all(1).reshape(b, t)
    if bool(both.any()):
        assert float(out.detach().cpu()[both].abs().max()) == 0.0
