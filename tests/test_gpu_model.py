"""The full training step on the HIP kernels against the oracle model (same seeded weights and tokens)."""
import pytest
import torch

from helpers import rel_l2

pytestmark = pytest.mark.gpu


def test_small_model_losses_and_gradients_track_oracle(dev):
    from oracle.model import OracleGPT
    from trainium_frontier_them_bones_amd.model import GPT, GPTConfig, zipf_tokens
    cfg = GPTConfig(n_layer=2, d_model=256, n_head=4, d_ff=1024, vocab=1024, seq_len=256)
    m = GPT(cfg, dev, seed=1)
    o = OracleGPT(cfg, m.init_values)
    idx, tg = zipf_tokens(2, 256, cfg.vocab, seed=3)
    loss = m.forward(idx.to(dev), tg.to(dev))
    m.backward(loss)
    lo = o.forward(idx, tg)
    lo.backward()
    assert abs(loss.item() - lo.item()) < 1e-3 * lo.item()
    # the head's gradients: its operand is the stream after every fp8 block, so the fp8 path's bar; the blocks themselves
    # are held, one by one and without compounding, by test_each_block_against_the_oracle_on_the_blocks_own_inputs
    assert rel_l2(m.p["lm_head"].grad_buf, o.p["lm_head"].grad) < 2e-2
    assert rel_l2(m.p["norm_f"].grad_buf, o.p["norm_f"].grad) < 2e-2
    m2, o2 = GPT(cfg, dev, seed=1), OracleGPT(cfg, m.init_values)
    for _ in range(4):
        a = m2.train_step(idx.to(dev), tg.to(dev)).item()
        b = o2.train_step(idx, tg).item()
        assert abs(a - b) < 1e-3 * b
    assert a < 6.5                                                  # it learns


def test_each_half_block_against_the_oracle_on_its_own_inputs(dev):
    """No compounding: each half of every block of the HIP model (attention with its norm and projections; the fp8 MLP
    with its norm) is compared with the oracle's half fed the HIP half's OWN input stream and the HIP model's OWN gradient
    of its output stream. The attention half is a bf16 path: output, input gradient and the gradients of norm1, w_qkv, w_o
    within 5e-3. The MLP half is the fp8 path: output, input gradient and the gradients of norm2, w_fc, w_proj within 2e-2."""
    from oracle.model import OracleGPT
    from trainium_frontier_them_bones_amd.model import GPT, GPTConfig, zipf_tokens
    cfg = GPTConfig(n_layer=3, d_model=256, n_head=4, d_ff=1024, vocab=1024, seq_len=256)
    m = GPT(cfg, dev, seed=1)
    o = OracleGPT(cfg, m.init_values)
    idx, tg = zipf_tokens(2, 256, cfg.vocab, seed=3)
    m.trace = []
    m.zero_grad()
    m.backward(m.forward(idx.to(dev), tg.to(dev)))
    assert len(m.trace) == 2 * cfg.n_layer + 1
    halves = (("attention", o.attention_half, ("norm1", "w_qkv", "w_o"), 5e-3), ("mlp", o.mlp_half, ("norm2", "w_fc", "w_proj"), 2e-2))
    for i in range(cfg.n_layer):
        for j, (what, fn, names, tol) in enumerate(halves):
            print("block %d %s half" % (i, what), flush=True)
            t_in, t_out = m.trace[2 * i + j], m.trace[2 * i + j + 1]
            for t in o.p.values():
                t.grad = None
            x_in = t_in.detach().cpu().clone().requires_grad_(True)
            x_out = fn(i, x_in)
            assert rel_l2(t_out, x_out) < tol, (i, what)
            x_out.backward(t_out.grad.cpu())
            assert rel_l2(t_in.grad, x_in.grad) < tol, (i, what)
            for name in names:
                key = "%s.%d" % (name, i)
                assert rel_l2(m.p[key].grad_buf, o.p[key].grad) < tol, key


def test_full_size_model_on_one_sequence_against_the_oracle(dev):
    """Configuration 4 of BASELINE.json at its real model size (12 layers, d 768, 12 heads, MLP 3072, vocab 32768) on ONE
    sequence of 2048 tokens: the loss of the first step and, after one AdamW update of every parameter, of the second,
    against the oracle model on the same tokens, within 1e-3 relative."""
    from oracle.model import OracleGPT
    from trainium_frontier_them_bones_amd.model import GPT, GPTConfig, zipf_tokens
    cfg = GPTConfig()
    m = GPT(cfg, dev, seed=0)
    o = OracleGPT(cfg, m.init_values)
    idx, tg = zipf_tokens(16, cfg.seq_len, cfg.vocab, seed=0)
    idx, tg = idx[:1], tg[:1]
    for step in range(2):
        print("full-size model, one sequence, step %d" % step, flush=True)
        a = m.train_step(idx.to(dev), tg.to(dev)).item()
        b = o.train_step(idx, tg).item()
        assert abs(a - b) < 1e-3 * b, (step, a, b)


@pytest.mark.parametrize("fp8_attn", [False, True])
def test_folded_residual_path_is_bit_identical_to_the_separate_passes(dev, fp8_attn):
    """GPTConfig.fuse_residual moves the residual adds into the projections' stores and the fp8 operand casts into the
    norms; every value, hence the loss and every gradient, must stay the same bit for bit."""
    from trainium_frontier_them_bones_amd.model import GPT, GPTConfig, zipf_tokens
    idx, tg = zipf_tokens(2, 256, 1024, seed=5)
    out = []
    for fuse in (False, True):
        cfg = GPTConfig(n_layer=2, d_model=256, n_head=4, d_ff=1024, vocab=1024, seq_len=256, fuse_residual=fuse,
                        fp8_attn_proj=fp8_attn)
        m = GPT(cfg, dev, seed=1)
        loss = m.forward(idx.to(dev), tg.to(dev))
        m.backward(loss)
        out.append((loss.item(), {k: v.grad_buf.clone() for k, v in m.p.items()}))
    assert out[0][0] == out[1][0]
    for k in out[0][1]:
        if k == "wte":   # the stream's and the first norm's gradients meet in one launch (one rounding) instead of a bf16 add
            assert rel_l2(out[0][1][k], out[1][1][k]) < 2e-3
        else:
            assert torch.equal(out[0][1][k], out[1][1][k]), k


def test_gradient_accumulation_in_place(dev):
    from trainium_frontier_them_bones_amd.model import GPT, GPTConfig, zipf_tokens
    cfg = GPTConfig(n_layer=1, d_model=256, n_head=4, d_ff=512, vocab=512, seq_len=128)
    m = GPT(cfg, dev, seed=2)
    idx, tg = zipf_tokens(4, 128, cfg.vocab, seed=4)
    idx, tg = idx.to(dev), tg.to(dev)
    m.zero_grad()
    m.backward(m.forward(idx, tg))
    once = {k: p.grad_buf.clone() for k, p in m.p.items()}
    m.backward(m.forward(idx, tg))                                  # second micro-step adds into the same buffers
    for k, p in m.p.items():
        assert rel_l2(p.grad_buf, 2 * once[k].float()) < 1e-2, k


def test_full_size_batch_first_loss_against_the_oracle(dev):
    """Configuration 4 of BASELINE.json at its stated batch (16 sequences of 2048 tokens): the loss of the first forward pass
    against the mean of the oracle's sixteen per-sequence forward losses (equal lengths, no ignored target: the batch mean),
    within 1e-3 relative."""
    from oracle.model import OracleGPT
    from trainium_frontier_them_bones_amd.model import GPT, GPTConfig, zipf_tokens
    cfg = GPTConfig()
    m = GPT(cfg, dev, seed=0)
    o = OracleGPT(cfg, m.init_values)
    idx, tg = zipf_tokens(16, cfg.seq_len, cfg.vocab, seed=0)
    got = m.forward(idx.to(dev), tg.to(dev)).item()
    per = []
    with torch.no_grad():
        for b in range(16):
            print("oracle forward, sequence %d" % b, flush=True)
            per.append(o.forward(idx[b:b + 1], tg[b:b + 1]).item())
    want = sum(per) / len(per)
    assert abs(got - want) < 1e-3 * want, (got, want)


def test_full_size_step_runs_and_loss_is_sane(dev):
    from trainium_frontier_them_bones_amd.model import GPT, GPTConfig, zipf_tokens
    import math
    cfg = GPTConfig()
    m = GPT(cfg, dev, seed=0)
    idx, tg = zipf_tokens(16, cfg.seq_len, cfg.vocab, seed=0)
    l0 = m.train_step(idx.to(dev), tg.to(dev)).item()
    assert abs(l0 - math.log(cfg.vocab)) < 0.5                     # random init: loss ~ ln V + var(logits) / 2
    for _ in range(3):
        l = m.train_step(idx.to(dev), tg.to(dev)).item()
    assert l < l0 and math.isfinite(l)


def test_benchmark_line_on_a_short_run(dev):
    """bench.py end to end (2 steps, no CPU leg): one JSON line with the contract's fields, and the entry point it times
    with events is one the step really calls (roofline.launch_ms > 0)."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--steps", "2", "--warmup", "1", "--no-cpu"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 2 and out["value"] > 0 and out["vs_baseline"] is None
    rf = out["roofline"]
    assert rf["bound"] == "mfma" and rf["launch_ms"] > 0 and 0 < rf["frac"] < 1 and abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-3
    r2 = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=60)
    assert r2.returncode != 0 and "one GPU" in r2.stderr
