"""Benchmark: train tokens/s of the 12-layer d768 T2048 step (fwd + bwd + AdamW) on one MI355X, entirely on the
HIP kernels, with the roofline position of the dominant kernel and the CPU oracle timed beside it.

python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--fp8-dw] [--unfused-residual]
Prints ONE JSON line. --fp8-dw (not the default, not the headline configuration) also runs the MLP's two weight-gradient
GEMMs in fp8, as the recipe of the reference's round1 sources does; the line's config then says so. --unfused-residual runs the same
arithmetic with the residual adds and the MLP's fp8 operand cast as passes of their own (for comparison; same values).

python bench.py --ns-probe        (Muon's Newton-Schulz call on the benchmark model's four stacks of 12 hidden matrices:
one line per stack with its time and flop rate; not part of the AdamW step the headline line times)

python bench.py --config-probe c1|c2|c3|c5|all   (the standalone configurations beside the full step, fwd + bwd each:
one line per configuration; run under rocprofv3 --kernel-trace --stats for the per-kernel durations)

python bench.py --traffic-probe   (for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs: a 256 MiB device copy as the
counters' calibration, then attention forward + backward at the benchmark shape; prints nothing)
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0
# HBM-side bytes one tfb_attn_bwd_rope call moves at B16 H12 T2048 D64 (delta + dkdv + dq kernels), from the FETCH_SIZE and
# WRITE_SIZE counters scaled by a 256 MiB copy (profiles/attn_c2_hbm_traffic.md): 570 MB fetched + 154 MB written.
ATTN_BWD_TRAFFIC_BYTES = 7.241e8


def flops_per_token(cfg):
    """The reference's own formula (round1/source/train.py:8964-8976): 6 x matmul params + 12 L h D (T / 2)."""
    d, F, L, V = cfg.d_model, cfg.d_ff, cfg.n_layer, cfg.vocab
    mm = L * (4 * d * d + 2 * d * F) + d * V
    return 6 * mm + 12 * L * cfg.n_head * cfg.head_dim * (cfg.seq_len // 2)


def cpu_baseline(cfg, init_values):
    """The oracle model's step on the host cores, on ONE sequence of the same 16 x 2048 batch."""
    import torch
    from oracle.model import OracleGPT
    from trainium_frontier_them_bones_amd.model import zipf_tokens
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    o = OracleGPT(cfg, init_values)
    idx, tg = zipf_tokens(16, cfg.seq_len, cfg.vocab, seed=0)
    t0 = time.perf_counter()
    o.train_step(idx[:1], tg[:1])
    dt = time.perf_counter() - t0
    return {"value": round(cfg.seq_len / dt, 2), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": "1 of the 16 sequences (2048 tokens) through the full 12-layer model, fwd+bwd+AdamW, 1 repetition"}


def traffic_probe():
    import torch
    from trainium_frontier_them_bones_amd import ops
    dev = torch.device("cuda:0")
    B, H, T, D = 16, 12, 2048, 64
    torch.manual_seed(0)
    q = torch.randn(B, H, T, D, device=dev).bfloat16()
    k, v = torch.randn_like(q), torch.randn_like(q)
    do = torch.randn(B, T, H, D, device=dev).bfloat16()
    src = torch.randn(64 * 1024 * 1024, device=dev)   # 256 MiB fp32
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)                                 # calibration: reads 256 MiB, writes 256 MiB
        o, lse = ops.attn_fwd(q, k, v, 0.125)
        ops.attn_bwd(q, k, v, o, do, lse, 0.125)
    torch.cuda.synchronize()


def ns_probe():
    import torch
    from trainium_frontier_them_bones_amd import ops
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    for (K, r, c) in ((12, 3072, 768), (12, 768, 3072), (12, 2304, 768), (12, 768, 768)):
        g = torch.randn(K, r, c, device=dev) * 0.02
        d = g.bfloat16().norm(dim=(-2, -1)) * 1.01 + 1e-6
        for _ in range(3):
            ops.ns5(g, d)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(10):
            ops.ns5(g, d)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / 10
        M, N = max(r, c), min(r, c)
        flop = 5 * K * (4 * M * N * N + 2 * N * N * N)   # per iteration: X^T X, X B (2 M N^2 each) and G G (2 N^3)
        print("ns5 K=%d %dx%d: %.3f ms, %.0f TFLOP/s" % (K, r, c, dt * 1e3, flop / dt / 1e12), flush=True)


def config_probe(which):
    """The standalone configurations beside the full step, each fwd + bwd through the autograd layer, 3 untimed and 5 timed
    repetitions: c1 RMSNorm -> LM head -> cross-entropy on 8192 tokens; c2 causal attention 16 x 12 x 2048 x 64; c3 the
    fp8 MLP on 16384 tokens with a per-tensor amax activation scale; c5 the 8-expert top-2 fp8 layer on 16384 tokens,
    balanced and with +2.0 on two experts' router logits. Prints one line per configuration with its time per repetition."""
    import torch
    from trainium_frontier_them_bones_amd import autograd as A
    from trainium_frontier_them_bones_amd import ops
    dev = torch.device("cuda:0")
    bf = torch.bfloat16

    def timed(name, fn, flop):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / 5
        print("%s: %.3f ms per fwd+bwd, %.0f TFLOP/s of algorithmic work" % (name, dt * 1e3, flop / dt / 1e12), flush=True)

    def leaf(t):
        return t.to(dev).requires_grad_(True)

    def clear(*ts):
        for t in ts:
            t.grad = None

    if which in ("c1", "all"):
        g = torch.Generator().manual_seed(20261)
        N, d, V = 8192, 768, 32768
        x = leaf(torch.randn(N, d, generator=g).to(bf))
        nw = leaf((1 + 0.02 * torch.randn(d, generator=g)).to(bf))
        W = leaf((0.02 * torch.randn(V, d, generator=g)).to(bf))
        t = torch.randint(0, V, (N,), generator=g).to(dev)

        def c1():
            clear(x, nw, W)
            A.LmHeadLossFn.apply(A.RMSNormFn.apply(x, nw, 1e-6), W, t, 0.0, "mean").backward()
        timed("c1 norm + LM head + loss, 8192 tokens", c1, 3 * 2.0 * N * d * V)
        del x, W
    if which in ("c2", "all"):
        g = torch.Generator().manual_seed(20262)
        B, H, T, D = 16, 12, 2048, 64
        q, k, v = (leaf(torch.randn(B, H, T, D, generator=g).to(bf)) for _ in range(3))
        do = torch.randn(B, T, H, D, generator=g).to(bf).to(dev)

        def c2():
            clear(q, k, v)
            A.CausalAttentionFn.apply(q, k, v, 0.125).backward(do)
        timed("c2 causal attention 16x12x2048x64", c2, 7.0 * B * H * T * T * D)
        del q, k, v, do
    if which in ("c3", "all"):
        g = torch.Generator().manual_seed(20263)
        M, d, F = 16384, 768, 3072
        x = leaf(torch.randn(M, d, generator=g).to(bf))
        wf = leaf((0.02 * torch.randn(d, F, generator=g)).to(bf).t().contiguous())
        wp = leaf((0.02 * torch.randn(F, d, generator=g)).to(bf).t().contiguous())
        dy = torch.randn(M, d, generator=g).to(bf).to(dev)
        st = A.Mlp8State(e4m3_limit=448.0)

        def c3():
            clear(x, wf, wp)
            st.x_scale = float(ops.amax_scale(x.detach(), 448.0, -20, 20)[0].item())   # power of two under amax
            st.refresh(wf, wp)
            A.Mlp8Fn.apply(x, wf, wp, st).backward(dy)
        timed("c3 fp8 MLP, 16384 tokens (scales and weight packs refreshed inside)", c3, 6 * 2.0 * M * d * F)
        del x, dy
    if which in ("c5", "all"):
        N, d, Fd, E = 16384, 1024, 2816, 8
        for skew in (0.0, 2.0):
            g = torch.Generator().manual_seed(20265)
            h = leaf(torch.randn(N, d, generator=g).to(bf))
            router = leaf(0.02 * torch.randn(E, d, generator=g))
            wf = leaf((0.02 * torch.randn(E, Fd, d, generator=g)).to(bf))
            wp = leaf((0.02 * torch.randn(E, d, Fd, generator=g)).to(bf))
            dy = torch.randn(N, d, generator=g).to(bf).to(dev)
            bias = torch.zeros(E)
            bias[:2] = skew
            b = bias.to(dev) if skew else None
            st = A.Moe8State()

            def c5():
                clear(h, router, wf, wp)
                st.refresh(wf, wp)
                A.MoeMlp8Fn.apply(h, router, wf, wp, st, 2, b).backward(dy)
            timed("c5 MoE layer, 16384 tokens top-2 of 8, router bias %+.1f on two experts" % skew, c5,
                  6 * 2.0 * (2 * N) * d * Fd)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--traffic-probe", action="store_true")
    ap.add_argument("--ns-probe", action="store_true")
    ap.add_argument("--config-probe", choices=("c1", "c2", "c3", "c5", "all"))
    ap.add_argument("--fp8-dw", action="store_true")
    ap.add_argument("--unfused-residual", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    if args.traffic_probe:
        traffic_probe()
        return
    if args.ns_probe:
        ns_probe()
        return
    if args.config_probe:
        config_probe(args.config_probe)
        return

    import torch
    from trainium_frontier_them_bones_amd import _lib
    from trainium_frontier_them_bones_amd.model import GPT, GPTConfig, zipf_tokens

    _lib.lib()
    dev = torch.device("cuda:0")
    cfg = GPTConfig()
    cfg.fp8_mlp_dw = bool(args.fp8_dw)
    cfg.fuse_residual = not args.unfused_residual
    model = GPT(cfg, dev, seed=0)
    B = 16
    idx, tg = zipf_tokens(B, cfg.seq_len, cfg.vocab, seed=0)
    idx, tg = idx.to(dev), tg.to(dev)
    for _ in range(args.warmup):
        model.train_step(idx, tg)
    torch.cuda.synchronize()

    rec = []
    _lib.TIMED["tfb_attn_bwd_rope"] = rec
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = model.train_step(idx, tg)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    del _lib.TIMED["tfb_attn_bwd_rope"]
    tokens = B * cfg.seq_len
    ms = dt / args.steps * 1e3

    # dominant entry point: attention backward (three launches: D = sum dO*O, dK/dV, dQ), timed with events on its stream
    if not rec:
        raise RuntimeError("the timed entry point was never called: roofline.achieved would be meaningless")
    k_ms = sum(s.elapsed_time(e) for s, e in rec) / len(rec)
    H, D, T = cfg.n_head, cfg.head_dim, cfg.seq_len
    k_flops = 5 * B * H * T * T * D   # causal-halved: 5 matmuls x 2 flop x 1/2
    achieved = k_flops / (k_ms * 1e-3) / 1e12 if k_ms > 0 else 0.0
    out = {
        "metric": "train tokens/s, 12L d768 T2048 fwd+bwd step; per-kernel % MFMA/HBM peak",
        "value": round(tokens / (dt / args.steps), 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 (fp8 e4m3/e5m2 MLP GEMMs)",
        "data": "synthetic: Zipf(1.1) token ids, N(0, 0.02) random-init weights",
        "config": {"workload": "C4 full step: 12 layers, d_model 768, 12 heads x 64, MLP 3072 squared-ReLU fp8, RMSNorm "
                               "pre-norm, RoPE, untied head, vocab 32768; batch 16 x 2048 tokens; fwd+bwd+AdamW"
                               + ("; MLP weight gradients in fp8 too (--fp8-dw)" if args.fp8_dw else "")
                               + ("; residual adds and fp8 casts as separate passes (--unfused-residual)"
                                  if args.unfused_residual else ""),
                   "global_batch": B, "seq_len": cfg.seq_len, "params": model.num_params(),
                   "step_tflops": round(flops_per_token(cfg) * tokens / 1e12, 2),
                   "model_tflops_per_s": round(flops_per_token(cfg) * tokens / (dt / args.steps) / 1e12, 1),
                   "final_loss": round(float(loss.item()), 4)},
        "roofline": {"kernel": "attention backward (tfb_attn_bwd_rope: attn64_delta + attn64_dkdv + attn64_dq), B16 H12 T2048 D64", "bound": "mfma",
                     "achieved": round(achieved, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_BF16_TFLOPS, 4), "traffic": ATTN_BWD_TRAFFIC_BYTES,
                     "launch_ms": round(k_ms, 4), "launches_timed": len(rec)},
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(cfg, model.init_values)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
