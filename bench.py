"""Benchmark: train tokens/s of the 12-layer d768 T2048 step (fwd + bwd + AdamW) on one MI355X, entirely on the
HIP kernels, with the roofline position of the dominant kernel and the CPU oracle timed beside it.

python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--bf16-dw] [--unfused-residual]
Prints ONE JSON line. All six GEMMs of the MLP run in fp8 (e4m3 forward, e5m2 gradients; the weight gradients from the
bytes the other GEMMs multiplied, as the reference's final recipe does); --bf16-dw keeps the MLP's two weight-gradient
GEMMs in bf16 for comparison and the line's config then says so. --unfused-residual runs the same
arithmetic with the residual adds and the MLP's fp8 operand cast as passes of their own (for comparison; same values).

python bench.py --ns-probe        (Muon's Newton-Schulz call on the benchmark model's four stacks of 12 hidden matrices:
one line per stack with its time and flop rate; not part of the AdamW step the headline line times)

python bench.py --config-probe c1|c2|c2d128|c3|c5|all   (the standalone configurations beside the full step, fwd + bwd each:
one line per configuration; run under rocprofv3 --kernel-trace --stats for the per-kernel durations; with --graphs a
second line per configuration: the same repetition recorded once as a HIP graph and replayed, without the host's launch work)

python bench.py --gemm-probe      (this library's bf16 GEMM beside torch.matmul, i.e. the vendor BLAS, on the step's own GEMM
shapes and 8192^3, in one process on one box: a yardstick only, the product never calls the vendor library)

python bench.py --power-probe     (the step's largest kernels timed on N(0, 1) operands and on all-zero operands, alternating:
identical instruction streams, so the difference is the clock the GPU sustains under its power limit)

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
# HBM-side bytes one tfb_attn_bwd_rope call moves at B16 H12 T2048 D64 (dq + dkdv kernels), from the FETCH_SIZE and
# WRITE_SIZE counters scaled by a 256 MiB copy (profiles/attn_c2_hbm_traffic.md): 513.5 MB fetched + 154.2 MB written.
ATTN_BWD_TRAFFIC_BYTES = 6.677e8


def flops_per_token(cfg):
    """The reference's own formula (round1/source/train.py:8964-8976): 6 x matmul params + 12 L h D (T / 2)."""
    d, F, L, V = cfg.d_model, cfg.d_ff, cfg.n_layer, cfg.vocab
    mm = L * (4 * d * d + 2 * d * F) + d * V
    return 6 * mm + 12 * L * cfg.n_head * cfg.head_dim * (cfg.seq_len // 2)


def cpu_baseline_and_parity(cfg, dev):
    """The oracle model's step on the host cores, on ONE sequence of the benchmark's first batch, timed; and the parity
    gate in the same pass: a fresh HIP model with the same initial weights takes the same two steps on the same
    sequence and the losses are compared (step 1 = the oracle's untimed warm-up repetition, the others the timed ones)."""
    import torch
    from oracle.model import OracleGPT
    from trainium_frontier_them_bones_amd.model import GPT, zipf_tokens
    host = os.cpu_count() or 1
    threads = min(host, 16)            # the GPU box gives one GPU's job 16 cores, whatever os.cpu_count() shows
    torch.set_num_threads(threads)
    m = GPT(cfg, dev, seed=0)
    o = OracleGPT(cfg, m.init_values)
    idx, tg = zipf_tokens(16, cfg.seq_len, cfg.vocab, seed=0)
    idx, tg = idx[:1], tg[:1]
    NT = 3                                                   # timed oracle steps: about 12 s of host work
    gpu = [m.train_step(idx.to(dev), tg.to(dev)).item() for _ in range(1 + NT)]
    cpu = [o.train_step(idx, tg).item()]                     # untimed warm-up repetition
    t0 = time.perf_counter()
    for _ in range(NT):
        cpu.append(o.train_step(idx, tg).item())
    dt = time.perf_counter() - t0
    rel = [abs(a - b) / abs(b) for a, b in zip(gpu, cpu)]
    base = {"value": round(NT * cfg.seq_len / dt, 2), "unit": "tokens/s", "cores": threads, "host_cpus": host, "kind": "port",
            "sample": "1 of the 16 sequences (2048 tokens) through the full 12-layer model, fwd+bwd+AdamW; 1 untimed "
                      "warm-up step, then %d timed steps (%.1f s)" % (NT, dt)}
    parity = {"loss_rel": round(max(rel), 6), "tolerance": 1e-3, "gpu_loss": [round(v, 5) for v in gpu],
              "oracle_loss": [round(v, 5) for v in cpu],
              "what": "HIP model vs CPU oracle, same initial weights, same 2048-token sequence, steps 1 to %d" % (1 + NT)}
    return base, parity


# ---- per-kernel roofline table: algorithmic work of one call of an entry point, from the arguments of the call --------
PEAK_FP8_TFLOPS = 5000.0
PEAK_HBM_GBS = 8000.0


def _work(name, a):
    """(label, bound, work) for one call: flop for "mfma" rows (against the bf16 or fp8 peak), bytes for "hbm" rows."""
    if name == "tfb_attn_bwd_rope":          # ..., B, H, T, D, scale, stream
        B, H, T, D = a[-6:-2]
        return "attention backward", "mfma", 5.0 * B * H * T * T * D
    if name == "tfb_attn_fwd":
        B, H, T, D = a[-6:-2]
        return "attention forward", "mfma", 2.0 * B * H * T * T * D
    if name == "tfb_qkv_rope_fwd":           # x, w, cos, sin, out, M, N, K, T, rot, stream
        M, N, K = a[5:8]
        return "QKV projection + RoPE %dx%dx%d" % (M, N, K), "mfma", 2.0 * M * N * K
    if name in ("tfb_gemm_bf16", "tfb_gemm_bf16_scaled"):   # A, B, C, M, N, K, ta, tb, ...
        M, N, K, ta, tb = a[3:8]
        return "bf16 GEMM %dx%dx%d %s%s" % (M, N, K, "T" if ta else "N", "T" if tb else "N"), "mfma", 2.0 * M * N * K
    if name == "tfb_gemm_bf16_res":          # A, B, res, C, M, N, K, tb, stream
        M, N, K = a[4:7]
        return "bf16 GEMM + residual %dx%dx%d" % (M, N, K), "mfma", 2.0 * M * N * K
    if name in ("tfb_mlp8_fwd", "tfb_mlp8_fwd_res", "tfb_mlp8_bwd", "tfb_mlp8_bwd_q"):
        M, d, F = a[-4:-1]
        return {"tfb_mlp8_fwd": "fp8 MLP forward", "tfb_mlp8_fwd_res": "fp8 MLP forward (+ residual)",
                "tfb_mlp8_bwd": "fp8 MLP backward", "tfb_mlp8_bwd_q": "fp8 MLP backward (+ e4m3 h)"}[name], "mfma8", 4.0 * M * d * F
    if name == "tfb_mlp8_dw8":               # ..., M, d, F, out_f32, accumulate, ws, ws_bytes, stream
        M, d, F = a[8:11]
        return "fp8 MLP weight gradients", "mfma8", 4.0 * M * d * F
    if name == "tfb_mlp_dw_proj":            # dy, r, dw, M, d, F, ...
        M, d, F = a[3:6]
        return "bf16 dW_proj (h = r^2 in the loader)", "mfma", 2.0 * M * d * F
    if name == "tfb_lmhead_fwd":             # ..., rows, d, V, softcap, stream
        N, d, V = a[-5:-2]
        return "LM head forward + lse", "mfma", 2.0 * N * d * V
    if name == "tfb_loss_fwd_bwd":           # ..., rows, V, softcap, stream
        N, V = a[-4:-2]
        return "loss forward + backward (one pass, dlogits in place)", "hbm", 2.0 * N * V * 2
    if name == "tfb_loss_bwd":               # ..., rows, V, softcap, stream
        N, V = a[-4:-2]
        return "loss backward (dlogits in place)", "hbm", 2.0 * N * V * 2
    if name in ("tfb_rmsnorm_fwd", "tfb_rmsnorm_fwd_q"):
        rows, C = a[-4:-2]
        return "RMSNorm forward", "hbm", rows * C * (2 * 2 + (1 if name.endswith("_q") else 0)) + 4.0 * rows
    if name in ("tfb_rmsnorm_bwd", "tfb_rmsnorm_bwd_amax"):   # ..., nrows, C, stream
        rows, C = a[-3:-1]
        return "RMSNorm backward", "hbm", rows * C * 2 * (4 if a[1] else 3)
    if name == "tfb_adamw":                  # p, g, g_f32, m, v, p16, n, ...
        n, gf32 = a[6], a[2]
        return "AdamW", "hbm", n * (24.0 if gf32 else 22.0)
    return name, None, 0.0


def per_kernel_table(rec, steps, top=8):
    """rec: (start, end, name, args) of every entry-point call over `steps` steps -> the `top` rows by time per step."""
    rows = {}
    for s, e, name, a in rec:
        label, bound, work = _work(name, a)
        r = rows.setdefault(label, {"kernel": label, "bound": bound, "ms": 0.0, "work": 0.0, "calls": 0})
        r["ms"] += s.elapsed_time(e)
        r["work"] += work
        r["calls"] += 1
    out = []
    total = sum(r["ms"] for r in rows.values())
    for r in sorted(rows.values(), key=lambda r: -r["ms"])[:top]:
        peak = {"mfma": PEAK_BF16_TFLOPS * 1e12, "mfma8": PEAK_FP8_TFLOPS * 1e12, "hbm": PEAK_HBM_GBS * 1e9}.get(r["bound"])
        row = {"kernel": r["kernel"], "bound": {"mfma8": "mfma"}.get(r["bound"], r["bound"]),
               "ms_per_step": round(r["ms"] / steps, 3), "calls_per_step": r["calls"] // steps,
               "share_of_timed": round(r["ms"] / total, 3)}
        if peak and r["ms"] > 0:
            row["frac"] = round(r["work"] / (r["ms"] * 1e-3) / peak, 4)
            row["peak"] = "fp8 5.0 PFLOP/s" if r["bound"] == "mfma8" else ("bf16 2.5 PFLOP/s" if r["bound"] == "mfma" else "HBM 8 TB/s")
        out.append(row)
    return out


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


def gemm_probe():
    """This library's bf16 GEMM (tfb_gemm_bf16) beside torch.matmul (the vendor BLAS) on the step's GEMM shapes, 20 timed
    calls each after 3 warm-up calls, alternating in one process; prints one table row per shape. The vendor library is the
    yardstick only: nothing in the package calls it."""
    import torch
    from trainium_frontier_them_bones_amd import ops
    dev = torch.device("cuda:0")

    def t(f, n=20):
        for _ in range(3):
            f()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(n):
            f()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / n * 1e3

    M = 32768
    shapes = [("QKV projection (NT)", M, 2304, 768, False, True), ("output projection (NT)", M, 768, 768, False, True),
              ("32768 x 3072 x 768 (NT)", M, 3072, 768, False, True), ("QKV dX (NN)", M, 768, 2304, False, False),
              ("output projection dX (NN)", M, 768, 768, False, False), ("QKV dW (TN)", 2304, 768, M, True, False),
              ("MLP-shaped dW (TN)", 3072, 768, M, True, False), ("LM head logits (NT)", M, 32768, 768, False, True),
              ("LM head dX (NN)", M, 768, 32768, False, False), ("LM head dW (TN)", 32768, 768, M, True, False),
              ("8192^3 (NT)", 8192, 8192, 8192, False, True)]
    print("| shape | m | n | k | vendor BLAS us | TFLOP/s | this library us | TFLOP/s | ratio | rel-L2 between them |")
    print("|---|---|---|---|---|---|---|---|---|---|")
    torch.manual_seed(0)
    for name, m, n, k, ta, tb in shapes:
        a = torch.randn((k, m) if ta else (m, k), device=dev).bfloat16()
        b = torch.randn((n, k) if tb else (k, n), device=dev).bfloat16()
        av, bv = (a.t() if ta else a), (b.t() if tb else b)
        out = torch.empty(m, n, device=dev, dtype=torch.bfloat16)
        tv = t(lambda: torch.matmul(av, bv, out=out))
        ref = out.float().clone()
        tl = t(lambda: ops.matmul(a, b, trans_a=ta, trans_b=tb, out=out))
        err = ((out.float() - ref).norm() / ref.norm()).item()
        fl = 2.0 * m * n * k
        print("| %s | %d | %d | %d | %.1f | %.0f | %.1f | %.0f | %.2f | %.1e |"
              % (name, m, n, k, tv, fl / tv / 1e6, tl, fl / tl / 1e6, tv / tl, err), flush=True)
        del a, b, out, ref


def power_probe():
    """The same launches timed on N(0, 1) operands and on all-zero operands, alternating (random, zeros, random, zeros):
    a GEMM's instruction stream does not depend on its data and the attention kernels' hardly does (no row maximum grows
    by 2^8 in either case), so what differs between the columns is the clock the GPU sustains under its power limit.
    20 timed calls after 5 warm-up calls per cell; one table row per kernel."""
    import torch
    from trainium_frontier_them_bones_amd import ops
    dev = torch.device("cuda:0")

    def t(f, n=20):
        for _ in range(5):
            f()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(n):
            f()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / n * 1e3

    def rnd(*shape):
        return torch.randn(*shape, device=dev).bfloat16()

    def zer(*shape):
        return torch.zeros(*shape, device=dev, dtype=torch.bfloat16)

    def gemm(m, n, k):
        def make(mk):
            a, b, out = mk(m, k), mk(n, k), torch.empty(m, n, device=dev, dtype=torch.bfloat16)
            return lambda: ops.matmul(a, b, trans_b=True, out=out)
        return make

    def attn(bwd):
        B, H, T, D = 16, 12, 2048, 64

        def make(mk):
            q, k, v, do = mk(B, H, T, D), mk(B, H, T, D), mk(B, H, T, D), mk(B, T, H, D)
            o, lse = ops.attn_fwd(q, k, v, 0.125)
            if bwd:
                return lambda: ops.attn_bwd(q, k, v, o, do, lse, 0.125)
            return lambda: ops.attn_fwd(q, k, v, 0.125)
        return make

    rows = [("bf16 GEMM 8192^3 (NT)", gemm(8192, 8192, 8192)), ("QKV projection 32768 x 2304 x 768", gemm(32768, 2304, 768)),
            ("LM head logits 32768 x 32768 x 768", gemm(32768, 32768, 768)),
            ("attention forward 16 x 12 x 2048 x 64", attn(False)), ("attention backward 16 x 12 x 2048 x 64", attn(True))]
    print("| kernel | random us | zeros us | random us | zeros us | zeros / random |")
    print("|---|---|---|---|---|---|")
    torch.manual_seed(0)
    for name, make in rows:
        fr, fz = make(rnd), make(zer)
        ts = [t(fr), t(fz), t(fr), t(fz)]
        print("| %s | %.1f | %.1f | %.1f | %.1f | %.2f |" % (name, *ts, (ts[1] + ts[3]) / (ts[0] + ts[2])), flush=True)
        del fr, fz


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


def config_probe(which, graphs=False):
    """The standalone configurations beside the full step, each fwd + bwd through the autograd layer, 3 untimed and 5 timed
    repetitions: c1 RMSNorm -> LM head -> cross-entropy on 8192 tokens; c2 causal attention 16 x 12 x 2048 x 64 (c2d128: 16 x 6 x
    2048 x 128); c3 the
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
        if not graphs:
            return
        # the same repetition recorded once as a HIP graph and replayed: what is left when the host's launch work (some
        # twenty Python calls per repetition) is out of the way. Warm-up on a side stream first, as torch's capture asks.
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            fn()
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(5):
            graph.replay()
        torch.cuda.synchronize()
        dg = (time.perf_counter() - t0) / 5
        print("%s, replayed as a HIP graph: %.3f ms per fwd+bwd, %.0f TFLOP/s of algorithmic work"
              % (name, dg * 1e3, flop / dg / 1e12), flush=True)

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
    if which in ("c2d128", "all"):
        # the same model width with the reference's own head dimension: 6 heads of 128
        g = torch.Generator().manual_seed(20266)
        B, H, T, D = 16, 6, 2048, 128
        q, k, v = (leaf(torch.randn(B, H, T, D, generator=g).to(bf)) for _ in range(3))
        do = torch.randn(B, T, H, D, generator=g).to(bf).to(dev)

        def c2d():
            clear(q, k, v)
            A.CausalAttentionFn.apply(q, k, v, D ** -0.5).backward(do)
        timed("c2d128 causal attention 16x6x2048x128", c2d, 7.0 * B * H * T * T * D)
        del q, k, v, do
    if which in ("c3", "all"):
        g = torch.Generator().manual_seed(20263)
        M, d, F = 16384, 768, 3072
        x = leaf(torch.randn(M, d, generator=g).to(bf))
        wf = leaf((0.02 * torch.randn(d, F, generator=g)).to(bf).t().contiguous())
        wp = leaf((0.02 * torch.randn(F, d, generator=g)).to(bf).t().contiguous())
        dy = torch.randn(M, d, generator=g).to(bf).to(dev)
        st = A.Mlp8State(e4m3_limit=448.0, dw_fp8=True)   # all six GEMMs in fp8: e4m3 forward, e5m2 gradients

        def c3():
            clear(x, wf, wp)
            st.x_scale = ops.amax_scale(x.detach(), 448.0, -20, 20)[0:1]   # power of two under amax, left on the device
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
            st = A.Moe8State(dw_fp8=True)

            def c5():
                clear(h, router, wf, wp)
                st.refresh(wf, wp)
                A.MoeMlp8Fn.apply(h, router, wf, wp, st, 2, b).backward(dy)
            timed("c5 MoE layer, 16384 tokens top-2 of 8, router bias %+.1f on two experts" % skew, c5,
                  6 * 2.0 * (2 * N) * d * Fd)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--traffic-probe", action="store_true")
    ap.add_argument("--ns-probe", action="store_true")
    ap.add_argument("--gemm-probe", action="store_true")
    ap.add_argument("--power-probe", action="store_true")
    ap.add_argument("--config-probe", choices=("c1", "c2", "c2d128", "c3", "c5", "all"))
    ap.add_argument("--graphs", action="store_true", help="with --config-probe: also time each repetition replayed as a HIP graph")
    ap.add_argument("--bf16-dw", action="store_true")
    ap.add_argument("--unfused-residual", action="store_true")
    ap.add_argument("--all-kernels", action="store_true", help="roofline.per_kernel lists every entry point, not the top 8")
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
    if args.gemm_probe:
        gemm_probe()
        return
    if args.power_probe:
        power_probe()
        return
    if args.config_probe:
        config_probe(args.config_probe, args.graphs)
        return

    import statistics

    import torch
    from trainium_frontier_them_bones_amd import _lib
    from trainium_frontier_them_bones_amd.model import GPT, GPTConfig, zipf_tokens

    _lib.lib()
    dev = torch.device("cuda:0")
    cfg = GPTConfig()
    cfg.fp8_mlp_dw = not args.bf16_dw
    cfg.fuse_residual = not args.unfused_residual
    model = GPT(cfg, dev, seed=0)
    B = 16
    # four distinct Zipf batches, resident in HBM, taken in turn: no step sees the buffers of the step before it
    batches = [tuple(t.to(dev) for t in zipf_tokens(B, cfg.seq_len, cfg.vocab, seed=s)) for s in range(4)]
    for i in range(args.warmup):
        model.train_step(*batches[i % 4])
    torch.cuda.synchronize()

    rec = []
    _lib.TIMED["tfb_attn_bwd_rope"] = rec
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(args.steps):
        loss = model.train_step(*batches[i % 4])
        marks[i + 1].record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    del _lib.TIMED["tfb_attn_bwd_rope"]
    tokens = B * cfg.seq_len
    ms = dt / args.steps * 1e3
    ms_median = statistics.median(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))

    # dominant entry point: attention backward (three launches: D = sum dO*O, dK/dV, dQ), timed with events on its stream
    if not rec:
        raise RuntimeError("the timed entry point was never called: roofline.achieved would be meaningless")
    k_ms = sum(r[0].elapsed_time(r[1]) for r in rec) / len(rec)
    H, D, T = cfg.n_head, cfg.head_dim, cfg.seq_len
    k_flops = 5 * B * H * T * T * D   # causal-halved: 5 matmuls x 2 flop x 1/2
    achieved = k_flops / (k_ms * 1e-3) / 1e12 if k_ms > 0 else 0.0

    # every entry point of the step, timed with events in three further (untimed) steps: the per-kernel table
    allrec = []
    _lib.TIMED["*"] = allrec
    for i in range(3):
        model.train_step(*batches[i % 4])
    torch.cuda.synchronize()
    del _lib.TIMED["*"]
    table = per_kernel_table(allrec, 3, top=1000 if args.all_kernels else 8)

    out = {
        "metric": "train tokens/s, 12L d768 T2048 fwd+bwd step; per-kernel % MFMA/HBM peak",
        "value": round(tokens / (dt / args.steps), 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 3),
        "ms_per_step_median": round(ms_median, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 (fp8 e4m3/e5m2 MLP GEMMs)",
        "data": "synthetic: 4 distinct batches of Zipf(1.1) token ids taken in turn, N(0, 0.02) random-init weights",
        "config": {"workload": "C4 full step: 12 layers, d_model 768, 12 heads x 64, MLP 3072 squared-ReLU fp8, RMSNorm "
                               "pre-norm, RoPE, untied head, vocab 32768; batch 16 x 2048 tokens; fwd+bwd+AdamW"
                               + ("; MLP weight gradients in bf16 (--bf16-dw)" if args.bf16_dw else "; all six MLP GEMMs in fp8")
                               + ("; residual adds and fp8 casts as separate passes (--unfused-residual)"
                                  if args.unfused_residual else ""),
                   "global_batch": B, "seq_len": cfg.seq_len, "params": model.num_params(),
                   "step_tflops": round(flops_per_token(cfg) * tokens / 1e12, 2),
                   "model_tflops_per_s": round(flops_per_token(cfg) * tokens / (dt / args.steps) / 1e12, 1),
                   "final_loss": round(float(loss.item()), 4)},
        "roofline": {"kernel": "attention backward (tfb_attn_bwd_rope: attn64_dq, which also makes the row statistics, + attn64_dkdv), B16 H12 T2048 D64", "bound": "mfma",
                     "achieved": round(achieved, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_BF16_TFLOPS, 4), "traffic": ATTN_BWD_TRAFFIC_BYTES,
                     "traffic_source": "constant from profiles/attn_c2_hbm_traffic.md (rocprofv3 --pmc), not measured in this run",
                     "launch_ms": round(k_ms, 4), "launches_timed": len(rec),
                     "per_kernel": table},
    }
    if not args.no_cpu:
        del model
        torch.cuda.empty_cache()
        out["cpu_baseline"], out["parity"] = cpu_baseline_and_parity(cfg, dev)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
