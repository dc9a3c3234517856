"""Writes tests/golden/ref_vectors.npz: small input/output vectors of the reference's own torch emulations of its kernels.

Run in the build container only (it needs the reference checkout; nothing else does):

    python tests/golden/make_ref_vectors.py [/root/reference]

It imports the reference's standalone kernel modules under round2/source/kernels/ (each needs only `os`, `math` and
`torch`; their `nki` imports are guarded) and calls the emulation functions on seeded inputs:

    nki_mlp_fused8.py   forward_scales, backward_scales, emulate8_forward, emulate8_backward, weight_grads
    nki_attn_bandpro.py emulate_forward, emulate_backward (+ the band forms)
    nki_dw8.py          emulate_dw
    nki_resmix.py       emulate
    nki_nsk.py          emulate_nsk

The fixture holds data only (inputs and the outputs the reference computed for them); bf16 tensors are stored as their
16-bit patterns. tests/test_oracle_golden.py holds the oracle to these outputs bit for bit on the CPU, and
tests/test_gpu_golden.py the HIP kernels to them within the path's tolerance on the GPU.
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "ref_vectors.npz")


def load(ref_root, name):
    path = os.path.join(ref_root, "round2", "source", "kernels", name + ".py")
    spec = importlib.util.spec_from_file_location("ref_" + name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def put(store, key, t):
    t = t.detach().contiguous()
    if t.dtype == torch.bfloat16:
        store[key + ":bf16"] = t.view(torch.int16).numpy().view(np.uint16)
    elif t.dtype in (torch.float32, torch.int64, torch.int32, torch.uint8):
        store[key] = t.numpy()
    else:
        raise TypeError(t.dtype)


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    torch.manual_seed(0)
    torch.set_num_threads(1)            # one summation order, whatever machine regenerates the file
    S = {}
    bf = torch.bfloat16

    # ---- fp8 fused MLP: scale rows, forward, backward, bf16 weight gradients (M 128, d 256, F 256) ----
    m8 = load(ref_root, "nki_mlp_fused8")
    g = torch.Generator().manual_seed(8101)
    M, d, F = 128, 256, 256
    x = torch.randn(M, d, generator=g).to(bf)
    w_fc = (0.04 * torch.randn(F, d, generator=g)).to(bf)
    w_proj = (0.04 * torch.randn(d, F, generator=g)).to(bf)
    dy = torch.randn(M, d, generator=g).to(bf)
    row = m8.forward_scales(w_fc, w_proj)
    y, rT = m8.emulate8_forward(x, w_fc, w_proj, row)
    brow = m8.backward_scales(dy, row)
    dx, h, dpre = m8.emulate8_backward(dy, rT, w_fc, w_proj, brow, 0)
    dw_fc, dw_proj = m8.weight_grads(dy, x, h, dpre, 0)
    for k, t in dict(x=x, w_fc=w_fc, w_proj=w_proj, dy=dy, row=row, y=y, rT=rT, brow=brow, dx=dx, h=h, dpre=dpre,
                     dw_fc=dw_fc, dw_proj=dw_proj).items():
        put(S, "mlp8." + k, t)
    # a second input, 12 times larger than the unit-RMS rows the scale bound assumes, so that a good share of the hidden
    # activations reaches the clamp: the clamp and the order "r saved before the clamp" become visible in y and dpre
    xc = (12.0 * torch.randn(M, d, generator=g)).to(bf)
    yc, rTc = m8.emulate8_forward(xc, w_fc, w_proj, row)
    dxc, hc, dprec = m8.emulate8_backward(dy, rTc, w_fc, w_proj, brow, 0)
    for k, t in dict(x=xc, y=yc, rT=rTc, dx=dxc, dpre=dprec).items():
        put(S, "mlp8c." + k, t)
    # scale rows alone over a spread of magnitudes (the exponent search and its window)
    rows = []
    mags = [2.0 ** e for e in (-30, -12, -3, 0, 5, 20, 45)]
    for i, mag in enumerate(mags):
        a = (mag * torch.randn(64, 128, generator=g)).to(bf)
        b = (mag * 0.5 * torch.randn(128, 64, generator=g)).to(bf)
        r0 = m8.forward_scales(a, b)
        gy = (mag * torch.randn(32, 128, generator=g)).to(bf)
        rows.append(torch.stack([r0, m8.backward_scales(gy, r0)]))
        put(S, "scales.%d.w_fc" % i, a)
        put(S, "scales.%d.w_proj" % i, b)
        put(S, "scales.%d.dy" % i, gy)
    put(S, "scales.rows", torch.stack(rows))

    # ---- attention: emulate_forward / emulate_backward, full causal and a band of 1 tile (B 1, H 2, T 256, D 64) ----
    ab = load(ref_root, "nki_attn_bandpro")
    g = torch.Generator().manual_seed(8102)
    B, H, T, D = 1, 2, 256, 64
    q, k, v = (torch.randn(B, H, T, D, generator=g).to(bf) for _ in range(3))
    # unit-RMS rows (the reference's fixed shift assumes QK-normed inputs)
    q = (q.float() * torch.rsqrt(q.float().square().mean(-1, keepdim=True))).to(bf)
    k = (k.float() * torch.rsqrt(k.float().square().mean(-1, keepdim=True))).to(bf)
    do3 = torch.randn(B, T, H * D, generator=g).to(bf)
    scale = 0.125
    shift = float(ab.fixed_shift(scale, D))
    o3, lse3 = ab.emulate_forward(q, k, v, scale, shift)
    dq, dk, dv3 = ab.emulate_backward(q, k, v, o3, do3, lse3, scale)
    o3b, lse3b = ab.emulate_forward_band(q, k, v, scale, shift, 1)
    dqb, dkb, dv3b = ab.emulate_backward_band(q, k, v, o3b, do3, lse3b, scale, 1)
    for kk, t in dict(q=q, k=k, v=v, do3=do3, o3=o3, lse3=lse3, dq=dq, dk=dk, dv3=dv3, o3b=o3b, lse3b=lse3b, dqb=dqb,
                      dkb=dkb, dv3b=dv3b).items():
        put(S, "attn." + kk, t)
    S["attn.shift"] = np.float32(shift)

    # ---- fp8 weight gradient: emulate_dw in both format pairings (M 256, O 128, D 128) ----
    dw = load(ref_root, "nki_dw8")
    g = torch.Generator().manual_seed(8103)
    g2 = (3e-3 * torch.randn(256, 128, generator=g)).to(bf)
    a2 = torch.randn(256, 128, generator=g).to(bf)
    s_g, s_a = 2.0 ** 20, 4.0
    put(S, "dw8.g2", g2)
    put(S, "dw8.a2", a2)
    put(S, "dw8.out_e5m2_e4m3", dw.emulate_dw(g2, a2, s_g, s_a, 1.0 / (s_g * s_a), dw.FMT_E5M2, dw.FMT_E4M3))
    hpos = (torch.randn(256, 128, generator=g).abs() * 3.0).to(bf)          # the clamped e4m3 form (h side)
    put(S, "dw8.h", hpos)
    put(S, "dw8.out_e4m3c_e5m2", dw.emulate_dw(hpos, g2, 64.0, s_g, 1.0 / (64.0 * s_g), dw.FMT_E4M3C, dw.FMT_E5M2))

    # ---- residual mix backward: emulate (M 256, d 128) ----
    rm = load(ref_root, "nki_resmix")
    g = torch.Generator().manual_seed(8104)
    gg, xx, x0 = (torch.randn(256, 128, generator=g).to(bf) for _ in range(3))
    a, b = torch.tensor([0.75]).to(bf), torch.tensor([-0.3125]).to(bf)
    dxr, dx0r, part = rm.emulate(gg, xx, x0, a, b)
    for kk, t in dict(g=gg, x=xx, x0=x0, a=a, b=b, dx=dxr, dx0=dx0r, part=part).items():
        put(S, "resmix." + kk, t)

    # ---- Newton-Schulz: emulate_nsk on one tall and one wide matrix (256 x 128) ----
    ns = load(ref_root, "nki_nsk")
    g = torch.Generator().manual_seed(8105)
    ga = torch.randn(1, 256, 128, generator=g).to(bf).float()      # bf16-representable, stored as bf16 (the kernel's
    gb = torch.randn(1, 128, 256, generator=g).to(bf).float()      # first step rounds g to bf16 anyway)
    d_a = ga.float().norm(dim=(-2, -1)) * 1.02 + 1e-6
    d_b = gb.float().norm(dim=(-2, -1)) * 1.02 + 1e-6
    ya, yb, va, vb = ns.emulate_nsk(ga, gb, d_a, d_b)
    for kk, t in dict(ga=ga.to(bf), gb=gb.to(bf), d_a=d_a, d_b=d_b, ya=ya, yb=yb, va=va, vb=vb).items():
        put(S, "nsk." + kk, t)
    S["nsk.coeffs"] = np.asarray(ns.NSK_COEFFS, dtype=np.float64)

    np.savez_compressed(OUT, **S)
    print("wrote %s: %d arrays, %.0f KB" % (OUT, len(S), os.path.getsize(OUT) / 1024))


if __name__ == "__main__":
    main()
