"""Pins oracle/model.py: its bf16-MLP variant against a straight fp32 nn.functional transformer, and closed forms."""
import math

import torch
import torch.nn.functional as F

from oracle.model import OracleGPT
from oracle import attention as OA
from trainium_frontier_them_bones_amd.model import GPTConfig, zipf_tokens


def _params(cfg, seed, head_zero=False):
    g = torch.Generator().manual_seed(seed)
    d, Fd, V = cfg.d_model, cfg.d_ff, cfg.vocab
    p = {"wte": torch.randn(V, d, generator=g) * 0.02}
    for i in range(cfg.n_layer):
        p["norm1.%d" % i] = 1 + 0.02 * torch.randn(d, generator=g)
        p["norm2.%d" % i] = 1 + 0.02 * torch.randn(d, generator=g)
        p["w_qkv.%d" % i] = torch.randn(3 * d, d, generator=g) * 0.02
        p["w_o.%d" % i] = torch.randn(d, d, generator=g) * 0.02
        p["w_fc.%d" % i] = torch.randn(Fd, d, generator=g) * 0.02
        p["w_proj.%d" % i] = torch.randn(d, Fd, generator=g) * 0.02
    p["norm_f"] = torch.ones(d)
    p["lm_head"] = torch.zeros(V, d) if head_zero else torch.randn(V, d, generator=g) * 0.02
    return {k: v.bfloat16() for k, v in p.items()}


def _plain_fp32(cfg, p, idx, tg):
    p = {k: v.float().clone().requires_grad_(True) for k, v in p.items()}
    B, T = idx.shape
    H, D = cfg.n_head, cfg.head_dim
    cos, sin = OA.rope_tables(T, D, cfg.rope_base)
    c, s = cos.float()[None, :, None, :], sin.float()[None, :, None, :]

    def rope(x):
        x1, x2 = x[..., : D // 2], x[..., D // 2:]
        return torch.cat((x1 * c + x2 * s, x2 * c - x1 * s), -1)

    x = F.embedding(idx, p["wte"])
    for i in range(cfg.n_layer):
        h = F.rms_norm(x, (cfg.d_model,), p["norm1.%d" % i], cfg.norm_eps)
        q, k, v = (t.reshape(B, T, H, D) for t in F.linear(h, p["w_qkv.%d" % i]).split(cfg.d_model, -1))
        o = F.scaled_dot_product_attention(rope(q).transpose(1, 2), rope(k).transpose(1, 2), v.transpose(1, 2), is_causal=True)
        x = x + F.linear(o.transpose(1, 2).reshape(B, T, cfg.d_model), p["w_o.%d" % i])
        h = F.rms_norm(x, (cfg.d_model,), p["norm2.%d" % i], cfg.norm_eps)
        x = x + F.linear(F.relu(F.linear(h, p["w_fc.%d" % i])).square(), p["w_proj.%d" % i])
    h = F.rms_norm(x, (cfg.d_model,), p["norm_f"], cfg.norm_eps)
    loss = F.cross_entropy(F.linear(h, p["lm_head"]).reshape(-1, cfg.vocab), tg.reshape(-1))
    loss.backward()
    return loss, p


def test_bf16_variant_tracks_plain_fp32_transformer():
    cfg = GPTConfig(n_layer=2, d_model=128, n_head=2, d_ff=512, vocab=512, seq_len=128)
    p = _params(cfg, 0)
    idx, tg = zipf_tokens(2, 128, cfg.vocab, seed=1)
    m = OracleGPT(cfg, p, fp8=False)
    loss = m.forward(idx, tg)
    loss.backward()
    ref, rp = _plain_fp32(cfg, p, idx, tg)
    assert abs(loss.item() - ref.item()) < 2e-3 * ref.item()
    for name in ("lm_head", "w_proj.1", "w_qkv.0", "wte"):
        a, b = m.p[name].grad.float(), rp[name].grad
        assert ((a - b).norm() / b.norm()).item() < 3e-2, name


def test_fp8_variant_stays_close_and_zero_head_gives_log_vocab():
    cfg = GPTConfig(n_layer=1, d_model=256, n_head=4, d_ff=512, vocab=512, seq_len=128)
    idx, tg = zipf_tokens(2, 128, cfg.vocab, seed=2)
    p = _params(cfg, 3, head_zero=True)
    assert abs(OracleGPT(cfg, p).forward(idx, tg).item() - math.log(512)) < 1e-5
    p = _params(cfg, 3)
    l8 = OracleGPT(cfg, p, fp8=True).forward(idx, tg).item()
    l16 = OracleGPT(cfg, p, fp8=False).forward(idx, tg).item()
    assert abs(l8 - l16) < 5e-3 * l16
