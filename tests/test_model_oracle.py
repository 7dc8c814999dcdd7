"""Pins oracle/model_oracle.py (the float32 restatement of the harness's decoder) independently of the code it
checks: rotary embedding against complex multiplication, attention against torch's scaled_dot_product_attention,
the whole model against causality and against a one-layer model written out with library calls."""
import math
from types import SimpleNamespace

import numpy as np
import torch
import torch.nn.functional as F

from oracle import model_oracle as M
from oracle import moe_oracle as O


def test_rotary_is_a_rotation_of_the_half_pairs_by_position_times_frequency():
    g = torch.Generator().manual_seed(0)
    n, heads, d, theta = 7, 3, 16, 10000.0
    x = torch.randn(n, heads, d, generator=g)
    pos = torch.tensor([0, 1, 2, 5, 9, 100, 4095])
    y = M.rotary(x, pos, theta)
    # pair (x[i], x[i + d/2]) as a complex number, multiplied by exp(j * pos * theta^(-2i/d))
    z = torch.complex(x[..., : d // 2].double(), x[..., d // 2:].double())
    freq = torch.tensor([theta ** (-2.0 * i / d) for i in range(d // 2)], dtype=torch.float64)
    rot = torch.polar(torch.ones(n, d // 2, dtype=torch.float64), pos.double()[:, None] * freq[None, :])
    want = z * rot[:, None, :]
    assert torch.allclose(y[..., : d // 2].double(), want.real, atol=2e-4)      # float32 angles at position 4095
    assert torch.allclose(y[..., d // 2:].double(), want.imag, atol=2e-4)
    assert torch.equal(M.rotary(x, torch.zeros(n, dtype=torch.int64), theta), x)         # position 0: identity
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-5)                     # a rotation keeps lengths


def test_attention_matches_the_library_with_repeated_kv_heads():
    g = torch.Generator().manual_seed(1)
    n, heads, kvh, d = 9, 8, 2, 16
    q, k, v = torch.randn(n, heads, d, generator=g), torch.randn(n, kvh, d, generator=g), torch.randn(n, kvh, d, generator=g)
    got = M.causal_gqa_attention(q, k, v)
    kk = k.repeat_interleave(heads // kvh, dim=1).transpose(0, 1)
    vv = v.repeat_interleave(heads // kvh, dim=1).transpose(0, 1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), kk, vv, is_causal=True).transpose(0, 1).reshape(n, -1)
    assert torch.allclose(got, want, atol=1e-5)
    assert torch.allclose(got[0], v[0].repeat_interleave(heads // kvh, dim=0).reshape(-1))   # position 0 sees itself only


def tiny(layers=2, seed=0):
    cfg = SimpleNamespace(vocab_size=50, hidden_size=32, intermediate_size=64, num_hidden_layers=layers,
                          num_attention_heads=4, num_key_value_heads=2, num_local_experts=4, num_experts_per_tok=2,
                          rms_norm_eps=1e-5, rope_theta=10000.0)
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g) * 0.2
    d = cfg.hidden_size // cfg.num_attention_heads
    p = {"model.embed_tokens.weight": r(cfg.vocab_size, 32), "model.norm.weight": 1 + r(32), "lm_head.weight": r(cfg.vocab_size, 32)}
    for li in range(layers):
        pre = f"model.layers.{li}."
        p[pre + "input_layernorm.weight"] = 1 + r(32)
        p[pre + "post_attention_layernorm.weight"] = 1 + r(32)
        p[pre + "self_attn.qkv_proj.weight"] = r((4 + 2 * 2) * d, 32)
        p[pre + "self_attn.o_proj.weight"] = r(32, 4 * d)
        p[pre + "block_sparse_moe.gate.weight"] = r(4, 32) * 10
        p[pre + "block_sparse_moe.experts.w13_weight"] = r(4, 128, 32)
        p[pre + "block_sparse_moe.experts.w2_weight"] = r(4, 32, 64)
    return cfg, p


def test_model_is_causal():
    cfg, p = tiny()
    ids = [3, 14, 15, 9, 2, 6, 5, 35, 8]
    full = M.model_logits(p, cfg, ids)
    assert full.shape == (len(ids), cfg.vocab_size)
    for n in (1, 4, 8):
        assert torch.allclose(M.model_logits(p, cfg, ids[:n]), full[:n], atol=1e-5)     # later tokens change nothing
    other = M.model_logits(p, cfg, ids[:4] + [40] + ids[5:])
    assert torch.allclose(other[:4], full[:4], atol=1e-5) and not torch.allclose(other[4:], full[4:], atol=1e-3)


def test_one_layer_model_against_library_calls():
    cfg, p = tiny(layers=1, seed=3)
    ids = torch.tensor([7, 1, 22, 49, 0, 13])
    n, heads, kvh, d = len(ids), 4, 2, 8
    pre = "model.layers.0."
    x = F.embedding(ids, p["model.embed_tokens.weight"])
    norm = lambda t, w: F.rms_norm(t, (32,), w, cfg.rms_norm_eps)
    qkv = F.linear(norm(x, p[pre + "input_layernorm.weight"]), p[pre + "self_attn.qkv_proj.weight"])
    q, k, v = qkv.split([heads * d, kvh * d, kvh * d], dim=-1)
    # rotary through complex numbers (see the first test), attention through the library
    def rope(t, h):
        t = t.reshape(n, h, d)
        z = torch.complex(t[..., : d // 2], t[..., d // 2:])
        freq = cfg.rope_theta ** (-torch.arange(0, d, 2, dtype=torch.float32) / d)
        z = z * torch.polar(torch.ones(n, d // 2), torch.arange(n, dtype=torch.float32)[:, None] * freq)[:, None, :]
        return torch.cat((z.real, z.imag), dim=-1)
    q, k = rope(q, heads).transpose(0, 1), rope(k, kvh).repeat_interleave(2, dim=1).transpose(0, 1)
    vv = v.reshape(n, kvh, d).repeat_interleave(2, dim=1).transpose(0, 1)
    att = F.scaled_dot_product_attention(q, k, vv, is_causal=True).transpose(0, 1).reshape(n, -1)
    res = x + F.linear(att, p[pre + "self_attn.o_proj.weight"])
    m = norm(res, p[pre + "post_attention_layernorm.weight"])
    # dense form of the MoE block: softmax over the bf16-rounded logits, top-2 renormalised, every expert evaluated
    lg = torch.from_numpy(O.gate_logits(m.numpy(), p[pre + "block_sparse_moe.gate.weight"].numpy()))
    probs = torch.softmax(lg, dim=-1)
    top, idx = probs.topk(2, dim=-1)
    assert (top[:, 0] - top[:, 1]).min() > 1e-6              # no ties in this draw, so torch.topk's order is safe
    wts = torch.zeros_like(probs).scatter(1, idx, top / top.sum(-1, keepdim=True))
    w13, w2 = p[pre + "block_sparse_moe.experts.w13_weight"], p[pre + "block_sparse_moe.experts.w2_weight"]
    hcat = torch.einsum("th,eih->tei", m, w13)
    moe = torch.einsum("tei,ehi->teh", F.silu(hcat[..., :64]) * hcat[..., 64:], w2)
    out = (moe * wts[..., None]).sum(1)
    want = F.linear(norm(out + res, p["model.norm.weight"]), p["lm_head.weight"])
    got = M.model_logits(p, cfg, ids.tolist())
    assert torch.allclose(got, want, atol=2e-5), float((got - want).abs().max())
