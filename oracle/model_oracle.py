"""CPU restatement, in float32 torch, of the Mixtral-shaped decoder the end-to-end harness runs.  TEST
INFRASTRUCTURE ONLY: imported by tests/ (and by nothing in the product path).

Follows the reference's model definition: decoder layer electrock_infer/models/mixtral.py:176-198 (input RMSNorm with
residual, attention, post-attention RMSNorm with residual, MoE block), attention mixtral.py:137-149 with rotate-half
rotary embedding (layers/rotary_embedding.py:6-16,39-55) and causal grouped-query attention (what flash_attn_varlen_func
computes, layers/attention.py:47-50), model mixtral.py:219-231, LM head layers/embed_head.py:61-66.  There is no KV
cache here: every call recomputes the whole sequence, which is what a paged cache must be equivalent to.

Pinned in tests/test_model_oracle.py: the rotary embedding against complex multiplication, the attention against
torch's scaled_dot_product_attention with repeated KV heads, causality of the whole model, and a one-layer model
against the same steps written out with library calls.  The MoE block is oracle.moe_oracle.moe_layer_fp32 on
oracle.moe_oracle.gate_logits (both pinned in tests/test_oracle.py).
"""
from typing import Dict

import numpy as np
import torch

from . import moe_oracle as O


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """layers/layernorm.py:17-27 in float32 (no intermediate rounding)."""
    var = x.pow(2).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(var + eps) * weight


def rotary(x: torch.Tensor, positions: torch.Tensor, theta: float) -> torch.Tensor:
    """Rotate-half rotary embedding of x [tokens, heads, head_dim]: the pair (x[i], x[i + d/2]) turns by
    positions * theta^(-2i/d) (rotary_embedding.py:6-16,29-36)."""
    d = x.shape[-1]
    inv_freq = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    ang = positions.float()[:, None] * inv_freq[None, :]
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    x1, x2 = x[..., : d // 2], x[..., d // 2:]
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1)


def causal_gqa_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """q [n, heads, d], k / v [n, kv_heads, d] of ONE sequence -> [n, heads * d]; query head h reads KV head
    h // (heads / kv_heads); position i attends to positions <= i; scale d^-0.5."""
    n, heads, d = q.shape
    group = heads // k.shape[1]
    out = torch.empty(n, heads, d)
    mask = torch.ones(n, n, dtype=torch.bool).tril()
    for h in range(heads):
        s = (q[:, h] @ k[:, h // group].t()) * d ** -0.5
        s = s.masked_fill(~mask, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, h // group]
    return out.reshape(n, heads * d)


def _bf16(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.bfloat16).float()


def _norm(x, residual, weight, eps, bf16_points: bool):
    """(normalised, new residual) of layers/layernorm.py:17-41; with `bf16_points` at the module's own rounding
    points (moe_oracle.rms_norm, "layer" semantics), else in plain float32."""
    if not bf16_points:
        s = x if residual is None else x + residual
        return rms_norm(s, weight, eps), s
    if residual is None:
        y = O.rms_norm(x.numpy(), weight.numpy(), eps)
        return torch.from_numpy(np.asarray(y)), x
    y, r = O.rms_norm(x.numpy(), weight.numpy(), eps, residual=residual.numpy())
    return torch.from_numpy(np.asarray(y)), torch.from_numpy(np.asarray(r))


def model_logits(params: Dict[str, torch.Tensor], cfg, token_ids, routing_margin: bool = False,
                 bf16_points: bool = False):
    """Logits [n, vocab] at every position of one sequence.  `params`: the model's state dict as float32 CPU
    tensors (names of the checkpoint layout: model.layers.N.self_attn.qkv_proj.weight, ...).

    ``bf16_points``: round to bf16 wherever a bf16 model stores a tensor (the outputs of the embedding, of every
    projection, of the rotary embedding, of the attention, of the norms at their own two rounding points, of the MoE
    block and of the LM head); every operation in between stays float32.  A bf16 model then differs from this only
    by the order of its sums and what its attention kernel rounds inside.

    With ``routing_margin`` also returns, per position, the smallest gap over the layers between the last selected
    and the first rejected expert's router logit, relative to the largest logit magnitude of that row: where it is
    small, a pipeline of another precision may legitimately pick another expert there (the layer is discontinuous in
    its router logits across that boundary), so a comparison has to know."""
    r = _bf16 if bf16_points else (lambda t: t)
    ids = torch.as_tensor(token_ids, dtype=torch.int64)
    pos = torch.arange(len(ids))
    heads, kvh, d = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.hidden_size // cfg.num_attention_heads
    h = params["model.embed_tokens.weight"][ids]
    residual = None
    for li in range(cfg.num_hidden_layers):
        p = f"model.layers.{li}."
        a, residual = _norm(h, residual, params[p + "input_layernorm.weight"], cfg.rms_norm_eps, bf16_points)
        qkv = r(a @ params[p + "self_attn.qkv_proj.weight"].t())
        q, k, v = qkv.split([heads * d, kvh * d, kvh * d], dim=-1)
        q = r(rotary(q.reshape(-1, heads, d), pos, cfg.rope_theta))
        k = r(rotary(k.reshape(-1, kvh, d), pos, cfg.rope_theta))
        att = r(r(causal_gqa_attention(q, k, v.reshape(-1, kvh, d))) @ params[p + "self_attn.o_proj.weight"].t())
        m, residual = _norm(att, residual, params[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps, bf16_points)
        logits = O.gate_logits(m.numpy().astype(np.float32), params[p + "block_sparse_moe.gate.weight"].numpy())
        top = np.sort(logits, axis=-1)[:, ::-1]
        kk = cfg.num_experts_per_tok
        gap = (top[:, kk - 1] - top[:, kk]) / np.abs(logits).max(axis=-1) if logits.shape[1] > kk else np.full(len(ids), np.inf)
        margin = gap if li == 0 else np.minimum(margin, gap)
        h = r(O.moe_layer_fp32(m, torch.from_numpy(logits), params[p + "block_sparse_moe.experts.w13_weight"],
                               params[p + "block_sparse_moe.experts.w2_weight"], topk=kk))
    final, _ = _norm(h, residual, params["model.norm.weight"], cfg.rms_norm_eps, bf16_points)
    out = r(final @ params["lm_head.weight"].t())
    return (out, torch.from_numpy(np.ascontiguousarray(margin))) if routing_margin else out
