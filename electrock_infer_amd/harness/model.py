"""Mixtral-shaped decoder-only model around the MoE block (counterpart of electrock_infer/models/mixtral.py:66-273,
layers/attention.py:9-63, layers/rotary_embedding.py:6-55, layers/embed_head.py:9-71, layers/sampler.py:5-18).

Per decoder layer (mixtral.py:176-198): input RMSNorm (+ residual) -> attention -> post-attention RMSNorm (+ residual)
-> MoE block.  The two RMSNorms and the MoE block are this package's kernels (the post-attention norm, the router gate,
the router and the experts in one library call); projections, rotary embedding and attention are torch ops -- the
reference uses flash_attn there, which this image does not have.
"""
import zlib
from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
import torch.nn.functional as F
from torch import nn

from ..layers.layernorm import RMSNorm
from ..layers.moe.mixtral_block import MixtralMoE, PostAttentionMoE
from .config import ModelConfig


@dataclass
class BatchContext:
    """What the attention layers need to know about the batch of one forward pass (utils/context.py:5-16)."""
    is_prefill: bool
    slot_mapping: torch.Tensor                       # [tokens] int64: flat cache slot of every token fed
    q_lens: List[int]                                # prefill: tokens fed per sequence
    k_lens: List[int]                                # prefill: context length per sequence (cached prefix + fed)
    block_tables: Optional[torch.Tensor] = None      # [seqs, max_blocks] int64, padded with 0
    context_lens: Optional[torch.Tensor] = None      # decode: [seqs] int64
    last_token_index: Optional[torch.Tensor] = None  # prefill: row of every sequence's last token
    decode_mask: Optional[torch.Tensor] = None       # decode: [seqs, 1, 1, max_blocks * block_size] bool, key < context length


class RotaryEmbedding(nn.Module):
    """Rotate-half ("neox") rotary embedding over the whole head (rotary_embedding.py:6-55); cos / sin are float32
    tables indexed by position, the rotation is computed in float32 and rounded once."""

    def __init__(self, head_dim: int, max_position: int, base: float):
        super().__init__()
        inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
        angles = torch.outer(torch.arange(max_position, dtype=torch.float32), inv_freq)
        self.register_buffer("cos", angles.cos(), persistent=False)
        self.register_buffer("sin", angles.sin(), persistent=False)

    def rotate(self, positions: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
        """x [tokens, heads, head_dim]"""
        cos, sin = self.cos[positions].unsqueeze(1), self.sin[positions].unsqueeze(1)
        x1, x2 = x.float().chunk(2, dim=-1)
        return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1).to(x.dtype)


class PagedAttention(nn.Module):
    """Causal grouped-query attention over a paged KV cache (layers/attention.py:26-63): the new keys and values are
    written into their cache slots first; a prefill sequence without a cached prefix attends over its own fresh keys,
    one with a cached prefix and every decode step over the keys gathered through the block table."""

    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int):
        super().__init__()
        self.num_heads, self.num_kv_heads, self.head_dim = num_heads, num_kv_heads, head_dim
        self.scale = head_dim ** -0.5
        self.k_cache = self.v_cache = None            # [blocks, block_size, kv_heads, head_dim], set by the runner
        self.kv_cache = None                          # the two as one tensor [2, blocks, block_size, kv_heads, head_dim]

    def _gathered(self, cache: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
        """[seqs, max_blocks * block_size, kv_heads, head_dim] from block ids [seqs, max_blocks]"""
        g = cache[table]
        return g.view(table.shape[0], -1, self.num_kv_heads, self.head_dim)

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, ctx: BatchContext) -> torch.Tensor:
        q = q.view(-1, self.num_heads, self.head_dim)
        k = k.view(-1, self.num_kv_heads, self.head_dim)
        v = v.view(-1, self.num_kv_heads, self.head_dim)
        self.k_cache.view(-1, self.num_kv_heads, self.head_dim).index_copy_(0, ctx.slot_mapping, k)
        self.v_cache.view(-1, self.num_kv_heads, self.head_dim).index_copy_(0, ctx.slot_mapping, v)
        if not ctx.is_prefill:
            # One new token per sequence: the query heads that share a KV head are laid out as the rows of one
            # small attention problem per (sequence, KV head), so the gathered keys are used as they are.
            B, group = q.shape[0], self.num_heads // self.num_kv_heads
            # keys and values of all sequences in one gather: [2, B, L, kvh, d] -> [B, kvh, L, d] each
            kv = self.kv_cache[:, ctx.block_tables].view(2, B, -1, self.num_kv_heads, self.head_dim).transpose(2, 3)
            o = F.scaled_dot_product_attention(q.view(B, self.num_kv_heads, group, self.head_dim), kv[0], kv[1],
                                               attn_mask=ctx.decode_mask, scale=self.scale)
            return o.reshape(B, self.num_heads * self.head_dim)
        out = torch.empty_like(q)
        row = 0
        for i, (ql, kl) in enumerate(zip(ctx.q_lens, ctx.k_lens)):
            qs = q[row:row + ql].transpose(0, 1).unsqueeze(0)                          # [1, heads, ql, d]
            if kl == ql:
                ks = k[row:row + ql].transpose(0, 1).unsqueeze(0)
                vs = v[row:row + ql].transpose(0, 1).unsqueeze(0)
                o = F.scaled_dot_product_attention(qs, ks, vs, is_causal=True, scale=self.scale, enable_gqa=True)
            else:   # cached prefix: keys come out of the cache; query j sits at position kl - ql + j
                table = ctx.block_tables[i:i + 1]
                ks = self._gathered(self.k_cache, table)[:, :kl].transpose(1, 2)
                vs = self._gathered(self.v_cache, table)[:, :kl].transpose(1, 2)
                qpos = torch.arange(kl - ql, kl, device=q.device)[:, None]
                mask = torch.arange(kl, device=q.device)[None, :] <= qpos
                o = F.scaled_dot_product_attention(qs, ks, vs, attn_mask=mask, scale=self.scale, enable_gqa=True)
            out[row:row + ql] = o[0].transpose(0, 1)
            row += ql
        return out.view(-1, self.num_heads * self.head_dim)


class MixtralAttention(nn.Module):
    """qkv projection -> rotary embedding of q and k -> paged attention -> output projection (mixtral.py:66-149)."""

    def __init__(self, cfg: ModelConfig):
        super().__init__()
        d, nh, nkv = cfg.head_dim, cfg.num_attention_heads, cfg.num_key_value_heads
        self.q_size, self.kv_size = nh * d, nkv * d
        # q, k and v rows stacked in one weight, as the reference's QKVParallelLinear keeps them
        self.qkv_proj = nn.Linear(cfg.hidden_size, self.q_size + 2 * self.kv_size, bias=False, dtype=cfg.torch_dtype)
        self.o_proj = nn.Linear(self.q_size, cfg.hidden_size, bias=False, dtype=cfg.torch_dtype)
        self.rotary_emb = RotaryEmbedding(d, cfg.max_position_embeddings, cfg.rope_theta)
        self.attn = PagedAttention(nh, nkv, d)

    def forward(self, positions: torch.Tensor, hidden_states: torch.Tensor, ctx: BatchContext) -> torch.Tensor:
        q, k, v = self.qkv_proj(hidden_states).split([self.q_size, self.kv_size, self.kv_size], dim=-1)
        q = self.rotary_emb.rotate(positions, q.reshape(-1, self.attn.num_heads, self.attn.head_dim))
        k = self.rotary_emb.rotate(positions, k.reshape(-1, self.attn.num_kv_heads, self.attn.head_dim))
        return self.o_proj(self.attn(q, k, v.contiguous(), ctx))


class MixtralDecoderLayer(nn.Module):

    def __init__(self, cfg: ModelConfig, fused_moe_tail: bool = True):
        super().__init__()
        self.self_attn = MixtralAttention(cfg)
        self.block_sparse_moe = MixtralMoE(cfg.num_local_experts, cfg.num_experts_per_tok, cfg.hidden_size,
                                           cfg.intermediate_size, params_dtype=cfg.torch_dtype, tp_size=1)
        self.input_layernorm = RMSNorm(cfg.hidden_size, eps=cfg.rms_norm_eps)
        self.post_attention_layernorm = RMSNorm(cfg.hidden_size, eps=cfg.rms_norm_eps)
        self.moe_tail = PostAttentionMoE(self.post_attention_layernorm, self.block_sparse_moe) if fused_moe_tail else None
        self.moe_events = None       # a list: (start, end) event pairs around the MoE tail are appended to it

    def forward(self, positions, hidden_states, residual, ctx: BatchContext):
        if residual is None:
            residual = hidden_states
            hidden_states = self.input_layernorm(hidden_states)
        else:
            hidden_states, residual = self.input_layernorm(hidden_states, residual)
        hidden_states = self.self_attn(positions, hidden_states, ctx)
        if self.moe_events is not None:
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
        if self.moe_tail is not None:
            hidden_states, residual = self.moe_tail(hidden_states, residual)
        else:
            hidden_states, residual = self.post_attention_layernorm(hidden_states, residual)
            hidden_states = self.block_sparse_moe(hidden_states)
        if self.moe_events is not None:
            end.record()
            self.moe_events.append((start, end))
        return hidden_states, residual


class MixtralForCausalLM(nn.Module):
    """Embedding, decoder layers, final norm, LM head (mixtral.py:201-273).  Parameter names follow the checkpoint
    layout the reference loads (`model.layers.N.block_sparse_moe.experts.w13_weight`, ...)."""

    experts_modules_mapping = {"w1": ("w13_weight", "w1"), "w3": ("w13_weight", "w3"), "w2": ("w2_weight", "w2")}

    def __init__(self, cfg: ModelConfig, fused_moe_tail: bool = True):
        super().__init__()
        self.cfg = cfg
        self.model = nn.Module()
        self.model.embed_tokens = nn.Embedding(cfg.vocab_size, cfg.hidden_size, dtype=cfg.torch_dtype)
        self.model.layers = nn.ModuleList([MixtralDecoderLayer(cfg, fused_moe_tail) for _ in range(cfg.num_hidden_layers)])
        self.model.norm = RMSNorm(cfg.hidden_size, eps=cfg.rms_norm_eps)
        self.lm_head = nn.Linear(cfg.hidden_size, cfg.vocab_size, bias=False, dtype=cfg.torch_dtype)

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, ctx: BatchContext) -> torch.Tensor:
        hidden_states, residual = self.model.embed_tokens(input_ids), None
        for layer in self.model.layers:
            hidden_states, residual = layer(positions, hidden_states, residual, ctx)
        hidden_states, _ = self.model.norm(hidden_states, residual)
        return hidden_states

    def compute_logits(self, hidden_states: torch.Tensor, ctx: BatchContext) -> torch.Tensor:
        """Logits of the position that predicts the next token of every sequence (embed_head.py:61-71)."""
        if ctx.is_prefill:
            hidden_states = hidden_states[ctx.last_token_index].contiguous()
        return self.lm_head(hidden_states)

    @torch.no_grad()
    def init_random_weights(self, seed: int = 0, std: float = 0.02, gate_std: Optional[float] = None) -> None:
        """Explicit random initialisation (no checkpoint exists here; the reference's parameters would stay
        torch.empty): N(0, std) for every matrix, drawn on the parameter's device expert by expert, 1 for the norms.
        The draws are rounded to the model's dtype first, as a checkpoint of that dtype would hold them, and then
        copied into the parameter (the experts' w2 may be held in another type)."""
        for li, layer in enumerate(self.model.layers):
            for name, p in layer.named_parameters():
                g = torch.Generator(device=p.device).manual_seed(seed * 100003 + li * 101 + (zlib.crc32(name.encode()) % 97))
                if name.endswith("layernorm.weight"):
                    p.fill_(1.0)
                elif p.dim() == 3:
                    for e in range(p.shape[0]):
                        p[e].copy_((torch.randn(p.shape[1:], generator=g, device=p.device, dtype=torch.float32) * std)
                                   .to(self.lm_head.weight.dtype))
                else:
                    s = gate_std if (gate_std is not None and name.endswith("gate.weight")) else std
                    p.copy_(torch.randn(p.shape, generator=g, device=p.device, dtype=torch.float32) * s)
        g = torch.Generator(device=self.lm_head.weight.device).manual_seed(seed + 7)
        self.model.embed_tokens.weight.copy_(torch.randn(self.model.embed_tokens.weight.shape, generator=g,
                                                         device=self.lm_head.weight.device) * std)
        self.lm_head.weight.copy_(torch.randn(self.lm_head.weight.shape, generator=g,
                                              device=self.lm_head.weight.device) * std)
        self.model.norm.weight.fill_(1.0)


class Sampler(nn.Module):
    """Greedy for temperature 0, else a draw from softmax(logits / temperature) by the exponential-race form of
    the Gumbel trick (layers/sampler.py:10-18)."""

    def forward(self, logits: torch.Tensor, temperatures: torch.Tensor) -> torch.Tensor:
        logits = logits.float()
        greedy = logits.argmax(dim=-1)
        if bool((temperatures == 0).all()):
            return greedy
        safe_t = torch.where(temperatures == 0, torch.ones_like(temperatures), temperatures)
        probs = torch.softmax(logits / safe_t.unsqueeze(1), dim=-1)
        draw = (probs / (torch.empty_like(probs).exponential_(1) + 1e-10)).argmax(dim=-1)
        return torch.where(temperatures == 0, greedy, draw)
