"""CPU oracle for the Mixtral MoE hot path.

TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, __graft_entry__.smoke()
and the cpu_baseline leg of bench.py may import this module; the product
package never does and has no CPU path of its own.

Every function restates one step of the reference (RouteTrace/electrock-infer,
paths relative to its root) and cites the lines it follows.  The reference
stores no golden vectors for this path (its tests draw unseeded random
inputs), so each function is pinned in tests/test_oracle.py by independent
means:

  topk_softmax              hand-worked tie cases, brute force over all orderings
                            of small rows, torch.softmax/torch.topk on tie-free rows
  moe_align_block_size      hand-worked cases, the sequential loop of the
                            reference's own test restated in pure Python
                            (moe_align_block_size_loop), structural invariants
  silu_and_mul / moe_sum    torch.nn.functional.silu / torch.sum library routines
  gate_logits               hand-worked case, torch.nn.functional.linear in float64
  rms_norm                  the reference's own torch op chains run by the library, exact small
                            cases, power-of-two scale invariance, a case where the two rounding
                            conventions differ
  moe_layer_fp32            dense all-experts formulation with torch.topk routing,
                            one-hot routing reducing to a plain SwiGLU MLP
  moe_layer_staged_bf16     its rounding points against moe_layer_fp32 within
                            bf16 error bounds (an emulation aid, not a parity target)

Parity status: no function here is "parity unpinned".  One behaviour of the
live reference is deliberately NOT reproduced: the tie order of torch.topk
inside topk_softmax_torch (softmax_topk.py:23-29), which no reference test
pins; ties go to the lowest expert index as in the reference's HIP router.
"""
from typing import Tuple

import numpy as np
import torch


# ----------------------------------------------------------------------------
# A8  tile configuration
# ----------------------------------------------------------------------------
def get_moe_config(num_tokens: int, num_experts: int) -> dict:
    """layers/moe/fused_moe.py:327-339."""
    if num_tokens <= num_experts:
        return {"BLOCK_SIZE_M": 16, "BLOCK_SIZE_N": 32, "BLOCK_SIZE_K": 64, "GROUP_SIZE_M": 1}
    return {"BLOCK_SIZE_M": 64, "BLOCK_SIZE_N": 64, "BLOCK_SIZE_K": 32, "GROUP_SIZE_M": 8}


# ----------------------------------------------------------------------------
# A9  router gate (the caller's step in front of the layer)
# ----------------------------------------------------------------------------
def to_bf16_f32(a: np.ndarray) -> np.ndarray:
    """Round float32 to the nearest bfloat16 (ties to even), returned as float32."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def gate_logits(x: np.ndarray, gate_w: np.ndarray, round_bf16: bool = True) -> np.ndarray:
    """Router logits of the model's MoE block: ``F.linear(x, weight)`` without bias
    (models/mixtral.py:40-42,59; layers/linear.py:53-54).

    x [T, H], gate_w [E, H] (values of bf16 tensors, any float dtype).  The dot products are
    taken in float64 and rounded once to float32 (a bf16 linear layer accumulates in fp32;
    its summation order is the library's), then to bf16 when ``round_bf16`` -- what the
    reference's bf16 linear returns.  -> float32 [T, E].
    """
    acc = np.asarray(x, dtype=np.float64) @ np.asarray(gate_w, dtype=np.float64).T
    out = acc.astype(np.float32)
    return to_bf16_f32(out) if round_bf16 else out


# ----------------------------------------------------------------------------
# the step in front of the MoE block: RMSNorm, optionally with the residual add
# ----------------------------------------------------------------------------
def round_to(a: np.ndarray, dtype: str) -> np.ndarray:
    """Round float32 values to the element type ("float32", "bfloat16", "float16"), returned as float32."""
    a = np.asarray(a, dtype=np.float32)
    if dtype == "bfloat16":
        return to_bf16_f32(a)
    if dtype == "float16":
        return a.astype(np.float16).astype(np.float32)
    if dtype == "float32":
        return a
    raise ValueError(dtype)


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float, residual: np.ndarray = None,
             semantics: str = "layer", dtype: str = "bfloat16"):
    """RMSNorm over the last axis, with the residual add when ``residual`` is given.

    x, residual [T, H] and weight [H] hold values of tensors of element type ``dtype`` (weight may also be
    float32) as float32 arrays.  Returns y, or (y, residual_out), as float32 arrays of ``dtype`` values.

    semantics "layer" -- what the model runs (layers/layernorm.py:17-41): the sum x + residual and its mean
    square stay float32; residual_out = T(sum); the normalised value is rounded to T before and after the
    multiplication by the weight.
    semantics "op" -- the native op (src/add_rms_norm.hip:47-52,76-80 and 103-106,130-133): the sum is
    rounded to T first and everything else uses the rounded value; one rounding of (value * weight) * rstd.

    The mean of squares is accumulated in float64 and rounded once to float32 (the reference sums in
    float32 in an order of its library's choosing); rsqrt is 1 / sqrt in float32.
    """
    x = np.asarray(x, dtype=np.float32)
    w = np.asarray(weight, dtype=np.float32)
    one = np.float32(1.0)
    res_out = None
    if residual is not None:
        s = x + np.asarray(residual, dtype=np.float32)      # float32 add
        res_out = round_to(s, dtype)
        if semantics == "op":
            s = res_out
    else:
        s = x
    var = (s.astype(np.float64) ** 2).mean(axis=-1, keepdims=True).astype(np.float32)
    rstd = one / np.sqrt(var + np.float32(eps), dtype=np.float32)
    if semantics == "layer":
        y = round_to(round_to(s * rstd, dtype) * w, dtype)
    elif semantics == "op":
        y = round_to((s * w) * rstd, dtype)
    else:
        raise ValueError(semantics)
    return y if residual is None else (y, res_out)


# ----------------------------------------------------------------------------
# A1/A2  router
# ----------------------------------------------------------------------------
def topk_softmax(logits: np.ndarray, topk: int, renormalize: bool) -> Tuple[np.ndarray, np.ndarray]:
    """Softmax + top-k on raw logits, ties to the lowest expert index.

    Selection: src/topk_softmax_kernels.hip:34-56 (strict '>' scan in ascending
    expert order == stable descending sort of the logits).
    Weights: exp(x - max) / sum in float32 (topk_softmax_kernels.hip:37-39,62-63;
    softmax_topk.py:23), then divided by the sum of the selected ones when
    renormalize (fused_moe.py:161-162).
    logits [T, E] any float dtype (evaluated as float32) -> (weights f32 [T,k], ids i32 [T,k]).
    """
    x = np.asarray(logits, dtype=np.float32)
    T, E = x.shape
    order = np.argsort(-x, axis=1, kind="stable")  # stable: equal logits keep ascending index
    ids = order[:, :topk].astype(np.int32)
    m = x.max(axis=1, keepdims=True)
    ex = np.exp(x - m, dtype=np.float32)
    denom = ex.sum(axis=1, keepdims=True, dtype=np.float32)
    probs = (ex / denom).astype(np.float32)
    w = np.take_along_axis(probs, ids.astype(np.int64), axis=1)
    if renormalize:
        w = (w / w.sum(axis=1, keepdims=True, dtype=np.float32)).astype(np.float32)
    return w.astype(np.float32), ids


def topk_scan_loop(row) -> Tuple[int, int]:
    """The reference's top-2 scan, literally (topk_softmax_kernels.hip:29-56).
    Pure Python; for small pinning cases."""
    top1_val, top1_idx, top2_val, top2_idx = -np.inf, -1, -np.inf, -1
    for i, v in enumerate(row):
        if v > top1_val:
            top2_val, top2_idx = top1_val, top1_idx
            top1_val, top1_idx = v, i
        elif v > top2_val:
            top2_val, top2_idx = v, i
    return top1_idx, top2_idx


# ----------------------------------------------------------------------------
# A3  expert sort
# ----------------------------------------------------------------------------
def align_buffer_sizes(numel: int, num_experts: int, block_size: int) -> Tuple[int, int]:
    """layers/moe/moe_align_block_size.py:32,41."""
    max_padded = numel + num_experts * (block_size - 1)
    return max_padded, -(-max_padded // block_size)


def moe_align_block_size(topk_ids: np.ndarray, num_experts: int, block_size: int,
                         sorted_len: int = None, expert_ids_len: int = None):
    """Stable counting sort of flat slot indices by expert with per-expert padding.

    Kernel: src/moe_align_block_size.hip:78-135 (count, pad to block, exclusive
    cumsum, stable scatter, block->expert table).  Buffer conventions of the
    wrapper, layers/moe/moe_align_block_size.py:32-48: sorted ids pre-filled -1
    (pads and tail), expert_ids pre-zeroed, lengths numel + E*(B-1) and
    cdiv(that, B).
    Returns (sorted_token_ids i32, expert_ids i32, num_tokens_post_pad i32[1]).
    """
    flat = np.asarray(topk_ids).reshape(-1).astype(np.int64)
    numel = flat.size
    dl, de = align_buffer_sizes(numel, num_experts, block_size)
    sorted_len = dl if sorted_len is None else sorted_len
    expert_ids_len = de if expert_ids_len is None else expert_ids_len
    cnt = np.bincount(flat, minlength=num_experts)[:num_experts]
    padded = -(-cnt // block_size) * block_size
    off = np.concatenate([[0], np.cumsum(padded)])
    sorted_ids = np.full(sorted_len, -1, dtype=np.int32)
    expert_ids = np.zeros(expert_ids_len, dtype=np.int32)
    order = np.argsort(flat, kind="stable")
    start = np.concatenate([[0], np.cumsum(cnt)])
    for e in range(num_experts):
        seg = order[start[e]:start[e + 1]]
        sorted_ids[off[e]:off[e] + cnt[e]] = seg
        expert_ids[off[e] // block_size: off[e + 1] // block_size] = e
    return sorted_ids, expert_ids, np.array([off[-1]], dtype=np.int32)


def moe_align_block_size_loop(topk_ids, num_experts: int, block_size: int):
    """Sequential restatement, one slot at a time, of the loop the reference's own
    test uses as ITS oracle (test/example/test_align_block.py:27-67), with the
    wrapper's buffer conventions.  Pure Python; for small pinning cases."""
    flat = [int(v) for v in np.asarray(topk_ids).reshape(-1)]
    counts = [0] * num_experts
    for e in flat:
        counts[e] += 1
    padded = [((c + block_size - 1) // block_size) * block_size for c in counts]
    offsets = [0] * num_experts
    for e in range(1, num_experts):
        offsets[e] = offsets[e - 1] + padded[e - 1]
    total = sum(padded)
    dl, de = align_buffer_sizes(len(flat), num_experts, block_size)
    sorted_ids = [-1] * dl
    expert_ids = [0] * de
    b = 0
    for e in range(num_experts):
        for _ in range(padded[e] // block_size):
            expert_ids[b] = e
            b += 1
    seen = [0] * num_experts
    for i, e in enumerate(flat):
        sorted_ids[offsets[e] + seen[e]] = i
        seen[e] += 1
    return (np.array(sorted_ids, dtype=np.int32), np.array(expert_ids, dtype=np.int32),
            np.array([total], dtype=np.int32))


# ----------------------------------------------------------------------------
# A5 / A7  element-wise ops (element type T in {float32, bfloat16, float16})
# ----------------------------------------------------------------------------
def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """out = T( T(silu_f32(gate)) * up ), gate = x[..., :d], up = x[..., d:]
    (src/activation_kernels.hip:35-45: SiLU in float32, rounded to T, then a
    multiply in T)."""
    d = x.shape[-1] // 2
    gate, up = x[..., :d], x[..., d:]
    g = gate.float()
    s = (g / (1.0 + torch.exp(-g))).to(x.dtype)
    return (s.float() * up.float()).to(x.dtype)


def moe_sum(x: torch.Tensor) -> torch.Tensor:
    """out[t] = T(T(0 + x[t,0]) + x[t,1]) ..., accumulated in T in ascending k
    (src/moe_sum.hip:36-45)."""
    acc = torch.zeros_like(x[:, 0])
    for k in range(x.shape[1]):
        acc = (acc.float() + x[:, k].float()).to(x.dtype)
    return acc


# ----------------------------------------------------------------------------
# whole layer
# ----------------------------------------------------------------------------
def moe_layer_fp32(x: torch.Tensor, router_logits: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor,
                   topk: int = 2, renormalize: bool = True, num_threads: int = None) -> torch.Tensor:
    """The layer in float32, expert by expert, as the reference's pure-torch MoE
    block does it (test/example/verify_hf_moe.py:59-86 ==
    models/modeling_mixtral.py:632-670), with the router of this module (ties
    to the lowest index) in place of torch.topk.

    x [T,H]; router_logits [T,E]; w13 [E,2I,H] (gate rows, then up rows:
    mixtral_moe.py:137-143); w2 [E,H,I].  Inputs of any float dtype are
    evaluated in float32.  Returns float32 [T,H].
    """
    if num_threads:
        torch.set_num_threads(num_threads)
    xf = x.float()
    T, H = xf.shape
    E, two_i, _ = w13.shape
    I = two_i // 2
    w, ids = topk_softmax(router_logits.float().numpy(), topk, renormalize)
    w_t, ids_t = torch.from_numpy(w), torch.from_numpy(ids.astype(np.int64))
    out = torch.zeros(T, H, dtype=torch.float32)
    for e in range(E):
        tok, slot = torch.where(ids_t == e)
        if tok.numel() == 0:
            continue
        cur = xf[tok]
        w13e = w13[e].float()
        h = torch.nn.functional.silu(cur @ w13e[:I].t()) * (cur @ w13e[I:].t())
        y = (h @ w2[e].float().t()) * w_t[tok, slot].unsqueeze(1)
        out.index_add_(0, tok, y)
    return out


def moe_layer_staged_bf16(x: torch.Tensor, router_logits: torch.Tensor, w13: torch.Tensor,
                          w2: torch.Tensor, topk: int = 2, renormalize: bool = True) -> dict:
    """The reference pipeline with its five roundings to bf16 made explicit
    (fused_moe.py:250-291): cache1 = bf16(x W13^T), cache2 = silu_and_mul(cache1),
    cache3 = bf16(f32(cache2 W2^T) * w), out = moe_sum(cache3).  Accumulation is
    float32 as in tl.dot.  Returns the intermediates keyed by the reference's names."""
    T, H = x.shape
    E, two_i, _ = w13.shape
    w, ids = topk_softmax(router_logits.float().numpy(), topk, renormalize)
    ids_t = torch.from_numpy(ids.astype(np.int64))
    w_t = torch.from_numpy(w)
    cache1 = torch.zeros(T, topk, two_i, dtype=torch.bfloat16)
    cache3 = torch.zeros(T, topk, H, dtype=torch.bfloat16)
    xf = x.float()
    for e in range(E):
        tok, slot = torch.where(ids_t == e)
        if tok.numel():
            cache1[tok, slot] = (xf[tok] @ w13[e].float().t()).to(torch.bfloat16)
    cache2 = silu_and_mul(cache1.view(-1, two_i)).view(T, topk, two_i // 2)
    for e in range(E):
        tok, slot = torch.where(ids_t == e)
        if tok.numel():
            acc = cache2[tok, slot].float() @ w2[e].float().t()
            cache3[tok, slot] = (acc * w_t[tok, slot].unsqueeze(1)).to(torch.bfloat16)
    return {"topk_weights": w, "topk_ids": ids, "cache1": cache1, "cache2": cache2, "cache3": cache3,
            "out": moe_sum(cache3)}


# ----------------------------------------------------------------------------
# seeded synthetic inputs of the benchmark configurations
# ----------------------------------------------------------------------------
def make_inputs(T: int, H: int, I: int, E: int = 8, seed: int = 0, dtype=torch.bfloat16,
                logits: str = "normal", logits_dtype=None):
    """x~N(0,1), router logits~N(0,1) (+ skew), w13/w2~N(0,0.02), drawn in float32
    from one generator in the fixed order x, logits, w13, w2 and then cast, so CPU
    and GPU see identical values.  `logits`: "normal" | "zipf" (per-expert bias
    log(rank^-1.2 / sum), experts permuted by the seed) | "two_experts" (+20 on
    experts 0 and 1)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g, dtype=torch.float32)
    lg = torch.randn(T, E, generator=g, dtype=torch.float32)
    w13 = torch.randn(E, 2 * I, H, generator=g, dtype=torch.float32) * 0.02
    w2 = torch.randn(E, H, I, generator=g, dtype=torch.float32) * 0.02
    if logits == "zipf":
        ranks = torch.arange(1, E + 1, dtype=torch.float32) ** -1.2
        bias = torch.log(ranks / ranks.sum())
        lg = lg + bias[torch.randperm(E, generator=g)]
    elif logits == "two_experts":
        lg[:, :2] += 20.0
    elif logits != "normal":
        raise ValueError(logits)
    return (x.to(dtype), lg.to(logits_dtype or dtype), w13.to(dtype), w2.to(dtype))
