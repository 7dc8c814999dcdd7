"""Host-side mirror of the reference layer: class surface, weight loading and
error behaviour (no kernel is launched; CPU tensors must be refused, not
silently computed)."""
import inspect

import pytest
import torch

import electrock_infer_amd as em
from electrock_infer_amd import FusedMoE, _C, fused_experts, fused_topk, moe_align_block_size
from electrock_infer_amd.layers.moe.fused_moe import _get_moe_config


def test_op_surface_matches_reference_binding():
    # names and keyword names of pytorch_bind.cpp:18-51
    assert list(inspect.signature(_C.silu_and_mul).parameters) == ["out", "input"]
    assert list(inspect.signature(_C.topk_softmax).parameters) == ["topk_weights", "topk_indices", "gating_output"]
    assert list(inspect.signature(_C.moe_sum).parameters) == ["input", "output"]
    assert list(inspect.signature(_C.moe_align_block_size).parameters) == [
        "topk_ids", "num_experts", "block_size", "sorted_token_ids", "expert_ids", "num_tokens_post_pad"]
    assert list(inspect.signature(moe_align_block_size).parameters) == ["topk_ids", "block_size", "num_experts"]
    assert list(inspect.signature(fused_experts).parameters)[:8] == [
        "hidden_states", "w1", "w2", "gating_output", "topk", "renormalize", "inplace", "activation"]
    assert list(inspect.signature(fused_topk).parameters) == ["hidden_states", "gating_output", "topk", "renormalize"]
    params = inspect.signature(FusedMoE.__init__).parameters
    assert list(params)[1:9] == [
        "num_experts", "top_k", "hidden_size", "intermediate_size", "tp_size", "params_dtype", "renormalize",
        "reduce_results"]
    # the additions are keyword-only and off by default
    assert list(params)[9:] == ["bf16_act", "w2_dtype"]
    assert all(params[k].kind is inspect.Parameter.KEYWORD_ONLY for k in ("bf16_act", "w2_dtype"))
    assert params["bf16_act"].default is False and params["w2_dtype"].default is None
    assert em._C is _C


def test_fusedmoe_keeps_w2_as_float16_where_the_tuned_kernels_run():
    """bfloat16 parameters: w2 is held as float16 (the w2 GEMM multiplies fp16 activations) unless the caller opts
    out, asks for bf16 activations, uses another parameter type, or the shape falls to the shape-generic kernels."""
    kw = dict(num_experts=8, top_k=2, hidden_size=256, intermediate_size=512, tp_size=1)
    m = FusedMoE(**kw, params_dtype=torch.bfloat16)
    assert m.w2_weight.dtype == torch.float16 and m.w13_weight.dtype == torch.bfloat16 and m.w2_dtype == torch.float16
    assert FusedMoE(**kw, params_dtype=torch.bfloat16, w2_dtype=torch.bfloat16).w2_weight.dtype == torch.bfloat16
    assert FusedMoE(**kw, params_dtype=torch.bfloat16, bf16_act=True).w2_weight.dtype == torch.bfloat16
    assert FusedMoE(**kw, params_dtype=torch.float32).w2_weight.dtype == torch.float32
    odd = dict(kw, hidden_size=136, intermediate_size=200)
    assert FusedMoE(**odd, params_dtype=torch.bfloat16).w2_weight.dtype == torch.bfloat16
    # the loader's copy converts: bf16 checkpoint values are exact in fp16 at these magnitudes
    w2 = (torch.randn(256, 512, generator=torch.Generator().manual_seed(1)) * 0.02).to(torch.bfloat16)
    m.weight_loader(m.w2_weight, w2, "w2", 3)
    big = w2.float().abs() >= 2.0 ** -14
    assert torch.equal(m.w2_weight[3].float()[big], w2.float()[big])
    assert float((m.w2_weight[3].float() - w2.float()).abs().max()) <= 2.0 ** -25


def test_moe_config_rule():
    assert _get_moe_config(8, 8, 14336, 2) == {"BLOCK_SIZE_M": 16, "BLOCK_SIZE_N": 32, "BLOCK_SIZE_K": 64,
                                               "GROUP_SIZE_M": 1}
    assert _get_moe_config(9, 8, 14336, 2)["BLOCK_SIZE_M"] == 64


def test_fusedmoe_parameters_and_weight_loader():
    m = FusedMoE(num_experts=4, top_k=2, hidden_size=16, intermediate_size=24, tp_size=1,
                 params_dtype=torch.bfloat16)
    assert m.w13_weight.shape == (4, 48, 16) and m.w2_weight.shape == (4, 16, 24)
    assert m.w13_weight.dtype == torch.bfloat16 and not m.w13_weight.requires_grad
    assert m.w13_weight.weight_loader == m.weight_loader and m.w2_weight.weight_loader == m.weight_loader
    m.w13_weight.data.zero_()
    m.w2_weight.data.zero_()
    g = torch.Generator().manual_seed(0)
    w1 = torch.randn(24, 16, generator=g).to(torch.bfloat16)
    w3 = torch.randn(24, 16, generator=g).to(torch.bfloat16)
    w2 = torch.randn(16, 24, generator=g).to(torch.bfloat16)
    m.weight_loader(m.w13_weight, w1, "w1", 2)
    m.weight_loader(m.w13_weight, w3, "w3", 2)
    m.weight_loader(m.w2_weight, w2, "w2", 2)
    assert torch.equal(m.w13_weight[2, :24], w1) and torch.equal(m.w13_weight[2, 24:], w3)
    assert torch.equal(m.w2_weight[2], w2)
    assert m.w13_weight[[0, 1, 3]].abs().sum() == 0 and m.w2_weight[[0, 1, 3]].abs().sum() == 0
    with pytest.raises(ValueError):
        m.weight_loader(m.w2_weight, w2, "w4", 0)


def test_fusedmoe_tp_shard_selection():
    m = FusedMoE(4, 2, 16, 24, tp_size=2, params_dtype=torch.float32)
    assert m.intermediate_size_per_partition == 12 and m.w13_weight.shape == (4, 24, 16)
    m.tp_rank = 1                                  # what dist.get_rank() would give on the second rank
    w1 = torch.arange(24 * 16, dtype=torch.float32).view(24, 16)
    w2 = torch.arange(16 * 24, dtype=torch.float32).view(16, 24)
    m.weight_loader(m.w13_weight, w1, "w1", 0)
    m.weight_loader(m.w2_weight, w2, "w2", 0)
    assert torch.equal(m.w13_weight[0, :12], w1[12:]) and torch.equal(m.w2_weight[0], w2[:, 12:])
    with pytest.raises(ValueError):
        FusedMoE(4, 2, 16, 25, tp_size=2)


def test_cpu_tensors_are_refused_not_computed():
    x = torch.zeros(4, 16, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        fused_experts(x, torch.zeros(8, 32, 16, dtype=torch.bfloat16), torch.zeros(8, 16, 16, dtype=torch.bfloat16),
                      torch.zeros(4, 8), 2)
    with pytest.raises(RuntimeError, match="GPU"):
        _C.silu_and_mul(torch.zeros(4, 8), torch.zeros(4, 16))
    with pytest.raises(RuntimeError, match="GPU"):
        _C.moe_sum(torch.zeros(4, 2, 8), torch.zeros(4, 8))
    with pytest.raises(RuntimeError, match="GPU"):
        fused_topk(x, torch.zeros(4, 8), 2, True)
    with pytest.raises(NotImplementedError):
        fused_experts(x, x, x, x, 2, activation="gelu")
