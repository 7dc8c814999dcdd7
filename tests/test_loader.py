"""Checkpoint loading into the package's modules with the reference's dispatch rules
(utils/loader.py:14-49, tensor names of utils/mixtral_info.txt:17-42).  Host logic only: CPU tensors."""
import pytest
import torch
from safetensors.torch import save_file
from torch import nn

from electrock_infer_amd import MixtralMoE, RMSNorm
from electrock_infer_amd.utils import load_model


class _Layer(nn.Module):
    def __init__(self, E, H, I):
        super().__init__()
        self.block_sparse_moe = MixtralMoE(E, 2, H, I, params_dtype=torch.bfloat16, tp_size=1)
        self.post_attention_layernorm = RMSNorm(H)


class _Model(nn.Module):
    def __init__(self, E, H, I, layers=2):
        super().__init__()
        self.model = nn.Module()
        self.model.layers = nn.ModuleList([_Layer(E, H, I) for _ in range(layers)])


def _checkpoint(tmp_path, E, H, I, layers=2, extra=True):
    g = torch.Generator().manual_seed(0)
    t = {}
    for l in range(layers):
        pre = f"model.layers.{l}."
        for e in range(E):
            t[pre + f"block_sparse_moe.experts.{e}.w1.weight"] = torch.randn(I, H, generator=g).to(torch.bfloat16)
            t[pre + f"block_sparse_moe.experts.{e}.w2.weight"] = torch.randn(H, I, generator=g).to(torch.bfloat16)
            t[pre + f"block_sparse_moe.experts.{e}.w3.weight"] = torch.randn(I, H, generator=g).to(torch.bfloat16)
        t[pre + "block_sparse_moe.gate.weight"] = torch.randn(E, H, generator=g).to(torch.bfloat16)
        t[pre + "post_attention_layernorm.weight"] = torch.randn(H, generator=g).to(torch.bfloat16)
        if extra:
            t[pre + "self_attn.k_proj.weight"] = torch.randn(8, H, generator=g).to(torch.bfloat16)
    # two files, as real checkpoints are sharded
    names = sorted(t)
    save_file({n: t[n] for n in names[::2]}, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file({n: t[n] for n in names[1::2]}, str(tmp_path / "model-00002-of-00002.safetensors"))
    return t


def test_load_model_stacks_expert_weights(tmp_path):
    E, H, I = 4, 16, 24
    t = _checkpoint(tmp_path, E, H, I)
    m = _Model(E, H, I)
    for p in m.parameters():
        p.data.zero_()
    loaded = load_model(m, str(tmp_path), strict=False)
    assert len(loaded) == len(t) - 2                      # the two attention tensors have no parameter here
    for l, layer in enumerate(m.model.layers):
        pre = f"model.layers.{l}."
        ex = layer.block_sparse_moe.experts
        for e in range(E):
            assert torch.equal(ex.w13_weight[e, :I], t[pre + f"block_sparse_moe.experts.{e}.w1.weight"])
            assert torch.equal(ex.w13_weight[e, I:], t[pre + f"block_sparse_moe.experts.{e}.w3.weight"])
            assert torch.equal(ex.w2_weight[e], t[pre + f"block_sparse_moe.experts.{e}.w2.weight"])
        assert torch.equal(layer.block_sparse_moe.gate.weight, t[pre + "block_sparse_moe.gate.weight"])
        assert torch.equal(layer.post_attention_layernorm.weight.to(torch.bfloat16), t[pre + "post_attention_layernorm.weight"])


def test_load_model_converts_w2_for_a_float16_w2_parameter(tmp_path):
    """w2_dtype=float16: the parameter is float16 and the loader's copy converts the checkpoint's bfloat16 tensors
    (exactly: these values lie inside the fp16 range)."""
    E, H, I = 2, 16, 24
    t = _checkpoint(tmp_path, E, H, I, layers=1, extra=False)
    m = _Model(E, H, I, layers=1)
    m.model.layers[0].block_sparse_moe = MixtralMoE(E, 2, H, I, params_dtype=torch.bfloat16, tp_size=1,
                                                    w2_dtype=torch.float16)
    load_model(m, str(tmp_path), strict=True)
    ex = m.model.layers[0].block_sparse_moe.experts
    assert ex.w2_weight.dtype == torch.float16 and ex.w13_weight.dtype == torch.bfloat16
    for e in range(E):
        src = t[f"model.layers.0.block_sparse_moe.experts.{e}.w2.weight"]
        assert torch.equal(ex.w2_weight[e].float(), src.float())


def test_load_model_strict_raises_on_unknown_tensor(tmp_path):
    _checkpoint(tmp_path, 2, 8, 8, layers=1)
    with pytest.raises(AttributeError):
        load_model(_Model(2, 8, 8, layers=1), str(tmp_path), strict=True)
    _checkpoint(tmp_path, 2, 8, 8, layers=1, extra=False)
    assert len(load_model(_Model(2, 8, 8, layers=1), str(tmp_path), strict=True)) == 2 * 3 + 2


def test_load_model_tp_shards(tmp_path):
    # with tp_size 2 every rank keeps its slice of the intermediate dimension (mixtral_moe.py:132-150)
    E, H, I = 2, 8, 16
    t = _checkpoint(tmp_path, E, H, I, layers=1, extra=False)

    class _M(nn.Module):
        def __init__(self, rank):
            super().__init__()
            self.model = nn.Module()
            layer = nn.Module()
            layer.block_sparse_moe = MixtralMoE(E, 2, H, I, params_dtype=torch.bfloat16, tp_size=2)
            layer.block_sparse_moe.experts.tp_rank = rank
            layer.post_attention_layernorm = RMSNorm(H)
            self.model.layers = nn.ModuleList([layer])

    for rank in (0, 1):
        m = _M(rank)
        load_model(m, str(tmp_path))
        ex = m.model.layers[0].block_sparse_moe.experts
        half = I // 2
        sl = slice(rank * half, (rank + 1) * half)
        assert ex.w13_weight.shape == (E, 2 * half, H)
        for e in range(E):
            assert torch.equal(ex.w13_weight[e, :half], t[f"model.layers.0.block_sparse_moe.experts.{e}.w1.weight"][sl])
            assert torch.equal(ex.w13_weight[e, half:], t[f"model.layers.0.block_sparse_moe.experts.{e}.w3.weight"][sl])
            assert torch.equal(ex.w2_weight[e], t[f"model.layers.0.block_sparse_moe.experts.{e}.w2.weight"][:, sl])
