"""Checkpoint -> device modules -> layer output.  A safetensors checkpoint with the tensor names of the reference's
Mixtral files (utils/mixtral_info.txt:17-42) is written by the test, loaded straight onto the GPU with the reference's
dispatch rules (utils/loader.py:18-53: safe_open(file, "pt", "cuda"); FusedMoE.weight_loader, mixtral_moe.py:121-152),
and the modules that hold the loaded parameters are run against the oracle evaluated on the checkpoint's own tensors."""
import numpy as np
import pytest
import torch
from safetensors.torch import save_file
from torch import nn

from electrock_infer_amd import MixtralMoE, PostAttentionMoE, RMSNorm
from electrock_infer_amd.utils import load_model
from oracle import moe_oracle as O
from tests.gpu_util import DEV, announce, error_stats

pytestmark = pytest.mark.gpu

E, H, I = 8, 512, 1024


class _Layer(nn.Module):
    def __init__(self, w2_dtype):
        super().__init__()
        self.block_sparse_moe = MixtralMoE(E, 2, H, I, params_dtype=torch.bfloat16, tp_size=1, w2_dtype=w2_dtype)
        self.post_attention_layernorm = RMSNorm(H)


class _Model(nn.Module):
    def __init__(self, layers, w2_dtype):
        super().__init__()
        self.model = nn.Module()
        self.model.layers = nn.ModuleList([_Layer(w2_dtype) for _ in range(layers)])


def _write_checkpoint(path, layers):
    g = torch.Generator().manual_seed(11)
    t = {}
    for l in range(layers):
        pre = f"model.layers.{l}."
        for e in range(E):
            t[pre + f"block_sparse_moe.experts.{e}.w1.weight"] = (torch.randn(I, H, generator=g) * 0.02).to(torch.bfloat16)
            t[pre + f"block_sparse_moe.experts.{e}.w2.weight"] = (torch.randn(H, I, generator=g) * 0.02).to(torch.bfloat16)
            t[pre + f"block_sparse_moe.experts.{e}.w3.weight"] = (torch.randn(I, H, generator=g) * 0.02).to(torch.bfloat16)
        t[pre + "block_sparse_moe.gate.weight"] = (torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16)
        t[pre + "post_attention_layernorm.weight"] = (1.0 + 0.1 * torch.randn(H, generator=g)).to(torch.bfloat16)
        t[pre + "self_attn.k_proj.weight"] = torch.randn(8, H, generator=g).to(torch.bfloat16)   # no parameter here
    names = sorted(t)
    save_file({n: t[n] for n in names[::2]}, str(path / "model-00001-of-00002.safetensors"))
    save_file({n: t[n] for n in names[1::2]}, str(path / "model-00002-of-00002.safetensors"))
    return t


def _oracle_layer(t, l, x, residual, eps):
    """norm(x + residual) -> gate -> experts on the checkpoint's tensors of layer l, in float."""
    pre = f"model.layers.{l}."
    w13 = torch.stack([torch.cat([t[pre + f"block_sparse_moe.experts.{e}.w1.weight"],
                                  t[pre + f"block_sparse_moe.experts.{e}.w3.weight"]]) for e in range(E)])
    w2 = torch.stack([t[pre + f"block_sparse_moe.experts.{e}.w2.weight"] for e in range(E)])
    h, res = O.rms_norm(x.float().numpy(), t[pre + "post_attention_layernorm.weight"].float().numpy(), eps,
                        residual=residual.float().numpy())
    h = torch.from_numpy(np.asarray(h)).to(torch.bfloat16)
    logits = O.gate_logits(h.float().numpy(), t[pre + "block_sparse_moe.gate.weight"].float().numpy())
    return O.moe_layer_fp32(h, torch.from_numpy(logits), w13, w2), h, torch.from_numpy(np.asarray(res))


@pytest.mark.parametrize("w2_dtype", [None, torch.bfloat16])
def test_checkpoint_loaded_onto_the_gpu_runs_the_layer(tmp_path, w2_dtype):
    """w2_dtype=None: the module's default, w2 held as float16 (the loader's copy converts the bfloat16 checkpoint);
    torch.bfloat16: the checkpoint's own type."""
    announce(f"load_model(device=cuda) -> MixtralMoE / PostAttentionMoE, w2_dtype={w2_dtype}")
    layers = 2
    t = _write_checkpoint(tmp_path, layers)
    model = _Model(layers, w2_dtype).to(DEV)
    for p in model.parameters():
        p.data.zero_()
    loaded = load_model(model, str(tmp_path), device=DEV, strict=False)
    assert len(loaded) == len(t) - layers
    g = torch.Generator().manual_seed(3)
    for l, layer in enumerate(model.model.layers):
        ex = layer.block_sparse_moe.experts
        assert ex.w13_weight.is_cuda and ex.w2_weight.is_cuda
        assert ex.w2_weight.dtype == (w2_dtype or torch.float16) and ex.w13_weight.dtype == torch.bfloat16
        pre = f"model.layers.{l}."
        for e in (0, E - 1):
            assert torch.equal(ex.w13_weight[e, :I].cpu(), t[pre + f"block_sparse_moe.experts.{e}.w1.weight"])
            assert torch.equal(ex.w13_weight[e, I:].cpu(), t[pre + f"block_sparse_moe.experts.{e}.w3.weight"])
            # (a float16 parameter holds every bf16 weight of magnitude >= 2^-14 exactly, smaller ones to 2^-25)
            d = (ex.w2_weight[e].float().cpu() - t[pre + f"block_sparse_moe.experts.{e}.w2.weight"].float()).abs()
            assert float(d.max()) <= (2.0 ** -25 if w2_dtype is None else 0.0)
        for T in (3, 70, 600):
            x = torch.randn(T, H, generator=g).to(torch.bfloat16)
            r = torch.randn(T, H, generator=g).to(torch.bfloat16)
            ref, h_ref, res_ref = _oracle_layer(t, l, x, r, layer.post_attention_layernorm.eps)
            # the MoE block alone on the oracle's normalised rows (in place, as the reference's block)
            out = layer.block_sparse_moe(h_ref.to(DEV).clone())
            st = error_stats(out.float(), ref)
            assert st["mean_rel"] <= 2e-3 and st["max_abs"] <= 2e-2, (l, T, st)     # bf16 output: 1.4e-3 of rounding
            # the decoder-layer tail: norm + gate + experts in one call
            tail = PostAttentionMoE(layer.post_attention_layernorm, layer.block_sparse_moe)
            out2, res2 = tail(x.to(DEV), r.to(DEV))
            assert torch.equal(res2.cpu().float(), res_ref.float().to(torch.bfloat16).float())
            st2 = error_stats(out2.float(), ref)
            assert st2["mean_rel"] <= 6e-3, (l, T, st2)   # a normalised value one bf16 step off moves a routing weight
