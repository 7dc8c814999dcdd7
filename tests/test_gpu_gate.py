"""GPU parity of the router gate fused with the router (em_gate_topk_softmax, em_moe_forward_gated)
against the oracle: logits = F.linear(x, gate_weight) of the model's MoE block
(models/mixtral.py:40-42,59), then the router's selection."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.gpu_util import DEV, announce, error_stats, gpu_inputs

pytestmark = pytest.mark.gpu


def gate_weight(E, H, seed):
    g = torch.Generator(device=DEV).manual_seed(1234 + seed)
    return (torch.randn(E, H, generator=g, device=DEV, dtype=torch.float32) * 0.05).to(torch.bfloat16)


def bf16_ulp(v: np.ndarray) -> np.ndarray:
    """spacing of bf16 numbers at |v| (8 significant bits)"""
    return np.maximum(2.0 ** (np.floor(np.log2(np.maximum(np.abs(v), 2.0 ** -126))) - 7), 2.0 ** -133)


@pytest.mark.parametrize("T,H,E", [(1, 4096, 8), (7, 4096, 8), (64, 4096, 8), (1000, 4096, 8), (8192, 4096, 8),
                                   (64, 6144, 8), (33, 1000, 8), (64, 2048, 16)])
@pytest.mark.parametrize("bf16_logits", [True, False])
def test_gate_topk_matches_oracle(T, H, E, bf16_logits):
    from electrock_infer_amd.layers.moe.fused_moe import gate_topk
    announce(f"gate_topk T={T} H={H} E={E} bf16_logits={bf16_logits}")
    g = torch.Generator(device=DEV).manual_seed(T + H)
    x = torch.randn(T, H, generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    gw = gate_weight(E, H, T)
    w, ids, logits = gate_topk(x, gw, 2, renormalize=True, bf16_logits=bf16_logits, return_logits=True)
    torch.cuda.synchronize()
    want = O.gate_logits(x.float().cpu().numpy(), gw.float().cpu().numpy(), round_bf16=bf16_logits)
    got = logits.float().cpu().numpy()
    if bf16_logits:
        # the fp32 sums differ from the oracle's in the last bits (summation order), so a logit that sits on a
        # rounding boundary may land on the neighbouring bf16 value: at most one bf16 step, and rarely
        # (for logits near zero a bf16 step is smaller than the fp32 rounding of the partial sums, whose size
        # follows sum |x_i * g_i|: allow that on top)
        sum_abs = np.abs(x.float().cpu().numpy()).astype(np.float64) @ np.abs(gw.float().cpu().numpy()).astype(np.float64).T
        err = np.abs(got - want)
        assert (err <= bf16_ulp(want) * (1.0 + 1e-6) + 4 * 2.0 ** -24 * sum_abs).all()
        assert (err > 0).sum() <= max(2, 2e-3 * err.size)   # (a small batch may hold one such logit)
    else:
        np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-5)
    # the selection must be the oracle's selection on the logits the kernel itself produced (bit-exact ids),
    # and the weights the oracle's weights for them
    w_ref, ids_ref = O.topk_softmax(got, 2, True)
    np.testing.assert_array_equal(ids.cpu().numpy(), ids_ref)
    np.testing.assert_allclose(w.cpu().numpy(), w_ref, rtol=3e-6, atol=1e-7)
    # against the oracle's own logits the ids may differ only where the two candidates are within a bf16 step
    _, ids_o = O.topk_softmax(want, 2, True)
    diff = np.nonzero((ids.cpu().numpy() != ids_o).any(axis=1))[0]
    for t in diff:
        srt = np.sort(want[t])[::-1]
        gaps = np.abs(np.diff(srt[:3]))
        assert gaps.min() <= 2 * bf16_ulp(srt[:3]).max(), (t, want[t], got[t])
    assert len(diff) <= max(1, T // 200)


def test_gate_bf16_logits_create_ties_that_go_to_lowest_index():
    from electrock_infer_amd.layers.moe.fused_moe import gate_topk
    announce("gate ties")
    T, H, E = 256, 512, 8
    x = torch.ones(T, H, device=DEV, dtype=torch.bfloat16)
    gw = torch.zeros(E, H, device=DEV, dtype=torch.bfloat16)
    gw[3] = 1.0 / 64
    gw[5] = 1.0 / 64          # experts 3 and 5 tie at 8.0, everything else 0
    gw[1, :8] = 1.0 / 64      # expert 1: 0.125
    w, ids = gate_topk(x, gw, 2, renormalize=True)
    assert (ids[:, 0] == 3).all() and (ids[:, 1] == 5).all()
    np.testing.assert_allclose(w.cpu().numpy(), 0.5, rtol=1e-6)


@pytest.mark.parametrize("T", [1, 64, 300, 2048])
def test_gated_layer_matches_two_step_path_and_oracle(T):
    from electrock_infer_amd.layers.moe.fused_moe import fused_experts, fused_experts_gated, gate_topk
    announce(f"gated layer T={T}")
    H, I, E = 512, 1024, 8
    x, _, w13, w2 = gpu_inputs(T, H, I, E, seed=T)
    gw = gate_weight(E, H, T)
    out = fused_experts_gated(x, gw, w13, w2, topk=2, renormalize=True, out_dtype=torch.float32)
    # same result as routing on the logits the gate kernel reports
    _, _, logits = gate_topk(x, gw, 2, return_logits=True)
    out2 = fused_experts(x, w13, w2, logits, topk=2, renormalize=True, out_dtype=torch.float32)
    assert torch.equal(out, out2)
    # and the fp32 definition on those logits
    ref = O.moe_layer_fp32(x.cpu(), logits.cpu(), w13.cpu(), w2.cpu())
    st = error_stats(out, ref)
    assert st["mean_rel"] <= 2.5e-3 and st["max_abs"] <= 4e-3 * float(ref.abs().max()), st


def test_mixtral_block_module():
    from electrock_infer_amd import MixtralMoE
    announce("MixtralMoE module")
    T, H, I, E = 48, 256, 512, 8
    torch.manual_seed(0)
    blk = MixtralMoE(E, 2, H, I, params_dtype=torch.bfloat16).to(DEV)
    blk.gate.weight.weight_loader(blk.gate.weight, (torch.randn(E, H) * 0.05).to(torch.bfloat16).to(DEV))
    for e in range(E):
        blk.experts.w13_weight.weight_loader(blk.experts.w13_weight, (torch.randn(I, H) * 0.02).to(torch.bfloat16).to(DEV), "w1", e)
        blk.experts.w13_weight.weight_loader(blk.experts.w13_weight, (torch.randn(I, H) * 0.02).to(torch.bfloat16).to(DEV), "w3", e)
        blk.experts.w2_weight.weight_loader(blk.experts.w2_weight, (torch.randn(H, I) * 0.02).to(torch.bfloat16).to(DEV), "w2", e)
    x = torch.randn(4, 12, H, device=DEV).to(torch.bfloat16)
    x0 = x.clone()
    y = blk(x)
    assert y.shape == x0.shape and y.data_ptr() == x.data_ptr()   # in place, original shape, as the reference
    logits = O.gate_logits(x0.view(-1, H).float().cpu().numpy(), blk.gate.weight.float().cpu().numpy())
    ref = O.moe_layer_fp32(x0.view(-1, H).cpu(), torch.from_numpy(logits), blk.experts.w13_weight.cpu(), blk.experts.w2_weight.cpu())
    st = error_stats(y.view(-1, H), ref)
    assert st["mean_rel"] <= 6e-3, st


def test_mixtral_block_module_with_float16_w2():
    """w2_dtype=float16 on the block: the same call as the default mode on the bf16 weights, without the conversion."""
    from electrock_infer_amd import MixtralMoE
    from electrock_infer_amd.layers.moe.fused_moe import fused_experts_gated
    announce("MixtralMoE module, float16 w2")
    T, H, I, E = 200, 256, 512, 8
    g = torch.Generator().manual_seed(5)
    blk = MixtralMoE(E, 2, H, I, params_dtype=torch.bfloat16, w2_dtype=torch.float16).to(DEV)
    assert blk.experts.w2_weight.dtype == torch.float16
    blk.gate.weight.data.copy_((torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16))
    blk.experts.w13_weight.data.copy_((torch.randn(E, 2 * I, H, generator=g) * 0.02).to(torch.bfloat16))
    w2 = (torch.randn(E, H, I, generator=g) * 0.02).to(torch.bfloat16).to(DEV)
    for e in range(E):
        blk.experts.weight_loader(blk.experts.w2_weight, w2[e], "w2", e)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(DEV)
    want = fused_experts_gated(x.clone(), blk.gate.weight, blk.experts.w13_weight, w2, topk=2, renormalize=True)
    got = blk(x.clone())
    assert float((got.float() - want.float()).abs().max()) <= 2.0 ** -8 * float(want.float().abs().max())
