"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

from oracle import moe_oracle as O

DEV = "cuda:0"


def announce(msg: str) -> None:
    """Name the case before any GPU work, so a lost box still tells which one ran."""
    print(f"[gpu-case] {msg}", flush=True)


def error_stats(got: torch.Tensor, ref: torch.Tensor) -> dict:
    """max-abs error and mean relative error  mean|d| / mean|ref|  against an fp32 reference."""
    d = (got.double().cpu() - ref.double().cpu()).abs()
    return {"max_abs": float(d.max()), "mean_rel": float(d.mean() / ref.double().abs().mean())}


def gpu_inputs(T, H, I, E=8, seed=0, logits="normal", logits_dtype=torch.bfloat16):
    """Full-size inputs drawn on the GPU (seeded), same distributions as
    oracle.make_inputs; returns device tensors."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    x = torch.randn(T, H, generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    lg = torch.randn(T, E, generator=g, device=DEV, dtype=torch.float32)
    w13 = torch.empty(E, 2 * I, H, device=DEV, dtype=torch.bfloat16)
    w2 = torch.empty(E, H, I, device=DEV, dtype=torch.bfloat16)
    for e in range(E):  # expert by expert keeps the fp32 staging small
        w13[e] = (torch.randn(2 * I, H, generator=g, device=DEV, dtype=torch.float32) * 0.02).to(torch.bfloat16)
        w2[e] = (torch.randn(H, I, generator=g, device=DEV, dtype=torch.float32) * 0.02).to(torch.bfloat16)
    if logits == "zipf":
        ranks = torch.arange(1, E + 1, dtype=torch.float32) ** -1.2
        bias = torch.log(ranks / ranks.sum())[torch.randperm(E, generator=torch.Generator().manual_seed(seed))]
        lg = lg + bias.to(DEV)
    elif logits == "two_experts":
        lg[:, :2] += 20.0
    return x, lg.to(logits_dtype), w13, w2


def oracle_rows(x, lg, w13_cpu, w2_cpu, rows):
    """fp32 oracle for a subset of tokens (the layer is token-wise)."""
    idx = torch.as_tensor(rows)
    return O.moe_layer_fp32(x[idx.to(x.device)].cpu(), lg[idx.to(lg.device)].cpu(), w13_cpu, w2_cpu)
