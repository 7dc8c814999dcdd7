"""Writes tests/golden/c1_seed0.npz: configuration 1 of the benchmark list
(T=64, hidden=256, intermediate=512, E=8, top-2 renormalised, fp32, seed 0).

The reference holds no stored vectors for the MoE path, so this fixture is made
from torch LIBRARY routines only — softmax, topk (the logits are tie-free fp32
normals, so its tie order is not exercised), sort, einsum, silu — in a dense
all-experts formulation that shares no code with oracle/.  It pins the oracle
(tests/test_oracle.py) and, through it, the GPU path.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch

T, H, I, E, K, BLOCK, SEED = 64, 256, 512, 8, 2, 64, 0


def main():
    g = torch.Generator().manual_seed(SEED)
    x = torch.randn(T, H, generator=g, dtype=torch.float32)
    logits = torch.randn(T, E, generator=g, dtype=torch.float32)
    w13 = torch.randn(E, 2 * I, H, generator=g, dtype=torch.float32) * 0.02
    w2 = torch.randn(E, H, I, generator=g, dtype=torch.float32) * 0.02
    assert all(len(set(r.tolist())) == E for r in logits), "tie-free logits expected"

    p = torch.softmax(logits, -1)
    tw, ti = torch.topk(p, K, -1)
    tw = tw / tw.sum(-1, keepdim=True)

    # expert sort from torch.sort(stable=True) on the flat expert ids
    flat = ti.reshape(-1)
    order = torch.sort(flat, stable=True).indices
    cnt = torch.bincount(flat, minlength=E)
    padded = (cnt + BLOCK - 1) // BLOCK * BLOCK
    total = int(padded.sum())
    sorted_len = T * K + E * (BLOCK - 1)
    sorted_ids = torch.full((sorted_len,), -1, dtype=torch.int32)
    expert_ids = torch.zeros(((sorted_len + BLOCK - 1) // BLOCK,), dtype=torch.int32)
    src = dst = 0
    for e in range(E):
        c = int(cnt[e])
        sorted_ids[dst:dst + c] = order[src:src + c].to(torch.int32)
        expert_ids[dst // BLOCK:(dst + int(padded[e])) // BLOCK] = e
        src += c
        dst += int(padded[e])

    route = torch.zeros(T, E, dtype=torch.float64).scatter_(1, ti, tw.double())
    xd, w13d, w2d = x.double(), w13.double(), w2.double()
    gate = torch.einsum("th,eih->tei", xd, w13d[:, :I])
    up = torch.einsum("th,eih->tei", xd, w13d[:, I:])
    y = torch.einsum("tei,ehi->teh", torch.nn.functional.silu(gate) * up, w2d)
    out = (route.unsqueeze(-1) * y).sum(1).float()

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c1_seed0.npz")
    np.savez_compressed(path, x_sum=np.float64(x.double().sum()), topk_ids=ti.numpy().astype(np.int32),
                        topk_weights=tw.numpy(), sorted_token_ids=sorted_ids.numpy(),
                        expert_ids=expert_ids.numpy(), num_tokens_post_pad=np.array([total], np.int32),
                        out=out.numpy())
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
