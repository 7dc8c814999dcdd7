"""Pins the CPU oracle by means independent of its own formulas: hand-worked
cases, brute force, library routines (torch.softmax/topk/silu/sum), a dense
all-experts formulation of the layer, and the committed golden fixture that
tests/golden/make_golden.py wrote from torch library calls only."""
import itertools
import os

import numpy as np
import pytest
import torch

from oracle import c_oracle, moe_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "c1_seed0.npz")


# ---------------------------------------------------------------- router ----
def test_router_hand_worked_ties():
    # survey probe row: torch.topk does NOT return [0, 1] here; the rule does
    w, ids = O.topk_softmax(np.array([[1, 1, 1, 0, 1, 0, 0, 0]], np.float32), 2, True)
    assert ids.tolist() == [[0, 1]]
    assert w.tolist() == [[0.5, 0.5]]
    # max later in the row, runner-up tie between experts 1 and 5 -> 1
    _, ids = O.topk_softmax(np.array([[0, 2, -1, 3, 0, 2, 1, 1]], np.float32), 2, True)
    assert ids.tolist() == [[3, 1]]
    # all equal -> the two lowest indices, weights 1/8 without renormalisation
    w, ids = O.topk_softmax(np.zeros((1, 8), np.float32), 2, False)
    assert ids.tolist() == [[0, 1]] and np.allclose(w, 0.125)
    # known closed form: logits (ln 3, ln 1) + six -inf-like -> probs 3/4, 1/4
    row = np.full((1, 8), -1e30, np.float32)
    row[0, 6], row[0, 2] = np.log(3.0), 0.0
    w, ids = O.topk_softmax(row, 2, False)
    assert ids.tolist() == [[6, 2]] and np.allclose(w, [[0.75, 0.25]], atol=1e-7)


def test_router_brute_force_small_rows():
    # every row over {0,1,2}^4: top-2 must equal the first two of a stable
    # descending sort done by plain Python, and the reference's literal scan
    for row in itertools.product([0.0, 1.0, 2.0], repeat=4):
        expect = sorted(range(4), key=lambda i: (-row[i], i))[:2]
        _, ids = O.topk_softmax(np.array([row], np.float32), 2, True)
        assert ids[0].tolist() == expect
        assert list(O.topk_scan_loop(row)) == expect
        _, cids = c_oracle.topk_softmax(np.array([row], np.float32), 2, True)
        assert cids[0].tolist() == expect


@pytest.mark.parametrize("renorm", [False, True])
def test_router_matches_torch_library_on_tie_free_rows(renorm):
    g = torch.Generator().manual_seed(1)
    logits = torch.randn(4096, 8, generator=g)
    assert all(len(set(r.tolist())) == 8 for r in logits[:64])  # fp32 normals: no ties
    p = torch.softmax(logits, dim=-1)
    tw, ti = torch.topk(p, 2, dim=-1)
    if renorm:
        tw = tw / tw.sum(-1, keepdim=True)
    w, ids = O.topk_softmax(logits.numpy(), 2, renorm)
    assert np.array_equal(ids, ti.numpy().astype(np.int32))
    np.testing.assert_allclose(w, tw.numpy(), rtol=2e-6, atol=1e-8)
    cw, cids = c_oracle.topk_softmax(logits.numpy(), 2, renorm)
    assert np.array_equal(cids, ids)
    np.testing.assert_allclose(cw, w, rtol=2e-6, atol=1e-8)


def test_router_invariants_with_bf16_ties():
    g = torch.Generator().manual_seed(2)
    logits = torch.randn(20000, 8, generator=g).to(torch.bfloat16).float().numpy()
    w, ids = O.topk_softmax(logits, 2, True)
    assert ((ids >= 0) & (ids < 8)).all() and (ids[:, 0] != ids[:, 1]).all()
    np.testing.assert_allclose(w.sum(1), 1.0, atol=2e-7)
    assert (w[:, 0] >= w[:, 1]).all()
    l0 = np.take_along_axis(logits, ids[:, :1].astype(np.int64), 1)[:, 0]
    l1 = np.take_along_axis(logits, ids[:, 1:].astype(np.int64), 1)[:, 0]
    assert (l0 == logits.max(1)).all()
    tie = l0 == l1
    assert tie.sum() > 10                       # bf16 logits do tie
    assert (ids[tie, 0] < ids[tie, 1]).all()    # ... and ties resolve to the lower index
    _, cids = c_oracle.topk_softmax(logits, 2, True)
    assert np.array_equal(cids, ids)


# ----------------------------------------------------------------- align ----
def test_gate_logits_hand_worked_and_library():
    # hand-worked: two tokens, two experts, exact small integers
    x = np.array([[1.0, 2.0, -3.0, 0.5], [0.0, -1.0, 4.0, 2.0]], dtype=np.float32)
    w = np.array([[2.0, 0.0, 1.0, 4.0], [-1.0, 1.0, 0.5, -2.0]], dtype=np.float32)
    #   token 0: [2 + 0 - 3 + 2, -1 + 2 - 1.5 - 1] = [1, -1.5];  token 1: [0 + 0 + 4 + 8, 0 - 1 + 2 - 4] = [12, -3]
    np.testing.assert_array_equal(O.gate_logits(x, w, round_bf16=False), np.array([[1.0, -1.5], [12.0, -3.0]], np.float32))
    # library routine: float64 linear layer of torch, rounded once; and torch's own bf16 rounding of the result
    g = torch.Generator().manual_seed(3)
    xt = torch.randn(37, 256, generator=g).to(torch.bfloat16)
    wt = (torch.randn(8, 256, generator=g) * 0.05).to(torch.bfloat16)
    ref64 = torch.nn.functional.linear(xt.double(), wt.double())
    got = O.gate_logits(xt.float().numpy(), wt.float().numpy(), round_bf16=False)
    np.testing.assert_array_equal(got, ref64.float().numpy())
    got_bf = O.gate_logits(xt.float().numpy(), wt.float().numpy(), round_bf16=True)
    np.testing.assert_array_equal(got_bf, ref64.float().to(torch.bfloat16).float().numpy())
    # a transposed weight or a dropped element changes the result
    assert not np.array_equal(O.gate_logits(x, w[::-1], round_bf16=False), O.gate_logits(x, w, round_bf16=False))


def test_to_bf16_rounding_is_nearest_even():
    # 1 + 2^-8 is exactly between bf16 1.0 and 1.0078125 -> even mantissa (1.0); 1 + 3 * 2^-8 -> 1.015625
    a = np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, -(1.0 + 2.0 ** -8), 3.0e38, 1e-40], dtype=np.float32)
    want = torch.from_numpy(a).to(torch.bfloat16).float().numpy()
    np.testing.assert_array_equal(O.to_bf16_f32(a), want)
    assert O.to_bf16_f32(a)[0] == 1.0 and O.to_bf16_f32(a)[1] == 1.015625


def test_align_hand_worked():
    # slots 0..5 -> experts [2,0,2,1,0,2], E=3, block 2:
    # counts 2,1,3 -> padded 2,2,4 -> offsets 0,2,4, total 8
    s, e, n = O.moe_align_block_size(np.array([2, 0, 2, 1, 0, 2]), 3, 2)
    assert n.tolist() == [8]
    assert s.tolist() == [1, 4, 3, -1, 0, 2, 5, -1, -1]      # length 6 + 3*(2-1) = 9
    assert e.tolist() == [0, 1, 2, 2, 0]                       # length cdiv(9, 2) = 5
    # T=1, top-2 -> experts (5, 3), E=8, block 16: lengths 122 / 8 as in the wrapper
    s, e, n = O.moe_align_block_size(np.array([[5, 3]]), 8, 16)
    assert s.size == 122 and e.size == 8 and n.tolist() == [32]
    assert s[0] == 1 and s[16] == 0 and (np.delete(s, [0, 16]) == -1).all()
    assert e.tolist() == [3, 5, 0, 0, 0, 0, 0, 0]


@pytest.mark.parametrize("numel,E,block", [(0, 8, 16), (2, 8, 16), (7, 3, 4), (64, 8, 16), (129, 8, 64),
                                           (300, 5, 1), (1000, 64, 8)])
def test_align_vectorised_equals_sequential_loop_and_c(numel, E, block):
    rng = np.random.default_rng(numel * 131 + E)
    ids = rng.integers(0, E, size=numel)
    a = O.moe_align_block_size(ids, E, block)
    b = O.moe_align_block_size_loop(ids, E, block)
    c = c_oracle.moe_align_block_size(ids, E, block)
    for x, y, z in zip(a, b, c):
        assert np.array_equal(x, y) and np.array_equal(x, z)


def check_align_invariants(ids, E, block, sorted_ids, expert_ids, post_pad):
    """Structural properties that fix the result uniquely (also used at full size on the GPU)."""
    flat = np.asarray(ids).reshape(-1)
    n = int(post_pad[0])
    cnt = np.bincount(flat, minlength=E)
    assert n == int((-(-cnt // block) * block).sum())
    assert n % block == 0 and n <= sorted_ids.size
    assert (sorted_ids[n:] == -1).all() and (expert_ids[n // block:] == 0).all()
    body = sorted_ids[:n]
    real = body[body >= 0]
    assert np.array_equal(np.sort(real), np.arange(flat.size))           # a permutation of all slots
    blk_expert = np.repeat(expert_ids[:n // block], block)
    assert np.array_equal(flat[real], blk_expert[body >= 0])            # every slot in its expert's block
    assert (np.diff(blk_expert) >= 0).all()                              # experts ascending
    for e in range(E):                                                    # stable + pads at segment end
        seg = body[blk_expert == e]
        k = int(cnt[e])
        assert (seg[:k] >= 0).all() and (seg[k:] == -1).all() and (np.diff(seg[:k]) > 0).all()


def test_align_invariants_and_special_cases():
    rng = np.random.default_rng(7)
    for ids, E, block in [(rng.integers(0, 8, 16384), 8, 64), (rng.integers(0, 2, 4096), 8, 64),
                          (np.full(100, 7), 8, 16), (np.array([3, 3]), 8, 16)]:
        check_align_invariants(ids, E, block, *O.moe_align_block_size(ids, E, block))
    # all tokens to experts {0,1}: two segments, six empty experts, no blocks for them
    ids = np.tile(np.array([0, 1]), 4096)
    s, e, n = O.moe_align_block_size(ids, 8, 64)
    assert n[0] == 8192 and set(e[:128].tolist()) == {0, 1} and (e[128:] == 0).all()
    assert np.array_equal(s[:4096], np.arange(0, 8192, 2)) and np.array_equal(s[4096:8192], np.arange(1, 8192, 2))


def test_align_buffer_lengths_match_reference_table():
    # (T, block) -> lengths listed for the wrapper's sizing rule numel + E*(B-1), cdiv(., B)
    for T, B, sl, el in [(1, 16, 122, 8), (8, 16, 136, 9), (32, 64, 568, 9), (64, 64, 632, 10),
                         (256, 64, 1016, 16), (4096, 64, 8696, 136), (8192, 64, 16888, 264)]:
        assert O.align_buffer_sizes(T * 2, 8, B) == (sl, el)
    assert O.get_moe_config(8, 8)["BLOCK_SIZE_M"] == 16 and O.get_moe_config(9, 8)["BLOCK_SIZE_M"] == 64


# ----------------------------------------------------------- element-wise ----
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-6), (torch.bfloat16, 1.6e-2), (torch.float16, 2e-3)])
def test_silu_and_mul_against_library(dtype, tol):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(33, 2 * 96, generator=g).to(dtype)
    ref = torch.nn.functional.silu(x[:, :96].float()) * x[:, 96:].float()
    got = O.silu_and_mul(x).float()
    assert got.dtype == torch.float32 and got.shape == (33, 96)
    assert ((got - ref).abs() <= tol * ref.abs() + 1e-6).all()
    # closed forms: silu(0) = 0; silu(x) -> x for large x
    z = torch.tensor([[0.0, 20.0, 3.0, 5.0]], dtype=dtype)
    assert torch.equal(O.silu_and_mul(z).float(), torch.tensor([[0.0, 100.0]]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_moe_sum_against_library(dtype):
    g = torch.Generator().manual_seed(4)
    x = torch.randn(17, 2, 40, generator=g).to(dtype)
    # for two addends one rounding of the exact sum is the definition
    assert torch.equal(O.moe_sum(x), (x[:, 0].float() + x[:, 1].float()).to(dtype))
    if dtype == torch.float32:
        assert torch.allclose(O.moe_sum(x), torch.sum(x, dim=1))


# ------------------------------------------------------------------ layer ----
def dense_layer(x, logits, w13, w2, topk=2):
    """Independent formulation: every expert on every token, mixed by a dense
    routing matrix built from torch.softmax + torch.topk (tie-free inputs only)."""
    T, H = x.shape
    E, two_i, _ = w13.shape
    I = two_i // 2
    p = torch.softmax(logits.float(), -1)
    tw, ti = torch.topk(p, topk, -1)
    tw = tw / tw.sum(-1, keepdim=True)
    route = torch.zeros(T, E).scatter_(1, ti, tw)
    g = torch.einsum("th,eih->tei", x.float(), w13[:, :I].float())
    u = torch.einsum("th,eih->tei", x.float(), w13[:, I:].float())
    y = torch.einsum("tei,ehi->teh", torch.nn.functional.silu(g) * u, w2.float())
    return (route.unsqueeze(-1) * y).sum(1)


def test_layer_fp32_equals_dense_formulation():
    x, lg, w13, w2 = O.make_inputs(40, 64, 96, E=8, seed=5, dtype=torch.float32)
    got = O.moe_layer_fp32(x, lg, w13, w2)
    ref = dense_layer(x, lg, w13, w2)
    assert torch.allclose(got, ref, rtol=1e-5, atol=1e-6)
    # a transposed w2 or swapped gate/up would not survive this
    swapped = torch.cat([w13[:, 96:], w13[:, :96]], 1)
    assert not torch.allclose(O.moe_layer_fp32(x, lg, swapped, w2), ref, rtol=1e-3, atol=1e-4)


def test_layer_one_hot_routing_reduces_to_swiglu_mlp():
    x, lg, w13, w2 = O.make_inputs(9, 32, 48, E=4, seed=6, dtype=torch.float32)
    lg = torch.full_like(lg, -50.0)
    lg[:, 2] = 50.0           # expert 2 takes weight 1 - O(e^-100); the runner-up contributes nothing
    got = O.moe_layer_fp32(x, lg, w13, w2)
    mlp = (torch.nn.functional.silu(x @ w13[2, :48].t()) * (x @ w13[2, 48:].t())) @ w2[2].t()
    assert torch.allclose(got, mlp, rtol=1e-5, atol=1e-7)


def test_layer_is_token_wise():
    x, lg, w13, w2 = O.make_inputs(16, 32, 48, E=8, seed=8, dtype=torch.float32)
    full = O.moe_layer_fp32(x, lg, w13, w2)
    part = O.moe_layer_fp32(x[5:9], lg[5:9], w13, w2)
    assert torch.allclose(full[5:9], part, rtol=1e-6, atol=1e-7)


def test_staged_bf16_pipeline_tracks_fp32_definition():
    x, lg, w13, w2 = O.make_inputs(32, 128, 256, E=8, seed=9)
    ref = O.moe_layer_fp32(x, lg, w13, w2)
    st = O.moe_layer_staged_bf16(x, lg, w13, w2)
    err = (st["out"].float() - ref).abs().mean() / ref.abs().mean()
    assert err < 1e-2
    assert st["cache1"].shape == (32, 2, 512) and st["cache2"].shape == (32, 2, 256)


def test_golden_fixture_c1():
    """Config 1 (T=64, H=256, I=512, E=8, fp32, seed 0): routing and output written
    by tests/golden/make_golden.py from torch library calls on tie-free inputs."""
    gold = np.load(GOLDEN)
    x, lg, w13, w2 = O.make_inputs(64, 256, 512, E=8, seed=0, dtype=torch.float32)
    assert abs(float(x.double().sum()) - float(gold["x_sum"])) < 1e-6
    w, ids = O.topk_softmax(lg.numpy(), 2, True)
    assert np.array_equal(ids, gold["topk_ids"])
    np.testing.assert_allclose(w, gold["topk_weights"], rtol=2e-6)
    s, e, n = O.moe_align_block_size(ids, 8, 64)
    assert np.array_equal(s, gold["sorted_token_ids"]) and np.array_equal(e, gold["expert_ids"])
    assert np.array_equal(n, gold["num_tokens_post_pad"])
    out = O.moe_layer_fp32(x, lg, w13, w2).numpy()
    np.testing.assert_allclose(out, gold["out"], rtol=1e-4, atol=1e-6)


# ----------------------------------------------------------------------------
# RMSNorm (the step in front of the MoE block)
# ----------------------------------------------------------------------------
_TORCH_DT = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}


def _ulp(v, dtype):
    bits = {"float32": 23, "bfloat16": 7, "float16": 10}[dtype]
    return 2.0 ** (np.floor(np.log2(np.maximum(np.abs(v), 2.0 ** -14))) - bits)


def _layer_chain(x, residual, weight, eps):
    """The reference module's own op chains (layers/layernorm.py:17-41), run by torch on the CPU."""
    orig = x.dtype
    if residual is None:
        xf = x.to(torch.float32)
        var = xf.pow(2).mean(dim=-1, keepdim=True)
        xf = xf * torch.rsqrt(var + eps)
        return xf.to(orig).mul_(weight), None
    xf = x.to(torch.float32).add_(residual.to(torch.float32))
    res = xf.to(orig)
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    xf = xf * torch.rsqrt(var + eps)
    return xf.to(orig).mul_(weight), res


def _op_chain(x, residual, weight, eps):
    """The native op's arithmetic (src/add_rms_norm.hip:47-52,76-80) written with torch library ops."""
    r = x if residual is None else (x + residual)           # add in the element type: one rounding
    var = r.to(torch.float32).pow(2).mean(dim=-1, keepdim=True)
    y = (r.to(torch.float32) * weight.to(torch.float32) * torch.rsqrt(var + eps)).to(x.dtype)
    return y, (None if residual is None else r)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16"])
@pytest.mark.parametrize("semantics", ["layer", "op"])
@pytest.mark.parametrize("with_residual", [False, True])
def test_rms_norm_matches_the_references_torch_chains(dtype, semantics, with_residual):
    g = torch.Generator().manual_seed(5)
    T, H, eps = 37, 512, 1e-5
    x = torch.randn(T, H, generator=g).to(_TORCH_DT[dtype])
    res = torch.randn(T, H, generator=g).to(_TORCH_DT[dtype]) if with_residual else None
    w = (1.0 + 0.1 * torch.randn(H, generator=g)).to(_TORCH_DT[dtype])
    chain = _layer_chain if semantics == "layer" else _op_chain
    y_ref, res_ref = chain(x.clone(), None if res is None else res.clone(), w, eps)
    out = O.rms_norm(x.float().numpy(), w.float().numpy(), eps, None if res is None else res.float().numpy(),
                     semantics=semantics, dtype=dtype)
    y, res_out = (out, None) if res is None else out
    if with_residual:
        np.testing.assert_array_equal(res_out, res_ref.float().numpy())       # one float32 add, one rounding: exact
    # the variance is summed in a different order (float64 here, float32 in the library): the results may sit on
    # neighbouring values of the element type where a product falls next to a rounding boundary
    if dtype == "float32":   # nothing is rounded to a coarser type: a few float32 steps from rstd and the products
        np.testing.assert_allclose(y, y_ref.numpy(), rtol=6e-7, atol=1e-9)
        return
    err = np.abs(y - y_ref.float().numpy())
    assert (err <= _ulp(y_ref.float().numpy(), dtype) * 1.0001).all()
    assert (err > 0).mean() < 0.01


def test_rms_norm_exact_small_cases():
    # var = 4, rstd = 1/2 exactly: y = w
    w = np.array([1.0, 2.0, 0.5, -1.0], dtype=np.float32)
    y = O.rms_norm(np.full((1, 4), 2.0, np.float32), w, 0.0)
    np.testing.assert_array_equal(y, w[None])
    # residual add first: 1 + 1 = 2, same result, residual_out = 2
    for sem in ("layer", "op"):
        y, r = O.rms_norm(np.ones((1, 4), np.float32), w, 0.0, np.ones((1, 4), np.float32), semantics=sem)
        np.testing.assert_array_equal(y, w[None])
        np.testing.assert_array_equal(r, np.full((1, 4), 2.0, np.float32))
    # eps matters: x = 0 gives 0, not NaN, as long as eps > 0
    assert np.all(O.rms_norm(np.zeros((2, 8), np.float32), np.ones(8, np.float32), 1e-5) == 0.0)
    # 3-4-5: mean square of (3, 4) is 12.5; y = x / sqrt(12.5) in float32
    y = O.rms_norm(np.array([[3.0, 4.0]], np.float32), np.ones(2, np.float32), 0.0, dtype="float32")
    np.testing.assert_allclose(y, np.array([[3.0, 4.0]]) / np.sqrt(12.5), rtol=2e-7)


@pytest.mark.parametrize("semantics", ["layer", "op"])
def test_rms_norm_power_of_two_scale_invariance(semantics):
    # with eps = 0 a scaling of the input by 2^k changes nothing, bit for bit; a scaling of the weight scales the output
    rng = np.random.default_rng(3)
    x = O.to_bf16_f32(rng.standard_normal((9, 256)).astype(np.float32))
    r = O.to_bf16_f32(rng.standard_normal((9, 256)).astype(np.float32))
    w = O.to_bf16_f32((1 + 0.1 * rng.standard_normal(256)).astype(np.float32))
    y0, r0 = O.rms_norm(x, w, 0.0, r, semantics=semantics)
    y1, r1 = O.rms_norm(x * 8, w, 0.0, r * 8, semantics=semantics)
    np.testing.assert_array_equal(y0, y1)
    np.testing.assert_array_equal(r0 * 8, r1)
    y2, _ = O.rms_norm(x, w * 4, 0.0, r, semantics=semantics)
    np.testing.assert_array_equal(y0 * 4, y2)
    # unit weight: every row of the (float32) result has mean square 1
    y = O.rms_norm(x, np.ones(256, np.float32), 0.0, dtype="float32")
    np.testing.assert_allclose((y.astype(np.float64) ** 2).mean(-1), 1.0, rtol=1e-6)


def test_rms_norm_rounding_conventions_differ_where_expected():
    # x + residual = 1 + 2^-8 is not a bf16 value: the layer keeps it for the variance and the product, the op
    # rounds it to 1 first
    x = np.array([[1.0, 3.0]], np.float32)
    r = np.array([[2.0 ** -8, 0.0]], np.float32)
    w = np.ones(2, np.float32)
    (yl, rl), (yo, ro) = (O.rms_norm(x, w, 0.0, r, semantics=s, dtype="float32") for s in ("layer", "op"))
    np.testing.assert_array_equal(rl, x + r)          # float32 element type: nothing is rounded
    (ylb, rlb), (yob, rob) = (O.rms_norm(x, w, 0.0, r, semantics=s, dtype="bfloat16") for s in ("layer", "op"))
    np.testing.assert_array_equal(rlb, np.array([[1.0, 3.0]], np.float32))   # both return the rounded sum
    np.testing.assert_array_equal(rob, rlb)
    # layer: var = ((1 + 2^-8)^2 + 9) / 2 ; op: var = (1 + 9) / 2 = 5 exactly
    np.testing.assert_allclose(yob[0, 1], O.to_bf16_f32(np.float32(3.0 / np.sqrt(5.0))), rtol=0)
    # double against single rounding: s * rstd = 1 + 2^-8 (a tie, rounds to 1), weight 1.5
    s = np.array([[1.0 + 2.0 ** -8, 1.0 + 2.0 ** -8]], np.float32)
    eps = float(np.float32(1.0) - (s.astype(np.float64) ** 2).mean().astype(np.float32))  # makes var + eps = 1
    w15 = np.full(2, 1.5, np.float32)
    yl2 = O.rms_norm(s, w15, eps, dtype="bfloat16", semantics="layer")
    yo2 = O.rms_norm(s, w15, eps, dtype="bfloat16", semantics="op")
    np.testing.assert_array_equal(yl2, np.full((1, 2), 1.5, np.float32))          # T(T(1.0039) * 1.5) = 1.5
    np.testing.assert_array_equal(yo2, np.full((1, 2), 1.5078125, np.float32))    # T(1.0039 * 1.5) = 1.5078125
