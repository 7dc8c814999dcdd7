"""GPU parity of RMSNorm / residual add + RMSNorm (em_rms_norm, em_add_rms_norm) against the oracle,
for the rounding points of the model's module (layers/layernorm.py:17-41) and of the native op
(src/add_rms_norm.hip:24-84,87-140)."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.gpu_util import DEV, announce

pytestmark = pytest.mark.gpu

_DT = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}
_BITS = {"float32": 23, "bfloat16": 7, "float16": 10}


def ulp(v, dtype):
    return 2.0 ** (np.floor(np.log2(np.maximum(np.abs(v), 2.0 ** -14))) - _BITS[dtype])


def inputs(T, H, dtype, seed, w32=False):
    g = torch.Generator(device=DEV).manual_seed(seed)
    x = torch.randn(T, H, generator=g, device=DEV).to(_DT[dtype])
    r = (2.0 * torch.randn(T, H, generator=g, device=DEV)).to(_DT[dtype])
    w = (1.0 + 0.1 * torch.randn(H, generator=g, device=DEV)).to(torch.float32 if w32 else _DT[dtype])
    return x, r, w


def check(y, y_ref, dtype, wmax=1.5):
    y = y.float().cpu().numpy()
    if dtype == "float32":
        np.testing.assert_allclose(y, y_ref, rtol=1e-6, atol=1e-9)
        return
    # the kernel sums the squares in float32 in its own order, so rstd may differ in its last bit: a product next
    # to a rounding boundary then lands on the neighbouring value of the element type.  With the module's two
    # roundings one step of the first, times the weight (|w| <= wmax), can read as 2 * wmax steps of a result
    # that sits below a power of two, where the spacing halves; rarely
    err = np.abs(y - y_ref)
    assert (err <= ulp(y_ref, dtype) * (2 * wmax + 0.6)).all()
    assert (err > 0).sum() <= max(2, 0.002 * err.size)


@pytest.mark.parametrize("dtype", ["bfloat16", "float16", "float32"])
@pytest.mark.parametrize("T,H", [(1, 4096), (7, 4096), (64, 4096), (2048, 4096), (33, 6144), (5, 1000), (3, 8192), (2, 16384)])
@pytest.mark.parametrize("w32", [False, True])
def test_module_semantics_match_oracle(dtype, T, H, w32):
    from electrock_infer_amd import RMSNorm
    if dtype == "float32" and H > 8192:
        pytest.skip("float32 rows are limited to 8192 elements")
    announce(f"RMSNorm module dtype={dtype} T={T} H={H} w32={w32}")
    x, r, w = inputs(T, H, dtype, T + H, w32 or dtype == "float32")
    m = RMSNorm(H, eps=1e-5).to(DEV)
    m.weight.data = w
    x0, r0 = x.clone(), r.clone()
    y = m(x)
    y2, res = m(x, r)
    torch.cuda.synchronize()
    assert torch.equal(x, x0) and torch.equal(r, r0)             # the module leaves its inputs alone
    xn, rn, wn = x.float().cpu().numpy(), r.float().cpu().numpy(), w.float().cpu().numpy()
    check(y, O.rms_norm(xn, wn, 1e-5, dtype=dtype), dtype)
    y_ref, res_ref = O.rms_norm(xn, wn, 1e-5, rn, dtype=dtype)
    np.testing.assert_array_equal(res.float().cpu().numpy(), res_ref)   # one add, one rounding: exact
    check(y2, y_ref, dtype)


@pytest.mark.parametrize("dtype", ["bfloat16", "float16", "float32"])
@pytest.mark.parametrize("T,H", [(1, 4096), (100, 4096), (19, 2048)])
def test_op_semantics_in_place_match_oracle(dtype, T, H):
    from electrock_infer_amd import _C
    announce(f"_C.rms_norm / add_rms_norm dtype={dtype} T={T} H={H}")
    x, r, w = inputs(T, H, dtype, 7 * T + H)
    xn, rn, wn = x.float().cpu().numpy(), r.float().cpu().numpy(), w.float().cpu().numpy()
    a = x.clone()
    _C.rms_norm(a, 1e-5, w)
    check(a, O.rms_norm(xn, wn, 1e-5, semantics="op", dtype=dtype), dtype)
    a, b = x.clone(), r.clone()
    _C.add_rms_norm(a, b, 1e-5, w)
    y_ref, res_ref = O.rms_norm(xn, wn, 1e-5, rn, semantics="op", dtype=dtype)
    np.testing.assert_array_equal(b.float().cpu().numpy(), res_ref)
    check(a, y_ref, dtype)


def test_rounding_conventions_are_distinct_on_the_gpu():
    from electrock_infer_amd import RMSNorm, _C
    announce("RMSNorm rounding conventions")
    # s * rstd = 1 + 2^-8 (a bf16 tie, rounds to 1), weight 1.5: the module gives T(T(.) * 1.5) = 1.5,
    # the op T(. * 1.5) = 1.5078125
    s = np.full((4, 8), 1.0 + 2.0 ** -8, np.float32)
    eps = float(np.float32(1.0) - (s.astype(np.float64) ** 2).mean().astype(np.float32))
    x = torch.ones(4, 8, device=DEV, dtype=torch.bfloat16)
    r = torch.full((4, 8), 2.0 ** -8, device=DEV, dtype=torch.bfloat16)
    w = torch.full((8,), 1.5, device=DEV, dtype=torch.bfloat16)
    m = RMSNorm(8, eps=eps).to(DEV)
    m.weight.data = w
    y, res = m(x, r)
    assert (y.float() == 1.5).all() and (res.float() == 1.0).all()
    # the op rounds the sum first: everything is 1.0, var + eps = 1 - 2^-7 or so, product 1.5 * rstd
    a, b = x.clone(), r.clone()
    _C.add_rms_norm(a, b, eps, w)
    y_ref, _ = O.rms_norm(np.ones((4, 8), np.float32), np.full(8, 1.5, np.float32), eps,
                          np.full((4, 8), 2.0 ** -8, np.float32), semantics="op")
    np.testing.assert_array_equal(a.float().cpu().numpy(), y_ref)
    assert not torch.equal(a, y)


def test_norm_rejects_what_it_cannot_do():
    from electrock_infer_amd import RMSNorm, _C
    announce("RMSNorm argument checks")
    m = RMSNorm(4096).to(DEV)
    with pytest.raises(RuntimeError):
        m(torch.zeros(2, 4096))                                            # CPU tensor: there is no CPU path
    with pytest.raises(RuntimeError):
        m(torch.zeros(2, 2048, device=DEV, dtype=torch.bfloat16))          # wrong hidden size
    with pytest.raises(RuntimeError):
        _C.rms_norm(torch.zeros(2, 4100, device=DEV, dtype=torch.bfloat16), 1e-5,
                    torch.ones(4100, device=DEV, dtype=torch.bfloat16))    # not a multiple of 8
    with pytest.raises(RuntimeError):
        _C.rms_norm(torch.zeros(2, 32768, device=DEV, dtype=torch.bfloat16), 1e-5,
                    torch.ones(32768, device=DEV, dtype=torch.bfloat16))   # row too long for one workgroup
    assert m(torch.zeros(0, 4096, device=DEV, dtype=torch.bfloat16)).shape == (0, 4096)


# ----------------------------------------------------------------------------
# RMSNorm + gate + router in one launch, and the decoder layer's tail in one call
# ----------------------------------------------------------------------------
def _gate_w(E, H, seed):
    g = torch.Generator(device=DEV).manual_seed(99 + seed)
    return (torch.randn(E, H, generator=g, device=DEV) * 0.05).to(torch.bfloat16)


@pytest.mark.parametrize("T,H,E", [(1, 4096, 8), (16, 4096, 8), (100, 4096, 8), (2048, 4096, 8), (40, 6144, 8),
                                   (33, 1000, 8), (50, 2048, 16)])
@pytest.mark.parametrize("with_residual", [True, False])
@pytest.mark.parametrize("w32", [False, True])
@pytest.mark.parametrize("op_rounding", [False, True])
def test_norm_gate_topk_matches_oracle(T, H, E, with_residual, w32, op_rounding):
    from electrock_infer_amd import norm_gate_topk
    announce(f"norm_gate_topk T={T} H={H} E={E} residual={with_residual} w32={w32} op={op_rounding}")
    x, r, w = inputs(T, H, "bfloat16", 3 * T + H, w32)
    gw = _gate_w(E, H, T)
    x0, r0 = x.clone(), r.clone()
    h, res, tw, ids, logits = norm_gate_topk(x, r if with_residual else None, w, 1e-5, gw, 2, return_logits=True,
                                             op_rounding=op_rounding)
    torch.cuda.synchronize()
    assert torch.equal(x, x0) and torch.equal(r, r0)
    sem = "op" if op_rounding else "layer"
    xn, rn, wn = x.float().cpu().numpy(), r.float().cpu().numpy(), w.float().cpu().numpy()
    if with_residual:
        h_ref, res_ref = O.rms_norm(xn, wn, 1e-5, rn, semantics=sem)
        np.testing.assert_array_equal(res.float().cpu().numpy(), res_ref)
    else:
        h_ref = O.rms_norm(xn, wn, 1e-5, semantics=sem)
        assert res is None
    check(h, h_ref, "bfloat16")
    # logits and routing on the rows the kernel itself wrote
    hn = h.float().cpu().numpy()
    lg_ref = O.gate_logits(hn, gw.float().cpu().numpy())
    lg = logits.float().cpu().numpy()
    sum_abs = np.abs(hn).astype(np.float64) @ np.abs(gw.float().cpu().numpy()).astype(np.float64).T
    err = np.abs(lg - lg_ref)
    bf16_step = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(lg_ref), 2.0 ** -126))) - 7)
    assert (err <= bf16_step * (1.0 + 1e-6) + 4 * 2.0 ** -24 * sum_abs).all()
    w_ref, ids_ref = O.topk_softmax(lg, 2, True)
    np.testing.assert_array_equal(ids.cpu().numpy(), ids_ref)
    np.testing.assert_allclose(tw.cpu().numpy(), w_ref, rtol=3e-6, atol=1e-7)


@pytest.mark.parametrize("T", [1, 64, 300, 2048])
def test_decoder_tail_in_one_call_matches_the_steps(T):
    from electrock_infer_amd import fused_experts, fused_experts_normed, norm_gate_topk
    from tests.gpu_util import error_stats, gpu_inputs
    announce(f"fused_experts_normed T={T}")
    H, I, E = 512, 1024, 8
    x, _, w13, w2 = gpu_inputs(T, H, I, E, seed=T)
    g = torch.Generator(device=DEV).manual_seed(T)
    r = torch.randn(T, H, generator=g, device=DEV).to(torch.bfloat16)
    nw = (1.0 + 0.1 * torch.randn(H, generator=g, device=DEV)).to(torch.bfloat16)
    gw = _gate_w(E, H, T)
    out, res = fused_experts_normed(x, r, nw, 1e-5, gw, w13, w2, topk=2, out_dtype=torch.float32)
    h, res2, _, _, logits = norm_gate_topk(x, r, nw, 1e-5, gw, 2, return_logits=True)
    assert torch.equal(res, res2)
    out2 = fused_experts(h, w13, w2, logits, topk=2, renormalize=True, out_dtype=torch.float32)
    assert torch.equal(out, out2)          # same kernels on the same rows and logits
    ref = O.moe_layer_fp32(h.cpu(), logits.cpu(), w13.cpu(), w2.cpu())
    st = error_stats(out, ref)
    assert st["mean_rel"] <= 2.5e-3 and st["max_abs"] <= 4e-3 * float(ref.abs().max()), st
    # bf16 result: written over the normalised rows
    out_b, _ = fused_experts_normed(x, r, nw, 1e-5, gw, w13, w2, topk=2)
    assert out_b.dtype == torch.bfloat16
    assert error_stats(out_b, ref)["mean_rel"] <= 3.5e-3


def test_post_attention_module():
    from electrock_infer_amd import MixtralMoE, PostAttentionMoE, RMSNorm
    announce("PostAttentionMoE module")
    T, H, I, E = 40, 256, 512, 8
    torch.manual_seed(1)
    norm = RMSNorm(H, eps=1e-5).to(DEV).to(torch.bfloat16)
    norm.weight.data = (1.0 + 0.1 * torch.randn(H)).to(torch.bfloat16).to(DEV)
    moe = MixtralMoE(E, 2, H, I, params_dtype=torch.bfloat16).to(DEV)
    moe.gate.weight.data = (torch.randn(E, H) * 0.05).to(torch.bfloat16).to(DEV)
    moe.experts.w13_weight.data = (torch.randn(E, 2 * I, H) * 0.02).to(torch.bfloat16).to(DEV)
    moe.experts.w2_weight.data = (torch.randn(E, H, I) * 0.02).to(torch.bfloat16).to(DEV)
    tail = PostAttentionMoE(norm, moe)
    x = torch.randn(4, 10, H, device=DEV).to(torch.bfloat16)
    r = torch.randn(4, 10, H, device=DEV).to(torch.bfloat16)
    y, res = tail(x, r)
    # the two lines of the reference's decoder layer, step by step
    h2, res2 = norm(x, r)
    y2 = moe(h2.clone())
    assert y.shape == x.shape and res.shape == x.shape
    assert torch.equal(res, res2)
    d = (y.float() - y2.float()).abs()
    assert float(d.mean()) <= 2e-3 * float(y2.float().abs().mean()) + 1e-6
