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


def check(y, y_ref, dtype):
    y = y.float().cpu().numpy()
    if dtype == "float32":
        np.testing.assert_allclose(y, y_ref, rtol=1e-6, atol=1e-9)
        return
    # the kernel sums the squares in float32 in its own order, so rstd may differ in its last bit: a product next
    # to a rounding boundary then lands on the neighbouring value of the element type (for the module's two
    # roundings, and across a power of two where the spacing halves, that can read as two steps); rarely
    err = np.abs(y - y_ref)
    assert (err <= ulp(y_ref, dtype) * 2.2).all()
    assert (err > 0).mean() < 0.002


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
