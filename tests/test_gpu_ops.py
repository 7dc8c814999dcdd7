"""GPU parity of the four `_C` ops against the CPU oracle, through the C ABI.
Integer outputs are compared bit for bit; float outputs within the tolerance
written at each assert."""
import numpy as np
import pytest
import torch

from electrock_infer_amd import _C, _lib, fused_topk, moe_align_block_size
from oracle import c_oracle, moe_oracle as O
from tests.gpu_util import DEV, announce
from tests.test_oracle import check_align_invariants

pytestmark = pytest.mark.gpu


# ---------------------------------------------------------------- router ----
@pytest.mark.parametrize("T", [1, 3, 64, 257, 8192])
def test_topk_softmax_op_fp32(T):
    announce(f"topk_softmax op T={T}")
    g = torch.Generator().manual_seed(T)
    logits = torch.randn(T, 8, generator=g)
    w = torch.full((T, 2), -7.0, device=DEV)
    ids = torch.full((T, 2), -7, dtype=torch.int32, device=DEV)
    assert _C.topk_softmax(w, ids, logits.to(DEV)) is None
    ow, oids = O.topk_softmax(logits.numpy(), 2, False)
    assert np.array_equal(ids.cpu().numpy(), oids)
    np.testing.assert_allclose(w.cpu().numpy(), ow, rtol=2e-6, atol=1e-9)   # fp32 exp/div: a few ulp


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("renorm", [True, False])
def test_fused_topk_ties_go_to_lowest_index(dtype, renorm):
    announce(f"fused_topk ties dtype={dtype} renorm={renorm}")
    g = torch.Generator().manual_seed(11)
    logits = torch.randn(30000, 8, generator=g).to(dtype)
    logits[:4] = torch.tensor([[1, 1, 1, 0, 1, 0, 0, 0], [0, 0, 0, 0, 0, 0, 0, 0], [0, 2, -1, 3, 0, 2, 1, 1],
                               [-3, -3, -3, -3, -3, -3, -3, 5]]).to(dtype)
    w, ids = fused_topk(torch.empty(30000, 1), logits.to(DEV), 2, renorm)
    ow, oids = O.topk_softmax(logits.float().numpy(), 2, renorm)
    assert ids.dtype == torch.int32 and w.dtype == torch.float32
    assert ids[:4].cpu().tolist() == [[0, 1], [0, 1], [3, 1], [7, 0]]
    assert np.array_equal(ids.cpu().numpy(), oids)
    np.testing.assert_allclose(w.cpu().numpy(), ow, rtol=2e-6, atol=1e-9)
    if dtype == torch.bfloat16:
        l = logits.float().numpy()
        tied = np.take_along_axis(l, oids[:, :1].astype(np.int64), 1) == np.take_along_axis(l, oids[:, 1:].astype(np.int64), 1)
        assert tied.sum() > 50      # the case the rule exists for is really exercised


@pytest.mark.parametrize("E,k", [(8, 1), (8, 4), (5, 2), (64, 2), (64, 8), (1, 1)])
def test_router_general_E_k(E, k):
    announce(f"router E={E} k={k}")
    g = torch.Generator().manual_seed(E * 10 + k)
    logits = torch.randn(777, E, generator=g).to(torch.bfloat16)
    w, ids = fused_topk(torch.empty(777, 1), logits.to(DEV), k, True)
    ow, oids = c_oracle.topk_softmax(logits.float().numpy(), k, True)
    assert np.array_equal(ids.cpu().numpy(), oids)
    np.testing.assert_allclose(w.cpu().numpy(), ow, rtol=4e-6, atol=1e-9)


def test_topk_softmax_op_rejects_what_the_reference_rejects():
    w = torch.empty(4, 2, device=DEV)
    ids = torch.empty(4, 2, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="num_experts=8"):
        _C.topk_softmax(w, ids, torch.zeros(4, 16, device=DEV))
    with pytest.raises(RuntimeError, match="top_k=2"):
        _C.topk_softmax(torch.empty(4, 3, device=DEV), torch.empty(4, 3, dtype=torch.int32, device=DEV),
                        torch.zeros(4, 8, device=DEV))
    with pytest.raises(RuntimeError):
        _C.topk_softmax(w, ids, torch.zeros(4, 8, device=DEV, dtype=torch.bfloat16))


# ----------------------------------------------------------------- align ----
ALIGN_CASES = [(1, 16), (8, 16), (32, 64), (64, 64), (256, 64), (4096, 64), (8192, 64), (32768, 64), (100, 128),
               (7, 1)]


@pytest.mark.parametrize("T,block", ALIGN_CASES)
def test_align_random_bit_exact(T, block):
    announce(f"align T={T} block={block}")
    rng = np.random.default_rng(T * 7 + block)
    ids = rng.integers(0, 8, size=(T, 2)).astype(np.int32)
    s, e, n = moe_align_block_size(torch.from_numpy(ids).to(DEV), block, 8)
    os_, oe, on = c_oracle.moe_align_block_size(ids, 8, block)
    assert s.dtype == e.dtype == n.dtype == torch.int32
    assert s.numel() == os_.size and e.numel() == oe.size           # the wrapper's buffer sizes
    assert np.array_equal(n.cpu().numpy(), on)
    assert np.array_equal(e.cpu().numpy(), oe)
    assert np.array_equal(s.cpu().numpy(), os_)
    check_align_invariants(ids, 8, block, s.cpu().numpy(), e.cpu().numpy(), n.cpu().numpy())


@pytest.mark.parametrize("name", ["two_experts", "one_expert", "empty_middle", "zipf", "reference_test_shape"])
def test_align_skewed_and_degenerate(name):
    announce(f"align case {name}")
    rng = np.random.default_rng(5)
    E, block = 8, 64
    if name == "two_experts":
        ids = np.tile(np.array([0, 1], np.int32), 8192)
    elif name == "one_expert":
        ids = np.full(3000, 7, np.int32)
    elif name == "empty_middle":
        ids = rng.choice(np.array([0, 2, 7], np.int32), size=5000)
    elif name == "zipf":
        p = np.arange(1, 9) ** -1.2
        ids = rng.choice(8, size=16384, p=p / p.sum()).astype(np.int32)
    else:  # the reference's own test input shape: 65536 tokens x top-2 (test_align_block.py:109-129)
        ids = rng.integers(0, 8, size=65536 * 2).astype(np.int32)
    s, e, n = moe_align_block_size(torch.from_numpy(ids).to(DEV), block, E)
    os_, oe, on = c_oracle.moe_align_block_size(ids, E, block)
    assert np.array_equal(n.cpu().numpy(), on) and np.array_equal(e.cpu().numpy(), oe)
    assert np.array_equal(s.cpu().numpy(), os_)


def test_align_defines_every_output_element_and_accepts_int64_and_exact_buffers():
    announce("align garbage-prefilled / int64 / exact-size buffers")
    rng = np.random.default_rng(9)
    ids = rng.integers(0, 8, size=1000)
    os_, oe, on = c_oracle.moe_align_block_size(ids, 8, 16)
    for dtype in (torch.int32, torch.int64):
        t = torch.from_numpy(ids).to(dtype).to(DEV)
        s = torch.full((os_.size,), 12345, dtype=torch.int32, device=DEV)
        e = torch.full((oe.size,), 12345, dtype=torch.int32, device=DEV)
        n = torch.full((1,), 12345, dtype=torch.int32, device=DEV)
        _C.moe_align_block_size(t, 8, 16, s, e, n)
        assert np.array_equal(s.cpu().numpy(), os_) and np.array_equal(e.cpu().numpy(), oe)
        assert np.array_equal(n.cpu().numpy(), on)
    # buffers sized exactly from the padded total, as the reference's test does
    total = int(on[0])
    s = torch.empty(total, dtype=torch.int32, device=DEV)
    e = torch.empty(total // 16, dtype=torch.int32, device=DEV)
    guard = torch.full((64,), 777, dtype=torch.int32, device=DEV)
    n = torch.empty(1, dtype=torch.int32, device=DEV)
    _C.moe_align_block_size(torch.from_numpy(ids).to(torch.int32).to(DEV), 8, 16, s, e, n)
    assert np.array_equal(s.cpu().numpy(), os_[:total]) and np.array_equal(e.cpu().numpy(), oe[:total // 16])
    assert (guard == 777).all()


def test_align_other_expert_counts():
    announce("align E in {1, 3, 64}")
    rng = np.random.default_rng(10)
    for E, block in [(1, 16), (3, 4), (64, 16)]:
        ids = rng.integers(0, E, size=5000).astype(np.int32)
        s, e, n = moe_align_block_size(torch.from_numpy(ids).to(DEV), block, E)
        os_, oe, on = c_oracle.moe_align_block_size(ids, E, block)
        assert np.array_equal(s.cpu().numpy(), os_) and np.array_equal(e.cpu().numpy(), oe)
        assert np.array_equal(n.cpu().numpy(), on)


# ----------------------------------------------------------- element-wise ----
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("rows,d", [(1024, 7168), (128, 14336), (3, 100), (5, 7), (2, 8)])
def test_silu_and_mul(dtype, rows, d):
    announce(f"silu_and_mul {dtype} rows={rows} d={d}")
    g = torch.Generator().manual_seed(rows + d)
    x = torch.randn(rows, 2 * d, generator=g).to(dtype)
    out = torch.full((rows, d), 99.0, dtype=dtype, device=DEV)
    assert _C.silu_and_mul(out, x.to(DEV)) is None
    ref = O.silu_and_mul(x)
    got = out.cpu()
    if dtype == torch.float32:
        assert torch.allclose(got, ref, rtol=1e-6, atol=1e-7)
    else:
        # the device exp may differ from the CPU's in the last ulp, which can move the
        # intermediate rounding by one unit and then the product's: allow 2 ulp of the
        # 16-bit type, with nearly all elements exact
        ulp = 2.0 ** -6 if dtype == torch.bfloat16 else 2.0 ** -9
        d_ = (got.float() - ref.float()).abs()
        floor = 6.2e-8 if dtype == torch.float16 else 1e-30      # fp16 results can be subnormal
        assert (d_ <= ulp * ref.float().abs() + floor).all()
        assert (d_ == 0).float().mean() > 0.98
    # the reference's own check (test/example/test_silu.py:16-27)
    lib = torch.nn.functional.silu(x[:, :d].float()) * x[:, d:].float()
    assert torch.allclose(got.float(), lib, atol=2e-2 if dtype != torch.float32 else 1e-5, rtol=2e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,H", [(1024, 4096), (1, 4096), (7, 100), (3, 6144)])
def test_moe_sum(dtype, T, H):
    announce(f"moe_sum {dtype} T={T} H={H}")
    g = torch.Generator().manual_seed(T + H)
    x = torch.randn(T, 2, H, generator=g).to(dtype)
    out = torch.full((T, H), 99.0, dtype=dtype, device=DEV)
    assert _C.moe_sum(x.to(DEV), out) is None
    assert torch.equal(out.cpu(), O.moe_sum(x))               # one rounding of an exact sum: bit-exact
    # the reference's own check is fp16 with atol 1e-2 (test_moe_sum.py:70-76); half a bf16 ulp near 8 is 3.1e-2
    assert torch.allclose(out.cpu().float(), torch.sum(x.float(), 1), atol=3.2e-2 if dtype == torch.bfloat16 else 1e-2)
    with pytest.raises(RuntimeError, match="top_k=2"):
        _C.moe_sum(torch.zeros(4, 3, 8, device=DEV, dtype=dtype), torch.zeros(4, 8, device=DEV, dtype=dtype))


def test_ops_run_on_the_callers_stream():
    announce("ops on a side stream")
    s = torch.cuda.Stream()
    x = torch.randn(64, 2, 512, device=DEV, dtype=torch.bfloat16)
    out = torch.zeros(64, 512, device=DEV, dtype=torch.bfloat16)
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        _C.moe_sum(x, out)
    s.synchronize()
    assert torch.equal(out, (x[:, 0].float() + x[:, 1].float()).to(torch.bfloat16))
    assert _lib.load().em_version() >= 100
