"""GPU parity of the whole MoE layer (em_moe_forward through fused_experts /
FusedMoE) against the fp32 CPU oracle.

Routing outputs (topk_ids, sorted_token_ids, expert_ids, num_tokens_post_pad)
must be bit-exact.  Layer outputs are float: the target stated for this path is
max-abs error 2e-2 and mean relative error 1e-3 against an fp32 reference.
Rounding an fp32 result to bf16 alone costs about 1.4e-3 mean relative error and up to
half a bf16 ulp (0.0156 for |v| in [4, 8), 0.031 for [8, 16)), so the target is asserted
on the float32 output of the default mode, and every case reports the measured errors of
all forms and asserts
    default, fp32 output : the stated target itself, max_abs <= 2e-2 and mean_rel <= 1e-3
    default, bf16 output : that fp32 output rounded once (within 1 bf16 ulp)
    FLAG_BF16_ACT (activations stored as bf16 between the GEMMs, the reference's storage type)
        fp32 output : mean_rel <= TOL_MEAN_REL_F32, max_abs <= TOL_MAX_ABS_F32 * max|ref|
                      (the activation rounding is a relative error, so the bound scales
                      with the output magnitude: max|ref| is ~9 at 8x7B and ~16 at 8x22B)
        bf16 output : equal to the rounded fp32 output within 1 bf16 ulp, and
                      mean_rel <= TOL_MEAN_REL_BF16
"""
import json
import os

import numpy as np
import pytest
import torch

from electrock_infer_amd import FusedMoE, _lib, fused_experts, moe_align_block_size
from electrock_infer_amd.layers.moe.fused_moe import get_workspace
from oracle import c_oracle, moe_oracle as O
from tests.gpu_util import DEV, announce, error_stats, gpu_inputs, oracle_rows

pytestmark = pytest.mark.gpu

TOL_MEAN_REL_F32 = 2.5e-3    # one bf16 rounding of the SiLU*mul activations feeds the w2 MFMA
TOL_MAX_ABS_F32 = 4e-3       # times max|ref|
TOL_MEAN_REL_BF16 = 3.5e-3   # + the final rounding of the output to bf16
TARGET_MAX_ABS, TARGET_MEAN_REL = 2e-2, 1e-3   # the stated target, asserted for the default mode with an fp32 output

REPORT = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "gpurun_out", "layer_errors.jsonl")


def record(case: str, **stats):
    os.makedirs(os.path.dirname(REPORT), exist_ok=True)
    with open(REPORT, "a") as f:
        f.write(json.dumps({"case": case, **stats}) + "\n")
    print(f"[layer-error] {case} {stats}", flush=True)


def check_routing(ws, lg_cpu_f32, T, E=8, k=2, renormalize=True):
    """Bit-exact comparison of everything the router and the sort left in the workspace."""
    ow, oids = O.topk_softmax(lg_cpu_f32.numpy(), k, renormalize)
    ids = ws.topk_ids().cpu().numpy()
    assert np.array_equal(ids, oids)
    np.testing.assert_allclose(ws.topk_weights().cpu().numpy(), ow, rtol=2e-6, atol=1e-9)
    B = ws.block_size
    os_, oe, on = c_oracle.moe_align_block_size(oids, E, B)
    s, e, n = ws.sorted_token_ids().cpu().numpy(), ws.expert_ids().cpu().numpy(), ws.num_tokens_post_pad().cpu().numpy()
    assert np.array_equal(n, on)
    m = min(s.size, os_.size)     # the workspace rounds the worst-case length up to whole blocks
    assert np.array_equal(s[:m], os_[:m]) and (s[m:] == -1).all()
    me = min(e.size, oe.size)
    assert np.array_equal(e[:me], oe[:me]) and (e[me:] == 0).all()


def one_ulp_excess(out_bf16, out_f32):
    """How far a bf16 output lies from its fp32 counterpart rounded once, beyond one bf16 ulp."""
    rounded = out_f32.to(torch.bfloat16).float()
    ulp = torch.maximum(rounded.abs(), torch.tensor(1e-30, device=rounded.device)) * 2.0 ** -7
    return float(((out_bf16.float() - rounded).abs() - ulp).clamp_min(0).max())


def check_outputs(case, out_f32, out_bf16, ref, out_def=None, def_bf16=None):
    """out_f32 / out_bf16: FLAG_BF16_ACT mode; out_def / def_bf16: default mode with fp32 / bf16 output."""
    f = error_stats(out_f32, ref)
    b = error_stats(out_bf16.float(), ref)
    a = error_stats(out_def, ref) if out_def is not None else None
    record(case, default=a, bf16act_f32=f, bf16act_bf16=b, ref_absmean=float(ref.abs().mean()),
           ref_absmax=float(ref.abs().max()))
    if a is not None:
        assert a["max_abs"] <= TARGET_MAX_ABS and a["mean_rel"] <= TARGET_MEAN_REL, (case, a)
    if def_bf16 is not None:
        assert one_ulp_excess(def_bf16, out_def) == 0.0, case
    assert f["mean_rel"] <= TOL_MEAN_REL_F32 and f["max_abs"] <= TOL_MAX_ABS_F32 * float(ref.abs().max()), (case, f)
    assert b["mean_rel"] <= TOL_MEAN_REL_BF16, (case, b)
    assert one_ulp_excess(out_bf16, out_f32) == 0.0, case   # the bf16 output is the fp32 output rounded once


def run_both(x, lg, w13, w2, flags=0):
    """The layer with bf16 activations between the GEMMs (the reference's storage type), fp32 and bf16 output."""
    flags |= _lib.FLAG_BF16_ACT
    out_f32 = fused_experts(x, w13, w2, lg, 2, renormalize=True, out_dtype=torch.float32, flags=flags)
    out_bf16 = fused_experts(x, w13, w2, lg, 2, renormalize=True, flags=flags)
    torch.cuda.synchronize()
    return out_f32, out_bf16


def run_default(x, lg, w13, w2, flags=0):
    """The default mode with an fp32 output: the form the stated target is asserted on."""
    out = fused_experts(x, w13, w2, lg, 2, renormalize=True, out_dtype=torch.float32, flags=flags)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("T", [1, 5, 16, 17, 64, 200])
def test_layer_config1_shape(T):
    """Tiny layer of configuration 1 (H=256, I=512, E=8) with bf16-rounded inputs."""
    announce(f"layer C1-shape T={T}")
    x, lg, w13, w2 = O.make_inputs(T, 256, 512, seed=0)
    ref = O.moe_layer_fp32(x, lg, w13, w2)
    xd, lgd, w13d, w2d = (t.to(DEV) for t in (x, lg, w13, w2))
    out_f32, out_bf16 = run_both(xd, lgd, w13d, w2d)
    out_def = run_default(xd, lgd, w13d, w2d)
    check_routing(get_workspace(DEV, T, 256, 512, 8, 2), lg.float(), T)
    check_outputs(f"c1_T{T}", out_f32.cpu(), out_bf16.cpu(), ref, out_def.cpu())


def test_layer_golden_fixture_c1():
    """Configuration 1 exactly (fp32 values, seed 0) against the committed fixture;
    the GPU path computes in bf16, so inputs are rounded to bf16 on both sides for the
    output check, while routing is compared on the fixture's own fp32 logits."""
    announce("layer golden c1_seed0")
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "c1_seed0.npz"))
    x, lg, w13, w2 = O.make_inputs(64, 256, 512, seed=0, dtype=torch.float32)
    xb, w13b, w2b = x.to(torch.bfloat16), w13.to(torch.bfloat16), w2.to(torch.bfloat16)
    out = fused_experts(xb.to(DEV), w13b.to(DEV), w2b.to(DEV), lg.to(DEV), 2, out_dtype=torch.float32)
    ws = get_workspace(DEV, 64, 256, 512, 8, 2)
    assert np.array_equal(ws.topk_ids().cpu().numpy(), gold["topk_ids"])
    np.testing.assert_allclose(ws.topk_weights().cpu().numpy(), gold["topk_weights"], rtol=4e-6)
    # the fixture's sort uses the reference's block size for T=64 (64 rows); the fused
    # path sorts for its own tile, so the op is run on the layer's topk_ids
    s_ids, e_ids, n_pad = moe_align_block_size(ws.topk_ids(), 64, 8)
    assert np.array_equal(s_ids.cpu().numpy(), gold["sorted_token_ids"])
    assert np.array_equal(e_ids.cpu().numpy(), gold["expert_ids"])
    assert np.array_equal(n_pad.cpu().numpy(), gold["num_tokens_post_pad"])
    # fp32-input fixture vs bf16-input GPU run: input rounding dominates (about 4e-3 relative)
    st = error_stats(out.cpu(), torch.from_numpy(gold["out"]))
    record("golden_c1", f32=st)
    assert st["mean_rel"] < 1e-2
    ref = O.moe_layer_fp32(xb, lg, w13b, w2b)
    st = error_stats(out.cpu(), ref)
    assert st["mean_rel"] <= TARGET_MEAN_REL and st["max_abs"] <= TARGET_MAX_ABS


@pytest.fixture(scope="module")
def mixtral_8x7b():
    announce("building 8x7B-shaped weights")
    x, lg, w13, w2 = gpu_inputs(8192, 4096, 14336, seed=0)
    return {"x": x, "lg": lg, "w13": w13, "w2": w2, "w13_cpu": w13.cpu(), "w2_cpu": w2.cpu()}


@pytest.mark.parametrize("T", [1, 8, 32, 64, 65, 130, 256])
def test_layer_8x7b_decode(mixtral_8x7b, T):
    """Configuration 2: H=4096, I=14336, E=8, top-2, bf16, decode batch sizes (from 65 tokens the w2 GEMM of this
    shape runs on the 256-row kernel)."""
    announce(f"layer 8x7B decode T={T}")
    m = mixtral_8x7b
    x, lg = m["x"][:T].contiguous(), m["lg"][:T].contiguous()
    out_f32, out_bf16 = run_both(x, lg, m["w13"], m["w2"])
    out_def = run_default(x, lg, m["w13"], m["w2"])
    def_bf16 = fused_experts(x, m["w13"], m["w2"], lg, 2)                    # what the drop-in layer returns
    check_routing(get_workspace(DEV, T, 4096, 14336, 8, 2), lg.float().cpu(), T)
    rows = list(range(T)) if T <= 64 else list(range(0, T, 4))
    ref = oracle_rows(x, lg, m["w13_cpu"], m["w2_cpu"], rows)
    check_outputs(f"8x7b_T{T}", out_f32[rows].cpu(), out_bf16[rows].cpu(), ref, out_def[rows].cpu(), def_bf16[rows].cpu())


@pytest.mark.parametrize("T", [17, 33, 48, 64])
def test_layer_config1_shape_two_busy_experts_in_a_decode_batch(T):
    """Decode batches whose tokens all pick experts 0 and 1: T rows per expert, i.e. two to four 16-row fragments in
    one pass of the streaming kernel over the weight rows (even routing gives one or two); every row against the
    oracle."""
    announce(f"layer C1-shape T={T}, all tokens to experts 0 and 1")
    x, lg, w13, w2 = O.make_inputs(T, 256, 512, seed=T, logits="two_experts")
    ref = O.moe_layer_fp32(x, lg, w13, w2)
    xd, lgd, w13d, w2d = (t.to(DEV) for t in (x, lg, w13, w2))
    out_f32, out_bf16 = run_both(xd, lgd, w13d, w2d)
    out_def = run_default(xd, lgd, w13d, w2d)
    check_routing(get_workspace(DEV, T, 256, 512, 8, 2), lg.float(), T)
    check_outputs(f"c1_T{T}_two_experts", out_f32.cpu(), out_bf16.cpu(), ref, out_def.cpu())


@pytest.mark.parametrize("T", [40, 64, 65, 200, 448])
def test_layer_8x7b_small_batches_with_two_busy_experts(mixtral_8x7b, T):
    """Small batches whose tokens all pick experts 0 and 1: six experts without rows, two with T rows each, on the
    kernels that even routing would give a few dozen rows per expert (up to 64 tokens: three and four fragments in one
    pass of the streaming kernel)."""
    announce(f"layer 8x7B T={T}, all tokens to experts 0 and 1")
    m = mixtral_8x7b
    lg = m["lg"][:T].float()
    lg[:, :2] += 20.0
    lg = lg.to(torch.bfloat16).contiguous()
    x = m["x"][:T].contiguous()
    out_f32, out_bf16 = run_both(x, lg, m["w13"], m["w2"])
    out_def = run_default(x, lg, m["w13"], m["w2"])
    check_routing(get_workspace(DEV, T, 4096, 14336, 8, 2), lg.float().cpu(), T)
    rows = list(range(0, T, max(1, T // 48)))
    ref = oracle_rows(x, lg, m["w13_cpu"], m["w2_cpu"], rows)
    check_outputs(f"8x7b_T{T}_two_experts", out_f32[rows].cpu(), out_bf16[rows].cpu(), ref, out_def[rows].cpu())


@pytest.mark.parametrize("logits", ["normal", "zipf", "two_experts"])
def test_layer_8x7b_prefill(mixtral_8x7b, logits):
    """Configuration 3: T=8192 with near-uniform, Zipf-skewed and all-to-{0,1} routing.
    The oracle is evaluated on a sample of tokens (the layer is token-wise)."""
    announce(f"layer 8x7B prefill T=8192 logits={logits}")
    m = mixtral_8x7b
    T = 8192
    g = torch.Generator().manual_seed(3)
    lg = m["lg"].float().cpu()
    if logits == "zipf":
        ranks = torch.arange(1, 9, dtype=torch.float32) ** -1.2
        lg = lg + torch.log(ranks / ranks.sum())[torch.randperm(8, generator=g)]
    elif logits == "two_experts":
        lg[:, :2] += 20.0
    lg = lg.to(torch.bfloat16).to(DEV)
    out_f32, out_bf16 = run_both(m["x"], lg, m["w13"], m["w2"])
    out_def = run_default(m["x"], lg, m["w13"], m["w2"])
    def_bf16 = fused_experts(m["x"], m["w13"], m["w2"], lg, 2)
    check_routing(get_workspace(DEV, T, 4096, 14336, 8, 2), lg.float().cpu(), T)
    rows = torch.randperm(T, generator=g)[:96].tolist() + [0, T - 1]
    ref = oracle_rows(m["x"], lg, m["w13_cpu"], m["w2_cpu"], rows)
    check_outputs(f"8x7b_prefill_{logits}", out_f32[rows].cpu(), out_bf16[rows].cpu(), ref, out_def[rows].cpu(),
                  def_bf16[rows].cpu())
    # size-independent properties on the full result
    assert torch.isfinite(out_f32).all()
    perm = torch.randperm(T, generator=g).to(DEV)     # token-wise layer: permuting tokens permutes outputs
    out_p = fused_experts(m["x"][perm].contiguous(), m["w13"], m["w2"], lg[perm].contiguous(), 2,
                          out_dtype=torch.float32)
    assert torch.allclose(out_p, out_def[perm], rtol=0, atol=1e-5)


@pytest.mark.parametrize("T", [2048, 8192])
def test_layer_8x7b_tuned_kernels_against_the_generic_kernels_on_every_row(mixtral_8x7b, T):
    """The oracle checks a sample of the rows of the large batches; here every element of the tuned kernels' output is
    compared with the shape-generic kernels' (another tiling, another copy path, no tile queue), which the oracle
    checks in full on the small shapes of this file: a wrong tile at one (expert, row tile, column tile) cannot hide.
    With bf16 activations and float32 partial sums both forms accumulate the same bf16 products in float32 through the
    same MFMA shape, K ascending, over the same two K slices: the results are equal to the last bit (measured:
    difference 0.0).  In the default form the tuned kernels keep the activations and the partial sums as fp16, the
    generic ones as a bf16 pair and float32: 2^-12 apart."""
    announce(f"layer 8x7B T={T}: tuned vs generic kernels, all rows")
    m = mixtral_8x7b
    x, lg = m["x"][:T].contiguous(), m["lg"][:T].contiguous()
    for mode in (0, _lib.FLAG_BF16_ACT | _lib.FLAG_F32_PARTIALS):
        tuned = fused_experts(x, m["w13"], m["w2"], lg, 2, out_dtype=torch.float32, flags=mode)
        generic = fused_experts(x, m["w13"], m["w2"], lg, 2, out_dtype=torch.float32, flags=mode | _lib.FLAG_FORCE_GENERIC)
        d = (tuned - generic).abs()
        scale = float(generic.abs().max())
        tol = (1e-5 if mode else 1.5e-3) * scale          # measured: 0.0 and 2.0e-4 * scale
        worst = float(d.max())
        record(f"8x7b_T{T}_tuned_vs_generic_flags{mode}", max_abs=worst, scale=scale, mean_abs=float(d.mean()))
        assert worst <= tol, (mode, worst, tol)
        assert float(d.mean()) <= (1e-6 if mode else 8e-4) * float(generic.abs().mean())


def assert_offsets_fit(T, H, I, E=8, k=2, flags=0):
    """Host-side bounds of a large case, checked before anything is launched: the tiled kernels form 32-bit byte
    offsets from x, from an expert's weights and from a 256-row tile of the activations, and slot indices are int32;
    the workspace the layout asks for must fit the device."""
    L = _lib.workspace_layout(T, H, I, E, k, flags)
    assert T * H * 2 < 2 ** 32 and 4 * I * H < 2 ** 32 and 256 * I * 2 < 2 ** 32
    assert L.sorted_len < 2 ** 31 and T * k < 2 ** 30 and L.sorted_len * I < 2 ** 62
    assert L.sorted_len == -(-(T * k + E * (L.block_size - 1)) // L.block_size) * L.block_size
    free, _ = torch.cuda.mem_get_info()
    assert L.total_bytes + T * H * 16 < free, (L.total_bytes, free)
    return L


def test_layer_8x7b_largest_engine_batch(mixtral_8x7b):
    """T = 32768, the reference's max_num_batched_tokens (config.py:9), the largest batch its engine hands the layer:
    routing bit-exact on all rows, the oracle on sampled rows, every row against the shape-generic kernels."""
    T = 32768
    announce(f"layer 8x7B T={T}")
    m = mixtral_8x7b
    assert_offsets_fit(T, 4096, 14336)
    assert_offsets_fit(T, 4096, 14336, flags=_lib.FLAG_FORCE_GENERIC)
    g = torch.Generator(device=DEV).manual_seed(77)
    x = torch.randn(T, 4096, generator=g, device=DEV).to(torch.bfloat16)
    lg = torch.randn(T, 8, generator=g, device=DEV)
    ranks = torch.arange(1, 9, dtype=torch.float32) ** -1.2
    lg = (lg + torch.log(ranks / ranks.sum())[torch.randperm(8, generator=torch.Generator().manual_seed(7))].to(DEV)).to(torch.bfloat16)
    out = run_default(x, lg, m["w13"], m["w2"])
    check_routing(get_workspace(DEV, T, 4096, 14336, 8, 2), lg.float().cpu(), T)
    assert int(get_workspace(DEV, T, 4096, 14336, 8, 2).saturated()) == 0
    rows = torch.randperm(T, generator=torch.Generator().manual_seed(5))[:96].tolist() + [0, T - 1]
    st = error_stats(out[rows].cpu(), oracle_rows(x, lg, m["w13_cpu"], m["w2_cpu"], rows))
    record(f"8x7b_T{T}", default=st)
    assert st["max_abs"] <= TARGET_MAX_ABS and st["mean_rel"] <= TARGET_MEAN_REL, st
    assert torch.isfinite(out).all()
    out16 = fused_experts(x, m["w13"], m["w2"].to(torch.float16), lg, 2, out_dtype=torch.float32)   # the module's default
    # (the weights below 2^-14 round differently on the two paths, by up to 2^-25 each: enough to flip the fp16
    # rounding of a partial sum here and there)
    assert float((out16 - out).abs().max()) <= 2.0 ** -10 * float(out.abs().max())
    assert float((out16 - out).abs().mean()) <= 1e-6 * float(out.abs().mean())
    del out16
    generic = fused_experts(x, m["w13"], m["w2"], lg, 2, out_dtype=torch.float32, flags=_lib.FLAG_FORCE_GENERIC)
    d = (out - generic).abs()
    scale = float(generic.abs().max())
    record(f"8x7b_T{T}_tuned_vs_generic", max_abs=float(d.max()), scale=scale, mean_abs=float(d.mean()))
    assert float(d.max()) <= 1.5e-3 * scale and float(d.mean()) <= 8e-4 * float(generic.abs().mean())
    from electrock_infer_amd.layers.moe.fused_moe import release_workspaces
    del generic, d, out
    release_workspaces()          # 6 GB of scratch that the rest of the file does not need
    torch.cuda.empty_cache()


def test_layer_8x7b_float16_w2(mixtral_8x7b):
    """w2 handed over as float16 at the full 8x7B shape (decode, mid-size and prefill kernels): the stated target
    against the oracle on sampled tokens."""
    m = mixtral_8x7b
    w2h = m["w2"].to(torch.float16)
    for T in (1, 64, 256, 8192):
        announce(f"layer 8x7B float16 w2 T={T}")
        x, lg = m["x"][:T].contiguous(), m["lg"][:T].contiguous()
        out = fused_experts(x, m["w13"], w2h, lg, 2, out_dtype=torch.float32)
        rows = list(range(T)) if T <= 64 else list(range(0, T, T // 64))
        st = error_stats(out[rows].cpu(), oracle_rows(x, lg, m["w13_cpu"], m["w2_cpu"], rows))
        record(f"8x7b_w2f16_T{T}", f32=st)
        assert st["max_abs"] <= TARGET_MAX_ABS and st["mean_rel"] <= TARGET_MEAN_REL, st


def test_layer_8x22b_shape():
    """Configuration 5: H=6144, I=16384; T in {1, 64} in full, T=100 (the w13 GEMM of this shape runs on the 256-row
    kernel from 65 tokens, the w2 GEMM on 128-row tiles), with even routing and with all tokens on experts 0 and 1, and
    T=4096 on sampled tokens."""
    announce("building 8x22B-shaped weights")
    x, lg, w13, w2 = gpu_inputs(4096, 6144, 16384, seed=1)
    w13_cpu, w2_cpu = w13.cpu(), w2.cpu()
    lg_two = lg[:100].float()
    lg_two[:, :2] += 20.0
    for T, lt in ((1, lg[:1]), (64, lg[:64]), (100, lg[:100]), (100, lg_two.to(torch.bfloat16)), (4096, lg)):
        announce(f"layer 8x22B T={T}")
        xt, lt = x[:T].contiguous(), lt.contiguous()
        out_f32, out_bf16 = run_both(xt, lt, w13, w2)
        out_def = run_default(xt, lt, w13, w2)
        def_bf16 = fused_experts(xt, w13, w2, lt, 2)
        check_routing(get_workspace(DEV, T, 6144, 16384, 8, 2), lt.float().cpu(), T)
        rows = list(range(T)) if T <= 64 else list(range(0, T, 64))
        ref = oracle_rows(xt, lt, w13_cpu, w2_cpu, rows)
        check_outputs(f"8x22b_T{T}", out_f32[rows].cpu(), out_bf16[rows].cpu(), ref, out_def[rows].cpu(), def_bf16[rows].cpu())
    # every row of the largest batch against the shape-generic kernels, as for the 8x7B shape
    T = 4096
    announce(f"layer 8x22B T={T}: tuned vs generic kernels, all rows")
    assert_offsets_fit(T, 6144, 16384)
    for mode in (0, _lib.FLAG_BF16_ACT | _lib.FLAG_F32_PARTIALS):
        tuned = fused_experts(x, w13, w2, lg, 2, out_dtype=torch.float32, flags=mode)
        generic = fused_experts(x, w13, w2, lg, 2, out_dtype=torch.float32, flags=mode | _lib.FLAG_FORCE_GENERIC)
        d = (tuned - generic).abs()
        scale = float(generic.abs().max())
        record(f"8x22b_T{T}_tuned_vs_generic_flags{mode}", max_abs=float(d.max()), scale=scale, mean_abs=float(d.mean()))
        assert float(d.max()) <= (1e-5 if mode else 1.5e-3) * scale, (mode, float(d.max()), scale)
        assert float(d.mean()) <= (1e-6 if mode else 8e-4) * float(generic.abs().mean())
    out16 = fused_experts(x, w13, w2.to(torch.float16), lg, 2, out_dtype=torch.float32)
    assert float((out16 - tuned).abs().max()) <= TOL_MAX_ABS_F32 * scale     # (tuned holds the bf16-activation form here)


def test_fusedmoe_module_runs_in_place_and_matches(mixtral_8x7b):
    announce("FusedMoE module, in place")
    m = mixtral_8x7b
    layer = FusedMoE(num_experts=8, top_k=2, hidden_size=4096, intermediate_size=14336, tp_size=1,
                     params_dtype=torch.bfloat16, renormalize=True, reduce_results=True, w2_dtype=torch.bfloat16).to(DEV)
    layer.w13_weight.data = m["w13"]          # share storage instead of a second 2.8 GB copy
    layer.w2_weight.data = m["w2"]
    x = m["x"][:48].clone()
    lg = m["lg"][:48].contiguous()
    expect = fused_experts(x.clone(), m["w13"], m["w2"], lg, 2, renormalize=True)
    ret = layer(x, lg)
    assert ret.data_ptr() == x.data_ptr()            # the input tensor is overwritten and returned
    assert torch.equal(ret, expect)
    layer.bf16_act = True                            # the keyword-only option of this build
    x2 = m["x"][:48].clone()
    expect = fused_experts(x2.clone(), m["w13"], m["w2"], lg, 2, renormalize=True, bf16_act=True)
    assert torch.equal(layer(x2, lg), expect) and not torch.equal(expect, ret)


def test_dense_equals_sparse_when_one_expert_wins():
    """With one expert far ahead the layer reduces to that expert's SwiGLU MLP,
    which torch's own bf16 GEMMs can evaluate on the GPU."""
    announce("layer one-hot routing vs plain MLP")
    T, H, I = 128, 512, 1024
    x, lg, w13, w2 = O.make_inputs(T, H, I, seed=4)
    lg = torch.full((T, 8), -40.0)
    lg[:, 5] = 40.0
    out = fused_experts(x.to(DEV), w13.to(DEV), w2.to(DEV), lg.to(DEV), 2, out_dtype=torch.float32).cpu()
    xf = x.float()
    mlp = (torch.nn.functional.silu(xf @ w13[5, :I].float().t()) * (xf @ w13[5, I:].float().t())) @ w2[5].float().t()
    st = error_stats(out, mlp)
    assert st["mean_rel"] <= TARGET_MEAN_REL, st


def test_unsupported_inputs_raise():
    x = torch.zeros(4, 256, device=DEV, dtype=torch.float16)
    w13 = torch.zeros(8, 1024, 256, device=DEV, dtype=torch.float16)
    w2 = torch.zeros(8, 256, 512, device=DEV, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="bfloat16"):
        fused_experts(x, w13, w2, torch.zeros(4, 8, device=DEV), 2)
    xb = x.to(torch.bfloat16)
    with pytest.raises(RuntimeError, match="shapes"):
        fused_experts(xb, w13.to(torch.bfloat16)[:, :, :128].contiguous(), w2.to(torch.bfloat16),
                      torch.zeros(4, 8, device=DEV), 2)
    assert fused_experts(xb[:0], w13.to(torch.bfloat16), w2.to(torch.bfloat16), torch.zeros(0, 8, device=DEV), 2).shape == (0, 256)


# ---- shapes and routings that exercise every tile case of the GEMM kernels on a layer the oracle runs in full ----
MID = dict(H=512, I=1024)


def mid_inputs(T, routing, seed):
    x, lg, w13, w2 = O.make_inputs(T, MID["H"], MID["I"], seed=seed, logits=routing if routing != "one_expert" else "normal")
    if routing == "one_expert":
        lg = lg.float()
        lg[:, 3] += 30.0      # expert 3 takes every token's first slot; the second slot spreads over the rest
        lg = lg.to(torch.bfloat16)
    return x, lg, w13, w2


@pytest.mark.parametrize("routing", ["normal", "zipf", "two_experts", "one_expert"])
@pytest.mark.parametrize("T", [65, 96, 300, 400, 513, 777, 1500, 4100])
def test_layer_mid_shape_all_tile_cases(T, routing):
    """T just above the streaming limit, around the split-K switch (512), experts with 0, 1 and several
    256-row tiles, last tiles of every height; tuned kernels and the generic kernel against the oracle."""
    announce(f"layer mid shape T={T} routing={routing}")
    x, lg, w13, w2 = mid_inputs(T, routing, seed=T)
    ref = O.moe_layer_fp32(x, lg, w13, w2)
    xd, lgd, w13d, w2d = (t.to(DEV) for t in (x, lg, w13, w2))
    out_f32, out_bf16 = run_both(xd, lgd, w13d, w2d)
    out_def = run_default(xd, lgd, w13d, w2d)
    check_routing(get_workspace(DEV, T, MID["H"], MID["I"], 8, 2), lg.float(), T)
    check_outputs(f"mid_T{T}_{routing}", out_f32.cpu(), out_bf16.cpu(), ref, out_def.cpu())
    gen_f32, gen_bf16 = run_both(xd, lgd, w13d, w2d, flags=_lib.FLAG_FORCE_GENERIC)
    gen_def = run_default(xd, lgd, w13d, w2d, flags=_lib.FLAG_FORCE_GENERIC)    # activations as a bf16 pair
    check_outputs(f"mid_T{T}_{routing}_generic", gen_f32.cpu(), gen_bf16.cpu(), ref, gen_def.cpu())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T", [1, 129, 2048, 2049])
def test_layer_router_and_sort_in_one_launch(T, dtype):
    """Up to 2048 tokens (4096 selected experts) the layer routes and sorts in one kernel, above in two: both
    leave the oracle's routing in the workspace, for every logits type, rows of ties included."""
    announce(f"layer routing front T={T} logits {dtype}")
    x, lg, w13, w2 = O.make_inputs(T, 256, 512, seed=T)
    lg = lg.float()
    lg[::7] = lg[::7].round()                      # rows with many ties
    lg[::11, 3] = 60000.0                          # one expert far ahead (finite in every logits type)
    lg = lg.to(dtype)
    out = fused_experts(x.to(DEV), w13.to(DEV), w2.to(DEV), lg.to(DEV), 2, out_dtype=torch.float32)
    assert out.shape == (T, 256)
    check_routing(get_workspace(DEV, T, 256, 512, 8, 2), lg.float(), T)


@pytest.mark.parametrize("E,k", [(8, 2), (16, 4), (5, 1), (64, 8)])
@pytest.mark.parametrize("T", [2048, 4096, 4097, 5000, 12289, 40000])
@pytest.mark.parametrize("routing", ["normal", "two_experts"])
def test_layer_sort_on_several_workgroups_writes_the_same_bytes(T, E, k, routing):
    """From 8192 routed slots the layer sorts on several workgroups (two launches, histogram rows in the workspace):
    every byte of sorted_token_ids, expert_ids, num_tokens_post_pad and the segment starts equals what the
    one-workgroup kernel writes, pads and tails included, and the oracle's routing."""
    if T * k < 8192:
        pytest.skip("fewer than 8192 routed slots: the one-workgroup sort runs either way")
    announce(f"sort on several workgroups: T={T} E={E} top-{k} {routing}")
    H, I = 256, 128
    x, lg, w13, w2 = O.make_inputs(T, H, I, E=E, seed=T + E, logits=routing)
    xd, lgd, w13d, w2d = (t.to(DEV) for t in (x, lg, w13, w2))
    ws = get_workspace(DEV, T, H, I, E, k)
    L = ws.layout
    head = slice(0, L.act_off)                     # everything in front of the activations
    ws.buffer[head].fill_(0x5A)
    fused_experts(xd, w13d, w2d, lgd, k, out_dtype=torch.float32, flags=_lib.FLAG_ONE_GROUP_SORT)
    one = ws.buffer[head].clone()
    ws.buffer[head].fill_(0xA5)
    fused_experts(xd, w13d, w2d, lgd, k, out_dtype=torch.float32)
    check_routing(ws, lg.float(), T, E=E, k=k)
    many = ws.buffer[head]
    for off, n in ((L.sorted_ids_off, L.sorted_len), (L.expert_ids_off, L.expert_ids_len), (L.post_pad_off, 1),
                   (L.seg_begin_off, E + 1), (L.topk_ids_off, T * k)):
        assert torch.equal(one[off:off + 4 * n], many[off:off + 4 * n]), (off, n)


@pytest.mark.parametrize("T", [1, 7, 33, 64, 200, 400, 777, 2100])
def test_layer_with_float16_w2(T):
    """w2 handed over as float16 (converted once from bf16: exact in this range) runs the default mode's arithmetic
    without the conversion inside the w2 kernels: the same results as the default mode on the bf16 weights up to the
    rounding of the few weights below 2^-14 in magnitude (fp16 subnormals: torch rounds them to nearest, the kernels'
    conversion towards zero), and the stated target against the oracle.  The generic kernels refuse float16 w2."""
    announce(f"layer with float16 w2, T={T}")
    x, lg, w13, w2 = mid_inputs(T, "zipf", seed=5 * T)
    ref = O.moe_layer_fp32(x, lg, w13, w2)
    xd, lgd, w13d, w2d = (t.to(DEV) for t in (x, lg, w13, w2))
    w2h = w2d.to(torch.float16)
    out = fused_experts(xd, w13d, w2h, lgd, 2, renormalize=True, out_dtype=torch.float32)
    st = error_stats(out.cpu(), ref)
    record(f"w2f16_T{T}", f32=st)
    assert st["max_abs"] <= TARGET_MAX_ABS and st["mean_rel"] <= TARGET_MEAN_REL, st
    acc = run_default(xd, lgd, w13d, w2d)
    # (above 448 tokens the partial sums are fp16: a difference of 2^-25 in a weight can flip the rounding of one)
    assert float((out - acc).abs().max()) <= (1e-6 if T <= 448 else 2.0 ** -10) * float(ref.abs().max())
    assert float((out - acc).abs().mean()) <= 1e-6 * float(ref.abs().mean())
    with pytest.raises(RuntimeError):
        fused_experts(xd, w13d, w2h, lgd, 2, flags=_lib.FLAG_FORCE_GENERIC)
    with pytest.raises(RuntimeError):       # fp16 weights multiply fp16 activations only
        fused_experts(xd, w13d, w2h, lgd, 2, bf16_act=True)


@pytest.mark.parametrize("w2_dtype", [None, torch.float16])
def test_fusedmoe_module_with_float16_w2(w2_dtype):
    """The module holds w2 as float16 by default (bfloat16 parameters, a shape the tuned kernels take)."""
    announce(f"FusedMoE module, w2_dtype={w2_dtype}")
    x, lg, w13, w2 = O.make_inputs(70, MID["H"], MID["I"], seed=70)
    layer = FusedMoE(num_experts=8, top_k=2, hidden_size=MID["H"], intermediate_size=MID["I"], tp_size=1,
                     params_dtype=torch.bfloat16, w2_dtype=w2_dtype).to(DEV)
    assert layer.w2_weight.dtype == torch.float16 and layer.w13_weight.dtype == torch.bfloat16
    for e in range(8):   # the reference loader's calls (utils/loader.py:36-49): the copy converts w2
        layer.weight_loader(layer.w13_weight, w13[e, :MID["I"]].to(DEV), "w1", e)
        layer.weight_loader(layer.w13_weight, w13[e, MID["I"]:].to(DEV), "w3", e)
        layer.weight_loader(layer.w2_weight, w2[e].to(DEV), "w2", e)
    xd = x.to(DEV)
    expect = fused_experts(xd.clone(), w13.to(DEV), w2.to(DEV), lg.to(DEV), 2)
    assert torch.equal(layer(xd, lg.to(DEV)), expect)


@pytest.mark.parametrize("T", [5, 100, 600])
def test_default_mode_clamps_activations_at_the_fp16_range(T):
    """The documented difference between the two modes: fp16 activations saturate at +-65504, bf16 ones do not.
    Inputs whose SiLU*mul values pass that bound: FLAG_BF16_ACT follows the fp32 definition, the default mode the
    definition with the activations clamped."""
    announce(f"activation range, T={T}")
    x, lg, w13, w2 = mid_inputs(T, "normal", seed=900 + T)
    x, w13 = (x.float() * 30).to(torch.bfloat16), (w13.float() * 50).to(torch.bfloat16)
    I = MID["I"]
    w, ids = O.topk_softmax(lg.float().numpy(), 2, True)
    ref = torch.zeros(T, MID["H"])
    ref_clamped = torch.zeros(T, MID["H"])
    over = 0
    for t in range(T):
        for j in range(2):
            e = int(ids[t, j])
            h = w13[e].float() @ x[t].float()
            act = torch.nn.functional.silu(h[:I]) * h[I:]
            over += int((act.abs() > 65504).sum())
            ref[t] += float(w[t, j]) * (w2[e].float() @ act)
            ref_clamped[t] += float(w[t, j]) * (w2[e].float() @ act.clamp(-65504, 65504))
    assert over > 10 * T                                   # the bound really is passed, many times per token
    xd, lgd, w13d, w2d = (t.to(DEV) for t in (x, lg, w13, w2))
    out = fused_experts(xd, w13d, w2d, lgd, 2, out_dtype=torch.float32, bf16_act=True).cpu()
    acc = fused_experts(xd, w13d, w2d, lgd, 2, out_dtype=torch.float32).cpu()
    assert torch.isfinite(out).all() and torch.isfinite(acc).all()
    scale = float(ref.abs().max())
    assert float((out - ref).abs().max()) <= TOL_MAX_ABS_F32 * scale
    assert float((acc - ref_clamped).abs().max()) <= 1e-3 * scale
    assert float((ref - ref_clamped).abs().max()) > 20e-3 * scale      # the two definitions are well apart here


@pytest.mark.parametrize("T", [5, 40, 100, 300, 600, 2100])
def test_saturated_counter_reports_clamped_activations(T):
    """A caller of the default mode can tell that activations were clamped: the workspace's `saturated` counter holds
    the number of SiLU*mul values of routed rows beyond +-65504 after the call (streaming, 64- / 128-row and 256-row
    kernels), and 0 after a call with ordinary magnitudes or with bf16 activations.  Padding rows do not count."""
    announce(f"saturated counter, T={T}")
    x, lg, w13, w2 = mid_inputs(T, "zipf", seed=1900 + T)
    xb, w13b = (x.float() * 30).to(torch.bfloat16), (w13.float() * 50).to(torch.bfloat16)
    I = MID["I"]
    _, ids = O.topk_softmax(lg.float().numpy(), 2, True)
    over, near = 0, 0
    for e in range(8):
        rows = np.nonzero((ids == e).any(axis=1))[0]
        if rows.size == 0:
            continue
        h = xb[rows].double() @ w13b[e].double().t()
        act = (h[:, :I] / (1.0 + torch.exp(-h[:, :I]))) * h[:, I:]
        over += int((act.abs() > 65504).sum())
        near += int(((act.abs() > 65504 * 0.999) & (act.abs() < 65504 * 1.001)).sum())   # the MFMA's sum may differ
    assert over > 10 * T
    xd, lgd, w13d, w2d = (t.to(DEV) for t in (xb, lg, w13b, w2))
    ws = get_workspace(DEV, T, MID["H"], I, 8, 2)
    fused_experts(xd, w13d, w2d, lgd, 2, out_dtype=torch.float32)
    got = int(ws.saturated())
    assert abs(got - over) <= near, (got, over, near)
    # the next call clears the counter: bf16 activations never clamp, ordinary magnitudes do not reach the bound
    fused_experts(xd, w13d, w2d, lgd, 2, out_dtype=torch.float32, bf16_act=True)
    assert int(get_workspace(DEV, T, MID["H"], I, 8, 2, _lib.FLAG_BF16_ACT).saturated()) == 0
    fused_experts(x.to(DEV), w13.to(DEV), w2d, lgd, 2, out_dtype=torch.float32)
    assert int(ws.saturated()) == 0
    fused_experts(xd, w13d, w2d.to(torch.float16), lgd, 2)          # the drop-in layer's form: fp16 w2, bf16 output
    assert abs(int(ws.saturated()) - over) <= near


@pytest.mark.parametrize("T", [300, 600, 2100])
def test_partial_sums_follow_the_definition_at_any_magnitude(T):
    """The partial sums of the w2 GEMM are float32 up to 448 tokens and fp16 above, where a value beyond the fp16 range
    is marked by the fp16 infinity and kept as float32 beside it: the layer follows the definition at any magnitude
    bf16 holds, with either format, and equals the all-float32 form (FLAG_F32_PARTIALS) wherever a partial sum
    escaped."""
    announce(f"output range, T={T}")
    x, lg, w13, w2 = mid_inputs(T, "normal", seed=31 + T)
    # large outputs from large w2 entries: the activations themselves stay far inside the fp16 range
    x, w2 = (x.float() * 8).to(torch.bfloat16), (w2.float() * 1e5).to(torch.bfloat16)
    w2[3, :, :] = (w2[3].float() * 1e-5).to(torch.bfloat16)          # ... and one expert with ordinary ones
    ref = O.moe_layer_fp32(x, lg, w13, w2)
    scale = float(ref.abs().max())
    assert scale > 4 * 65504
    xd, lgd, w13d, w2d = (t.to(DEV) for t in (x, lg, w13, w2))
    for mode in (0, _lib.FLAG_BF16_ACT):
        out = fused_experts(xd, w13d, w2d, lgd, 2, flags=mode).float().cpu()
        assert torch.isfinite(out).all()
        assert float((out - ref).abs().max()) <= 2.0 ** -7 * scale
        out32 = fused_experts(xd, w13d, w2d, lgd, 2, out_dtype=torch.float32, flags=mode)
        wide32 = fused_experts(xd, w13d, w2d, lgd, 2, out_dtype=torch.float32, flags=mode | _lib.FLAG_F32_PARTIALS)
        assert one_ulp_excess(out.to(torch.bfloat16).to(DEV), out32) == 0.0    # the same sums, rounded once more
        # partial sums beyond 65520 went through the float32 array; the others carry their fp16 rounding
        assert float((out32 - wide32).abs().max()) <= 2.0 ** -10 * scale
        big = wide32.abs() > 8 * 65504                               # rows of numbers whose every partial sum escaped
        if T > 448 and bool(big.any()):
            assert float(((out32 - wide32).abs() / wide32.abs())[big].max()) <= 2.0 ** -8
    if T > 448:          # infinities and NaNs among the partial sums come out as what they are
        w2n = w2d.clone()
        w2n[5, 7, :] = float("inf")
        w2n[6, 9, 0] = float("nan")
        got = fused_experts(xd, w13d, w2n, lgd, 2, out_dtype=torch.float32).cpu()
        want = fused_experts(xd, w13d, w2n, lgd, 2, out_dtype=torch.float32, flags=_lib.FLAG_F32_PARTIALS).cpu()
        assert torch.equal(torch.isnan(got), torch.isnan(want)) and torch.equal(torch.isinf(got), torch.isinf(want))
        assert bool(torch.isnan(want).any())


@pytest.mark.parametrize("T", [449, 777, 2100])
def test_fp16_partial_sums_within_their_rounding(T):
    """Above 448 tokens the partial sums are fp16 on ordinary magnitudes: against the all-float32 form
    (FLAG_F32_PARTIALS) the result differs by the rounding of the partial results (relative step 2^-11 each; where
    they cancel it shows in absolute terms, asserted with max|out| standing for the largest partial result), and the
    bf16 output is the fp32 output rounded once."""
    announce(f"fp16 partial sums, T={T}")
    x, lg, w13, w2 = (t.to(DEV) for t in mid_inputs(T, "zipf", seed=13 * T))
    for mode in (0, _lib.FLAG_BF16_ACT):
        f32 = fused_experts(x, w13, w2, lg, 2, out_dtype=torch.float32, flags=mode | _lib.FLAG_F32_PARTIALS)
        half = fused_experts(x, w13, w2, lg, 2, flags=mode)
        assert half.dtype == torch.bfloat16
        assert one_ulp_excess(half, f32) <= 2.0 ** -10 * float(f32.abs().max())
        half32 = fused_experts(x, w13, w2, lg, 2, out_dtype=torch.float32, flags=mode)
        assert half32.dtype == torch.float32 and not torch.equal(half32, f32)
        assert float((half32 - f32).abs().max()) <= 2.0 ** -10 * float(f32.abs().max())
        assert one_ulp_excess(half, half32) == 0.0
        if mode == 0:   # the stated target holds with either format
            ref = O.moe_layer_fp32(*(t.cpu() for t in (x, lg, w13, w2)))
            for out in (half32, f32):
                st = error_stats(out.cpu(), ref)
                assert st["max_abs"] <= 2e-2 and st["mean_rel"] <= 1e-3, st


@pytest.mark.parametrize("T", [7, 64, 300, 777])
def test_layer_default_mode_with_bf16_output(T):
    """The default mode is asserted against the stated target with an fp32 output everywhere else; with the bf16
    output of the drop-in layer the result is that fp32 output rounded once."""
    announce(f"layer default mode, bf16 out T={T}")
    x, lg, w13, w2 = (t.to(DEV) for t in O.make_inputs(T, MID["H"], MID["I"], seed=7 * T))
    acc_f32 = run_default(x, lg, w13, w2)
    acc_bf16 = fused_experts(x, w13, w2, lg, 2, renormalize=True)
    assert acc_bf16.dtype == torch.bfloat16
    assert one_ulp_excess(acc_bf16, acc_f32) == 0.0


@pytest.mark.parametrize("routing", ["normal", "one_expert"])
@pytest.mark.parametrize("I", [8192, 10240, 12288])
@pytest.mark.parametrize("T", [96, 300])
def test_layer_mid_kernel_many_column_tiles(T, I, routing):
    """Wide intermediate sizes with H = 256: w13 launches of the 64- / 128-row kernel with two or three whole rounds
    of 256-row weight tiles (I = 10240: plus a last round of 128-row tiles)."""
    announce(f"layer H=256 I={I} T={T} {routing}")
    x, lg, w13, w2 = O.make_inputs(T, 256, I, seed=T + I)
    if routing == "one_expert":
        lg = lg.float()
        lg[:, 2] += 30.0
        lg = lg.to(torch.bfloat16)
    ref = O.moe_layer_fp32(x, lg, w13, w2)
    xd, lgd, w13d, w2d = (t.to(DEV) for t in (x, lg, w13, w2))
    out_f32, out_bf16 = run_both(xd, lgd, w13d, w2d)
    out_def = run_default(xd, lgd, w13d, w2d)
    check_outputs(f"wideI{I}_T{T}_{routing}", out_f32.cpu(), out_bf16.cpu(), ref, out_def.cpu())


@pytest.mark.parametrize("T", [8, 9, 16, 17, 63, 64, 191, 192, 193, 255, 256, 257, 351, 352, 353, 447, 448, 449, 895, 896, 897,
                               1023, 1024, 1025, 1279, 1280, 1281, 2047, 2048, 2049])
def test_layer_at_every_kernel_switch(T):
    """The batch sizes on both sides of every point where the layer changes kernels, K slices, sorted block,
    routing front or the format of the partial results."""
    announce(f"layer at a kernel switch, T={T}")
    x, lg, w13, w2 = mid_inputs(T, "zipf", seed=11 * T)
    ref = O.moe_layer_fp32(x, lg, w13, w2)
    xd, lgd, w13d, w2d = (t.to(DEV) for t in (x, lg, w13, w2))
    out_f32, out_bf16 = run_both(xd, lgd, w13d, w2d)
    out_def = run_default(xd, lgd, w13d, w2d)
    check_routing(get_workspace(DEV, T, MID["H"], MID["I"], 8, 2), lg.float(), T)
    check_outputs(f"switch_T{T}", out_f32.cpu(), out_bf16.cpu(), ref, out_def.cpu())


@pytest.mark.parametrize("routing", ["normal", "one_expert"])
@pytest.mark.parametrize("T", [40, 100, 300, 600, 1500])
def test_layer_column_tiles_not_a_multiple_of_eight(T, routing):
    """H = 768 and I = 1152 give 3 and 9 column tiles: the tile orders that do not deal whole columns to the XCDs,
    and launches of the 64- / 128-row kernel whose tile count fills no whole round."""
    announce(f"layer H=768 I=1152 T={T} {routing}")
    x, lg, w13, w2 = O.make_inputs(T, 768, 1152, seed=3 * T)
    if routing == "one_expert":
        lg = lg.float()
        lg[:, 5] += 30.0
        lg = lg.to(torch.bfloat16)
    ref = O.moe_layer_fp32(x, lg, w13, w2)
    xd, lgd, w13d, w2d = (t.to(DEV) for t in (x, lg, w13, w2))
    out_f32, out_bf16 = run_both(xd, lgd, w13d, w2d)
    out_def = run_default(xd, lgd, w13d, w2d)
    check_routing(get_workspace(DEV, T, 768, 1152, 8, 2), lg.float(), T)
    check_outputs(f"h768_T{T}_{routing}", out_f32.cpu(), out_bf16.cpu(), ref, out_def.cpu())


@pytest.mark.parametrize("E,k", [(4, 1), (16, 4), (64, 8)])
@pytest.mark.parametrize("T", [9, 70, 500])
def test_layer_other_expert_counts(T, E, k):
    """The path is built for 8 experts and top-2; other counts go through the same kernels (streaming, 64- / 128-row
    and 256-row tiles) with the two-launch routing front."""
    announce(f"layer E={E} top-{k} T={T}")
    x, lg, w13, w2 = O.make_inputs(T, 256, 512, E=E, seed=T + E)
    ref = O.moe_layer_fp32(x, lg, w13, w2, topk=k)
    xd, lgd, w13d, w2d = (t.to(DEV) for t in (x, lg, w13, w2))
    out = fused_experts(xd, w13d, w2d, lgd, k, renormalize=True, out_dtype=torch.float32, bf16_act=True)
    check_routing(get_workspace(DEV, T, 256, 512, E, k), lg.float(), T, E=E, k=k)
    st = error_stats(out.cpu(), ref)
    record(f"E{E}_k{k}_T{T}", f32=st)
    assert st["mean_rel"] <= TOL_MEAN_REL_F32 and st["max_abs"] <= TOL_MAX_ABS_F32 * float(ref.abs().max()), st
    acc = fused_experts(xd, w13d, w2d, lgd, k, renormalize=True, out_dtype=torch.float32)
    sa = error_stats(acc.cpu(), ref)
    assert sa["max_abs"] <= TARGET_MAX_ABS and sa["mean_rel"] <= TARGET_MEAN_REL, sa


@pytest.mark.parametrize("T", [96, 300])
def test_layer_mid_kernel_wide_w13_tiles(T):
    """I = 4096 makes 8 experts x 32 column tiles = one full round of CUs, so the w13 GEMM of the 64- and
    128-row kernels keeps its 256-row weight tiles (the other shapes in this file get the 128-row ones)."""
    announce(f"layer H=256 I=4096 T={T}")
    x, lg, w13, w2 = O.make_inputs(T, 256, 4096, seed=T)
    ref = O.moe_layer_fp32(x, lg, w13, w2)
    dev = [t.to(DEV) for t in (x, lg, w13, w2)]
    out_f32, out_bf16 = run_both(*dev)
    check_outputs(f"wide_T{T}", out_f32.cpu(), out_bf16.cpu(), ref, run_default(*dev).cpu())


@pytest.mark.parametrize("T", [1, 7, 33, 64])
@pytest.mark.parametrize("routing", ["normal", "two_experts", "one_expert"])
def test_layer_mid_shape_decode_cases(T, routing):
    """Streaming kernel: experts with no tokens, with more than two 16-row fragments (second pass), generic cross-check."""
    announce(f"layer mid shape decode T={T} routing={routing}")
    x, lg, w13, w2 = mid_inputs(T, routing, seed=100 + T)
    ref = O.moe_layer_fp32(x, lg, w13, w2)
    xd, lgd, w13d, w2d = (t.to(DEV) for t in (x, lg, w13, w2))
    out_f32, out_bf16 = run_both(xd, lgd, w13d, w2d)
    out_def = run_default(xd, lgd, w13d, w2d)
    check_routing(get_workspace(DEV, T, MID["H"], MID["I"], 8, 2), lg.float(), T)
    check_outputs(f"mid_dec_T{T}_{routing}", out_f32.cpu(), out_bf16.cpu(), ref, out_def.cpu())
    gen_f32, gen_bf16 = run_both(xd, lgd, w13d, w2d, flags=_lib.FLAG_FORCE_GENERIC)
    gen_def = run_default(xd, lgd, w13d, w2d, flags=_lib.FLAG_FORCE_GENERIC)
    check_outputs(f"mid_dec_T{T}_{routing}_generic", gen_f32.cpu(), gen_bf16.cpu(), ref, gen_def.cpu())


def _drawn_case(seed):
    """Shape, batch and routing of one drawn case (a fixed function of the seed)."""
    rng = np.random.default_rng(1000 + seed)
    H = int(rng.choice([64, 136, 256, 320, 512, 768, 1024, 1280, 2048]))
    I = int(rng.choice([64, 200, 256, 384, 512, 640, 1024, 1152, 1536, 2048, 3584]))
    E, k = [(8, 2), (8, 2), (8, 2), (8, 1), (4, 2), (16, 2), (2, 2), (32, 3), (64, 6)][int(rng.integers(9))]
    T = int(rng.choice([1, 2, 5, 8, 9, 16, 17, 31, 48, 64, 65, 100, 129, 192, 193, 250, 288, 352, 353, 449, 600, 897, 1300, 2049, 2100]))
    routing = ["normal", "zipf", "two_experts"][int(rng.integers(3))]
    logits_dtype = [torch.bfloat16, torch.float16, torch.float32][int(rng.integers(3))]
    return H, I, E, k, T, routing, logits_dtype, bool(rng.integers(2))


@pytest.mark.parametrize("seed", range(48))
def test_layer_drawn_shapes(seed):
    """Shapes, expert counts, batch sizes, routing skews, logit types and the renormalise switch drawn together: whatever
    kernels the library picks for the combination, routing bit-exact and outputs within the tolerances."""
    H, I, E, k, T, routing, logits_dtype, renorm = _drawn_case(seed)
    announce(f"drawn case {seed}: H={H} I={I} E={E} top-{k} T={T} {routing} logits={logits_dtype} renormalize={renorm}")
    x, lg, w13, w2 = O.make_inputs(T, H, I, E=E, seed=seed, logits=routing, logits_dtype=logits_dtype)
    ref = O.moe_layer_fp32(x, lg, w13, w2, topk=k, renormalize=renorm)
    xd, lgd, w13d, w2d = (t.to(DEV) for t in (x, lg, w13, w2))
    out = fused_experts(xd, w13d, w2d, lgd, k, renormalize=renorm, out_dtype=torch.float32, bf16_act=True)
    check_routing(get_workspace(DEV, T, H, I, E, k), lg.float(), T, E=E, k=k, renormalize=renorm)
    st = error_stats(out.cpu(), ref)
    record(f"drawn_{seed}", f32=st)
    assert st["mean_rel"] <= TOL_MEAN_REL_F32 and st["max_abs"] <= TOL_MAX_ABS_F32 * float(ref.abs().max()), st
    acc = fused_experts(xd, w13d, w2d, lgd, k, renormalize=renorm, out_dtype=torch.float32)
    sa = error_stats(acc.cpu(), ref)
    assert sa["max_abs"] <= TARGET_MAX_ABS and sa["mean_rel"] <= TARGET_MEAN_REL, sa
    out_b = fused_experts(xd, w13d, w2d, lgd, k, renormalize=renorm)
    sb = error_stats(out_b.float().cpu(), ref)
    assert sb["mean_rel"] <= TOL_MEAN_REL_BF16, sb


@pytest.mark.parametrize("I", [128, 256, 384, 512, 640])
@pytest.mark.parametrize("T", [500, 1300])
def test_layer_256_row_kernel_with_short_reductions(T, I):
    """The 256-row kernels request their operands one to three K steps ahead; with I / 2 = 64 ... 320 the w2 GEMM has
    one to five K steps per slice (H = 256: four for the w13 GEMM), which walks the first and last steps of the copy
    schedule without the steady state in between, in every flag combination that changes that schedule."""
    announce(f"256-row kernel, short reductions: T={T} H=256 I={I}")
    x, lg, w13, w2 = O.make_inputs(T, 256, I, seed=T + I, logits="zipf")
    ref = O.moe_layer_fp32(x, lg, w13, w2)
    xd, lgd, w13d, w2d = (t.to(DEV) for t in (x, lg, w13, w2))
    outs = {}
    for name, flags in (("default", 0), ("no_queue", _lib.FLAG_NO_PERSIST), ("bf16_act", _lib.FLAG_BF16_ACT)):
        outs[name] = fused_experts(xd, w13d, w2d, lgd, 2, out_dtype=torch.float32, flags=flags)
    outs["w2_f16"] = fused_experts(xd, w13d, w2d.to(torch.float16), lgd, 2, out_dtype=torch.float32)
    check_routing(get_workspace(DEV, T, 256, I, 8, 2), lg.float(), T)
    for name, out in outs.items():
        st = error_stats(out.cpu(), ref)
        if name == "bf16_act":
            assert st["mean_rel"] <= TOL_MEAN_REL_F32 and st["max_abs"] <= TOL_MAX_ABS_F32 * float(ref.abs().max()), (name, st)
        else:
            assert st["max_abs"] <= TARGET_MAX_ABS and st["mean_rel"] <= TARGET_MEAN_REL, (name, st)
    assert torch.equal(outs["default"], outs["no_queue"])


def test_layer_shape_only_the_generic_kernel_supports():
    """H and I that are multiples of 8 but fit neither tuned kernel."""
    announce("layer odd shape H=136 I=200")
    for T in (5, 70, 300):
        x, lg, w13, w2 = O.make_inputs(T, 136, 200, seed=T)
        ref = O.moe_layer_fp32(x, lg, w13, w2)
        dev = [t.to(DEV) for t in (x, lg, w13, w2)]
        out_f32, out_bf16 = run_both(*dev)
        check_outputs(f"odd_T{T}", out_f32.cpu(), out_bf16.cpu(), ref, run_default(*dev).cpu())
