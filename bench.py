#!/usr/bin/env python3
"""Benchmark of the Mixtral MoE layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--tokens T] [--shape 8x7b|8x22b] [--mode MODE]
                    [--routing normal|zipf|two_experts|balanced] [--no-cpu] [--no-table] [--no-e2e] [--detail FILE]

A "step" is one call of the layer (router, expert sort, w13 GEMM + SiLU*mul,
w2 GEMM, top-k combine) on one batch of T tokens resident in HBM.  The headline
workload is the decode batch T=64 of the 8x7B shape (H=4096, I=14336, E=8,
top-2 renormalised, bf16, N(0,1) router logits); `value` is T / (time per step).

Modes (flag sets of em_moe_forward; every row names its mode and carries the errors of that very
mode against the fp32 oracle on sampled tokens):
  default_f32out   what the drop-in FusedMoE layer computes (w2 held as float16 by the loader, fp16
                   activations, w2 partial sums of large batches as fp16 with a float32 escape) with a float32 output -- the form the stated tolerance
                   (max-abs 2e-2, mean relative 1e-3 against an fp32 reference) is defined on.  The headline.
  default          the same with the bf16 output FusedMoE.forward returns (the output rounding alone is
                   1.4e-3 mean relative)
  w2_bf16_f32out   w2 left in the checkpoint's bfloat16 (FusedMoE(..., w2_dtype=torch.bfloat16), flags = 0 of
                   the C ABI): the w2 kernel converts its weight fragments on the way to the MFMA
  bf16_act         activations stored as bf16 between the GEMMs (the reference's type), bf16 w2, bf16 output
  f32_partials_f32out
                   the headline's form with float32 partial sums of the w2 GEMM at every batch size

One JSON line is printed, short enough to survive an 8 KB tail.  Besides the contract fields it carries
  roofline      the dominant kernel of the headline batch (w13 GEMM + SiLU*mul), timed alone with HIP events on
                the stream it is launched on, against 8 TB/s of HBM; nested in it `prefill`: the same kernel of
                the T=8192 batch against the dense bf16 MFMA peak
  cpu_baseline  the reference-style torch CPU expert loop (oracle port) timed on the host cores on the same workload
  rows          one compact row per (shape, T, routing, mode): ms per call, tokens/s, fraction of the HBM and of the
                MFMA roofline (algorithmic bytes / flops of the layer), errors, and whether the tolerance is met;
                the 8x22B shape and the end-to-end generation run are rows too
--detail FILE writes the unabridged measurements (stage times, latency percentiles) as JSON.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 (fp16 is the same)
SHAPES = {"8x7b": (4096, 14336), "8x22b": (6144, 16384)}
H, I, E, TOPK = 4096, 14336, 8, 2
SHAPE = "8x7b"


def set_shape(name):
    global H, I, SHAPE
    SHAPE = name
    H, I = SHAPES[name]


OPERANDS = "gaussian"
# mode name -> flags of em_moe_forward (numeric values of include/electrock_moe.h)
F_OUT_F32, F_W2_F16, F_BF16_ACT, F_F32_PARTIALS = 1 << 0, 1 << 3, 1 << 5, 1 << 7
MODES = {
    "default_f32out": F_W2_F16 | F_OUT_F32,
    "default": F_W2_F16,
    "w2_bf16_f32out": F_OUT_F32,
    "bf16_act": F_BF16_ACT,
    "f32_partials_f32out": F_W2_F16 | F_F32_PARTIALS | F_OUT_F32,
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--tokens", type=int, default=64, help="batch size T of the headline workload")
    ap.add_argument("--routing", choices=["normal", "zipf", "two_experts", "balanced"], default="normal",
                    help="router logits of the headline workload: N(0,1) (default), N(0,1) + a Zipf bias per expert, "
                         "two experts far ahead, or exactly 2T/E rows per expert (the best case of the tiled kernels)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-table", action="store_true", help="skip the other batch sizes")
    ap.add_argument("--no-e2e", action="store_true", help="skip the end-to-end generation row")
    ap.add_argument("--e2e-layers", type=int, default=32, help="decoder layers of the end-to-end model")
    ap.add_argument("--e2e-requests", type=int, default=100, help="requests of the end-to-end run")
    ap.add_argument("--shape", choices=sorted(SHAPES), default="8x7b",
                    help="8x7b: H=4096 I=14336 (the headline); 8x22b: H=6144 I=16384")
    ap.add_argument("--mode", choices=sorted(MODES), default="default_f32out",
                    help="flag set of the headline workload (see the module docstring)")
    ap.add_argument("--extra-flags", type=lambda v: int(v, 0), default=0,
                    help="diagnostic: flag bits OR-ed into every layer call (include/electrock_moe_diag.h, "
                         "e.g. 0x20000 = EM_FLAG_NO_PERSIST)")
    ap.add_argument("--no-errors", action="store_true",
                    help="skip the error measurement against the fp32 oracle (it copies the weights to the host)")
    ap.add_argument("--weight-sets", type=int, default=1,
                    help="cycle the calls through N independently drawn sets of expert weights (N x 2.8 GB), so that no "
                         "call finds the weights of the one before in a cache")
    ap.add_argument("--operands", choices=["gaussian", "zeros"], default="gaussian",
                    help="values of x and the expert weights.  'zeros' is a diagnostic: the matrix pipes then draw "
                         "little power and the same kernels run at the full shader clock, which separates the "
                         "board's power limit from the kernels' own stalls; never the headline")
    ap.add_argument("--vendor-gemm", action="store_true",
                    help="diagnostic: time the library's dense bf16 GEMM of the w13 GEMM's size (torch.matmul, "
                         "[tokens*top_k, H] x [2I, H]^T) on the same operand distributions, print it and exit")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run three device copies of 1 GiB (a plain copy kernel of known size that the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run are scaled by)")
    ap.add_argument("--detail", default=None, help="write the unabridged measurements to this JSON file")
    return ap.parse_args()


def make_weights(torch, dev, seed=0):
    g = torch.Generator(device=dev).manual_seed(seed)
    if OPERANDS == "zeros":
        return (torch.zeros(E, 2 * I, H, device=dev, dtype=torch.bfloat16),
                torch.zeros(E, H, I, device=dev, dtype=torch.bfloat16))
    w13 = torch.empty(E, 2 * I, H, device=dev, dtype=torch.bfloat16)
    w2 = torch.empty(E, H, I, device=dev, dtype=torch.bfloat16)
    for e in range(E):
        w13[e] = (torch.randn(2 * I, H, generator=g, device=dev, dtype=torch.float32) * 0.02).to(torch.bfloat16)
        w2[e] = (torch.randn(H, I, generator=g, device=dev, dtype=torch.float32) * 0.02).to(torch.bfloat16)
    return w13, w2


def make_batch(torch, dev, T, seed=0, logits="normal"):
    g = torch.Generator(device=dev).manual_seed(1000 + seed)
    x = torch.randn(T, H, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    if OPERANDS == "zeros":
        x.zero_()
    lg = torch.randn(T, E, generator=g, device=dev, dtype=torch.float32)
    if logits == "zipf":
        ranks = torch.arange(1, E + 1, dtype=torch.float32) ** -1.2
        perm = torch.randperm(E, generator=torch.Generator().manual_seed(seed))
        lg = lg + torch.log(ranks / ranks.sum())[perm].to(dev)
    elif logits == "two_experts":
        lg[:, :2] += 20.0
    elif logits == "balanced":  # token t -> experts 2t, 2t+1 (mod E): every expert gets exactly 2T/E rows
        t = torch.arange(T, device=dev)
        lg = torch.full_like(lg, -10.0)
        lg[t, (2 * t) % E] = 10.0
        lg[t, (2 * t + 1) % E] = 5.0
    return x, lg.to(torch.bfloat16)


class Weights:
    """One set of expert weights on the device: w13 and w2 as drawn (bfloat16, the checkpoint's type) and, made once
    on first use, the float16 copy of w2 that the loader of the drop-in layer keeps."""

    def __init__(self, w13, w2):
        self.w13, self.w2_bf16, self._w2_f16 = w13, w2, None

    def w2(self, torch, flags):
        if not flags & F_W2_F16:
            return self.w2_bf16
        if self._w2_f16 is None:
            self._w2_f16 = self.w2_bf16.to(torch.float16)
        return self._w2_f16


class LayerRunner:
    """Calls em_moe_forward through the C ABI with pre-allocated buffers."""

    extra_weight_sets = []      # [Weights, ...] cycled through together with the set given to the constructor
    extra_flags = 0             # diagnostic flag bits added to every call

    def __init__(self, torch, T, weights, x, lg, mode_flags):
        import ctypes
        from electrock_infer_amd import _lib
        from electrock_infer_amd.layers.moe.fused_moe import MoeWorkspace
        self.torch, self._lib, self.ctypes = torch, _lib, ctypes
        self.T, self.x, self.lg, self.mode_flags = T, x, lg, mode_flags
        # every set's w2 in the type the mode takes, converted here, outside every timed call
        self.sets = [(w.w13, w.w2(torch, mode_flags)) for w in [weights] + LayerRunner.extra_weight_sets]
        self.calls = 0
        self.ws = MoeWorkspace(x.device, T, H, I, E, TOPK, mode_flags)
        self.out = torch.empty(T, H, device=x.device, dtype=torch.float32 if mode_flags & F_OUT_F32 else torch.bfloat16)
        self.lib = _lib.load()

    def __call__(self, flags=0):
        w13, w2 = self.sets[self.calls % len(self.sets)]
        self.calls += 1
        code = self.lib.em_moe_forward(
            self.x.data_ptr(), self.lg.data_ptr(), self._lib.DTYPE_BF16, w13.data_ptr(), w2.data_ptr(),
            self.out.data_ptr(), self.T, H, I, E, TOPK, 1, self.ws.buffer.data_ptr(),
            self.ctypes.c_size_t(self.ws.buffer.numel()), flags | self.mode_flags | LayerRunner.extra_flags,
            self.torch.cuda.current_stream().cuda_stream)
        self._lib.check(code, "em_moe_forward")

    def n_active(self):
        return int(self.ws.topk_ids().unique().numel())


def time_calls(torch, fn, steps, warmup):
    """Average milliseconds per call: HIP events on the current stream around `steps` calls."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return start.elapsed_time(stop) / steps, wall_ms


def latency_percentiles(torch, fn, calls):
    """p10 / p50 / p90 of single calls in microseconds, each between its own pair of events."""
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(calls)]
    for a, b in ev:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    us = sorted(a.elapsed_time(b) * 1e3 for a, b in ev)
    return {"p10": us[len(us) // 10], "p50": us[len(us) // 2], "p90": us[(len(us) * 9) // 10], "calls": calls}


def layer_bytes(T, n_active):
    """Algorithmic HBM bytes of one layer call: active expert weights once, x in, out, logits."""
    return n_active * 3 * H * I * 2 + 2 * T * H * 2 + T * E * 2


def layer_flops(T):
    return T * TOPK * 6 * H * I


class HostWeights:
    """fp32 copies of the expert weights on the host, for the oracle (error measurement and CPU baseline)."""

    def __init__(self, weights):
        self.w13, self.w2 = weights.w13.cpu().float(), weights.w2_bf16.cpu().float()


def layer_errors(torch, run, host, max_rows=64):
    """max-abs and mean relative error of the runner's last output against the fp32 oracle on up to `max_rows`
    tokens spread over the batch (the layer is token-wise).  Outside every timed region."""
    from oracle import moe_oracle as O
    T = run.T
    rows = list(range(T)) if T <= max_rows else [int(i * (T - 1) / (max_rows - 1)) for i in range(max_rows)]
    idx = torch.as_tensor(rows, device=run.x.device)
    ref = O.moe_layer_fp32(run.x[idx].float().cpu(), run.lg[idx].float().cpu(), host.w13, host.w2)
    d = (run.out[idx].double().cpu() - ref.double()).abs()
    return {"max_abs": float(d.max()), "mean_rel": float(d.mean() / ref.double().abs().mean()), "rows": len(rows),
            "against": "oracle.moe_layer_fp32"}


def measure(torch, T, weights, steps, warmup, logits="normal", mode="default_f32out", host=None, stages=False,
            percentiles=False):
    from electrock_infer_amd import _lib
    x, lg = make_batch(torch, weights.w13.device, T, logits=logits)
    run = LayerRunner(torch, T, weights, x, lg, MODES[mode])
    run()
    torch.cuda.synchronize()
    na = run.n_active()
    # with several weight sets the last output belongs to another set than the host copy: no error figures then
    errors = layer_errors(torch, run, host) if host is not None and len(run.sets) == 1 else None
    ms, wall_ms = time_calls(torch, run, steps, warmup)
    pct = latency_percentiles(torch, run, min(steps, 100)) if percentiles else None
    only = lambda keep: (_lib.FLAG_SKIP_ROUTER | _lib.FLAG_SKIP_ALIGN | _lib.FLAG_SKIP_GEMM1 |
                         _lib.FLAG_SKIP_GEMM2 | _lib.FLAG_SKIP_COMBINE) & ~keep
    stage = {}
    if stages:
        for name, flag in (("gemm1", _lib.FLAG_SKIP_GEMM1), ("gemm2", _lib.FLAG_SKIP_GEMM2),
                           ("router", _lib.FLAG_SKIP_ROUTER), ("align", _lib.FLAG_SKIP_ALIGN),
                           ("combine", _lib.FLAG_SKIP_COMBINE)):
            stage[name] = time_calls(torch, lambda f=only(flag): run(f), steps, max(2, warmup // 4))[0]
    r = {"shape": SHAPE, "T": T, "logits": logits, "mode": mode, "ms": ms, "wall_ms": wall_ms, "n_active": na,
         "stage_ms": stage, "latency_us": pct, "tokens_per_s": T / ms * 1e3, "hbm_gbs": layer_bytes(T, na) / ms / 1e6,
         "tflops": layer_flops(T) / ms / 1e9, "errors": errors,
         "errors_note": None if errors is not None or host is None else "not measured: the calls cycle through several weight sets"}
    r["hbm_frac"] = r["hbm_gbs"] / HBM_PEAK_GBS
    r["mfma_frac"] = r["tflops"] / MFMA_BF16_PEAK_TFLOPS
    if errors is not None:
        r["meets_tolerance"] = bool(errors["max_abs"] <= 2e-2 and errors["mean_rel"] <= 1e-3)
    return r


def sig(v, digits=4):
    """A float rounded to `digits` significant digits (the JSON line has to stay short)."""
    return None if v is None else float(f"{v:.{digits}g}")


def compact(r):
    """One short row of the printed line."""
    e = r.get("errors") or {}
    return {"shape": r["shape"], "T": r["T"], "routing": r["logits"], "mode": r["mode"], "ms": sig(r["ms"]),
            "tok_s": sig(r["tokens_per_s"]), "hbm": sig(r["hbm_frac"], 3), "mfma": sig(r["mfma_frac"], 3),
            "max_abs": sig(e.get("max_abs"), 3), "mean_rel": sig(e.get("mean_rel"), 3), "ok": r.get("meets_tolerance")}


def cpu_baseline(torch, T, dev, host):
    """Reference-style torch CPU expert loop (oracle port) on the same workload, host cores."""
    from oracle import moe_oracle as O
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or (os.cpu_count() or 1))
    torch.set_num_threads(cores)
    x, lg = make_batch(torch, dev, T)
    xc, lc = x.float().cpu(), lg.float().cpu()
    w13c, w2c = host.w13, host.w2                        # the CPU path holds fp32 weights
    O.moe_layer_fp32(xc, lc, w13c, w2c)                  # warm-up
    iters, t0 = 0, time.perf_counter()
    while iters < 3 or (time.perf_counter() - t0 < 10.0 and iters < 200):
        O.moe_layer_fp32(xc, lc, w13c, w2c)
        iters += 1
    sec = (time.perf_counter() - t0) / iters
    return {"value": sig(T / sec, 5), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"{iters} calls of oracle.moe_layer_fp32 (fp32 torch expert loop), same T={T} batch, "
                      f"{sec * 1e3:.0f} ms per call"}


def measured_traffic(T):
    """HBM bytes per launch of the dominant kernel from the committed rocprofv3 --pmc summary
    (FETCH_SIZE + WRITE_SIZE, scaled by the copy-kernel calibration) and where that figure comes from; (None, None)
    when no summary covers this shape and batch size.  It is a property of the kernel, measured in profiler runs of
    their own (counters cannot be read inside this process), not of this run."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            entry = json.load(f).get(f"T{T}" if SHAPE == "8x7b" else f"{SHAPE}_T{T}")
    except (OSError, ValueError):
        return None, None
    if not entry:
        return None, None
    return entry.get("dominant_kernel_hbm_bytes"), entry.get("summary")


def w13_roofline(r):
    """The roofline object of the w13 GEMM + SiLU*mul launch of measured row `r` (needs its stage times)."""
    T, g1_ms = r["T"], r["stage_ms"]["gemm1"]
    traffic, src = measured_traffic(T)
    if T <= 1024:
        # the w13 GEMM streams 2/3 of the weight bytes; HBM-bound
        work = r["n_active"] * 2 * I * H * 2 + T * H * 2   # w13 of the active experts + x
        out = {"kernel": "w13 GEMM + SiLU*mul", "bound": "hbm", "achieved": work / g1_ms / 1e6, "peak": HBM_PEAK_GBS,
               "unit": "GB/s"}
    else:
        # 4*H*I flops per routed slot in the w13 GEMM; MFMA-bound
        work = T * TOPK * 4 * H * I
        out = {"kernel": "w13 GEMM + SiLU*mul", "bound": "mfma", "achieved": work / g1_ms / 1e9,
               "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s"}
    out.update({"frac": out["achieved"] / out["peak"], "traffic": traffic, "traffic_source": src, "per_launch": work,
                "avg_launch_ms": g1_ms, "tokens": T})
    return out


def calibrate_copy(torch, dev):
    src = torch.ones(1 << 28, dtype=torch.float32, device=dev)   # 1 GiB read + 1 GiB written per copy
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst


def vendor_gemm(torch, dev, T, steps, warmup):
    """What the same board does on a dense problem of the w13 GEMM's flops: a yardstick for the power limit."""
    M, N, K = T * TOPK, 2 * I, H
    if OPERANDS == "zeros":
        a = torch.zeros(M, K, device=dev, dtype=torch.bfloat16)
        b = torch.zeros(N, K, device=dev, dtype=torch.bfloat16)
    else:
        g = torch.Generator(device=dev).manual_seed(0)
        a = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
        b = (torch.randn(N, K, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    c = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
    bt = b.t()
    ms, _ = time_calls(torch, lambda: torch.matmul(a, bt, out=c), steps, warmup)
    return {"diagnostic": "library dense bf16 GEMM (torch.matmul)", "M": M, "N": N, "K": K, "operands": OPERANDS,
            "ms": ms, "tflops": 2.0 * M * N * K / ms / 1e9, "frac_of_peak": 2.0 * M * N * K / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS}


def e2e_row(torch, layers, num_requests):
    """The end-to-end configuration: a Mixtral-8x7B-shaped random-init bf16 model (GQA 32q/8kv heads, head_dim 128,
    vocab 32000) generating for `num_requests` requests with prompts of 100-1024 uniform token ids and 100-256 output
    tokens (ignore_eos, temperature 0.6) through the harness's scheduler and paged KV cache, as the reference's
    bench.py:8-32 does.  Reports output tokens/s and the share of the GPU time spent in the MoE tail of the decoder
    layers (post-attention norm + gate + router + experts), from HIP events around those calls."""
    from random import Random
    from electrock_infer_amd.harness import LLMEngine, ModelConfig, SamplingParams
    rnd = Random(0)
    t0 = time.perf_counter()
    engine = LLMEngine(ModelConfig(num_hidden_layers=layers), max_model_len=4096, max_num_seqs=300,
                       max_num_batched_tokens=32768, gpu_memory_utilization=0.90)
    build_s = time.perf_counter() - t0
    prompts = [[rnd.randrange(0, 32000) for _ in range(rnd.randint(100, 1024))] for _ in range(num_requests)]
    sps = [SamplingParams(temperature=0.6, ignore_eos=True, max_tokens=rnd.randint(100, 256)) for _ in range(num_requests)]
    engine.generate([[rnd.randrange(0, 32000) for _ in range(40)]], SamplingParams(temperature=0.6, max_tokens=8, ignore_eos=True))
    events = []
    for layer in engine.model_runner.model.model.layers:
        layer.moe_events = events
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    outs = engine.generate(prompts, sps)
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    moe_ms = sum(a.elapsed_time(b) for a, b in events)
    gpu_ms = start.elapsed_time(stop)
    out_tokens = sum(len(o["token_ids"]) for o in outs)
    st = engine.stats
    row = {"row": "e2e", "layers": layers, "requests": num_requests, "prompt_tokens": sum(len(p) for p in prompts),
           "output_tokens": out_tokens, "wall_s": wall, "output_tokens_per_s": out_tokens / wall,
           "moe_share_of_gpu_time": moe_ms / gpu_ms, "moe_ms": moe_ms, "gpu_ms": gpu_ms,
           "prefill_tokens_per_s": st["prefill_tokens"] / max(st["prefill_s"], 1e-9),
           "decode_tokens_per_s": st["decode_tokens"] / max(st["decode_s"], 1e-9), "engine_stats": st,
           "kv_blocks": engine.config.num_kvcache_blocks, "model_build_s": build_s,
           "attention": "torch scaled_dot_product_attention over the gathered paged cache (harness, not the hot path)"}
    del engine, events
    from electrock_infer_amd.layers.moe.fused_moe import release_workspaces
    release_workspaces()
    torch.cuda.empty_cache()
    return row


def compact_e2e(r):
    return {"row": "e2e", "layers": r["layers"], "requests": r["requests"], "wall_s": sig(r["wall_s"]),
            "out_tok_s": sig(r["output_tokens_per_s"]), "prefill_tok_s": sig(r["prefill_tokens_per_s"]),
            "decode_tok_s": sig(r["decode_tokens_per_s"]), "moe_share": sig(r["moe_share_of_gpu_time"], 3)}


def main():
    global OPERANDS
    args = parse_args()
    OPERANDS = args.operands
    set_shape(args.shape)
    if args.gpus != 1:
        print("bench.py measures one GPU: all experts are resident on a single MI355X and the layer uses "
              "no collectives; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    from electrock_infer_amd import _lib
    _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.calibrate_copy:
        calibrate_copy(torch, dev)
    if args.vendor_gemm:
        print(json.dumps(vendor_gemm(torch, dev, args.tokens, min(args.steps, 30), min(args.warmup, 5))))
        return
    weights = Weights(*make_weights(torch, dev))
    LayerRunner.extra_flags = args.extra_flags
    LayerRunner.extra_weight_sets = [Weights(*make_weights(torch, dev, seed=s)) for s in range(1, args.weight_sets)]
    need_host = not (args.no_cpu and args.no_errors) and OPERANDS == "gaussian"
    host = HostWeights(weights) if need_host else None
    err_host = None if args.no_errors else host

    T = args.tokens
    head = measure(torch, T, weights, args.steps, args.warmup, logits=args.routing, mode=args.mode, host=err_host,
                   stages=True, percentiles=True)
    roofline = w13_roofline(head)

    detail = []
    if not args.no_table:
        # (the rows' own step counts: short runs of a few calls right after a change of batch size scatter by 10 %)
        half_steps, half_warm = max(50, args.steps // 2), max(10, args.warmup // 2)
        big = 8192 if args.shape == "8x7b" else 4096
        # the tolerance-meeting mode at every named batch size
        for t in ((1, 8, 32, 64, 256, 512, 1024, 2048) if args.shape == "8x7b" else (1, 64)):
            if t != T or args.mode != "default_f32out":
                detail.append(measure(torch, t, weights, half_steps if t <= 256 else 30, half_warm, host=err_host))
        if args.shape == "8x7b":
            # uneven routing at decode and mid sizes (the kernels there are chosen by batch size: an expert far above the
            # average must not cost a second pass over its weights)
            for t in (64, 256):
                detail.append(measure(torch, t, weights, half_steps, half_warm, logits="zipf", host=err_host))
        for lgk in (("normal", "zipf", "two_experts") if args.shape == "8x7b" else ("normal",)):
            detail.append(measure(torch, big, weights, 20, 5, logits=lgk, host=err_host, stages=lgk == "normal"))
            if lgk == "normal":
                pre = w13_roofline(detail[-1])
                g2_ms = detail[-1]["stage_ms"]["gemm2"]
                roofline["prefill"] = {k: pre[k] for k in ("tokens", "kernel", "bound", "achieved", "peak", "unit", "frac",
                                                           "per_launch", "avg_launch_ms", "traffic", "traffic_source")}
                roofline["prefill"].update({"w2_launch_ms": g2_ms,
                                            "w2_frac": big * TOPK * 2 * H * I / g2_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS,
                                            "layer_frac": detail[-1]["mfma_frac"]})
        # the other modes at the headline batch and at the prefill batch
        for mode in ("default", "w2_bf16_f32out", "bf16_act"):
            if mode != args.mode:
                detail.append(measure(torch, T, weights, half_steps, half_warm, mode=mode, host=err_host))
        for mode in ("default", "w2_bf16_f32out", "f32_partials_f32out", "bf16_act"):
            detail.append(measure(torch, big, weights, 20, 5, mode=mode, host=err_host))

    cpu = None if (args.no_cpu or host is None) else cpu_baseline(torch, T, dev, host)
    rows = [compact(r) for r in detail]
    if not args.no_table and args.shape == "8x7b" and OPERANDS == "gaussian":
        # the other Mixtral shape: H=6144, I=16384 (4.8 GB of expert weights), on weights of its own
        del weights, host, err_host
        LayerRunner.extra_weight_sets = []
        torch.cuda.empty_cache()
        set_shape("8x22b")
        w22 = Weights(*make_weights(torch, dev, seed=22))
        host22 = None if args.no_errors else HostWeights(w22)
        for t in (1, 64, 4096):
            detail.append(measure(torch, t, w22, 50 if t <= 64 else 20, 10 if t <= 64 else 5, host=host22))
            rows.append(compact(detail[-1]))
        del w22, host22
        set_shape(args.shape)
        torch.cuda.empty_cache()
        if not args.no_e2e:
            detail.append(e2e_row(torch, args.e2e_layers, args.e2e_requests))
            rows.append(compact_e2e(detail[-1]))

    for k in ("achieved", "frac", "avg_launch_ms"):
        roofline[k] = sig(roofline[k], 5)
    if "prefill" in roofline:
        for k in ("achieved", "frac", "avg_launch_ms", "w2_launch_ms", "w2_frac", "layer_frac"):
            roofline["prefill"][k] = sig(roofline["prefill"][k], 5)
    e = head["errors"] or {}
    result = {
        "metric": f"Mixtral-{args.shape.upper().replace('X', 'x')} MoE layer tokens/s", "value": head["tokens_per_s"], "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic" if args.operands == "gaussian" else "synthetic, all-zero x and weights (diagnostic)",
        "config": {"workload": f"Mixtral-{args.shape} MoE layer T={T}: H={H} I={I} E={E} top-{TOPK} renormalised, "
                               f"x~N(0,1), w~N(0,0.02), logits~N(0,1)" +
                               ("" if args.routing == "normal" else f", routing {args.routing}"),
                   "tokens": T, "n_active_experts": head["n_active"], "mode": args.mode, "flags": MODES[args.mode],
                   "w2_dtype": "f16 copy of the bf16 weights (loader)" if MODES[args.mode] & F_W2_F16 else "bf16",
                   "max_abs_err": sig(e.get("max_abs"), 3), "mean_rel_err": sig(e.get("mean_rel"), 3),
                   "err_rows": e.get("rows"), "err_against": e.get("against"),
                   "meets_tolerance_2e-2_1e-3": head.get("meets_tolerance"), "weight_sets": args.weight_sets},
        "latency_us": {k: sig(v) for k, v in head["latency_us"].items()},
        "layer_hbm_frac": sig(head["hbm_frac"]), "stage_ms": {k: sig(v) for k, v in head["stage_ms"].items()},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "rows": rows,
    }
    if args.detail:
        with open(args.detail, "w") as f:
            json.dump({"head": head, "rows": detail, "line": result}, f, indent=1)
    print(json.dumps(result, separators=(",", ":")))


if __name__ == "__main__":
    main()
