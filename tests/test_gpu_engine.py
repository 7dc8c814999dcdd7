"""The end-to-end harness on a scaled-down Mixtral (2 layers) against oracle/model_oracle.py, the float32 CPU
restatement without a KV cache: greedy generation of fixed prompts with a KV cache small enough to force a preemption
and two prompts that share a two-block prefix (a prefix-cache hit).

The GPU model computes in bf16, so the comparison is made where it is meaningful: at every step of every request the
engine's next-token logits must match, for the same token prefix, (a) the restatement evaluated with a bf16 model's
rounding points (float32 arithmetic between them) to a few bf16 steps of the logits, and (b) the plain float32
restatement within the noise of bf16 storage; and the token the engine picked must be the restatement's arg-max or
within that tolerance of it (a bf16 pipeline cannot resolve closer calls).  Positions at which two experts' router
logits nearly tie are held to a loose bound only: the layer is discontinuous there."""
import pytest
import torch

from electrock_infer_amd.harness import LLMEngine, ModelConfig, SamplingParams
from oracle import model_oracle as M
from tests.gpu_util import announce

pytestmark = pytest.mark.gpu

LOGIT_TOL_MAX = 0.04      # against the bf16-point restatement; logits reach +-2 here, where a bf16 step is 0.0078
LOGIT_TOL_MEAN_REL = 2e-2  # against the float32 restatement (logits have a standard deviation of about 0.45)
# Where the router logits of the last selected and the first rejected expert lie closer than this (relative to the
# row's largest logit), the bf16 pipeline may pick the other expert: the layer jumps there, so such positions get the
# loose bound only.  bf16 hidden states move a router logit by about 1 % of its magnitude.
ROUTING_MARGIN = 0.04
LOGIT_TOL_MAX_AMBIGUOUS = 0.4


def small_config():
    return ModelConfig(vocab_size=1000, hidden_size=512, intermediate_size=1024, num_hidden_layers=2,
                       num_attention_heads=8, num_key_value_heads=2, num_local_experts=8, num_experts_per_tok=2,
                       rope_theta=10000.0, max_position_embeddings=512)


def make_prompts():
    g = torch.Generator().manual_seed(1234)
    draw = lambda n: torch.randint(0, 1000, (n,), generator=g).tolist()
    shared = draw(64)                                   # two whole KV blocks
    prompts = [draw(70), shared + draw(9), draw(33), shared + draw(30), draw(100), draw(5)]
    max_tokens = [24, 10, 40, 12, 8, 30]
    return prompts, max_tokens


@pytest.mark.parametrize("fused_tail", [True, False])
def test_greedy_generation_matches_the_float32_restatement(fused_tail):
    announce(f"engine harness, 2-layer model, fused_moe_tail={fused_tail}")
    cfg = small_config()
    engine = LLMEngine(cfg, num_kvcache_blocks=13, max_num_batched_tokens=256, max_num_seqs=8, max_model_len=512,
                       eos=-1, seed=5, fused_moe_tail=fused_tail)
    model = engine.model_runner.model
    model.init_random_weights(seed=5, gate_std=0.05)
    params = {k: v.detach().float().cpu() for k, v in model.state_dict().items() if ".moe_tail." not in k}

    seen = []          # (seq_id, tokens the logits were computed from, logits row, cached tokens at that step)
    def hook(seqs, is_prefill, logits):
        rows = logits.float().cpu()
        for s, row in zip(seqs, rows):
            seen.append((s.seq_id, list(s.token_ids), row, s.num_cached_tokens if is_prefill else -1))
    engine.step_hook = hook

    prompts, max_tokens = make_prompts()
    outs = engine.generate(prompts, [SamplingParams(temperature=0.0, max_tokens=m, ignore_eos=True) for m in max_tokens])
    assert [len(o["token_ids"]) for o in outs] == max_tokens
    st = engine.stats
    assert st["preemptions"] >= 1, st                                     # the small cache did force one
    assert any(c >= 64 for _, _, _, c in seen), "no prefill step found its prefix in the cache"
    assert st["prefill_steps"] >= 2 and st["decode_steps"] >= max(max_tokens) - 1
    assert engine.planner.pool.num_free == 13      # everything was given back

    # one restatement pass per request over its final tokens gives the logits of every prefix
    final = {}
    for (sid, toks, _, _) in seen:
        if sid not in final or len(toks) > len(final[sid]):
            final[sid] = toks
    ref, ref32, margin = {}, {}, {}
    for sid, toks in final.items():
        # the last step's prefix is the longest one seen; its successor token is not needed
        ref[sid], margin[sid] = M.model_logits(params, cfg, toks, routing_margin=True, bf16_points=True)
        ref32[sid], m32 = M.model_logits(params, cfg, toks, routing_margin=True)
        margin[sid] = torch.minimum(margin[sid], m32)
    worst_abs, sum_abs, sum_ref, close_calls, ambiguous = 0.0, 0.0, 0.0, 0, 0
    by_seq, per_step = {}, []
    for sid, toks, row, cached in seen:
        want = ref[sid][len(toks) - 1]
        d = (row - want).abs()
        picked = int(row.argmax())
        by_seq.setdefault(sid, []).append((len(toks), picked))
        if float(margin[sid][len(toks) - 1]) < ROUTING_MARGIN:
            ambiguous += 1
            assert float(d.max()) <= LOGIT_TOL_MAX_AMBIGUOUS, (sid, len(toks), float(d.max()))
            continue
        per_step.append((round(float(d.max()), 4), sid, len(toks), cached))
        worst_abs = max(worst_abs, float(d.max()))
        want32 = ref32[sid][len(toks) - 1]
        sum_abs += float((row - want32).abs().sum())
        sum_ref += float(want32.abs().sum())
        gap = float(want.max() - want[picked])
        assert gap <= 2 * LOGIT_TOL_MAX, (sid, len(toks), gap)            # the engine's pick is the arg-max, or a near tie
        close_calls += gap > 0
    print(f"[engine] largest step errors (max-abs, request, tokens, cached tokens or -1 for decode): {sorted(per_step)[-6:]}")
    print(f"[engine] {len(seen)} steps, {ambiguous} of them with an ambiguous routing; the others: max-abs {worst_abs:.4f} against the bf16-point restatement, mean-rel {sum_abs / sum_ref:.2e} against float32, "
          f"{close_calls} near ties, stats {st}", flush=True)
    assert ambiguous <= len(seen) // 3
    assert worst_abs <= LOGIT_TOL_MAX and sum_abs / sum_ref <= LOGIT_TOL_MEAN_REL
    # the completions are the tokens picked step by step (a re-prefilled request repeats a step: same pick expected)
    order = sorted(final)
    for o, sid, prompt in zip(outs, order, prompts):
        picks = dict(by_seq[sid])
        assert o["token_ids"] == [picks[n] for n in range(len(prompt), len(prompt) + len(o["token_ids"]))]


def test_sampled_generation_runs_and_respects_limits():
    announce("engine harness, temperature sampling")
    engine = LLMEngine(small_config(), num_kvcache_blocks=40, max_num_batched_tokens=512, max_num_seqs=4,
                       max_model_len=512, eos=7, seed=1)
    prompts, _ = make_prompts()
    sps = [SamplingParams(temperature=0.8, max_tokens=6 + i, ignore_eos=(i % 2 == 0)) for i in range(len(prompts))]
    outs = engine.generate(prompts, sps)
    for i, (o, sp) in enumerate(zip(outs, sps)):
        toks = o["token_ids"]
        assert 1 <= len(toks) <= sp.max_tokens and all(0 <= t < 1000 for t in toks)
        if sp.ignore_eos:
            assert len(toks) == sp.max_tokens
        elif len(toks) < sp.max_tokens:
            assert toks[-1] == 7
    assert engine.is_finished()
