"""Serving benchmark on one MI355X: decode tokens a second of the Llama 3.2 1B
shape with random weights (BASELINE.json configs[2]), plus prefill speed and the
decode step's share of the memory roofline.

    python bench.py --gpus 1 --steps K --warmup W

A "step" is one decode step of the engine (schedule, model step, sampling,
bookkeeping) with every request bringing one token.  One JSON line is printed.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12          # bytes/s, MI355X
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}

MODEL = dict(  # BASELINE.json configs[2]: Llama 3.2 1B shape
    architectures=["LlamaForCausalLM"], vocab_size=128256, hidden_size=2048, intermediate_size=8192,
    num_hidden_layers=16, num_attention_heads=32, num_key_value_heads=8, head_dim=64, max_position_embeddings=8192,
    rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True,
    rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192))
# The larger shapes of BASELINE.json (configs[3] and [4]), for measurements beside the headline.
SHAPES = {
    "1b": MODEL,
    "3b": dict(MODEL, hidden_size=3072, num_hidden_layers=28, num_attention_heads=24, head_dim=128),
    "8b": dict(MODEL, hidden_size=4096, intermediate_size=14336, num_hidden_layers=32, head_dim=128,
               tie_word_embeddings=False, rope_scaling=dict(MODEL["rope_scaling"], factor=8.0)),
}


def build_engine(layers, dtype, num_blocks, max_num_seqs, block_size, budget, shape=MODEL, rounded=False):
    """``rounded``: the random weights are rounded to bfloat16 whatever the engine's precision."""
    import torch

    from lyapunov_engine_amd.config import EngineConfig, LlamaConfig
    from lyapunov_engine_amd.engine.core import EngineCore
    from lyapunov_engine_amd.engine.llm_engine import LLMEngine
    from lyapunov_engine_amd.models import build_model
    from lyapunov_engine_amd.models.llama import llama_spec
    from lyapunov_engine_amd.weights import DictSource, load_weights, random_tensors

    cfg = LlamaConfig.from_dict(dict(shape, num_hidden_layers=layers))
    model = build_model(llama_spec(cfg))
    tdtype = torch.bfloat16 if dtype == "bf16" else torch.float32
    tensors = dict(random_tensors(model, 4, torch.bfloat16 if rounded else tdtype, device="cuda:0"))   # seed 4, N(0, 0.02)
    tensors = {k: v.to(tdtype) for k, v in tensors.items()}
    load_weights(model, DictSource(tensors), tdtype, "cuda:0")
    del tensors
    core = EngineCore(model, cfg, dtype=tdtype, device="cuda:0", num_blocks=num_blocks, block_size=block_size,
                      num_state_slots=max_num_seqs)
    engine = LLMEngine(core, EngineConfig(dtype=tdtype, num_blocks=num_blocks, block_size=block_size,
                                          max_num_seqs=max_num_seqs, max_num_batched_tokens=budget,
                                          max_model_len=cfg.max_position_embeddings))
    return engine, cfg


def weight_bytes(cfg, esz):
    h, i = cfg.hidden_size, cfg.intermediate_size
    q, kv = cfg.num_attention_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim
    per_layer = (q + 2 * kv) * h + h * q + 3 * i * h + 2 * h
    return (cfg.num_hidden_layers * per_layer + cfg.vocab_size * h + h) * esz   # the head matrix once per step


def kv_bytes_per_token(cfg, esz):
    return 2 * cfg.num_hidden_layers * cfg.num_key_value_heads * cfg.head_dim * esz


def prefill_flops(cfg, T):
    h, i = cfg.hidden_size, cfg.intermediate_size
    q, kv = cfg.num_attention_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim
    linear = 2 * T * ((q + 2 * kv) * h + h * q + 3 * i * h)
    attn = 2 * cfg.num_attention_heads * cfg.head_dim * T * T       # causal: half of 4 nh hd T^2
    return cfg.num_hidden_layers * (linear + attn) + 2 * cfg.vocab_size * h   # logits of the last token


def random_prompt(n, vocab, seed):
    import torch

    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def measure_decode(engine, cfg, batch, context, steps, warmup, seed):
    """`batch` requests are brought to just under `context` tokens, then warmup +
    steps decode steps run with all of them decoding together.  Requests that
    finish their prompt first decode while the others are still in their prompt,
    so the prompts are shortened by the number of steps that takes.  Returns
    (seconds per step, mean context length over the timed steps)."""
    import torch

    from lyapunov_engine_amd.sampling.params import SamplingParams

    budget = engine.config.max_num_batched_tokens
    ctx_start = context - (warmup + steps) - 4
    ctx_start -= batch * (-(-ctx_start // budget)) + batch      # steps the prompts take, at worst
    assert ctx_start > 0
    sp = SamplingParams(temperature=0.0, max_tokens=context, ignore_eos=True)
    names = [f"d{seed}-{b}" for b in range(batch)]
    for b, name in enumerate(names):
        engine.add_request(name, random_prompt(ctx_start, cfg.vocab_size, seed * 1000 + b), sp)
    seqs = [engine._by_request[n] for n in names]
    while engine.scheduler.num_waiting() or any(
            engine.scheduler.info(s).num_computed < engine.scheduler.info(s).prompt_len for s in seqs):
        engine.step()                       # prompt portions until every request is decoding
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    ctx0 = sum(engine.scheduler.info(s).total_len for s in seqs) / batch
    t0 = time.perf_counter()
    for _ in range(steps):
        out = engine.step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    assert len(out) == batch and not any(o.finished for o in out), "every request must decode in every timed step"
    ctx1 = sum(engine.scheduler.info(s).total_len for s in seqs) / batch
    assert ctx1 - ctx0 == steps and ctx1 <= context
    for name in names:
        engine.abort_request(name)
    return dt, (ctx0 + ctx1 - 1) / 2.0


def measure_prefill(engine, cfg, tokens, repeats=5):
    import torch

    from lyapunov_engine_amd.sampling.params import SamplingParams

    times = []
    for r in range(repeats + 2):
        engine.add_request(f"p{r}", random_prompt(tokens, cfg.vocab_size, 5 + r),
                           SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = engine.step()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        assert out and out[0].finished
    times = sorted(times[2:])
    return times[len(times) // 2]


def measure_mixed(engine, cfg, requests=64, seed=0):
    """BASELINE.json configs[3]'s workload: a continuous batch of `requests` requests with prompts
    of 128 to 4096 random tokens and 128 to 512 output tokens each, prompts taken in portions of at
    most 512 tokens.  Returns (seconds, prompt tokens, generated tokens, steps, latencies): per
    request the time from the start of the run (all requests are added at once) to its first token,
    and the mean time between its tokens after that, as the reference's serving bench reports them
    for its batches (benchmarks/bench_serving.py:54-77: TTFT and average inter-token latency)."""
    import random

    import torch

    from lyapunov_engine_amd.config import EngineConfig
    from lyapunov_engine_amd.engine.llm_engine import LLMEngine
    from lyapunov_engine_amd.sampling.params import SamplingParams

    ec = engine.config
    mixed = LLMEngine(engine.core, EngineConfig(dtype=ec.dtype, num_blocks=ec.num_blocks, block_size=ec.block_size,
                                                max_num_seqs=requests, max_num_batched_tokens=2048, max_chunk=512,
                                                max_model_len=cfg.max_position_embeddings))
    rng = random.Random(seed)
    prompts = [random_prompt(rng.randint(128, 4096), cfg.vocab_size, 100 + i) for i in range(requests)]
    params = [SamplingParams(temperature=0.0, max_tokens=rng.randint(128, 512), ignore_eos=True) for _ in prompts]
    # The workload runs twice and the second run is timed: the first captures the graphs of every
    # batch and context bucket the workload passes through (a serving engine does that once in its life).
    for timed in (False, True):
        for p_, sp in zip(prompts, params):
            mixed.add_request(p_, sp)
        torch.cuda.synchronize()
        t0, steps = time.perf_counter(), 0
        first, last, count = {}, {}, {}
        while mixed.has_unfinished_requests():
            outs = mixed.step()
            now = time.perf_counter() - t0     # the step's tokens have reached the host
            steps += 1
            for o in outs:
                if o.output_tokens and o.request_id not in first:
                    first[o.request_id] = now
                if o.finished:
                    last[o.request_id], count[o.request_id] = now, len(o.output_tokens)
        torch.cuda.synchronize()
    secs = time.perf_counter() - t0
    ttft = sorted(first.values())
    itl = sorted((last[r] - first[r]) / max(count[r] - 1, 1) for r in last)

    def spread(xs):
        return {"mean": round(sum(xs) / len(xs) * 1e3, 3), "p50": round(xs[len(xs) // 2] * 1e3, 3),
                "p99": round(xs[min(len(xs) - 1, int(0.99 * len(xs)))] * 1e3, 3), "max": round(xs[-1] * 1e3, 3)}

    latencies = {"time_to_first_token_ms": spread(ttft), "inter_token_ms": spread(itl)}
    return secs, sum(len(p_) for p_ in prompts), sum(sp.max_tokens for sp in params), steps, latencies


# Largest bf16-against-fp32 logit difference over the largest logit that passes, per layer of the
# model.  Measured at context 8,192 with random weights (whose logits are nearly flat, so that the
# largest logit is a small yardstick): 1B shape 0.8 % through 2 layers and 1.9 % through all 16, 3B
# shape 3.8 % through 28, 8B shape 5.1 % through 32; at context 32,768 the 1B shape shows 1.8 %.
# Allowed: a quarter of a per cent per layer, about one and a half times the largest of these.
CHECK_LIMIT_PER_LAYER = 0.0025


def check_limit(layers):
    return max(0.02, CHECK_LIMIT_PER_LAYER * layers)


def check_logits(shape=MODEL, layers=None, context=8192, portion=2048):
    """The bfloat16 engine against the 32-bit engine at the benchmark's context, on the same shape
    at its full depth (``layers`` None) and the same weights (random, rounded to bfloat16 for both, so that only the
    arithmetic differs): a prompt of context - 1 tokens in portions, through the eager step, then
    one decoded token through the recorded graph of that context.  Returns, for the last prompt
    position and for the decoded position, the largest difference of the logits relative to the
    largest logit, and whether both engines agree on the best token."""
    import numpy as np
    import torch

    from lyapunov_engine_amd.engine.graphs import DecodeGraphs
    from lyapunov_engine_amd.engine.runner import StepEntry

    prompt = random_prompt(context, shape["vocab_size"], 6)
    layers = layers or shape["num_hidden_layers"]
    logits = {}
    for dtype in ("fp32", "bf16"):
        engine, _ = build_engine(layers, dtype, num_blocks=context // 16 + 8, max_num_seqs=1, block_size=16,
                                 budget=portion, shape=shape, rounded=True)
        core = engine.core
        core.cache.add(0)
        rows = []
        for lo in range(0, context - 1, portion):
            hi = min(context - 1, lo + portion)
            core.cache.extend(0, hi)
            out = core.step([StepEntry(0, prompt[lo:hi], lo, [hi - lo - 1] if hi == context - 1 else [])])
            core.cache.commit(0, hi)
        rows.append(out.float().cpu()[0])
        core.cache.extend(0, context)
        graphs = DecodeGraphs(core.runner, max_batch=1)
        out = graphs.step_arrays(np.zeros(1, np.int64), np.asarray([context - 1], np.int32),
                                 np.asarray(prompt[-1:], np.int32)).values
        rows.append(out.float().cpu()[0])
        assert list(graphs.captured) == [(1, context)]
        core.cache.commit(0, context)
        core.cache.free(0)
        logits[dtype] = rows
        del engine, core, graphs
        torch.cuda.empty_cache()
    rel = [float((b - a).abs().max() / a.abs().max()) for a, b in zip(logits["fp32"], logits["bf16"])]
    # the best token is the same, or the 32-bit logits of the two candidates are closer than the two
    # engines' logits differ (random weights give nearly flat logits: such ties are the rule there)
    same = [bool(a.argmax() == b.argmax()) or float(a.max() - a[b.argmax()]) <= 2 * float((b - a).abs().max())
            for a, b in zip(logits["fp32"], logits["bf16"])]
    return rel, same


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=8192, help="context length the decode steps run at")
    ap.add_argument("--shape", default="1b", choices=sorted(SHAPES), help="1b is the headline configuration")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0: all of them)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--workload", default="decode", choices=["decode", "mixed"],
                    help="mixed: the continuous batch of BASELINE.json configs[3] instead of the headline")
    ap.add_argument("--skip-points", action="store_true", help="only the headline decode and the prefill")
    ap.add_argument("--skip-check", action="store_true", help="no comparison of bfloat16 logits with a 32-bit run")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch

    esz = 2 if args.dtype == "bf16" else 4
    block_size = 16
    max_batch = 64
    # the pool holds the largest batch that runs: 64 for the points beside the headline
    pool_batch = max(args.batch, 1) if args.skip_points and args.workload == "decode" else max_batch
    num_blocks = pool_batch * (args.context // block_size + 1) + 64
    shape = SHAPES[args.shape]
    if args.context > shape["max_position_embeddings"]:     # a longer context than the baseline's: the models allow it
        shape = dict(shape, max_position_embeddings=args.context)
    full_layers = shape["num_hidden_layers"]
    engine, cfg = build_engine(args.layers or full_layers, args.dtype, num_blocks, max_batch, block_size, budget=8192,
                               shape=shape)

    if args.workload == "mixed":
        secs, n_prompt, n_gen, steps, latencies = measure_mixed(engine, cfg)
        print(json.dumps({
            "metric": "generated tok/s of a mixed continuous batch", "value": round(n_gen / secs, 1), "unit": "tok/s",
            "n_gpus": 1, "steps": steps, "warmup": 0, "ms_per_step": round(secs / steps * 1e3, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
            "data": "synthetic (random weights seed 4, random token ids)",
            "config": {"model": f"llama-{args.shape}-shape", "num_hidden_layers": cfg.num_hidden_layers,
                       "full_layers": full_layers, "requests": 64, "prompt_tokens": n_prompt,
                       "generated_tokens": n_gen, "prompt_portion": 512, "step_token_budget": 2048,
                       "kv_block_size": block_size, "parallelism": "single-gpu", "graphs": True},
            "total_tokens_per_s": round((n_prompt + n_gen) / secs, 1), **latencies}))
        return 0

    lookahead = bool(engine.config.lookahead)
    prefill_s = measure_prefill(engine, cfg, 2048)
    step_s, mean_ctx = measure_decode(engine, cfg, args.batch, args.context, args.steps, args.warmup, seed=1)
    value = args.batch / step_s
    step_bytes = weight_bytes(cfg, esz) + args.batch * mean_ctx * kv_bytes_per_token(cfg, esz)
    achieved = step_bytes / step_s

    points = {}
    if not args.skip_points:
        for b in (1, 64):
            s, _ = measure_decode(engine, cfg, b, args.context, min(args.steps, 64), min(args.warmup, 8), seed=10 + b)
            points[f"decode_b{b}"] = round(b / s, 1)
        # the decode workload as configs[2] words it: 2048-token prompts, 256 steps -> contexts up to 2304
        for b in (1, 8, 64):
            s, _ = measure_decode(engine, cfg, b, 2304, min(args.steps, 64), min(args.warmup, 8), seed=20 + b)
            points[f"decode_b{b}_ctx2048"] = round(b / s, 1)

    check = None
    if not args.skip_check:
        del engine
        torch.cuda.empty_cache()
        rel, same = check_logits(shape, layers=cfg.num_hidden_layers, context=args.context)
        check = {"what": f"bf16 against fp32 logits, same bf16-rounded weights, {cfg.num_hidden_layers} layers, prompt of {args.context - 1} "
                         f"tokens in portions of 2048 (eager), then one decoded token at context {args.context} "
                         f"through the recorded graph; largest difference over largest logit",
                 "prompt_last": round(rel[0], 5), "decoded_through_graph": round(rel[1], 5),
                 "limit": check_limit(cfg.num_hidden_layers),
                 "best_token_same_or_tied": all(same), "ok": max(rel) <= check_limit(cfg.num_hidden_layers) and all(same)}

    peak = MFMA_PEAK[args.dtype]
    line = {
        "metric": "decode tok/s at batch 1/8/64; prefill tok/s at 2048 tokens; % of roofline",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic (random weights seed 4, random token ids)",
        "config": {
            "model": f"llama-{args.shape}-shape" if args.shape != "1b" else "llama-3.2-1b-shape",
            "num_hidden_layers": cfg.num_hidden_layers, "full_layers": full_layers,
            "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
            "num_attention_heads": cfg.num_attention_heads, "num_key_value_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "vocab_size": cfg.vocab_size, "tie_word_embeddings": bool(shape["tie_word_embeddings"]),
            "rope_scaling": f"llama3 factor {shape['rope_scaling']['factor']:g}", "global_batch": args.batch, "seq_len": int(round(mean_ctx)),
            "context_len": args.context, "kv_block_size": block_size, "prefill_tokens": 2048,
            "parallelism": "single-gpu", "graphs": True, "lookahead": lookahead,
            "logits_check": "skipped" if check is None else
                            f"bf16 vs fp32 engine, {cfg.num_hidden_layers} layers, context {args.context}: "
                            f"{max(rel):.4f} of the largest logit (limit {check['limit']}), {'ok' if check['ok'] else 'FAILED'}",
        },
        "prefill": {"value": round(2048 / prefill_s, 1), "tokens": 2048, "ms": round(prefill_s * 1e3, 3),
                    "frac": round(prefill_flops(cfg, 2048) / prefill_s / peak, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4)},
        "points": points,
        "logits_check": check,
    }
    print(json.dumps(line))
    if check is not None and not check["ok"]:
        print(f"bench.py: bfloat16 logits at context {args.context} are off by {max(rel):.4f} of the largest logit "
              f"(limit {check['limit']}), or the two engines' best tokens differ beyond a tie", file=sys.stderr)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
