"""The whole model through the engine's step function, cache and kernels,
against the plain implementation: whole prompts, decoding token by token,
portions of changing size, and mixed batches with pages used again; in 32-bit
and in bfloat16, for the tiny configurations."""
import json
import os
import random
import subprocess
import sys

import numpy as np
import pytest

from conftest import ROOT, TINY
from trace_util import (Trace, compare, compare_with_alone, plain_logits, plain_logits_at, random_tokens, random_trace,
                        replay)

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
LENGTHS = {"A": {"a": 5, "b": 17, "c": 33, "d": 70}, "B": {"a": 1, "b": 9, "c": 64, "d": 130},
           "C": {"a": 3, "b": 20, "c": 48, "d": 81}}


def requests_for(name, extra=None):
    vocab = TINY[name][0]["vocab_size"]
    lens = dict(LENGTHS[name], **(extra or {}))
    return {rid: random_tokens(n, vocab, seed=100 + i) for i, (rid, n) in enumerate(sorted(lens.items()))}


@pytest.fixture(scope="module")
def plain(model_folders):
    cache = {}

    def get(name, reqs):
        key = (name, tuple(sorted((k, tuple(v)) for k, v in reqs.items())))
        if key not in cache:
            cache[key] = plain_logits(model_folders[name]["float32"], reqs)
        return cache[key]

    return get


def folder(model_folders, name, dtype):
    # the 32-bit engine reads 32-bit files; the bfloat16 engine reads bfloat16 files,
    # and is compared with the plain model of the same (rounded) weights
    return model_folders[name][dtype]


def plain_for(model_folders, name, dtype, reqs):
    return plain_logits(model_folders[name][dtype], reqs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_each_request_alone_and_whole(model_folders, name, dtype):
    reqs = requests_for(name)
    want = plain_for(model_folders, name, dtype, reqs)
    for rid, toks in reqs.items():
        t = Trace({rid: toks})
        t.step([(rid, len(toks))], end=[rid])
        compare(t, replay(folder(model_folders, name, dtype), dtype, t), want, dtype, f"whole {rid}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_most_in_one_step_then_token_by_token(model_folders, name, dtype):
    reqs = requests_for(name, {"e": 100})
    want = plain_for(model_folders, name, dtype, reqs)
    for rid, toks in reqs.items():
        if len(toks) <= 33:
            continue
        t = Trace({rid: toks})
        t.step([(rid, len(toks) - 32)], want="last")
        for _ in range(32):
            t.step([(rid, 1)])
        got = replay(folder(model_folders, name, dtype), dtype, t)
        compare(t, got, want, dtype, f"decode {rid}")
        compare_with_alone(t, got, folder(model_folders, name, dtype), dtype, f"decode {rid}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_portions_of_changing_size(model_folders, name, dtype):
    reqs = requests_for(name, {"e": 100})
    want = plain_for(model_folders, name, dtype, reqs)
    sizes = [7, 2, 5, 3, 16, 2, 31, 4, 2, 9]
    for rid, toks in reqs.items():
        if len(toks) < 9:
            continue
        t = Trace({rid: toks})
        left, i = len(toks), 0
        while left:
            n = min(sizes[i % len(sizes)], left)
            if left - n == 1:
                n += 1  # never leave a single token: portions go down to two
            t.step([(rid, n)])
            left -= n
            i += 1
        got = replay(folder(model_folders, name, dtype), dtype, t)
        compare(t, got, want, dtype, f"portions {rid}")
        compare_with_alone(t, got, folder(model_folders, name, dtype), dtype, f"portions {rid}")


def mixed_trace(reqs):
    """Up to four live requests; portions of some beside single tokens of
    others; requests end and later ones take their pages."""
    t = Trace(reqs)
    t.step([("d", 40), ("a", len(reqs["a"]))], end=["a"])
    t.step([("d", 2), ("b", len(reqs["b"]) - 3), ("c", 20)])
    t.step([("d", 1), ("b", 1), ("c", 2), ("e", 30)])
    t.step([("b", 1), ("c", 1), ("e", 7)])                     # d sits this one out
    t.step([("d", len(reqs["d"]) - 43), ("b", 1), ("c", len(reqs["c"]) - 23)], end=["b", "c"])
    t.step([("e", 1), ("f", 64), ("g", 3)], end=["d"])
    t.step([("e", 2), ("f", 1), ("g", 2), ("h", 33)])
    for _ in range(5):
        t.step([("e", 1), ("f", 1), ("g", 1), ("h", 1)])
    t.step([("e", len(reqs["e"]) - 45), ("f", len(reqs["f"]) - 70), ("g", len(reqs["g"]) - 10),
            ("h", len(reqs["h"]) - 38)], end=["e", "f", "g", "h"])
    return t


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_batches_with_pages_used_again(model_folders, name, dtype):
    reqs = requests_for(name, {"e": 100, "f": 90, "g": 12, "h": 50})
    want = plain_for(model_folders, name, dtype, reqs)
    t = mixed_trace(reqs)
    total = sum(64 * -(-len(v) // 64) for v in reqs.values())
    assert t.max_tokens < total, "the pool is meant to be too small for all requests at once"
    got = replay(folder(model_folders, name, dtype), dtype, t)
    compare(t, got, want, dtype, "mixed")
    compare_with_alone(t, got, folder(model_folders, name, dtype), dtype, "mixed")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_random_schedules(model_folders, name, dtype):
    """Twelve random sets of requests under random schedules each, against the plain model and
    against the same requests alone and whole.  (Sweeps of thousands of seeds of this generator are
    where the tolerances of trace_util come from; in 32-bit they found no logits that depend on the
    schedule beyond 2e-6.)"""
    cfg = TINY[name][0]
    for seed in range(12):
        rng = random.Random(1000 * seed + ord(name))
        reqs, t = random_trace(rng, cfg["vocab_size"], min(200, cfg["max_position_embeddings"] - 1))
        want = plain_for(model_folders, name, dtype, reqs)
        got = replay(folder(model_folders, name, dtype), dtype, t)
        compare(t, got, want, dtype, f"random schedule {seed}")
        compare_with_alone(t, got, folder(model_folders, name, dtype), dtype, f"random schedule {seed}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_steps_of_few_rows_take_the_folded_kernels(model_folders, dtype, monkeypatch):
    """Configuration C is there so that decode steps run the kernels a large
    model's decode steps run: the norm folded into the products around it.  Count
    how often that happens in a token-by-token replay (and compare, as above)."""
    from lyapunov_engine_amd.kernels import ops

    taken = {"norm": 0, "qkv": 0, "gate_up": 0}
    pending, rope_kv, swiglu = ops.rmsnorm_pending, ops.linear_rope_kv, ops.linear_swiglu

    def count_pending(*a, **k):
        out = pending(*a, **k)
        taken["norm"] += out[0] is not None
        return out

    def count_rope_kv(x, *a, **k):
        taken["qkv"] += isinstance(x, ops.PendingNorm)
        return rope_kv(x, *a, **k)

    def count_swiglu(x, *a, **k):
        taken["gate_up"] += isinstance(x, ops.PendingNorm)
        return swiglu(x, *a, **k)

    monkeypatch.setattr(ops, "rmsnorm_pending", count_pending)
    monkeypatch.setattr(ops, "linear_rope_kv", count_rope_kv)
    monkeypatch.setattr(ops, "linear_swiglu", count_swiglu)
    reqs = {"a": random_tokens(40, TINY["C"][0]["vocab_size"], seed=7)}
    want = plain_for(model_folders, "C", dtype, reqs)
    t = Trace(reqs)
    t.step([("a", 30)], want="last")
    for _ in range(10):
        t.step([("a", 1)])
    compare(t, replay(folder(model_folders, "C", dtype), dtype, t), want, dtype, "folded")
    layers = TINY["C"][0]["num_hidden_layers"]
    # per decode step: the norm before every feed-forward and before every attention but the first
    assert taken["norm"] == 10 * (2 * layers - 1), taken
    assert taken["gate_up"] == 10 * layers and taken["qkv"] == 10 * (layers - 1), taken


ODD = dict(architectures=["LlamaForCausalLM"], max_position_embeddings=256, rms_norm_eps=1e-5, rope_theta=10000.0,
           rope_scaling=None, tie_word_embeddings=True, num_hidden_layers=2)
ODD_SIZES = {
    # a width that is no multiple of 8, as many key/value heads as query heads, head size 48
    "wide-heads": dict(ODD, vocab_size=1001, hidden_size=100, intermediate_size=300, num_attention_heads=5,
                       num_key_value_heads=5, head_dim=48),
    # nine heads in groups of three, the smallest head size, a separate output head
    "small-heads": dict(ODD, vocab_size=257, hidden_size=72, intermediate_size=136, num_attention_heads=9,
                        num_key_value_heads=3, head_dim=16, tie_word_embeddings=False),
    # one key/value head for twenty query heads (more than a 16-column tile holds), head size 80
    "one-kv-head": dict(ODD, vocab_size=333, hidden_size=192, intermediate_size=320, num_attention_heads=20,
                        num_key_value_heads=1, head_dim=80),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(ODD_SIZES))
def test_sizes_that_are_no_powers_of_two(tmp_path, name, dtype):
    """Whole models of awkward sizes, a mixed trace with portions and decoded
    tokens: every kernel takes them or the engine says why not; never a wrong
    result."""
    from lyapunov_engine_amd.weights import write_random_model

    cfg = ODD_SIZES[name]
    write_random_model(dict(cfg), str(tmp_path), 3, dtype, init_std=0.1, norm_init_std=0.1)
    reqs = {"a": random_tokens(70, cfg["vocab_size"], 1), "b": random_tokens(9, cfg["vocab_size"], 2)}
    want = plain_logits(str(tmp_path), reqs)
    t = Trace(reqs)
    t.step([("a", 37), ("b", 2)])
    t.step([("a", 2), ("b", 7)], end=["b"])
    t.step([("a", 20)])
    for _ in range(11):
        t.step([("a", 1)])
    compare(t, replay(str(tmp_path), dtype, t), want, dtype, name)


@pytest.mark.parametrize("dtype", DTYPES)
def test_few_new_tokens_over_many_keys(tmp_path, dtype, monkeypatch):
    """Portions of a prompt at the end of 1,300 tokens: in bfloat16 the attention kernel then cuts the
    keys into runs for workgroups of their own (checked), and the logits stay the plain model's."""
    from lyapunov_engine_amd.kernels import ops
    from lyapunov_engine_amd.weights import write_random_model

    cfg = dict(TINY["C"][0], max_position_embeddings=2048, num_hidden_layers=1)
    write_random_model(dict(cfg), str(tmp_path), 11, dtype, init_std=0.1, norm_init_std=0.1)
    reqs = {"a": random_tokens(1300, cfg["vocab_size"], 4), "b": random_tokens(1150, cfg["vocab_size"], 5)}
    want = plain_logits(str(tmp_path), reqs)
    seen, plan = [], ops.attn_prefill_plan
    monkeypatch.setattr(ops, "attn_prefill_plan", lambda *a: seen.append(plan(*a)) or seen[-1])
    t = Trace(reqs)
    t.step([("a", 1100), ("b", 1024)], want="last")
    t.step([("a", 70), ("b", 2)])            # 70 and 2 new tokens over 1,170 and 1,026 keys
    t.step([("a", 100), ("b", 64)], want="last")
    t.step([("a", 30), ("b", 60)], end=["a", "b"])
    compare(t, replay(str(tmp_path), dtype, t), want, dtype, "many keys")
    assert (max(seen) > 1) == (dtype == "bfloat16"), seen


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(model_folders, dtype):
    name = "B"
    reqs = {"long": random_tokens(400, TINY[name][0]["vocab_size"], seed=9)}
    want = plain_for(model_folders, name, dtype, reqs)
    t = Trace(reqs)
    t.step([("long", 3)])
    for _ in range(397):
        t.step([("long", 1)])
    compare(t, replay(folder(model_folders, name, dtype), dtype, t), want, dtype, "long decode")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens_of_a_sequence(model_folders, name, dtype):
    """A one-token prompt, then single tokens: positions 0, 1, 2 have no page
    edge and no history to hide behind."""
    reqs = {"s": random_tokens(6, TINY[name][0]["vocab_size"], seed=11)}
    want = plain_for(model_folders, name, dtype, reqs)
    t = Trace(reqs)
    for _ in range(6):
        t.step([("s", 1)])
    compare(t, replay(folder(model_folders, name, dtype), dtype, t), want, dtype, "first tokens")


def test_trace_run_program(model_folders, tmp_path):
    """The program itself, as a user starts it: steps on stdin, a "done" line
    per step, files of little-endian floats."""
    name, dtype = "A", "float32"
    reqs = requests_for(name)
    want = plain_for(model_folders, name, dtype, reqs)
    t = Trace(reqs)
    t.step([("c", 20), ("a", 5)], end=["a"])
    t.step([("c", 2)], want="none")
    t.step([("c", 11), ("b", 17)], end=["b", "c"], want="last")
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_folders[name][dtype], "--dtype", dtype,
         "--out", str(out), "--max-tokens", str(t.max_tokens)],
        input="".join(json.dumps(s) + "\n" for s in t.steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    vocab = TINY[name][0]["vocab_size"]
    got = {n: np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, vocab) for n in t.rows}
    assert not (out / "1.f32").exists()
    compare(t, got, want, dtype, "trace_run")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,heads,head_dim", [(2048, 32, 64), (3072, 24, 128)])
def test_a_layer_of_the_benchmark_shape(tmp_path, dtype, hidden, heads, head_dim):
    """One layer as wide as the Llama 3.2 1B shape, and one as wide as the 3B
    shape (the sizes the benchmark runs at: products over 2,048 / 3,072 and
    8,192 values, 32 heads of 64 or 24 of 128 over 8, llama3 scaling), through
    steps of 100 rows (the vendor library's products in bfloat16, the tiled
    32-bit kernel in float32), 58 rows, 11 rows (a portion beside decoded
    tokens, the folded kernels of up to 16 rows) and 3 rows, against the plain
    implementation."""
    from lyapunov_engine_amd.weights import write_random_model

    cfg = dict(architectures=["LlamaForCausalLM"], vocab_size=1000, hidden_size=hidden, intermediate_size=8192,
               num_hidden_layers=1, num_attention_heads=heads, num_key_value_heads=8, head_dim=head_dim,
               max_position_embeddings=512, rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True,
               rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                 original_max_position_embeddings=128))
    d = str(tmp_path / "wide")
    os.makedirs(d)
    write_random_model(cfg, d, 11, dtype, init_std=0.03, norm_init_std=0.1)
    reqs = {"a": random_tokens(150, 1000, seed=1), "b": random_tokens(60, 1000, seed=2), "c": random_tokens(20, 1000, seed=3)}
    t = Trace(reqs)
    t.step([("a", 100)])
    t.step([("a", 18), ("b", 40)], want="last")
    t.step([("a", 1), ("b", 1), ("c", 9)])
    for _ in range(8):
        t.step([("a", 1), ("b", 1), ("c", 1)])
    t.step([("a", 23), ("b", 11), ("c", 3)], end=["a", "b", "c"])
    compare(t, replay(d, dtype, t), plain_logits(d, reqs), dtype, "wide layer")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_wide_layer_over_a_long_context(tmp_path, dtype):
    """The same layer at 2,400 tokens: the prompt in two uneven portions (the
    second one's workgroups take the keys of the first in runs), a portion of 40
    tokens at the end of it, and decoded tokens over all of it in partitions."""
    from lyapunov_engine_amd.weights import write_random_model

    cfg = dict(architectures=["LlamaForCausalLM"], vocab_size=1000, hidden_size=2048, intermediate_size=8192,
               num_hidden_layers=1, num_attention_heads=32, num_key_value_heads=8, head_dim=64,
               max_position_embeddings=4096, rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True,
               rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                 original_max_position_embeddings=1024))
    d = str(tmp_path / "wide")
    os.makedirs(d)
    write_random_model(cfg, d, 12, dtype, init_std=0.03, norm_init_std=0.1)
    reqs = {"a": random_tokens(2400, 1000, seed=4), "b": random_tokens(30, 1000, seed=5)}
    t = Trace(reqs)
    t.step([("a", 1900)], want="last")
    t.step([("a", 450), ("b", 20)], want="last")
    t.step([("a", 40), ("b", 1)])
    for _ in range(9):
        t.step([("a", 1), ("b", 1)])
    t.step([("a", 1)], end=["a", "b"])
    compare(t, replay(d, dtype, t), plain_logits(d, reqs), dtype, "wide layer, long context")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_wide_layer_at_the_benchmarks_context(tmp_path, dtype):
    """The 1B shape's layer to 8,300 tokens, where the benchmark runs: the prompt in portions of
    2,048 (each one's keys beyond the first in runs for workgroups of their own), a last portion of
    92 beside the prompt of a second, short request, then sixteen decoded tokens of both (the long
    one's keys in many partitions, block tables over 512 entries wide), against the plain model."""
    from lyapunov_engine_amd.weights import write_random_model

    cfg = dict(architectures=["LlamaForCausalLM"], vocab_size=1000, hidden_size=2048, intermediate_size=8192,
               num_hidden_layers=1, num_attention_heads=32, num_key_value_heads=8, head_dim=64,
               max_position_embeddings=8448, rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True,
               rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                 original_max_position_embeddings=2048))
    d = str(tmp_path / "wide")
    os.makedirs(d)
    write_random_model(cfg, d, 13, dtype, init_std=0.03, norm_init_std=0.1)
    reqs = {"a": random_tokens(8300, 1000, seed=6), "b": random_tokens(40, 1000, seed=7)}
    t = Trace(reqs)
    for _ in range(4):
        t.step([("a", 2048)], want="last")
    t.step([("a", 92), ("b", 24)], want="last")
    for _ in range(16):
        t.step([("a", 1), ("b", 1)])
    t.steps[-1]["end"] = ["a", "b"]
    t.live.clear()
    rows_a = sorted(pos for rows in t.rows.values() for rid, pos in rows if rid == "a")
    want = {"a": plain_logits_at(d, reqs["a"], rows_a), "b": plain_logits(d, {"b": reqs["b"]})["b"]}
    compare(t, replay(d, dtype, t), want, dtype, "wide layer at 8,300 tokens")


def test_the_largest_bfloat16_error_a_sweep_found(model_folders):
    """Seed 1098 of configuration A in a sweep of 3,000 random schedules: at position 32 of its
    first request the bfloat16 logits are 7.3 % of the largest logit off the plain model's, the
    largest such error seen.  It is rounding: the request run alone and whole is off by the same
    amount there, the mixed schedule agrees with that run to 3 %, and the 32-bit engine is exact.
    The case is kept so that the per-row bound stays where measurement put it."""
    name = "A"
    vocab = TINY[name][0]["vocab_size"]
    made = [(69, 713405), (3, 36094), (2, 167777), (3, 176177), (108, 911988), (1, 834276), (3, 610150)]
    reqs = {f"r{i}": random_tokens(n, vocab, seed) for i, (n, seed) in enumerate(made)}
    steps = [([("r0", 23)], [], "last"), ([("r0", 15), ("r1", 2), ("r2", 2), ("r3", 1)], [], "all"),
             ([("r3", 2)], ["r2"], "all"), ([("r0", 1), ("r1", 1)], ["r1"], "all"), ([("r0", 24)], [], "all"),
             ([("r0", 2), ("r4", 1), ("r5", 1)], ["r3", "r5"], "all"), ([("r0", 1)], [], "all"),
             ([("r0", 3), ("r6", 2)], [], "all"), ([("r4", 6), ("r6", 1)], ["r0", "r6"], "last")]
    for dtype in DTYPES:
        t = Trace(reqs)
        for portions, end, want in steps:
            t.step(portions, end=end, want=want)
        f = folder(model_folders, name, dtype)
        got = replay(f, dtype, t)
        rel = compare(t, got, plain_for(model_folders, name, dtype, reqs), dtype, "seed 1098")
        compare_with_alone(t, got, f, dtype, "seed 1098")
        if dtype == "bfloat16":   # (kernels that round better may bring it down; nothing may bring it up)
            assert max(rel) < 0.08, f"the case is kept for its error of 7.3 %; it now shows {max(rel):.3f}"


def test_bfloat16_without_the_vendor_library(model_folders, tmp_path, monkeypatch):
    """LYAPUNOV_AMD_GEMM=own: every bfloat16 product in this package's kernels (the tiled one where
    the library would stand).  Configuration C through a mixed trace, and the 1B shape's layer
    through steps of 100, 58, 11 and 3 rows, against the plain model."""
    from lyapunov_engine_amd.kernels import ops
    from lyapunov_engine_amd.weights import write_random_model

    monkeypatch.setattr(ops, "LIBRARY_GEMM", False)
    called = []
    monkeypatch.setattr(ops, "library_gemm_nt", lambda *a, **k: called.append(1))
    dtype = "bfloat16"
    reqs = requests_for("C", {"e": 100, "f": 90, "g": 12, "h": 50})
    t = mixed_trace(reqs)
    compare(t, replay(folder(model_folders, "C", dtype), dtype, t), plain_for(model_folders, "C", dtype, reqs), dtype,
            "own products, mixed")

    cfg = dict(architectures=["LlamaForCausalLM"], vocab_size=1000, hidden_size=2048, intermediate_size=8192,
               num_hidden_layers=1, num_attention_heads=32, num_key_value_heads=8, head_dim=64,
               max_position_embeddings=512, rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True)
    d = str(tmp_path / "wide")
    write_random_model(cfg, d, 11, dtype, init_std=0.03, norm_init_std=0.1)
    reqs = {"a": random_tokens(150, 1000, seed=1), "b": random_tokens(60, 1000, seed=2), "c": random_tokens(20, 1000, seed=3)}
    t = Trace(reqs)
    t.step([("a", 100)])
    t.step([("a", 18), ("b", 40)], want="last")
    t.step([("a", 1), ("b", 1), ("c", 9)])
    for _ in range(4):
        t.step([("a", 1), ("b", 1), ("c", 1)])
    t.step([("a", 27), ("b", 15), ("c", 7)], end=["a", "b", "c"])
    compare(t, replay(d, dtype, t), plain_logits(d, reqs), dtype, "own products, wide layer")
    assert not called


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_prompts_do_not_depend_on_their_portions(tmp_path, dtype):
    """The 1B shape's layer over 20,000 tokens, where no plain model reaches in the time a test has:
    the logits at the end of the prompt and of 3 decoded tokens are the same whether the prompt came
    in portions of 4,096 or of 777 tokens (in 32-bit to 5e-5 of the largest logit; in bfloat16 to what
    the kernels' roundings differ by, see trace_util).  Block tables are 1,250 entries wide here and
    a late portion's keys are cut into runs."""
    from lyapunov_engine_amd.weights import write_random_model
    from trace_util import TOL_ALONE

    cfg = dict(architectures=["LlamaForCausalLM"], vocab_size=1000, hidden_size=2048, intermediate_size=8192,
               num_hidden_layers=1, num_attention_heads=32, num_key_value_heads=8, head_dim=64,
               max_position_embeddings=32768, rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True,
               rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                 original_max_position_embeddings=8192))
    d = str(tmp_path / "wide")
    write_random_model(cfg, d, 14, dtype, init_std=0.03, norm_init_std=0.1)
    n = 20000
    reqs = {"a": random_tokens(n + 3, 1000, seed=8)}
    got = {}
    for portion in (4096, 777):
        t = Trace(reqs)
        left = n
        while left:
            take = min(portion, left)
            t.step([("a", take)], want="last" if take == left else "none")
            left -= take
        for _ in range(3):
            t.step([("a", 1)])
        t.steps[-1]["end"] = ["a"]
        t.live.clear()
        out = replay(d, dtype, t)
        got[portion] = np.concatenate([out[s] for s in sorted(out)])
    assert got[4096].shape == (4, 1000)
    scale = np.abs(got[4096]).max(axis=1, keepdims=True)
    err = np.abs(got[777] - got[4096]) / np.maximum(scale, 1.0)
    assert err.max() <= TOL_ALONE[dtype]["atol"], f"portions of 777 against 4,096: {err.max(axis=1)}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B", "C"])
def test_recorded_prompt_steps_meet_the_plain_model(model_folders, name, dtype):
    """A prompt of 100 tokens and one of 17, each alone in its step, through the step that the
    generating engine records for short prompts (128 and 32 token rows, the rest padding, the unused
    tile entries beyond any request): the last token's logits against the plain model, on the
    capture's first run and on replays."""
    from lyapunov_engine_amd.engine.core import EngineCore
    from lyapunov_engine_amd.engine.graphs import StepGraphs
    from trace_util import TOL

    f = folder(model_folders, name, dtype)
    vocab = TINY[name][0]["vocab_size"]
    reqs = {"long": random_tokens(100, vocab, seed=301), "short": random_tokens(17, vocab, seed=302)}
    want = plain_for(model_folders, name, dtype, reqs)
    core = EngineCore.from_folder(f, dtype=dtype, num_blocks=32, block_size=TINY[name][1]["block_size"], num_state_slots=4)
    graphs = StepGraphs(core.runner, max_batch=4)
    tol = TOL[dtype]
    for turn in range(3):
        for i, (rid, toks) in enumerate(reqs.items()):
            sid = 10 * turn + i
            core.cache.add(sid)
            core.cache.extend(sid, len(toks))
            counts = np.asarray([len(toks)], np.int32)
            assert graphs.prompt_usable(counts)
            got = graphs.prompt_step_arrays(np.asarray([sid], np.int64), np.zeros(1, np.int32), counts,
                                            np.asarray(toks, np.int32)).values[0].float().cpu().numpy()
            ref = np.asarray(want[rid][len(toks) - 1], dtype=np.float64)
            scale = max(1.0, float(np.abs(ref).max()))
            err = np.abs(got.astype(np.float64) - ref)
            assert (err <= tol["atol"] * scale + tol["rtol"] * np.abs(ref)).all(), \
                f"{rid}, turn {turn}: max error {err.max():.3e} at scale {scale:.3f}"
            core.cache.commit(sid, len(toks))
            core.cache.free(sid)              # the next turn's requests get these pages, stale contents and all
    assert sorted(k[2] for k in graphs.captured) == [32, 128]
    core.cache.check()


def test_bfloat16_error_against_depth(tmp_path):
    """One layer and four layers as wide as the 1B shape's, to 2,400 tokens in bfloat16 against the
    plain model: how the rounding error grows with depth.  Measured: the median over the rows goes
    from 1.0e-2 of the largest logit (one layer) to 1.9e-2 (four; largest row 2.6e-2), about the square root of the
    depth; the per-row bound of the tiny models' traces holds at four layers, their median bound
    (set on models of two and three layers) does not, so the deeper model gets twice that."""
    from lyapunov_engine_amd.weights import write_random_model
    from trace_util import TOL

    medians = {}
    for layers in (1, 4):
        cfg = dict(architectures=["LlamaForCausalLM"], vocab_size=1000, hidden_size=2048, intermediate_size=8192,
                   num_hidden_layers=layers, num_attention_heads=32, num_key_value_heads=8, head_dim=64,
                   max_position_embeddings=4096, rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True,
                   rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                     original_max_position_embeddings=1024))
        d = str(tmp_path / f"deep{layers}")
        os.makedirs(d)
        write_random_model(cfg, d, 12, "bfloat16", init_std=0.03, norm_init_std=0.1)
        reqs = {"a": random_tokens(2400, 1000, seed=4)}
        t = Trace(reqs)
        t.step([("a", 1900)], want="last")
        t.step([("a", 460)], want="last")
        t.step([("a", 30)])
        for _ in range(10):
            t.step([("a", 1)])
        t.steps[-1]["end"] = ["a"]
        t.live.clear()
        rows = sorted(pos for rs in t.rows.values() for _, pos in rs)
        tol = dict(TOL["bfloat16"], median=TOL["bfloat16"]["median"] * (2 if layers > 3 else 1))
        rel = compare(t, replay(d, "bfloat16", t), {"a": plain_logits_at(d, reqs["a"], rows)}, "bfloat16",
                      f"{layers} wide layers", tol=tol)
        medians[layers] = float(np.median(rel))
        print(f"{layers} wide layer(s), bfloat16: median {np.median(rel):.4f}, largest {max(rel):.4f} of the largest logit")
    assert medians[4] <= 3.0 * medians[1], f"the error grew faster than depth accounts for: {medians}"
