"""Generation through the entry points: the scheduler, the step function, the
sampler and the graphs together, against greedy decoding with the plain model."""
import os
import subprocess
import sys

import pytest
import torch

from conftest import ROOT, TINY
from plain import llama_plain as P
from trace_util import random_tokens

pytestmark = pytest.mark.gpu


def plain_greedy(folder, prompt, n):
    w, cfg = P.read_model(folder)
    toks, margins = list(prompt), []
    for _ in range(n):
        logits = P.forward(w, cfg, toks)[-1]
        top = torch.topk(logits, 2).values
        margins.append(float(top[0] - top[1]))
        toks.append(P.greedy(logits))
    return toks[len(prompt):], margins


def check_against_plain(folder, prompt, got, dtype):
    """In 32-bit the tokens are the plain model's.  In bfloat16 a token may
    differ only where the plain model's best two logits are closer than what
    bfloat16 resolves; the comparison then stops (the continuations differ)."""
    want, margins = plain_greedy(folder, prompt, len(got))
    for i, (g, w_) in enumerate(zip(got, want)):
        if g != w_:
            assert dtype == "bfloat16" and margins[i] < 0.25, f"token {i}: engine {g}, plain {w_}, margin {margins[i]}"
            return
    assert len(got) == len(want)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_point(model_folders, name, dtype):
    import lyapunov_engine_amd as L

    folder = model_folders[name][dtype]
    vocab = TINY[name][0]["vocab_size"]
    prompts = [random_tokens(n, vocab, seed=50 + n) for n in (5, 17, 33)]
    llm = L.LLM(folder, dtype=dtype, num_blocks=64, block_size=TINY[name][1]["block_size"])
    outs = llm.generate(prompts, L.SamplingParams(temperature=0.0, max_tokens=16, ignore_eos=True))
    assert [o.request_id for o in outs] == [0, 1, 2]
    for prompt, o in zip(prompts, outs):
        assert o.finished and o.finish_reason == "length" and o.prompt_tokens == prompt and len(o.output_tokens) == 16
        check_against_plain(folder, prompt, o.output_tokens, dtype)


@pytest.mark.parametrize("graphs", [True, False])
def test_portions_preemption_and_graphs_do_not_change_the_tokens(model_folders, graphs):
    """A token budget smaller than the prompts, and so few pages that requests
    are preempted and recomputed: greedy tokens stay those of the plain model."""
    from lyapunov_engine_amd.config import EngineConfig
    from lyapunov_engine_amd.engine.llm_engine import LLMEngine
    from lyapunov_engine_amd.sampling.params import SamplingParams

    folder = model_folders["A"]["float32"]
    prompts = [random_tokens(n, 256, seed=70 + n) for n in (30, 9, 21, 40)]
    engine = LLMEngine(folder, EngineConfig(dtype="float32", num_blocks=30, block_size=4, max_num_seqs=4,
                                            max_num_batched_tokens=16, enable_graphs=graphs))
    for i, p in enumerate(prompts):
        engine.add_request(f"r{i}", p, SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True))
    done, steps = {}, 0
    while engine.has_unfinished_requests():
        for out in engine.step():
            if out.finished:
                done[out.request_id] = out
        steps += 1
        engine.core.cache.check()
        assert steps < 2000
    assert engine.scheduler.counters()["preemptions"] > 0, "the pool was meant to be too small"
    assert engine.core.cache.num_requests() == 0 and engine.core.cache.num_free_pages() == 30
    for i, p in enumerate(prompts):
        check_against_plain(folder, p, done[f"r{i}"].output_tokens, "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_started_ahead_give_the_same_tokens(model_folders, dtype):
    """Decode steps started before the tokens of the step before them have reached the host
    (greedy and seeded sampling, end-of-sequence tokens, requests that arrive and end at different
    times, few pages): the same tokens as without looking ahead, to the last one."""
    from lyapunov_engine_amd.config import EngineConfig
    from lyapunov_engine_amd.engine.llm_engine import LLMEngine
    from lyapunov_engine_amd.sampling.params import SamplingParams

    folder = model_folders["B"][dtype]
    prompts = [random_tokens(n, 515, seed=90 + n) for n in (30, 9, 21, 40, 3)]
    params = [SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True),
              SamplingParams(temperature=0.9, top_k=40, max_tokens=25, seed=5, ignore_eos=True),
              SamplingParams(temperature=0.0, max_tokens=33),
              SamplingParams(temperature=0.7, top_p=0.9, max_tokens=48, seed=6),
              SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True)]
    arrive = [0, 0, 3, 10, 30]

    def run(lookahead, eos):
        engine = LLMEngine(folder, EngineConfig(dtype=dtype, num_blocks=24, block_size=16, max_num_seqs=4,
                                                max_num_batched_tokens=32, lookahead=lookahead, eos_token_ids=eos))
        done, steps, added = {}, 0, 0
        while added < len(prompts) or engine.has_unfinished_requests():
            while added < len(prompts) and arrive[added] <= steps:
                engine.add_request(f"r{added}", prompts[added], params[added])
                added += 1
            for out in engine.step():
                if out.finished:
                    done[out.request_id] = (list(out.output_tokens), out.finish_reason)
            steps += 1
            engine.core.cache.check()
            assert steps < 1000
        assert engine.core.cache.num_requests() == 0 and engine.core.cache.num_free_pages() == 24
        return done, engine.steps_taken_ahead

    plain_run, none_ahead = run(False, ())
    assert none_ahead == 0
    # tokens that the third and fourth request produce somewhere in the middle end them
    eos = (plain_run["r2"][0][12], plain_run["r3"][0][20])
    want, _ = run(False, eos)
    got, taken_ahead = run(True, eos)
    assert got == want
    assert want["r2"][1] == "stop" and len(want["r2"][0]) <= 13
    assert taken_ahead > 20, "most decode steps were meant to be started ahead"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_across_the_graphs_context_buckets(model_folders, dtype):
    """Three requests decode from under 256 tokens to over 256 (a new graph is captured while a step
    started ahead is still running) and one of them on to 500: the tokens are those of the engine
    without graphs, and in 32-bit those of the plain model at the places checked."""
    from lyapunov_engine_amd.config import EngineConfig
    from lyapunov_engine_amd.engine.llm_engine import LLMEngine
    from lyapunov_engine_amd.sampling.params import SamplingParams

    folder = model_folders["B"][dtype]
    prompts = [random_tokens(n, 515, seed=30 + n) for n in (200, 90, 250)]
    lengths = [290, 200, 40]

    def run(graphs):
        engine = LLMEngine(folder, EngineConfig(dtype=dtype, num_blocks=80, block_size=16, max_num_seqs=4,
                                                enable_graphs=graphs))
        for i, p in enumerate(prompts):
            engine.add_request(i, p, SamplingParams(temperature=0.0, max_tokens=lengths[i], ignore_eos=True))
        done = {}
        while engine.has_unfinished_requests():
            for out in engine.step():
                if out.finished:
                    done[out.request_id] = list(out.output_tokens)
        return done, engine

    with_graphs, engine = run(True)
    assert len({key[1] for key in engine.graphs.captured}) >= 2 and engine.steps_taken_ahead > 200
    eager, _ = run(False)
    assert with_graphs == eager
    if dtype == "float32":
        check_against_plain(folder, prompts[2], with_graphs[2], dtype)


def test_a_step_that_does_not_fit_the_cache_is_refused(model_folders):
    """What the step function will not run, with the reason: a request the
    cache does not know, a gap or an overlap in its positions, tokens without
    pages, a token outside the vocabulary, a position beyond the model's,
    logits at a place the step does not bring, a request twice."""
    from lyapunov_engine_amd.engine.core import EngineCore, StepEntry
    from lyapunov_engine_amd.engine.runner import StepError

    core = EngineCore.from_folder(model_folders["A"]["float32"], dtype="float32", num_blocks=80, block_size=4)
    core.cache.add(0)
    core.cache.extend(0, 8)
    for entries, words in [
        ([], "at least one entry"),
        ([StepEntry(3, [1, 2], 0, [])], "request 3 is not known"),
        ([StepEntry(0, [], 0, [])], "brings no tokens"),
        ([StepEntry(0, [1, 2], 1, [])], "continues at 1 but its cache holds 0"),
        ([StepEntry(0, list(range(9)), 0, [])], "has pages for 8 tokens, the step needs 9"),
        ([StepEntry(0, [1, 256], 0, [])], "outside the vocabulary of 256"),
        ([StepEntry(0, [1, 2], 0, [2])], "wants logits at a place it does not bring"),
        ([StepEntry(0, [1], 0, []), StepEntry(0, [2], 1, [])], "twice"),
    ]:
        with pytest.raises(StepError, match=words):
            core.step(entries)
    core.cache.extend(0, 300)
    with pytest.raises(StepError, match="beyond the 256 positions"):
        core.step([StepEntry(0, [1] * 257, 0, [])])
    logits = core.step([StepEntry(0, [1, 2, 3], 0, [2])])       # and what fits still runs
    assert tuple(logits.shape) == (1, 256) and bool(torch.isfinite(logits).all())


def test_graph_steps_equal_eager_steps(model_folders):
    """The same decode steps through a captured graph, replayed several times
    with other work in between, and eagerly: equal logits every time."""
    from lyapunov_engine_amd.engine.core import EngineCore, StepEntry
    from lyapunov_engine_amd.engine.graphs import DecodeGraphs

    core = EngineCore.from_folder(model_folders["B"]["bfloat16"], dtype="bfloat16", num_blocks=64, block_size=16)
    graphs = DecodeGraphs(core.runner, max_batch=8)
    seqs = {i: random_tokens(n, 515, seed=i) for i, n in enumerate((40, 3, 17))}
    for i, toks in seqs.items():
        core.cache.add(i)
        core.cache.extend(i, len(toks) + 8)
        core.step([StepEntry(i, toks, 0, [])])
        core.cache.commit(i, len(toks))
    for k in range(6):
        entries = [StepEntry(i, [(7 * k + i) % 515], len(seqs[i]) + k, [0]) for i in seqs]
        eager = core.step(entries).clone()              # writes the same slots the graph is about to write
        assert graphs.usable(entries)
        torch.cuda.synchronize()
        replayed = graphs.step(entries).clone()
        torch.testing.assert_close(replayed, eager, rtol=0, atol=0)
        for e in entries:
            core.cache.commit(e.seq_id, e.start + 1)
    assert len(graphs.captured) == 1


def test_graph_of_many_rows_with_library_products_equals_eager(tmp_path):
    """A layer as wide as the 1B shape's, so that the products of a decode step
    of 40 requests go to the vendor's library (in the graph with algorithms
    chosen by measurement for the graph's 48 rows, eagerly with the library's
    first choice for 40): every replay of the graph, with eager steps between
    the replays, gives the eager step's logits up to bfloat16 rounding."""
    from lyapunov_engine_amd.engine.core import EngineCore, StepEntry
    from lyapunov_engine_amd.engine.graphs import DecodeGraphs
    from lyapunov_engine_amd.kernels import ops
    from lyapunov_engine_amd.weights import write_random_model

    cfg = dict(architectures=["LlamaForCausalLM"], vocab_size=512, hidden_size=2048, intermediate_size=8192,
               num_hidden_layers=1, num_attention_heads=32, num_key_value_heads=8, head_dim=64,
               max_position_embeddings=256, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=True)
    folder = str(tmp_path / "wide")
    os.makedirs(folder)
    write_random_model(cfg, folder, 3, "bfloat16", init_std=0.02)
    n = 40
    # the gate/up product is the library's at this many rows (several rounds of this package's workgroups);
    # the o product, one small round when its inner dimension is cut into slices, is this package's
    assert ops._library_product(n, 2 * 8192, 2048, torch.bfloat16)
    assert not ops._library_product(n, 2048, 2048, torch.bfloat16, sliced=True)   # the o product: one small round
    core = EngineCore.from_folder(folder, dtype="bfloat16", num_blocks=n * 4 + 8, block_size=16, num_state_slots=64)
    graphs = DecodeGraphs(core.runner, max_batch=64)
    lens = [3 + (5 * i) % 17 for i in range(n)]
    for i in range(n):
        core.cache.add(i)
        core.cache.extend(i, lens[i] + 8)
        core.step([StepEntry(i, random_tokens(lens[i], 512, seed=i), 0, [])])
        core.cache.commit(i, lens[i])
    plans_before = ops.blas().lyp_library_gemm_plans()
    for k in range(5):
        entries = [StepEntry(i, [(11 * k + 3 * i) % 512], lens[i] + k, [0]) for i in range(n)]
        eager = core.step(entries).clone()
        torch.cuda.synchronize()
        replayed = graphs.step(entries).clone()
        scale = float(eager.abs().max())
        assert float((replayed - eager).abs().max()) <= 0.03 * scale, f"replay {k}"
        for e in entries:
            core.cache.commit(e.seq_id, e.start + 1)
    assert [key[0] for key in graphs.captured] == [48]
    assert ops.blas().lyp_library_gemm_plans() > plans_before       # the library was used, for 40 and for 48 rows


def test_seeded_sampling_does_not_depend_on_batch_mates(model_folders):
    import lyapunov_engine_amd as L

    folder = model_folders["B"]["float32"]
    prompt = random_tokens(9, 515, seed=1)
    sp = L.SamplingParams(temperature=0.8, top_k=50, top_p=0.95, max_tokens=24, ignore_eos=True, seed=1234)
    alone = L.LLM(folder, dtype="float32", num_blocks=64).generate([prompt], sp)[0].output_tokens
    others = [random_tokens(n, 515, seed=n) for n in (1, 64, 130)]
    sps = [L.SamplingParams(temperature=0.8, max_tokens=24, ignore_eos=True, seed=s) for s in (1, 2, 3)]
    mixed = L.LLM(folder, dtype="float32", num_blocks=64, max_num_batched_tokens=48).generate(
        others[:2] + [prompt] + others[2:], sps[:2] + [sp] + sps[2:])
    assert mixed[2].output_tokens == alone
    other_seed = L.SamplingParams(temperature=0.8, top_k=50, top_p=0.95, max_tokens=24, ignore_eos=True, seed=99)
    assert L.LLM(folder, dtype="float32", num_blocks=64).generate([prompt], other_seed)[0].output_tokens != alone
    assert len(set(alone)) > 4  # it does sample: greedy on this model repeats itself quickly


def test_requests_that_make_no_sense_are_refused_when_added(model_folders):
    import lyapunov_engine_amd as L

    engine = L.LLM(model_folders["A"]["float32"], dtype="float32", num_blocks=32, block_size=4).engine
    sp = L.SamplingParams(temperature=0.0, max_tokens=4)
    for prompt, words in [([1, 2, 256], "token ids below"), ([1, -1], "token ids below"), ([1.5, 2.0], "token ids below"),
                          ([[1, 2], [3, 4]], "token ids below"), ([], "empty prompt"), ([1] * 256, "max_model_len"),
                          ([1] * 200, "pages")]:
        with pytest.raises((ValueError, RuntimeError), match=words):
            engine.add_request("bad", prompt, sp)
        assert not engine.has_unfinished_requests()
    engine.add_request("a", [1, 2, 3], sp)
    with pytest.raises(ValueError, match="in use"):
        engine.add_request("a", [4, 5], sp)
    first = engine.add_request([4, 5], sp)              # an anonymous request gets a number of its own
    assert first != "a" and engine.add_request(first + 1, [6], sp) == first + 1
    assert engine.add_request([7, 8], sp) not in ("a", first, first + 1)
    done = {}
    while engine.has_unfinished_requests():
        for out in engine.step():
            if out.finished:
                done[out.request_id] = out
    assert len(done) == 4 and all(len(o.output_tokens) == 4 for o in done.values())


def test_eos_stops_a_request(model_folders):
    import lyapunov_engine_amd as L

    folder = model_folders["A"]["float32"]
    prompt = random_tokens(12, 256, seed=3)
    want, _ = plain_greedy(folder, prompt, 10)
    stop_at = 4
    llm = L.LLM(folder, dtype="float32", num_blocks=32, block_size=4, eos_token_ids=(want[stop_at],))
    out = llm.generate([prompt], L.SamplingParams(temperature=0.0, max_tokens=10))[0]
    first = want.index(want[stop_at])
    assert out.output_tokens == want[: first + 1] and out.finish_reason == "stop"
    out = llm.generate([prompt], L.SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))[0]
    assert out.output_tokens == want and out.finish_reason == "length"


def test_command_line_generate(model_folders):
    folder = model_folders["A"]["float32"]
    prompt = random_tokens(7, 256, seed=8)
    want, _ = plain_greedy(folder, prompt, 8)
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "lyapunov"), "generate", "--model", folder,
                           "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "8", "--temperature", "0",
                           "--dtype", "float32", "--block-size", "4", "--num-blocks", "32"],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "--- Output Generation ---" in proc.stdout
    assert proc.stdout.strip().splitlines()[-1].split() == [str(t) for t in want]


def test_a_step_ahead_that_cannot_start_does_not_break_the_planned_step(model_folders, capsys):
    """Starting the next step early is optional work: if it raises (a new graph that cannot be
    recorded, no memory for it), the planned step's tokens still reach the scheduler, looking ahead
    is switched off with a note, and generation gives the tokens it gives without looking ahead."""
    from lyapunov_engine_amd.config import EngineConfig
    from lyapunov_engine_amd.engine.graphs import RecordingFailed
    from lyapunov_engine_amd.engine.llm_engine import LLMEngine
    from lyapunov_engine_amd.sampling.params import SamplingParams

    folder = model_folders["B"]["float32"]
    prompts = [random_tokens(n, 515, seed=70 + n) for n in (12, 5)]
    params = SamplingParams(temperature=0.0, max_tokens=15, ignore_eos=True)

    def run(lookahead, break_it):
        engine = LLMEngine(folder, EngineConfig(dtype="float32", num_blocks=24, block_size=16, max_num_seqs=4,
                                                lookahead=lookahead))
        if break_it:
            real = engine.graphs.step_arrays

            def failing(ids, starts, tokens, tokens_dev=None):
                if tokens_dev is not None:
                    raise RecordingFailed("no memory for a new graph")
                return real(ids, starts, tokens)

            engine.graphs.step_arrays = failing
        outs = engine.generate(prompts, params)
        engine.core.cache.check()
        assert engine.core.cache.num_requests() == 0 and engine.core.cache.num_free_pages() == 24
        return [o.output_tokens for o in outs], engine

    want, _ = run(False, False)
    got, engine = run(True, True)
    assert got == want and engine._look_ahead is False and engine.steps_taken_ahead == 0
    assert "looking ahead switched off" in capsys.readouterr().err
    assert len(engine.recording_failures) == 1 and engine.counters()["recording_failures"] == 1


def test_sampled_tokens_are_the_plain_rules_at_the_engines_uniform_numbers(model_folders):
    """Temperature, top-k and top-p through the whole engine, in 32-bit: every token is the one the
    reference's rules give (python/lyapunov_engine/engine/sampling.py:40-69: scale, keep the k
    largest, cut the tail beyond p, draw) on the plain model's logits, at the uniform number the
    engine derives from (engine seed, request seed, index of the token)."""
    import lyapunov_engine_amd as L
    from lyapunov_engine_amd.sampling.sampler import uniform

    folder = model_folders["B"]["float32"]
    w, cfg = P.read_model(folder)
    for seed, temperature, top_k, top_p in ((1234, 0.8, 50, 0.95), (77, 1.3, -1, 0.7), (5, 0.6, 8, 1.0)):
        prompt = random_tokens(9, 515, seed=seed)
        sp = L.SamplingParams(temperature=temperature, top_k=top_k, top_p=top_p, max_tokens=20, ignore_eos=True, seed=seed)
        got = L.LLM(folder, dtype="float32", num_blocks=64, seed=3).generate([prompt], sp)[0].output_tokens
        toks = list(prompt)
        for i, t in enumerate(got):
            probs = P.sample_filter(P.forward(w, cfg, toks)[-1], temperature, top_k, top_p)
            u = uniform(3, seed, i)
            if t != P.inverse_cdf(probs, u):
                # only where the uniform number falls on the border between two tokens' shares
                cdf = torch.cumsum(probs, 0)
                assert probs[t] > 0 and float(cdf[t] - probs[t]) - 2e-5 <= u <= float(cdf[t]) + 2e-5, \
                    f"seed {seed}, token {i}: engine {t}, plain {P.inverse_cdf(probs, u)} at u = {u}"
            toks.append(t)
        assert len(set(got)) > 4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_short_prompts_run_as_recorded_steps(model_folders, dtype):
    """A prompt of up to 128 tokens alone in its step is replayed from a graph recorded for the next
    bucket of token rows (the rows past its tokens are padding): the tokens it leads to are those of
    the engine without graphs, for lengths at and around the buckets' edges, for a prompt whose last
    portion starts in the middle of its pages, and with the graphs used again for other prompts."""
    import lyapunov_engine_amd as L

    folder = model_folders["B"][dtype]
    lengths = [2, 5, 16, 17, 40, 64, 100, 128, 129, 200]
    prompts = [random_tokens(n, 515, seed=300 + n) for n in lengths]
    sp = L.SamplingParams(temperature=0.0, max_tokens=5, ignore_eos=True)

    def run(graphs):
        llm = L.LLM(folder, dtype=dtype, num_blocks=64, block_size=16, max_num_batched_tokens=128, enable_graphs=graphs)
        outs = [llm.generate([p], sp)[0].output_tokens for p in prompts]       # one at a time: alone in its step
        outs += [llm.generate([p], sp)[0].output_tokens for p in prompts[:4]]   # the recorded steps again
        return outs, llm.engine

    with_graphs, engine = run(True)
    prompt_keys = sorted(key for key in engine.graphs.captured if len(key) == 3)
    assert {key[2] for key in prompt_keys} == {16, 32, 64, 128}, prompt_keys
    eager, _ = run(False)
    assert with_graphs == eager
    assert with_graphs[:4] == with_graphs[len(prompts):]
    for p, got in zip(prompts[:8], with_graphs):
        check_against_plain(folder, p, got, dtype)
    engine.core.cache.check()
    assert engine.core.cache.num_requests() == 0


def test_a_recorded_prompt_step_of_two_requests_equals_the_eager_step(model_folders):
    """The table builder's recorded layout with prompt tokens, beyond what the engine uses it for:
    two requests in one recorded step (a portion of 9 tokens from position 20 and a whole prompt of
    30), replayed with other requests and lengths, against the same steps run eagerly."""
    import numpy as np

    from lyapunov_engine_amd.engine.core import EngineCore, StepEntry
    from lyapunov_engine_amd.engine.graphs import _Captured
    from lyapunov_engine_amd.parts.base import FixedStep

    core = EngineCore.from_folder(model_folders["C"]["float32"], dtype="float32", num_blocks=64, block_size=16)
    cache, runner = core.cache, core.runner
    cap = _Captured(runner, FixedStep(rows=2, max_context=256, tokens=64), torch.cuda.graph_pool_handle())
    toks = {i: random_tokens(90, 320, seed=40 + i) for i in range(4)}
    for i in toks:
        cache.add(i)

    def both(entries):
        for e in entries:
            cache.extend(e.seq_id, e.start + len(e.tokens))
        eager = core.step(entries).clone()
        ids = np.asarray([e.seq_id for e in entries], dtype=np.int64)
        starts = np.asarray([e.start for e in entries], dtype=np.int32)
        counts = np.asarray([len(e.tokens) for e in entries], dtype=np.int32)
        flat = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in entries])
        replayed = cap.run(runner, ids, starts, flat, counts=counts).values.clone()
        for e in entries:
            cache.commit(e.seq_id, e.start + len(e.tokens))
        torch.testing.assert_close(replayed, eager, rtol=1e-5, atol=1e-5)
        return eager

    cache.extend(0, 20)
    core.step([StepEntry(0, toks[0][:20], 0, [])])
    cache.commit(0, 20)
    both([StepEntry(0, toks[0][20:29], 20, [8]), StepEntry(1, toks[1][:30], 0, [29])])
    both([StepEntry(2, toks[2][:64], 0, [63])])                              # one request, every token row live
    both([StepEntry(1, toks[1][30:31], 30, [0]), StepEntry(0, toks[0][29:70], 29, [40])])   # a single token beside a portion
    both([StepEntry(3, toks[3][:2], 0, [1]), StepEntry(2, toks[2][64:66], 64, [1])])


def test_a_step_that_cannot_be_recorded_runs_eagerly(model_folders, capsys):
    """Recording a step is an optimisation: when it fails, the planned step runs the eager way, later
    steps too, and generation gives the tokens it gives without graphs."""
    import lyapunov_engine_amd as L
    from lyapunov_engine_amd.engine import graphs as G

    folder = model_folders["B"]["float32"]
    prompts = [random_tokens(n, 515, seed=60 + n) for n in (12, 70)]
    sp = L.SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True)
    want = [o.output_tokens for o in L.LLM(folder, dtype="float32", num_blocks=24, enable_graphs=False).generate(prompts, sp)]

    llm = L.LLM(folder, dtype="float32", num_blocks=24)
    calls = []

    def failing(self, fixed):
        calls.append(fixed)
        raise G.RecordingFailed("out of memory while recording")

    real = G.StepGraphs._captured
    G.StepGraphs._captured = failing
    try:
        got = [o.output_tokens for o in llm.generate(prompts, sp)]
    finally:
        G.StepGraphs._captured = real
    assert got == want and len(calls) == 1 and llm.engine.graphs.safe is False
    assert "recorded steps switched off" in capsys.readouterr().err
    assert llm.engine.recording_failures == ["out of memory while recording"]
    llm.engine.core.cache.check()


def test_a_defect_in_a_recorded_step_is_raised_not_swallowed(model_folders):
    """Only a shortage while recording is answered by stepping eagerly; an error from the step's
    tables or from a kernel's own checks comes out as it is."""
    import lyapunov_engine_amd as L
    from lyapunov_engine_amd.engine import graphs as G
    from lyapunov_engine_amd.kernels.ops import KernelError

    folder = model_folders["B"]["float32"]
    llm = L.LLM(folder, dtype="float32", num_blocks=24)

    def broken(self, fixed):
        raise KernelError("attention: partition workspace too small")

    real = G.StepGraphs._captured
    G.StepGraphs._captured = broken
    try:
        with pytest.raises(KernelError, match="workspace too small"):
            llm.generate([random_tokens(12, 515, seed=3)], L.SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))
    finally:
        G.StepGraphs._captured = real
    assert llm.engine.graphs.safe is True and llm.engine.recording_failures == []


# ------------------------------------------- recorded prompt steps at long contexts, windows
LONG = dict(architectures=["LlamaForCausalLM"], vocab_size=300, hidden_size=128, intermediate_size=192,
            num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=32,
            max_position_embeddings=8192, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=True)


def register_windowed(name, windows):
    """A Llama whose layer i sees the last ``windows[i]`` keys (0: all of them), registered from here."""
    from lyapunov_engine_amd.config import LlamaConfig, register_architecture
    from lyapunov_engine_amd.config.specs import LayerSpec, ModelSpec, PartSpec
    from lyapunov_engine_amd.models.llama import llama_spec

    def to_spec(cfg):
        spec = llama_spec(cfg)
        layers = []
        for layer, w in zip(spec.layers, windows):
            mixer = PartSpec(layer.mixer.kind, dict(layer.mixer.params, window=w))
            layers.append(LayerSpec(layer.block, mixer, layer.ffn, layer.norm1, layer.norm2, layer.names))
        fields = {f: getattr(spec, f) for f in spec.__dataclass_fields__}
        return ModelSpec(**dict(fields, layers=tuple(layers)))

    register_architecture(name, LlamaConfig, to_spec, replace=True)


@pytest.mark.parametrize("windows", [(0, 0), (0, 48)], ids=["all keys", "a windowed layer"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_recorded_last_portion_at_a_long_context_equals_the_eager_step(tmp_path, dtype, windows):
    """The last portion of a long prompt, alone in its step, replays a recorded step whose bound is
    the context's bucket: in bfloat16 its keys are cut into runs for workgroups of their own, the
    unused tile entries pass through the merging kernel, and a windowed layer walks its window only.
    Against the same step run eagerly on the same cache (the step writes the same keys to the same
    slots again), logits and all."""
    import numpy as np

    from lyapunov_engine_amd.config import ARCHITECTURES
    from lyapunov_engine_amd.engine.core import EngineCore, StepEntry
    from lyapunov_engine_amd.engine.graphs import StepGraphs
    from lyapunov_engine_amd.weights import write_random_model

    arch = "WindowedLlamaForCausalLM"
    register_windowed(arch, windows)
    try:
        folder = str(tmp_path / "long")
        write_random_model(dict(LONG, architectures=[arch]), folder, seed=11, dtype=dtype, init_std=0.1, norm_init_std=0.1)
        core = EngineCore.from_folder(folder, dtype=dtype, num_blocks=520, block_size=16, num_state_slots=2)
        total, last = 4170, 90
        toks = random_tokens(total, 300, seed=12)
        core.cache.add(0)
        for lo in range(0, total - last, 1020):
            hi = min(total - last, lo + 1020)
            core.cache.extend(0, hi)
            core.step([StepEntry(0, toks[lo:hi], lo, [])])
            core.cache.commit(0, hi)
        core.cache.extend(0, total)
        eager = core.step([StepEntry(0, toks[total - last:], total - last, [last - 1])]).clone()
        graphs = StepGraphs(core.runner, max_batch=2)
        ids, starts = np.zeros(1, np.int64), np.asarray([total - last], np.int32)
        counts, flat = np.asarray([last], np.int32), np.asarray(toks[total - last:], np.int32)
        assert graphs.prompt_usable(counts)
        for _ in range(3):      # the capture, then replays
            replayed = graphs.prompt_step_arrays(ids, starts, counts, flat).values.clone()
            scale = float(eager.abs().max())
            limit = 1e-5 if dtype == "float32" else 2e-2
            assert float((replayed - eager).abs().max()) <= limit * scale
        (key,) = graphs.captured
        assert key == (1, 8192, 128)
        if dtype == "bfloat16":  # the bound's keys in runs: the recorded launch merges partial results
            meta = graphs.captured[key].ctx.plans[core.runner.model.layers[0].mixer.step_planner().key].meta
            launch = core.runner.model.layers[0].mixer.prefill_launch(meta, core.dtype, 16)
            assert launch["parts"] > 1 and launch["n_tiles"] == 3
        core.cache.check()
    finally:
        ARCHITECTURES.unregister(arch)


def test_a_model_of_windows_alone_generates_past_its_pool(tmp_path):
    """Every layer keeps a window: pages come back as the window passes, so a request is bound by the
    model's length, not by the pool.  Through the entry point, with a pool far smaller than the
    request: the tokens are those of an engine whose pool holds the whole request."""
    import lyapunov_engine_amd as L
    from lyapunov_engine_amd.config import ARCHITECTURES
    from lyapunov_engine_amd.weights import write_random_model

    arch = "WindowsOnlyLlamaForCausalLM"
    register_windowed(arch, (40, 24))
    try:
        folder = str(tmp_path / "windows")
        write_random_model(dict(LONG, architectures=[arch], max_position_embeddings=1024), folder, seed=13,
                           dtype="float32", init_std=0.1, norm_init_std=0.1)
        prompt = random_tokens(50, 300, seed=14)
        sp = L.SamplingParams(temperature=0.0, max_tokens=260, ignore_eos=True)
        roomy = L.LLM(folder, dtype="float32", num_blocks=64, block_size=16, max_chunk=32)
        want = roomy.generate([prompt], sp)[0].output_tokens
        small = L.LLM(folder, dtype="float32", num_blocks=10, block_size=16, max_chunk=32)   # 160 tokens of pages
        assert small.engine.core.runner.max_position == 1024          # not the pool's 160
        got = small.generate([prompt], sp)[0]
        assert got.output_tokens == want and len(want) == 260 and got.finish_reason == "length"
        small.engine.core.cache.check()
        assert small.engine.core.cache.counters()["window_returns"] > 0
    finally:
        ARCHITECTURES.unregister(arch)
