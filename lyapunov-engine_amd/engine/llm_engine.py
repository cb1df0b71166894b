"""The generating engine: requests in, tokens out.

Names and meanings follow the reference's LLMEngine
(python/lyapunov_engine/engine/llm_engine.py:93-312): ``add_request`` in both of
its forms (:165-212), ``has_unfinished_requests`` (:214-217), ``step`` returning
a ``RequestOutput`` per scheduled request with the tokens produced so far
(:219-310), and ``RequestOutput``'s fields (:41-55).  Added: ``abort_request``,
``generate`` (the loop of entrypoints/cli.py:41-46 over a list of prompts), a
finish reason that tells "stop" from "length" (the reference always says
"stop", :307), and a request counter that moves once per request (the reference
bumps it twice for an anonymous request, :184-185, 193-194).

One step: the scheduler plans (prompt portions and decoded tokens, pages taken),
the step function runs the plan as one batch, the sampler picks a token for
every request whose known tokens are now all in the cache, the scheduler takes
the tokens and finishes or frees what is done.

Looking ahead: when a step only decodes, through a captured graph, and nothing
can change the set of requests before the next step (nobody waits, nobody reaches
its length), the next step is started on the device before this step's tokens
have reached the host: it reads them from the sampler's device buffer, and its
pages are taken a step early.  The scheduler is not told; the next call plans as
ever, and if its plan is the step that is already running, that step's results
are taken, otherwise (a request ended on an end-of-sequence token, was aborted,
was added) they are dropped and the plan runs.  A dropped step has only written
keys and values of its own requests at positions that the plan writes again or
whose pages were given back; later work on the stream overwrites what it
reuses before reading it.  A model with per-request state of its own (which a
step changes in place) does not look ahead.
"""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from ..config.engine_config import EngineConfig
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from ..utils import log
from .core import EngineCore
from .graphs import RecordingFailed
from .scheduler import FINISH_REASON, STATUS, Scheduler


class RequestOutput:
    def __init__(self, request_id, prompt_tokens: list, output_tokens: list, finished: bool,
                 finish_reason: Optional[str] = None):
        self.request_id = request_id
        self.prompt_tokens = prompt_tokens
        self.output_tokens = output_tokens
        self.finished = finished
        self.is_finished = finished
        self.finish_reason = finish_reason

    def __repr__(self):
        return (f"RequestOutput(request_id={self.request_id!r}, output_tokens={self.output_tokens}, "
                f"finished={self.finished}, finish_reason={self.finish_reason!r})")


class _Request:
    __slots__ = ("request_id", "params", "stream", "prompt", "outputs")

    def __init__(self, request_id, params, stream, prompt):
        self.request_id, self.params, self.stream, self.prompt = request_id, params, stream, prompt
        self.outputs: list = []


class _Ahead:
    """A decode step that is running before the scheduler has planned it."""
    __slots__ = ("ids", "start", "pending")

    def __init__(self, ids, start, pending):
        self.ids, self.start, self.pending = ids, start, pending

    def is_plan(self, ids, start) -> bool:
        return len(ids) == len(self.ids) and bool((ids == self.ids).all()) and bool((start == self.start).all())


class LLMEngine:
    def __init__(self, model, config: Optional[EngineConfig] = None, **kw):
        """``model`` is an ``EngineCore``, or a model folder (then the core is
        built from ``config``)."""
        config = config or EngineConfig(**kw)
        self.config = config
        if isinstance(model, EngineCore):
            self.core = model
        else:
            self.core = EngineCore.from_folder(str(model), dtype=config.dtype, device=config.device,
                                               num_blocks=config.num_blocks, block_size=config.block_size,
                                               cache_groups=config.cache_groups, num_state_slots=config.max_num_seqs,
                                               max_model_len=config.max_model_len)
        spec = self.core.model.spec
        # (the model's position tables may have fewer rows than spec.max_position: as many as a request
        # can reach, EngineCore.reach; where a pool that keeps every token is the bound, a longer request
        # is refused for its pages, not its length)
        self.max_model_len = min(config.max_model_len or spec.max_position, spec.max_position)
        eos = config.eos_token_ids if config.eos_token_ids is not None else spec.eos_token_ids
        self.scheduler = Scheduler(self.core.cache, max_num_seqs=config.max_num_seqs,
                                   max_num_batched_tokens=config.max_num_batched_tokens,
                                   max_model_len=self.max_model_len, max_chunk=config.max_chunk,
                                   eos_token_ids=tuple(eos))
        self.sampler = Sampler(self.core.device, seed=config.seed)
        self.req_counter = 0
        self._requests: dict = {}     # seq id -> _Request
        self._by_request: dict = {}   # request id -> seq id
        self.graphs = None
        if config.enable_graphs:
            from .graphs import DecodeGraphs
            self.graphs = DecodeGraphs(self.core.runner, max_batch=config.max_num_seqs)
        # A step that is dropped is run again: harmless for keys and values (the same values to the
        # same slots), not for a mixer's own state, which the step changes in place.
        self._look_ahead = bool(config.lookahead) and not self.core.pools.state
        self._ahead: Optional[_Ahead] = None
        self.steps_taken_ahead = 0    # steps whose results came from a step started ahead
        self.recording_failures: list = []   # why recorded steps or looking ahead were switched off, if they were
        if config.warmup:
            self._warm_up()

    def counters(self) -> dict:
        """What the scheduler and the cache manager counted so far, and what this engine did beside them."""
        return dict(scheduler=self.scheduler.counters(), cache=self.core.cache.counters(),
                    steps_taken_ahead=self.steps_taken_ahead,
                    graphs_recorded=len(self.graphs.captured) if self.graphs is not None else 0,
                    recording_failures=len(self.recording_failures))

    def __del__(self):
        try:
            if log.level() == "debug" and hasattr(self, "scheduler"):
                log.debug(f"engine dropped: {self.counters()}")
        except Exception:  # noqa: BLE001  (an interpreter that is shutting down may have taken the modules away)
            pass

    WARMUP_ID = -1   # the cache manager's name for the warm-up step's request; the scheduler counts from 0

    def _warm_up(self) -> None:
        """Steps of as many tokens as a step may bring (as far as the model's
        length and the pages go), and of every power of two from 128 up to
        that, by a request that is gone afterwards.  They load the kernels a
        full step needs, and the products of that many rows are given the
        fastest of the vendor library's algorithms by measurement
        (``ops.library_gemm_tuning``) rather than the library's first guess; a
        prompt portion of any other length later takes the choice measured for
        the nearest of these sizes."""
        from ..kernels import ops

        cache, cfg = self.core.cache, self.config
        room = min(cache.num_free_pages(g) * gc.page_size for g, gc in enumerate(cache.groups))  # tokens a step may bring
        sizes = {cfg.max_num_batched_tokens}
        if cfg.max_chunk:
            sizes.add(min(cfg.max_chunk, cfg.max_num_batched_tokens))
        if ops.LIBRARY_GEMM and ops.LIBRARY_TUNE_CANDIDATES > 1 and self.core.dtype == torch.bfloat16:
            n = 128
            while n < cfg.max_num_batched_tokens:
                sizes.add(n)
                n *= 2
        for n in sorted({min(s, self.max_model_len, room) for s in sizes}):
            if n < 1 or cache.has(self.WARMUP_ID) or cache.num_free_slots() < 1:
                continue
            cache.add(self.WARMUP_ID)
            try:
                cache.extend(self.WARMUP_ID, n)
                if len(sizes) > 2:
                    log.info(f"warm-up: a step of {n} tokens (matrix-product algorithms chosen by measurement)")
                with ops.library_gemm_tuning():
                    self.core.runner.step_arrays(np.asarray([self.WARMUP_ID], dtype=np.int64), np.zeros(1, dtype=np.int32),
                                                 np.asarray([n], dtype=np.int32), np.zeros(n, dtype=np.int32),
                                                 np.asarray([n - 1], dtype=np.int32))
                torch.cuda.synchronize(self.core.device)
            finally:
                cache.free(self.WARMUP_ID)

    # ---------------------------------------------------------------- requests
    def add_request(self, arg1, arg2=None, arg3=None):
        """``add_request(prompt_tokens, sampling_params)`` or
        ``add_request(request_id, prompt_tokens, sampling_params)``."""
        if isinstance(arg1, (int, str)) and isinstance(arg2, (list, tuple)):
            request_id, prompt, params = arg1, list(arg2), arg3 or SamplingParams()
        elif isinstance(arg1, (list, tuple)):
            request_id, prompt = self.req_counter, list(arg1)
            while request_id in self._by_request:    # a caller's own id may be this number already
                request_id += 1
            params = arg2 if isinstance(arg2, SamplingParams) else SamplingParams()
        else:
            raise TypeError("Invalid arguments provided to add_request")
        if request_id in self._by_request:
            raise ValueError(f"request id {request_id!r} is in use")
        vocab = self.core.model.spec.vocab_size
        ids = np.asarray(prompt)
        if ids.ndim != 1 or (ids.size and (ids.dtype.kind not in "iu" or int(ids.min()) < 0 or int(ids.max()) >= vocab)):
            raise ValueError(f"a prompt is a list of token ids below the vocabulary's {vocab}")
        seq_id = self.req_counter
        self.req_counter += 1
        self.scheduler.add(seq_id, prompt, params)
        stream = params.seed if params.seed is not None else seq_id
        self._requests[seq_id] = _Request(request_id, params, stream, prompt)
        self._by_request[request_id] = seq_id
        return request_id

    def abort_request(self, request_id) -> bool:
        seq_id = self._by_request.get(request_id)
        if seq_id is None:
            return False
        done = self.scheduler.abort(seq_id)
        self._drop(seq_id)
        return done

    def _drop(self, seq_id: int) -> None:
        req = self._requests.pop(seq_id)
        self._by_request.pop(req.request_id, None)
        self.scheduler.forget(seq_id)

    def has_unfinished_requests(self) -> bool:
        return self.scheduler.has_unfinished()

    # -------------------------------------------------------------------- step
    def step(self) -> list:
        """One iteration.  Returns a RequestOutput for every request that took
        part; ``output_tokens`` of an unfinished request is the engine's own
        growing list (copy it to keep a snapshot)."""
        if not self.has_unfinished_requests():
            self._ahead = None
            return []
        ids, start, count, wants = self.scheduler.schedule_arrays()
        ahead, self._ahead = self._ahead, None
        n = len(ids)
        if n == 0:
            return []  # everything running was preempted; the next step admits again
        tokens = self.scheduler.plan_tokens()
        reqs = [self._requests[int(i)] for i in ids]
        decoding = self.graphs is not None and self.graphs.safe and n <= self.graphs.max_batch and \
            bool((count == 1).all()) and bool(wants.all())
        if ahead is not None and decoding and ahead.is_plan(ids, start):
            pending = ahead.pending
            self.steps_taken_ahead += 1
        else:
            logits = None
            recorded = decoding or (self.graphs is not None and bool(wants.all()) and self.graphs.prompt_usable(count))
            if recorded:
                # A recorded step that cannot be had for lack of memory is no reason to lose the step: it
                # runs eagerly, and so do all later ones (``recording_failures`` says so to whoever asks).
                # Anything else that goes wrong in a recorded step (its tables, a kernel's check) is a
                # defect and is raised.
                try:
                    if decoding:
                        logits = self.graphs.step_arrays(ids, start, tokens)
                    else:   # a short prompt alone in its step
                        logits = self.graphs.prompt_step_arrays(ids, start, count, tokens)
                except RecordingFailed as err:
                    self.graphs.safe, self._look_ahead, decoding = False, False, False
                    self.recording_failures.append(str(err))
                    log.warn(f"recorded steps switched off: {err}")
            if logits is None:
                rows = (np.cumsum(count, dtype=np.int32) - 1)[wants != 0]   # the last token of each request that wants
                logits = self.core.runner.step_arrays(ids, start, count, tokens, rows)
            wanting = [r for r, w in zip(reqs, wants) if w]
            pending = None
            if wanting:
                pending = self.sampler.launch(logits, [r.params for r in wanting], [r.stream for r in wanting],
                                              [len(r.outputs) for r in wanting])
        if decoding and self._look_ahead:
            # Optional work must not break the planned step: when the next one cannot be started
            # because a new graph cannot be recorded (no memory for it), this step's tokens still
            # reach the scheduler; looking ahead is then switched off.
            try:
                self._ahead = self._start_ahead(ids, start, reqs, pending)
            except RecordingFailed as err:
                self._ahead, self._look_ahead = None, False
                self.recording_failures.append(str(err))
                log.warn(f"looking ahead switched off: {err}")
        sampled = pending.result() if pending is not None else []
        status = self.scheduler.post_step_status(sampled)
        outputs, k = [], 0
        for i in range(n):
            req = reqs[i]
            if wants[i]:
                req.outputs.append(sampled[k])
                k += 1
            code = int(status[i])
            finished = code >= 2
            outputs.append(RequestOutput(req.request_id, req.prompt, req.outputs, finished,
                                         FINISH_REASON.get(STATUS[code])))
            if finished:
                self._drop(int(ids[i]))
        return outputs

    def _start_ahead(self, ids, start, reqs, pending) -> Optional[_Ahead]:
        """Start the decode step that follows the planned one (same requests, one
        position on, the tokens that ``pending`` is choosing), if nothing but an
        end-of-sequence token can keep the next plan from being that step."""
        if self.scheduler.num_waiting():
            return None
        next_start = start + 1
        if int(next_start.max()) + 1 >= self.max_model_len or \
                any(len(r.outputs) + 1 >= r.params.max_tokens for r in reqs):
            return None  # somebody reaches a length in the planned step
        ids = ids.copy()
        if not self.core.cache.reserve(ids, next_start + 1):
            return None  # no pages to take early
        logits = self.graphs.step_arrays(ids, next_start, np.zeros(len(ids), dtype=np.int32), tokens_dev=pending.tokens)
        return _Ahead(ids, next_start, self.sampler.launch(logits, [r.params for r in reqs], [r.stream for r in reqs],
                                                           [len(r.outputs) + 1 for r in reqs]))

    def generate(self, prompts: list, params=None) -> list:
        """Run the prompts (lists of token ids) to the end; one RequestOutput
        per prompt, in order.  ``params`` is one SamplingParams or one per prompt."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        ids = [self.add_request(list(p), sp) for p, sp in zip(prompts, params)]
        done: dict = {}
        while self.has_unfinished_requests():
            for out in self.step():
                if out.finished:
                    done[out.request_id] = out
        return [done[i] for i in ids]


class LLM:
    """``LLM(folder, dtype="bfloat16", num_blocks=..., ...).generate(prompts, params)``."""

    def __init__(self, model: str, **engine_options):
        self.engine = LLMEngine(model, EngineConfig(**engine_options))

    def generate(self, prompts: list, params=None) -> list:
        return self.engine.generate(prompts, params)


def generate(model: str, prompts: list, params=None, **engine_options) -> list:
    return LLM(model, **engine_options).generate(prompts, params)


__all__ = ["LLMEngine", "LLM", "RequestOutput", "generate", "SamplingParams", "EngineConfig", "torch"]
