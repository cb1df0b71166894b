"""The scheduler as Python sees it: a thin wrapper of the C++ class in
csrc/runtime/scheduler.hpp (after the reference's ContinuousScheduler,
csrc/engine/scheduler.cpp:7-138, bound there with pybind11,
csrc/bindings.cpp:552-621)."""
from __future__ import annotations

from ctypes import POINTER, c_int32, c_int64
from dataclasses import dataclass

import numpy as np

from ..cache import runtime_lib
from ..cache.manager import CacheManager
from ..sampling.params import SamplingParams

STATUS = ("waiting", "running", "finished_stopped", "finished_length_capped", "finished_aborted")
FINISH_REASON = {"finished_stopped": "stop", "finished_length_capped": "length", "finished_aborted": "abort"}


class SchedulerError(RuntimeError):
    pass


@dataclass
class Scheduled:
    seq_id: int
    start: int
    count: int
    wants_logits: bool


@dataclass
class SequenceInfo:
    prompt_len: int
    total_len: int
    num_computed: int
    status: str
    preemptions: int

    @property
    def finished(self) -> bool:
        return self.status.startswith("finished")


class Scheduler:
    def __init__(self, cache: CacheManager, *, max_num_seqs: int, max_num_batched_tokens: int, max_model_len: int,
                 max_chunk: int = 0, eos_token_ids=()):
        self._lib = runtime_lib.lib()
        self.cache = cache  # keeps the C++ cache manager alive as long as the scheduler
        eos = (c_int32 * max(1, len(eos_token_ids)))(*eos_token_ids)
        self._h = self._lib.lyp_sched_create(cache.handle, max_num_seqs, max_num_batched_tokens, max_model_len,
                                             max_chunk, eos, len(eos_token_ids))
        if not self._h:
            raise SchedulerError(runtime_lib.last_error())
        self._cap = max(max_num_seqs, 1) + 8
        self._ids = np.zeros(self._cap, dtype=np.int64)
        self._start = np.zeros(self._cap, dtype=np.int32)
        self._count = np.zeros(self._cap, dtype=np.int32)
        self._wants = np.zeros(self._cap, dtype=np.int32)
        self._status = np.zeros(self._cap, dtype=np.int32)
        self._tokens = np.zeros(max(max_num_batched_tokens, 1), dtype=np.int32)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.lyp_sched_destroy(h)

    def _rc(self, rc: int) -> int:
        if rc < 0:
            raise SchedulerError(runtime_lib.last_error())
        return rc

    def add(self, seq_id: int, prompt: list, params: SamplingParams) -> None:
        arr = np.ascontiguousarray(prompt, dtype=np.int32)
        # the scheduler gets what decides when a request ends; how tokens are chosen stays with the sampler
        self._rc(self._lib.lyp_sched_add(self._h, seq_id, arr.ctypes.data_as(POINTER(c_int32)), len(arr),
                                         params.max_tokens, int(params.ignore_eos)))

    def abort(self, seq_id: int) -> bool:
        return bool(self._rc(self._lib.lyp_sched_abort(self._h, seq_id)))

    def has_unfinished(self) -> bool:
        return bool(self._lib.lyp_sched_has_unfinished(self._h))

    def num_waiting(self) -> int:
        return self._lib.lyp_sched_num_waiting(self._h)

    def num_running(self) -> int:
        return self._lib.lyp_sched_num_running(self._h)

    def schedule_arrays(self):
        """Plan a step -> (ids, start, count, wants): numpy views, valid until
        the next call."""
        n = self._rc(self._lib.lyp_sched_schedule(self._h, self._ids.ctypes.data, self._start.ctypes.data,
                                                  self._count.ctypes.data, self._wants.ctypes.data, self._cap))
        return self._ids[:n], self._start[:n], self._count[:n], self._wants[:n]

    def schedule(self) -> list:
        ids, start, count, wants = self.schedule_arrays()
        return [Scheduled(int(i), int(s), int(c), bool(w)) for i, s, c, w in zip(ids, start, count, wants)]

    def plan_tokens(self):
        """The tokens of the planned portions, one after the other (a numpy
        view, valid until the next call)."""
        n = self._rc(self._lib.lyp_sched_plan_tokens(self._h, self._tokens.ctypes.data, len(self._tokens)))
        return self._tokens[:n]

    def post_step_status(self, sampled):
        """post_step, returning the status code of every planned request after
        the step (index into STATUS), in the order of the plan."""
        arr = np.ascontiguousarray(sampled, dtype=np.int32)
        n = self._rc(self._lib.lyp_sched_post_step_status(self._h, arr.ctypes.data, len(arr),
                                                          self._status.ctypes.data, self._cap))
        return self._status[:n]

    def post_step(self, sampled: list) -> None:
        arr = (c_int32 * max(1, len(sampled)))(*sampled)
        self._rc(self._lib.lyp_sched_post_step(self._h, arr, len(sampled)))

    def last_preempted(self) -> list:
        buf = (c_int64 * self._cap)()
        n = self._lib.lyp_sched_last_preempted(self._h, buf, self._cap)
        return list(buf[:min(n, self._cap)])

    def info(self, seq_id: int) -> SequenceInfo:
        out = (c_int32 * 5)()
        self._rc(self._lib.lyp_sched_info(self._h, seq_id, out))
        return SequenceInfo(out[0], out[1], out[2], STATUS[out[3]], out[4])

    def tokens(self, seq_id: int, start: int = 0, count: int | None = None) -> list:
        if count is None:
            count = self.info(seq_id).total_len - start
        buf = (c_int32 * max(1, count))()
        n = self._rc(self._lib.lyp_sched_tokens(self._h, seq_id, start, buf, count))
        return list(buf[:n])

    def forget(self, seq_id: int) -> None:
        self._rc(self._lib.lyp_sched_forget(self._h, seq_id))

    def counters(self) -> dict:
        out = (c_int64 * 4)()
        self._lib.lyp_sched_counters(self._h, out)
        return dict(steps=out[0], scheduled_tokens=out[1], preemptions=out[2], finished=out[3])
