"""Scheduler: the Python face of the host core's scheduler (csrc/host/scheduler.h).

It decides, step by step, which requests run and with how many tokens: every running request
whose next token is known decodes, then prompts go on in portions, under a token budget.
What happens when pages run out is the policy: "reserve" admits a request only if its peak
need can be set aside (nothing ever runs out in mid-run); "preempt" takes pages step by step,
and when a running request cannot get one, the youngest running request gives all its pages
back and returns to the head of the queue, to be recomputed from its known tokens.
"""
from __future__ import annotations

import ctypes
from ctypes import c_int
from dataclasses import dataclass
from typing import List, Tuple

import numpy as np

from ..cache.manager import CacheManager, host_library

POLICIES = {"preempt": 0, "reserve": 1}

EMPTY_PROMPT, PROMPT_TOO_LONG, NEVER_FITS, DUPLICATE, UNKNOWN, BAD_STATE = -10, -11, -12, -13, -14, -15
_NAMES = {EMPTY_PROMPT: "the prompt is empty",
          PROMPT_TOO_LONG: "the prompt is longer than the model's positions",
          NEVER_FITS: "the request needs more pages than the cache has, even alone",
          DUPLICATE: "request id is in use", UNKNOWN: "unknown request id",
          BAD_STATE: "the request is not in a state that allows this"}


class SchedulerError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        super().__init__(f"{what}: {_NAMES.get(code, code)}")


@dataclass(frozen=True)
class Planned:
    rid: int
    start: int       # tokens in the cache before the step
    count: int       # tokens to feed
    samples: bool    # the step brings the request to its last known token


class Scheduler:
    def __init__(self, cache: CacheManager, *, max_live: int, max_batch_tokens: int, prefill_chunk: int,
                 policy: str, max_positions: int):
        self._lib = host_library()
        self._cache = cache   # keeps the manager alive as long as the scheduler
        self._h = self._lib.dn_sched_create(cache._h, max_live, max_batch_tokens, prefill_chunk,
                                            POLICIES[policy], max_positions)
        if not self._h:
            raise ValueError("scheduler: bad arguments")
        self._cap = max(max_live, 1)
        self._rid = np.empty(self._cap, dtype=np.int64)
        self._start = np.empty(self._cap, dtype=np.int32)
        self._count = np.empty(self._cap, dtype=np.int32)
        self._samples = np.empty(self._cap, dtype=np.int32)
        self._pre = np.empty(self._cap, dtype=np.int64)

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.dn_sched_destroy(self._h)
            self._h = None

    def _chk(self, rc, what):
        if rc < 0:
            raise SchedulerError(rc, what)
        return rc

    def add(self, rid: int, prompt_len: int, max_new: int) -> int:
        """Queues a request; -> max_new after clamping to the positions left."""
        return self._chk(self._lib.dn_sched_add(self._h, rid, prompt_len, max_new), f"add request {rid}")

    def schedule(self) -> Tuple[List[Planned], List[int]]:
        """-> (this step's entries, requests preempted while planning it)."""
        n_pre = c_int(0)
        n = self._lib.dn_sched_schedule(self._h, self._rid.ctypes.data, self._start.ctypes.data,
                                        self._count.ctypes.data, self._samples.ctypes.data, self._cap,
                                        self._pre.ctypes.data, ctypes.byref(n_pre), self._cap)
        if n < 0:
            raise RuntimeError("scheduler: more entries than live requests")
        plan = [Planned(int(self._rid[i]), int(self._start[i]), int(self._count[i]), bool(self._samples[i]))
                for i in range(n)]
        return plan, [int(self._pre[i]) for i in range(n_pre.value)]

    def step_done(self, rid: int, count: int):
        self._chk(self._lib.dn_sched_step_done(self._h, rid, count), f"step done for request {rid}")

    def token_sampled(self, rid: int) -> bool:
        """One more token is known; -> True if it was the request's last (length)."""
        return bool(self._chk(self._lib.dn_sched_token_sampled(self._h, rid), f"token for request {rid}"))

    def steps_done(self, rids: np.ndarray, counts: np.ndarray):
        """step_done for all entries of a step (rids int64, counts int32)."""
        failed = c_int(0)
        rc = self._lib.dn_sched_steps_done(self._h, rids.ctypes.data, counts.ctypes.data, len(rids), ctypes.byref(failed))
        if rc < 0:
            raise SchedulerError(rc, f"step done for request {int(rids[failed.value])}")

    def tokens_sampled(self, rids: np.ndarray) -> np.ndarray:
        """token_sampled for all of them; -> int32 array, 1 where the token was the request's last."""
        last = np.zeros(len(rids), dtype=np.int32)
        failed = c_int(0)
        rc = self._lib.dn_sched_tokens_sampled(self._h, rids.ctypes.data, len(rids), last.ctypes.data, ctypes.byref(failed))
        if rc < 0:
            raise SchedulerError(rc, f"token for request {int(rids[failed.value])}")
        return last

    def finish(self, rid: int):
        self._chk(self._lib.dn_sched_finish(self._h, rid), f"finish request {rid}")

    def n_waiting(self) -> int:
        return self._lib.dn_sched_n_waiting(self._h)

    def n_running(self) -> int:
        return self._lib.dn_sched_n_running(self._h)

    def known(self, rid: int) -> int:
        """The tokens the scheduler knows of the request; -1 if it has no such request (any more)."""
        rc = self._lib.dn_sched_known(self._h, rid)
        return -1 if rc == UNKNOWN else self._chk(rc, f"request {rid}")

    def computed(self, rid: int) -> int:
        return self._chk(self._lib.dn_sched_computed(self._h, rid), f"request {rid}")

    def generated(self, rid: int) -> int:
        return self._chk(self._lib.dn_sched_generated(self._h, rid), f"request {rid}")
