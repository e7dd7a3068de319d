"""Engine: requests in, tokens out.  It joins the model runner (weights, cache, the step
function), the scheduler and the sampler.

The reference's engine goes begin_chat -> install_session -> step_chat / step_chat_batch ->
release_session (crates/denno-engine/src/engine.rs:810-817, 532-545, 946-966, 1309-1342,
707-737).  Here: add_request -> step (each call runs one mixed batch and samples) -> the
request is released when it finishes.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Dict, Iterable, List, Optional, Sequence

import numpy as np
import torch

from ..config import EngineOptions
from ..sampling import Sampler, SamplingParams, entropy_seed
from .batch import StepEntry
from .runner import ModelRunner
from .scheduler import Scheduler, SchedulerError


@dataclass
class Request:
    rid: int
    prompt: List[int]
    params: SamplingParams
    seed: int
    max_new: int
    tokens: List[int] = field(default_factory=list)    # prompt + generated
    finished: bool = False
    finish_reason: Optional[str] = None                 # "eos", "length", "error"
    preemptions: int = 0

    @property
    def generated(self) -> List[int]:
        return self.tokens[len(self.prompt):]


@dataclass
class StepOutput:
    rid: int
    token: Optional[int]       # the token sampled in this step, if any
    finished: bool
    finish_reason: Optional[str]


@dataclass
class StepRecord:
    """What one step ran: for measurement and tests."""
    rows: int
    decode_rows: int
    prefill_rows: int
    requests: int
    preempted: int
    host_ms: float = 0.0     # wall time of Engine.step on the host (it ends with the read of the sampled tokens)


class Engine:
    def __init__(self, runner: ModelRunner, options: Optional[EngineOptions] = None):
        self.runner = runner
        self.options = options or runner.options
        self.spec = runner.spec
        self.scheduler = Scheduler(
            runner.cache.manager, max_live=self.options.max_live,
            max_batch_tokens=self.options.max_batch_tokens, prefill_chunk=self.options.prefill_chunk,
            policy=self.options.kv_policy, max_positions=self.spec.max_positions)
        self.sampler = Sampler(runner.device)
        self.requests: Dict[int, Request] = {}
        self._next_rid = 0
        self.records: List[StepRecord] = []
        self.fail_next_step = False    # test hook: the next step raises after its pages were taken

    @classmethod
    def from_folder(cls, model_dir: str, options: Optional[EngineOptions] = None, cast_matrices=False):
        options = options or EngineOptions()
        return cls(ModelRunner.from_folder(model_dir, options, cast_matrices), options)

    @classmethod
    def from_random(cls, config: dict, seed: int, options: Optional[EngineOptions] = None, stored=None):
        options = options or EngineOptions()
        return cls(ModelRunner.from_random(config, seed, options, stored), options)

    # -- requests ------------------------------------------------------------------------
    def add_request(self, prompt: Sequence[int], params: Optional[SamplingParams] = None) -> int:
        """Queues a request; raises on an empty prompt, a prompt that fills the context, a token
        outside the vocabulary, or a request that could never fit the cache."""
        params = (params or SamplingParams()).validate()
        prompt = [int(t) for t in prompt]
        for t in prompt:
            if not 0 <= t < self.spec.vocab:
                raise ValueError(f"token id {t} is outside the vocabulary of {self.spec.vocab}")
        rid = self._next_rid
        max_new = self.scheduler.add(rid, len(prompt), params.max_tokens)   # clamped to the positions left
        self._next_rid += 1
        seed = params.seed if params.seed is not None else (
            self.options.seed if self.options.seed is not None else entropy_seed())
        self.requests[rid] = Request(rid, prompt, params, seed, max_new, list(prompt))
        return rid

    def has_unfinished(self) -> bool:
        return self.scheduler.n_waiting() + self.scheduler.n_running() > 0

    def abort(self, rid: int):
        req = self.requests.get(rid)
        if req is None or req.finished:
            return
        self.scheduler.finish(rid)
        req.finished, req.finish_reason = True, "aborted"

    # -- one step ------------------------------------------------------------------------
    def step(self) -> List[StepOutput]:
        t_begin = time.perf_counter()
        plan, preempted = self.scheduler.schedule()
        for rid in preempted:
            self.requests[rid].preemptions += 1
        if not plan:
            if self.has_unfinished():
                raise RuntimeError("scheduler: requests are waiting but none can run "
                                   "(a request larger than the cache should have been refused)")
            return []
        entries, sampled = [], []
        manager = self.runner.cache.manager
        for p in plan:
            req = self.requests[p.rid]
            if p.start == 0:
                # admitted (or admitted again after preemption): fixed-size states start at zero, and the
                # request's slot record gets its generator (seed, numbers drawn so far: a request that
                # comes back after preemption goes on where it was, so its samples do not change)
                self.runner.cache.reset_states(manager.slot(p.rid))
                manager.set_rng(p.rid, req.seed, len(req.generated))
            wants = p.samples and len(req.generated) < req.max_new
            entries.append(StepEntry(p.rid, req.tokens[p.start:p.start + p.count], [p.count - 1] if wants else []))
            if wants:
                sampled.append(req)
        try:
            if self.fail_next_step:
                self.fail_next_step = False
                raise RuntimeError("step failed (injected)")
            logits = self.runner.step(entries)
            for p in plan:
                self.scheduler.step_done(p.rid, p.count)
            # each request's generator lives in its slot record: the seed and the count of numbers drawn
            seeds, drawn = manager.rng_states(np.asarray([r.rid for r in sampled], dtype=np.int64))
            tokens = self.sampler.sample(logits, [r.params for r in sampled], seeds.tolist(), drawn.tolist(),
                                         [r.tokens for r in sampled])
            for r, tok in zip(sampled, tokens):
                manager.note_sampled(r.rid, int(tok))
        except Exception:
            # the step's requests are dropped, their pages go back, the engine stays usable
            # (crates/denno-server/src/scheduler.rs:362-370, 457-469)
            for p in plan:
                req = self.requests[p.rid]
                self.scheduler.finish(p.rid)
                req.finished, req.finish_reason = True, "error"
            raise
        self.records.append(StepRecord(
            rows=sum(p.count for p in plan), decode_rows=sum(1 for p in plan if p.count == 1 and p.start > 0),
            prefill_rows=sum(p.count for p in plan if not (p.count == 1 and p.start > 0)),
            requests=len(plan), preempted=len(preempted)))
        record = self.records[-1]
        outputs = []
        by_rid = {r.rid: t for r, t in zip(sampled, tokens)}
        eos = set(self.spec.eos_token_ids)
        for p in plan:
            req = self.requests[p.rid]
            tok = by_rid.get(p.rid)
            if tok is not None:
                req.tokens.append(int(tok))
                last = self.scheduler.token_sampled(p.rid)
                # the end-of-sequence token counts as generated (crates/denno-engine/src/engine.rs:1125-1129)
                if int(tok) in eos and not req.params.ignore_eos:
                    req.finish_reason = "eos"
                elif last:
                    req.finish_reason = "length"
            elif p.samples and len(req.generated) >= req.max_new:
                req.finish_reason = "length"      # max_tokens = 0: the prompt is computed, nothing is sampled
            if req.finish_reason is not None:
                req.finished = True
                self.scheduler.finish(p.rid)
            outputs.append(StepOutput(p.rid, None if tok is None else int(tok), req.finished, req.finish_reason))
        record.host_ms = (time.perf_counter() - t_begin) * 1e3
        return outputs

    # -- whole generations ---------------------------------------------------------------
    def generate(self, prompts: Iterable[Sequence[int]], params=None) -> List[List[int]]:
        """Runs the prompts to their ends; -> generated tokens of each, in the prompts' order.
        params: one SamplingParams for all, or one per prompt."""
        prompts = list(prompts)
        plist = params if isinstance(params, (list, tuple)) else [params] * len(prompts)
        rids = [self.add_request(p, sp) for p, sp in zip(prompts, plist)]
        while self.has_unfinished():
            self.step()
        out = [self.requests[r].generated for r in rids]
        return out

    def finish_reason(self, rid: int) -> Optional[str]:
        return self.requests[rid].finish_reason
