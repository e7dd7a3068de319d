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
    finish_reason: Optional[str] = None                 # "eos", "length", "stop_sequence", "error", "aborted"
    text: Optional[str] = None                          # the generated text, where the engine has a detokenizer
    stop_sequence: Optional[str] = None                 # the stop sequence that ended it
    preemptions: int = 0
    n_sampled: int = 0     # tokens sampled for it so far, the one that the host has not read yet among them

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
    ran_ahead: bool = False  # launched before the step before it had given its tokens to the host
    host_ms: float = 0.0     # wall time of the step's two halves on the host (the second ends with the read of the tokens)


@dataclass
class _Launched:
    """A step whose kernels are issued and whose sampled tokens are not read yet."""
    plan: list
    sampled: List[Request]           # the requests that are sampled, in the order of the logits' rows
    last: Dict[int, bool]            # request id -> the token being sampled is its last (length)
    alive: List[Request]             # the sampled requests that go on after this step
    pending: object                  # sampling.sampler.Pending
    record: StepRecord


class _AheadFailed(Exception):
    """The step that was launched ahead could not run; its requests are not dropped yet (`plan`)."""

    def __init__(self, plan):
        super().__init__("the step launched ahead failed")
        self.plan = plan


class Engine:
    def __init__(self, runner: ModelRunner, options: Optional[EngineOptions] = None, detokenize=None):
        """detokenize: token ids -> text, for requests with stop sequences (and for `Request.text`)."""
        self.runner = runner
        self.detokenize = detokenize
        self.options = options or runner.options
        self.spec = runner.spec
        self.scheduler = Scheduler(
            runner.cache.manager, max_live=self.options.max_live,
            max_batch_tokens=self.options.max_batch_tokens, prefill_chunk=self.options.prefill_chunk,
            policy=self.options.kv_policy, max_positions=self.spec.max_positions)
        self.sampler = Sampler(runner.device, self.options.max_live, self.spec.max_positions + 1)
        self.requests: Dict[int, Request] = {}
        self._next_rid = 0
        self.records: List[StepRecord] = []
        self.fail_next_step = False    # test hook: the next step raises after its pages were taken
        self._ahead: Optional[_Launched] = None      # the step that was launched before the last one was read
        self._failed_ahead: Optional[Exception] = None

    @classmethod
    def from_folder(cls, model_dir: str, options: Optional[EngineOptions] = None, cast_matrices=False,
                    detokenize=None):
        options = options or EngineOptions()
        return cls(ModelRunner.from_folder(model_dir, options, cast_matrices), options, detokenize)

    @classmethod
    def from_random(cls, config: dict, seed: int, options: Optional[EngineOptions] = None, stored=None):
        options = options or EngineOptions()
        return cls(ModelRunner.from_random(config, seed, options, stored), options)

    # -- requests ------------------------------------------------------------------------
    def add_request(self, prompt: Sequence[int], params: Optional[SamplingParams] = None) -> int:
        """Queues a request; raises on an empty prompt, a prompt that fills the context, a token
        outside the vocabulary, or a request that could never fit the cache."""
        params = (params or SamplingParams()).validate()
        if any(params.stop_sequences) and self.detokenize is None:
            raise ValueError("stop_sequences are texts: the engine needs a detokenizer for them (Engine(..., detokenize=))")
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
        """Requests are waiting or running, a launched step's tokens have not been read yet, or the failure
        of a step that was launched ahead has not been reported yet (the next `step` raises it)."""
        return (self.scheduler.n_waiting() + self.scheduler.n_running() > 0 or self._ahead is not None
                or self._failed_ahead is not None)

    def _release(self, rid: int):
        """The request's pages and slot go back, unless they have (its last token was already on its way)."""
        if self.scheduler.known(rid) >= 0:
            self.scheduler.finish(rid)

    def abort(self, rid: int):
        req = self.requests.get(rid)
        if req is None or req.finished:
            return
        self._release(rid)
        req.finished, req.finish_reason = True, "aborted"

    # -- one step ------------------------------------------------------------------------
    # A step has two halves: `_launch` plans it, issues its kernels and the sampling kernels and does the
    # bookkeeping that needs counts only; `_complete` waits for the sampled tokens and does what needs the
    # tokens themselves (the request's token list, the end-of-sequence check).  In steady decoding the next
    # step is launched between the two, with its tokens taken from the device where the sampling kernel
    # left them (`run_ahead`): the host's work on a step then hides behind the GPU's work on the next one,
    # and a request that ends with an end-of-sequence token has run one step too many, whose token is
    # thrown away.
    def step(self) -> List[StepOutput]:
        if self._failed_ahead is not None:          # the step that was launched ahead could not run
            exc, self._failed_ahead = self._failed_ahead, None
            raise exc
        launched, self._ahead = self._ahead, None
        if launched is not None and all(r.finished for r in launched.sampled):
            launched = None                         # launched ahead for requests that have all ended since
        if launched is None:
            launched = self._launch(None)
        if launched is None:
            return []
        failed_plan = None
        if self._may_run_ahead(launched):
            try:
                self._ahead = self._launch(launched)
            except _AheadFailed as failure:
                # This step's tokens are sampled already and are the requests' own: they are read and told first.
                # Then the failed step's requests are dropped, and the caller hears the error from the next
                # `step`, which `has_unfinished` keeps it calling for.
                failed_plan, self._failed_ahead = failure.plan, failure.__cause__
        outputs = self._complete(launched)
        if failed_plan is not None:
            dropped = self._drop(failed_plan)
            for o in outputs:
                if o.rid in dropped:
                    o.finished, o.finish_reason = True, "error"
        return outputs

    def _drop(self, plan) -> set:
        """A step that failed: its requests end with an error and their pages go back, so that the engine stays
        usable (crates/denno-server/src/scheduler.rs:362-370, 457-469).  -> the requests dropped here."""
        dropped = set()
        for p in plan:
            req = self.requests[p.rid]
            if not req.finished:
                self._release(p.rid)
                req.finished, req.finish_reason = True, "error"
                dropped.add(p.rid)
        return dropped

    def _may_run_ahead(self, launched: "_Launched") -> bool:
        """The next step can be planned and launched before this one's tokens are known on the host: it will
        be single tokens of requests that were all sampled in this one, replayed from a graph, and nothing
        about it depends on the tokens' values."""
        if not (self.options.run_ahead and self.runner.runs_ahead() and launched.pending.final):
            return False
        if self.scheduler.n_waiting() > 0 or self.scheduler.n_running() == 0:
            return False
        return self.scheduler.n_running() == len(launched.alive)     # (else: a running request not sampled in this step)

    def _launch(self, before: Optional["_Launched"]) -> Optional["_Launched"]:
        """before: the step whose sampled tokens are still on the device only (then this step takes them
        from there)."""
        t_begin = time.perf_counter()
        plan, preempted = self.scheduler.schedule()
        for rid in preempted:
            self.requests[rid].preemptions += 1
        if not plan:
            if self.has_unfinished() and before is None:
                raise RuntimeError("scheduler: requests are waiting but none can run "
                                   "(a request larger than the cache should have been refused)")
            return None
        entries, sampled = [], []
        manager = self.runner.cache.manager
        for p in plan:
            req = self.requests[p.rid]
            if p.start == 0:
                # admitted (or admitted again after preemption): fixed-size states start at zero, and the
                # request's slot record gets its generator (seed, numbers drawn so far: a request that
                # comes back after preemption goes on where it was, so its samples do not change)
                self.runner.cache.reset_states(manager.slot(p.rid))
                manager.set_rng(p.rid, req.seed, req.n_sampled)
                if req.params.has_penalties:      # what the penalties read lies on the device, beside the sampler
                    self.sampler.remember(manager.slot(p.rid), req.tokens)
            wants = p.samples and req.n_sampled < req.max_new
            tokens = req.tokens[p.start:p.start + p.count] if before is None else [0]     # ([0]: stands in for the token on the device)
            entries.append(StepEntry(p.rid, tokens, [p.count - 1] if wants else []))
            if wants:
                sampled.append(req)
        try:
            if self.fail_next_step:
                self.fail_next_step = False
                raise RuntimeError("step failed (injected)")
            device_tokens = None
            if before is not None:
                place = {r.rid: i for i, r in enumerate(before.sampled)}
                order = [place[p.rid] for p in plan]
                device_tokens = before.pending.tokens
                if order != list(range(len(before.sampled))):
                    device_tokens = device_tokens[torch.tensor(order, dtype=torch.long, device=device_tokens.device)]
            # (the sampling below is this stream's next work: the logits need not outlive the next step)
            logits = self.runner.step(entries, device_tokens, borrow=True)
            self.scheduler.steps_done(np.asarray([p.rid for p in plan], dtype=np.int64),
                                      np.asarray([p.count for p in plan], dtype=np.int32))
            # each request's generator lives in its slot record: the seed and the count of numbers drawn
            rids = np.asarray([r.rid for r in sampled], dtype=np.int64)
            seeds, drawn = manager.rng_states(rids)
            # (a request's history holds its known tokens and, where this step runs ahead, the one sampled
            # in the step before, which only the device knows yet)
            ahead = 0 if before is None else 1
            places = ([(manager.slot(r.rid), len(r.tokens) + ahead) for r in sampled]
                      if any(r.params.has_penalties for r in sampled) else None)
            pending = self.sampler.launch(logits, [r.params for r in sampled], seeds.tolist(), drawn.tolist(), places)
            manager.note_drawn_step(rids)
            last = self.scheduler.tokens_sampled(rids).tolist()
        except Exception as exc:
            if before is not None:       # launched ahead: the step before is told first (see `step`)
                raise _AheadFailed(plan) from exc
            self._drop(plan)
            raise
        alive = []
        for r, is_last in zip(sampled, last):
            r.n_sampled += 1
            if is_last:
                # the token that is being sampled is the request's last: nothing of it runs after this step
                # (its pages go back now: whoever gets them writes after this step on the device)
                self.scheduler.finish(r.rid)
            else:
                alive.append(r)
        self.records.append(StepRecord(
            rows=sum(p.count for p in plan), decode_rows=sum(1 for p in plan if p.count == 1 and p.start > 0),
            prefill_rows=sum(p.count for p in plan if not (p.count == 1 and p.start > 0)),
            requests=len(plan), preempted=len(preempted), ran_ahead=before is not None,
            host_ms=(time.perf_counter() - t_begin) * 1e3))
        return _Launched(plan, sampled, dict(zip((r.rid for r in sampled), last)), alive, pending, self.records[-1])

    def _complete(self, launched: "_Launched") -> List[StepOutput]:
        t_begin = time.perf_counter()
        tokens = self.sampler.read(launched.pending)
        manager = self.runner.cache.manager
        # (a request that ended meanwhile, by an end-of-sequence token of the step before, ran here for nothing)
        told = [(r, int(t)) for r, t in zip(launched.sampled, tokens) if not r.finished]
        manager.note_tokens_step(np.asarray([r.rid for r, _ in told], dtype=np.int64),
                                 np.asarray([t for _, t in told], dtype=np.int32))
        by_rid = {r.rid: t for r, t in told}
        eos = set(self.spec.eos_token_ids)
        outputs = []
        for p in launched.plan:
            req = self.requests[p.rid]
            if req.finished:
                continue
            tok = by_rid.get(p.rid)
            if tok is not None:
                req.tokens.append(tok)
                # the end-of-sequence token counts as generated (crates/denno-engine/src/engine.rs:1125-1129)
                if tok in eos and not req.params.ignore_eos:
                    req.finish_reason = "eos"
                    self._release(p.rid)
                elif any(req.params.stop_sequences) and self._stops(req):
                    req.finish_reason = "stop_sequence"
                    self._release(p.rid)
                elif launched.last[p.rid]:
                    req.finish_reason = "length"
            elif p.samples and req.n_sampled >= req.max_new:
                req.finish_reason = "length"      # max_tokens = 0: the prompt is computed, nothing is sampled
                self._release(p.rid)
            if req.finish_reason is not None:
                req.finished = True
                if self.detokenize is not None and req.text is None:
                    out = req.generated
                    if out and out[-1] in eos and req.finish_reason == "eos":
                        out = out[:-1]               # the end-of-sequence token is no text
                    req.text = self._text_of(out)
            outputs.append(StepOutput(p.rid, tok, req.finished, req.finish_reason))
        launched.record.host_ms += (time.perf_counter() - t_begin) * 1e3
        return outputs

    def _text_of(self, tokens: List[int]) -> str:
        """The text of the tokens; tokens at the end that leave a character unfinished (the detokenizer
        puts U+FFFD there) wait for the tokens that finish it (engine.rs:1209-1218)."""
        n = len(tokens)
        text = self.detokenize(tokens[:n])
        while n > 0 and text.endswith("\ufffd"):
            n -= 1
            text = self.detokenize(tokens[:n])
        return text

    def _stops(self, req: Request) -> bool:
        """Whether one of the request's stop sequences has appeared in its generated text: the text is cut
        where the earliest of them begins (engine.rs:1241-1257)."""
        text = self._text_of(req.generated)
        found = [(text.find(s), s) for s in req.params.stop_sequences if s and s in text]
        if not found:
            return False
        at, seq = min(found, key=lambda f: f[0])
        req.text, req.stop_sequence = text[:at], seq
        return True

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
