"""Sampler: from rows of logits to tokens, on the device.

Order, as the reference fixes it (crates/denno-engine/src/sampler.rs:164-179): repetition
penalty, frequency, presence, n-gram ban, then temperature, top-k, top-p, sample.  Rows of
one step are sampled together; each row has its own parameters and its own generator.
"""
from __future__ import annotations

from typing import List, Sequence

import torch

from ..kernels import ops
from .params import TOP_CANDIDATES, SamplingParams
from .rng import uniform


class Sampler:
    def __init__(self, device):
        self.device = device
        self._zeros = {}      # rows -> [2, rows] of zeros on the device: temperatures and uniforms of all-greedy steps

    def sample(self, logits, params, seeds, counters, contexts) -> List[int]:
        """launch and read at once."""
        return self.read(self.launch(logits, params, seeds, counters, contexts))

    def launch(self, logits: torch.Tensor, params: Sequence[SamplingParams], seeds: Sequence[int],
               counters: Sequence[int], contexts: Sequence[Sequence[int]]) -> "Pending":
        """Starts the sampling of a step's rows and does not wait for it.
        logits: [R, V] 32-bit (changed in place by penalties); row r belongs to a request
        with params[r], the seed seeds[r], counters[r] tokens sampled so far and the tokens
        contexts[r] (prompt + generated).  `read` gives the tokens; `Pending.tokens` holds them on the
        device as soon as the kernels have run, and is final if `Pending.final`."""
        R = logits.shape[0]
        if R == 0:
            return Pending(None, 0)
        dev = self.device
        if any(p.has_penalties for p in params):
            starts, flat = [0], []
            for p, c in zip(params, contexts):
                if p.has_penalties:
                    flat.extend(int(t) for t in c)
                starts.append(len(flat))
            f32 = lambda vals: torch.tensor(vals, dtype=torch.float32, device=dev)   # noqa: E731
            ops.penalties(
                logits, torch.tensor(flat or [0], dtype=torch.int32, device=dev),
                torch.tensor(starts, dtype=torch.int32, device=dev),
                f32([p.repetition_penalty if p.repetition_penalty is not None else 1.0 for p in params]),
                f32([p.frequency_penalty or 0.0 for p in params]),
                f32([p.presence_penalty or 0.0 for p in params]),
                torch.tensor([p.no_repeat_ngram_size or 0 for p in params], dtype=torch.int32, device=dev))
        # top_p = 1 without top_k restricts nothing: such a row takes the plain walk over the whole
        # vocabulary (the reference sorts it first, crates/denno-engine/src/sampler.rs:387-435, which
        # gives the same distribution)
        restricted = [r for r, p in enumerate(params)
                      if not p.greedy and (p.top_k is not None or (p.top_p is not None and p.top_p < 1.0))]
        n = len(restricted)
        both = torch.empty(R + n, dtype=torch.int32, device=dev)       # tokens, then which listed rows are undecided
        if all(p.greedy for p in params):
            # nothing to bring to the device: a step of greedy rows costs no copy
            tu = self._zeros.get(R)
            if tu is None:
                tu = self._zeros[R] = torch.zeros((2, R), dtype=torch.float32, device=dev)
        else:
            temps = [0.0 if p.greedy else p.effective_temperature for p in params]
            us = [0.0 if p.greedy else uniform(s, n_) for p, s, n_ in zip(params, seeds, counters)]
            tu = self._to_device([temps, us], torch.float32)      # one copy for both
        t_dev, u_dev = tu[0], tu[1]
        ops.sample(logits, t_dev, u_dev, both[:R])
        if restricted:
            top_p = [params[r].top_p if params[r].top_p is not None else 1.0 for r in restricted]
            ints = self._to_device([restricted, [params[r].top_k or 0 for r in restricted]], torch.int32)
            ps = self._to_device(top_p, torch.float32)
            ops.sample_top(logits, ints[0], t_dev, u_dev, ints[1], ps, both[:R], both[R:])
            if logits.shape[1] > TOP_CANDIDATES and any(params[r].top_k is None for r in restricted):
                # top-p alone whose cut lies beyond the 2,048 largest: the whole vocabulary, sorted.  Launched
                # behind the kernel that says which rows these are, and which it does not touch the others of:
                # the host need not read the flags first, so the step's tokens are final once the kernels
                # have run and the next step can be launched ahead
                ops.sample_full(logits, ints[0], t_dev, u_dev, ps, both[:R], only=both[R:])
        return Pending(both, R, *self._bring_home(both))

    def _to_device(self, values, dtype):
        """A small table for the sampling kernels.  Through pinned memory and without waiting: a copy from
        ordinary host memory holds the host until the stream has run dry, and with it the step that the engine
        launches ahead."""
        host = torch.tensor(values, dtype=dtype)
        if self.device.type != "cuda":
            return host.to(self.device)
        pinned = torch.empty(host.shape, dtype=dtype, pin_memory=True)
        pinned.copy_(host)
        return pinned.to(self.device, non_blocking=True)

    @staticmethod
    def _bring_home(both):
        """The copy of a step's tokens to the host is asked for here, behind the sampling kernels, and not when
        they are read: a copy asked for at the read would queue behind whatever was launched meanwhile (the
        whole next step, where the engine runs ahead), and the read would wait for all of that.  -> (the
        pinned host tensor, the event that says it is filled)."""
        if both.device.type != "cuda":
            return both, None
        host = torch.empty(both.shape, dtype=both.dtype, pin_memory=True)
        host.copy_(both, non_blocking=True)
        filled = torch.cuda.Event()
        filled.record()
        return host, filled

    def read(self, pending: "Pending") -> List[int]:
        """Waits for a launched sampling; -> the rows' tokens."""
        if pending.rows == 0:
            return []
        if pending.filled is not None:
            pending.filled.synchronize()
        return pending.host.tolist()[:pending.rows]


class Pending:
    """A launched sampling: `both[:rows]` are the tokens on the device, final as soon as the kernels have run."""

    def __init__(self, both, rows, host=None, filled=None):
        self.both, self.rows = both, rows
        self.host, self.filled = host, filled      # both on the host, and the event that says so (None: no wait)

    @property
    def tokens(self):
        return self.both[:self.rows]

    @property
    def final(self):
        return True
