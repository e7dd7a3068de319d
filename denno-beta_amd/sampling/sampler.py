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
    """slots, positions: the histories that the penalties read lie on the device, a row of `positions` tokens per
    slot (a request's slot in the cache manager).  A request with penalties is written there when it is admitted
    (`remember`), and every token sampled for it is added behind on the device, so that a step needs nothing of
    the tokens from the host, not even those of the step before."""

    def __init__(self, device, slots: int = 0, positions: int = 0):
        self.device = torch.device(device)
        self._zeros = {}      # rows -> [2, rows] of zeros on the device: temperatures and uniforms of all-greedy steps
        self.history = None
        if slots > 0 and positions > 0:
            if slots * positions >= 2 ** 31:      # the kernels address the table with 32-bit offsets
                raise ValueError(f"sampler: {slots} histories of {positions} tokens are more than the kernels address")
            self.history = torch.zeros((slots, positions), dtype=torch.int32, device=self.device)

    def remember(self, slot: int, tokens: Sequence[int]):
        """The tokens of the request in `slot` so far (prompt + generated), from the start."""
        n = len(tokens)
        if self.history is None or not (0 <= slot < self.history.shape[0]) or n > self.history.shape[1]:
            raise ValueError(f"sampler: no room for {n} tokens in slot {slot}")
        if n:
            self.history[slot, :n].copy_(self._to_device(list(tokens), torch.int32))

    def sample(self, logits, params, seeds, counters, contexts) -> List[int]:
        """launch and read at once, the rows' contexts (prompt + generated) given as lists: for a sampler that
        serves no engine, since the contexts are written over the histories of slots 0, 1, ..."""
        places = None
        if any(p.has_penalties for p in params):
            rows, width = len(contexts), max(len(c) for c in contexts) + 1
            if self.history is None or self.history.shape[0] < rows or self.history.shape[1] < width:
                # (every call writes its contexts anew, so a larger table need not keep the old one's rows)
                rows = max(rows, 0 if self.history is None else self.history.shape[0])
                width = max(width, 0 if self.history is None else self.history.shape[1])
                if rows * width >= 2 ** 31:
                    raise ValueError(f"sampler: {rows} histories of {width} tokens are more than the kernels address")
                self.history = torch.zeros((rows, width), dtype=torch.int32, device=self.device)
            places = []
            for r, (p, c) in enumerate(zip(params, contexts)):
                if p.has_penalties:
                    self.remember(r, c)
                places.append((r, len(c)))
        return self.read(self.launch(logits, params, seeds, counters, places))

    def launch(self, logits: torch.Tensor, params: Sequence[SamplingParams], seeds: Sequence[int],
               counters: Sequence[int], places: Sequence = None) -> "Pending":
        """Starts the sampling of a step's rows and does not wait for it.
        logits: [R, V] 32-bit (changed in place by penalties); row r belongs to a request
        with params[r], the seed seeds[r] and counters[r] tokens sampled so far; places[r] = (slot, n): its
        history's slot and how many tokens it holds (needed for rows with penalties only).  `read` gives the
        tokens; `Pending.tokens` holds them on the device as soon as the kernels have run."""
        R = logits.shape[0]
        if R == 0:
            return Pending(None, 0)
        dev = self.device
        punished = [r for r, p in enumerate(params) if p.has_penalties]
        if punished:
            if places is None or self.history is None:
                raise ValueError("sampler: rows with penalties need their histories' places")
            width = self.history.shape[1]
            for r in punished:
                slot, n = places[r]
                if not (0 <= slot < self.history.shape[0] and 0 <= n < width):
                    raise ValueError(f"sampler: a history of {n} tokens in slot {slot} does not fit")
            begin = [places[r][0] * width if p.has_penalties else 0 for r, p in enumerate(params)]
            length = [places[r][1] if p.has_penalties else 0 for r, p in enumerate(params)]
            where = self._to_device([begin, length, [p.no_repeat_ngram_size or 0 for p in params]], torch.int32)
            f = self._to_device([[p.repetition_penalty if p.repetition_penalty is not None else 1.0 for p in params],
                                 [p.frequency_penalty or 0.0 for p in params],
                                 [p.presence_penalty or 0.0 for p in params]], torch.float32)
            ops.penalties(logits, self.history.view(-1), where[0], where[1], f[0], f[1], f[2], where[2],
                          bounds=max(b + n for b, n in zip(begin, length)))
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
            # (the first kernel takes the restricted rows as greedy ones, which costs it a third of the walk:
            # the kernel after it decides their tokens)
            later = set(restricted)
            first = [[0.0 if r in later else t for r, t in enumerate(temps)]] if restricted else []
            tu = self._to_device([temps, us] + first, torch.float32)      # one copy for all
        t_dev, u_dev = tu[0], tu[1]
        ops.sample(logits, tu[2] if restricted else t_dev, u_dev, both[:R])
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
        if punished:
            # each sampled token behind its request's history, for the next step's penalties
            t = self._to_device([[begin[r] for r in punished], [length[r] for r in punished], punished], torch.int32)
            ops.history_append(self.history.view(-1), t[0], t[1], t[2], both,
                               bounds=(max(begin[r] + length[r] for r in punished), max(punished)))
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
