"""Decode steps replayed from captured HIP graphs.

A step in which every request brings one token launches some hundreds of small kernels; issued
one by one from Python they cost more than they run.  Such a step is captured once per
(batch bucket, context bucket) as a HIP graph (through torch.cuda.CUDAGraph) over fixed
buffers: the step's index tables are copied into the graph's input buffer, the graph is
replayed, the logits are read from its output buffer.  Requests beyond the real ones are
padding that every kernel skips or computes apart (rows never mix).

No memset is recorded into a graph: buffers are filled by kernels or by copies made before the
replay.
"""
from __future__ import annotations

import gc
import weakref
from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch

from ..kernels.ops import DECODE_SPLIT
from .batch import BatchError, GroupStep, StepContext, StepEntry

BUCKETS = (1, 2, 4, 8, 16, 32, 48, 64, 96, 128, 192, 256)


def batch_bucket(n: int, limit: int):
    for b in BUCKETS:
        if b >= n:
            return min(b, max(limit, n))
    return n


class DecodeGraph:
    def __init__(self, runner, batch: int, max_context: int):
        self.manager, self.B, self.max_context = runner.cache.manager, batch, max_context      # (no way back to the runner: no cycle)
        cache, dev = runner.cache, runner.device
        self.layouts = cache.layouts
        B = batch
        self.max_blocks = [(-(-runner.spec.max_positions // l.page_size) if l.kind == 0 else 0) for l in self.layouts]
        # layout of the int32 input buffer
        self.off, o = {}, 0
        def take(name, n):
            nonlocal o
            self.off[name] = (o, n)
            o += n
        for name, n in (("tokens", B), ("positions", B), ("logit_rows", B), ("state_slots", B),
                        ("row_start", B + 1), ("tiles", 4 * B)):
            take(name, n)
        for g, l in enumerate(self.layouts):
            if l.kind == 0:
                take(f"bt{g}", B * self.max_blocks[g])
                take(f"sm{g}", B)
        self.size = o
        self.host = [torch.empty(o, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self.copied = [None, None]
        self.turn = 0
        self.dev = torch.zeros(o, dtype=torch.int32, device=dev)
        v = self._view
        tiles = v("tiles").view(4, B)
        groups = []
        for g, l in enumerate(self.layouts):
            if l.kind != 0:
                groups.append(GroupStep(0, 0, None, None, None))
            else:
                groups.append(GroupStep(l.page_size, l.window, v(f"sm{g}"), v(f"bt{g}").view(B, self.max_blocks[g]),
                                        tiles, tiles, True, max_context))
        self.ctx = StepContext(T=B, S=B, R=B, tokens=v("tokens"), positions=v("positions"),
                               logit_rows=v("logit_rows"), state_slots=v("state_slots"), row_start=v("row_start"),
                               groups=groups, host_row_start=list(range(B + 1)), host_first_pos=[0] * B,
                               host_slots=[-1] * B, rids=[-1] * B)
        none = np.empty(0, dtype=np.int32)
        self._fill(self.host[0].numpy(), np.empty(0, dtype=np.int64), none, none, none)
        self.dev.copy_(self.host[0])
        # once outside the capture (libraries load, allocator warms up), then the capture
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            runner.model.forward(self.ctx, cache)
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize(dev)
        self.graph = torch.cuda.CUDAGraph()
        # The collector stays off while the stream records: a finalizer that gives device or pinned memory
        # back, or destroys another graph (whatever of an engine let go earlier sits in a cycle of references
        # waits for the collector, whenever its turn comes), is an error during a capture, raised inside a
        # destructor, which ends the process.  (It is not run first either: a full collection costs
        # milliseconds, and a serving run captures a graph per batch and context bucket as it goes.)
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(self.graph):
                self.logits = runner.model.forward(self.ctx, cache)
        finally:
            if collecting:
                gc.enable()

    def _view(self, name):
        b, n = self.off[name]
        return self.dev[b:b + n]

    def _fill(self, hv, rids, tokens, starts, slots):
        """The step's tables into a host buffer: rids int64 [n], tokens, starts, slots int32 [n]."""
        B, n = self.B, len(rids)
        mgr = self.manager

        def put(name, vals, fill):
            b, ln = self.off[name]
            hv[b:b + ln] = fill
            hv[b:b + n] = vals
        steps = np.arange(n + 1, dtype=np.int32)
        put("tokens", tokens, 0)
        put("positions", starts, 0)
        put("logit_rows", steps[:n], 0)
        put("state_slots", slots, -1)
        b, ln = self.off["row_start"]
        hv[b:b + ln] = n
        hv[b:b + n + 1] = steps
        b, ln = self.off["tiles"]
        t = hv[b:b + ln].reshape(4, B)
        t[0, :], t[1, :], t[2, :], t[3, :] = -1, 0, 1, 0
        t[0, :n], t[1, :n], t[3, :n] = steps[:n], steps[:n], starts
        ones = np.ones(n, dtype=np.int32)
        for g, l in enumerate(self.layouts):
            if l.kind != 0:
                continue
            (b0, n0), (b1, n1) = self.off[f"bt{g}"], self.off[f"sm{g}"]
            bad = mgr.step_tables(g, rids, starts, ones, hv[b0:b0 + n0].reshape(B, self.max_blocks[g]), hv[b1:b1 + n1])
            if bad >= 0:
                raise BatchError(f"request {int(rids[bad])}: a token's page was given back already")

    def run(self, rids, tokens, starts, slots, device_tokens=None) -> torch.Tensor:
        """device_tokens: the step's tokens as an int32 tensor on the device (a sampling that the host has
        not read yet), in place of `tokens`."""
        i = self.turn
        self.turn ^= 1
        if self.copied[i] is not None:
            self.copied[i].synchronize()      # the copy that last read this host buffer has ended
        self._fill(self.host[i].numpy(), rids, tokens, starts, slots)
        self.dev.copy_(self.host[i], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self.copied[i] = ev
        if device_tokens is not None:
            self._view("tokens")[:len(rids)].copy_(device_tokens)
        self.graph.replay()
        return self.logits


class DecodeGraphs:
    """The graphs of one runner, captured on demand."""

    def __init__(self, runner):
        self._runner = weakref.ref(runner)      # the runner owns these graphs; a reference back would be a cycle
        self.graphs: Dict[Tuple[int, int], DecodeGraph] = {}

    @property
    def runner(self):
        runner = self._runner()
        if runner is None:
            raise BatchError("the runner of these graphs is gone")
        return runner

    def takes(self, entries: Sequence[StepEntry]) -> bool:
        return self.runner.model.graph_safe and all(len(e.tokens) == 1 for e in entries)

    def step(self, entries: Sequence[StepEntry], device_tokens=None, borrow=False) -> torch.Tensor:
        """Runs a pure decode step; -> logits [R, vocab] at the wanted places: a copy, or with `borrow`, where every
        entry wants its logits, the graph's own buffer, which holds them until the same graph is replayed (enough
        for a caller that samples from them on this stream before its next step).
        device_tokens: int32 [entries] on the device: the entries' tokens, which the host does not know yet
        (the entries then hold any token of the vocabulary in their place)."""
        runner = self.runner
        mgr, spec = runner.cache.manager, runner.spec
        n = len(entries)
        rids = np.asarray([e.rid for e in entries], dtype=np.int64)
        tokens = np.asarray([e.tokens[0] for e in entries], dtype=np.int64)
        if device_tokens is not None and (device_tokens.dtype != torch.int32 or tuple(device_tokens.shape) != (n,)
                                          or device_tokens.device != runner.device):
            raise BatchError("device_tokens must be int32, one per entry, on the runner's device")
        starts = mgr.lengths(rids)
        if len(set(rids.tolist())) != n:
            raise BatchError("a request appears twice in one step")
        if int(starts.max()) + 1 > spec.max_positions:
            i = int(starts.argmax())
            raise BatchError(f"request {entries[i].rid}: {int(starts[i])} tokens in the cache + 1 exceed the model's "
                             f"{spec.max_positions} positions")
        if int(tokens.min()) < 0 or int(tokens.max()) >= spec.vocab:
            i = int(np.flatnonzero((tokens < 0) | (tokens >= spec.vocab))[0])
            raise BatchError(f"request {entries[i].rid}: token id {entries[i].tokens[0]} is outside the vocabulary of {spec.vocab}")
        rows = []
        for i, e in enumerate(entries):
            if len(e.want) > 0:
                if len(e.want) != 1 or e.want[0] != 0:
                    w = [w for w in e.want if w != 0]
                    raise BatchError(f"request {e.rid}: wanted place {w[0] if w else 0} is not among its 1 tokens")
                rows.append(i)
        new_lens = starts + 1
        slots = mgr.reserve_step(rids, new_lens)
        B = batch_bucket(n, runner.options.max_live)
        ctx_bucket = min(-(-int(new_lens.max()) // DECODE_SPLIT) * DECODE_SPLIT, -(-spec.max_positions // 16) * 16)
        key = (B, ctx_bucket)
        g = self.graphs.get(key)
        if g is None:
            g = self.graphs[key] = DecodeGraph(runner, B, ctx_bucket)
        logits = g.run(rids, tokens.astype(np.int32), starts, slots, device_tokens)
        if len(rows) == n:
            out = logits[:n] if borrow else logits[:n].clone()
        else:
            out = logits[torch.tensor(rows, dtype=torch.long, device=logits.device)] if rows else logits[:0].clone()
        mgr.commit_step(rids, new_lens)
        return out
