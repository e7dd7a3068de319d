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
        self.runner, self.B, self.max_context = runner, batch, max_context
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
        self._fill(self.host[0].numpy(), [], [], [])
        self.dev.copy_(self.host[0])
        # once outside the capture (libraries load, allocator warms up), then the capture
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            runner.model.forward(self.ctx, cache)
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize(dev)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits = runner.model.forward(self.ctx, cache)

    def _view(self, name):
        b, n = self.off[name]
        return self.dev[b:b + n]

    def _fill(self, hv, entries, starts, slots):
        B, n = self.B, len(entries)
        mgr = self.runner.cache.manager

        def put(name, vals, fill):
            b, ln = self.off[name]
            hv[b:b + ln] = fill
            hv[b:b + len(vals)] = vals
        put("tokens", [int(e.tokens[0]) for e in entries], 0)
        put("positions", starts, 0)
        put("logit_rows", list(range(n)), 0)
        put("state_slots", slots, -1)
        put("row_start", list(range(n + 1)), n)
        b, ln = self.off["tiles"]
        t = hv[b:b + ln].reshape(4, B)
        t[0, :], t[1, :], t[2, :], t[3, :] = -1, 0, 1, 0
        t[0, :n], t[1, :n], t[3, :n] = np.arange(n), np.arange(n), starts
        for g, l in enumerate(self.layouts):
            if l.kind != 0:
                continue
            b, ln = self.off[f"bt{g}"]
            bt = hv[b:b + ln].reshape(B, self.max_blocks[g])
            bt[:] = -1
            b, ln = self.off[f"sm{g}"]
            sm = hv[b:b + ln]
            sm[:] = -1
            for s, (e, start) in enumerate(zip(entries, starts)):
                tab = mgr.block_table(e.rid, g)
                bt[s, :len(tab)] = tab
                page = tab[start // l.page_size]
                if page < 0:
                    raise BatchError(f"request {e.rid}: a token's page was given back already")
                sm[s] = page * l.page_size + start % l.page_size

    def run(self, entries: Sequence[StepEntry], starts: List[int], slots: List[int]) -> torch.Tensor:
        i = self.turn
        self.turn ^= 1
        if self.copied[i] is not None:
            self.copied[i].synchronize()      # the copy that last read this host buffer has ended
        self._fill(self.host[i].numpy(), entries, starts, slots)
        self.dev.copy_(self.host[i], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self.copied[i] = ev
        self.graph.replay()
        return self.logits


class DecodeGraphs:
    """The graphs of one runner, captured on demand."""

    def __init__(self, runner):
        self.runner = runner
        self.graphs: Dict[Tuple[int, int], DecodeGraph] = {}

    def takes(self, entries: Sequence[StepEntry]) -> bool:
        return self.runner.model.graph_safe and all(len(e.tokens) == 1 for e in entries)

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Runs a pure decode step; -> logits [R, vocab] at the wanted places (a copy)."""
        runner = self.runner
        mgr, spec = runner.cache.manager, runner.spec
        starts = [mgr.length(e.rid) for e in entries]
        seen = set()
        for e, start in zip(entries, starts):
            if e.rid in seen:
                raise BatchError(f"request {e.rid} appears twice in one step")
            seen.add(e.rid)
            if start + 1 > spec.max_positions:
                raise BatchError(f"request {e.rid}: {start} tokens in the cache + 1 exceed the model's "
                                 f"{spec.max_positions} positions")
            if not 0 <= int(e.tokens[0]) < spec.vocab:
                raise BatchError(f"request {e.rid}: token id {e.tokens[0]} is outside the vocabulary of {spec.vocab}")
            for w in e.want:
                if w != 0:
                    raise BatchError(f"request {e.rid}: wanted place {w} is not among its 1 tokens")
        for e, start in zip(entries, starts):
            mgr.reserve(e.rid, start + 1)
        slots = [mgr.slot(e.rid) for e in entries]
        n = len(entries)
        B = batch_bucket(n, runner.options.max_live)
        ctx_bucket = min(-(-(max(starts) + 1) // DECODE_SPLIT) * DECODE_SPLIT, -(-spec.max_positions // 16) * 16)
        key = (B, ctx_bucket)
        g = self.graphs.get(key)
        if g is None:
            g = self.graphs[key] = DecodeGraph(runner, B, ctx_bucket)
        logits = g.run(entries, starts, slots)
        rows = [i for i, e in enumerate(entries) if len(e.want) > 0]
        if len(rows) == n:
            out = logits[:n].clone()
        else:
            out = logits[torch.tensor(rows, dtype=torch.long, device=logits.device)] if rows else logits[:0].clone()
        for e, start in zip(entries, starts):
            mgr.commit(e.rid, start + 1)
        return out
