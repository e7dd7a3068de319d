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


# -- steps that hold portions of prompts ---------------------------------------------------------------
# Issued kernel by kernel, a step costs the host some 12 us a launch, seven launches a layer: at 48 layers more than
# 4 ms, which a step of a few hundred rows does not keep the GPU busy for.  Such a step is captured too, over
# buffers of a bucket's size: T rows, S requests, R wanted rows, and as many attention tiles as T rows of S
# requests can make.  Rows, requests and tiles beyond the real ones are padding: a padding row has token 0,
# position 0 and slot -1 (its keys and values go nowhere), belongs to no tile (attention leaves it alone) and is
# wanted by nobody; rows never mix, so whatever a padding row holds stays in it.  A bucket is captured when a step
# falls into it for the second time: a shape that comes once runs kernel by kernel.
PORTION_ROWS = (16, 32, 48, 64, 96, 128, 192, 256, 384, 512)
PORTION_REQUESTS = (1, 2, 4, 8, 16, 32, 64, 128, 256, 512)
PORTION_GRAPHS_MAX = 48      # captured buckets per runner; steps of further shapes run kernel by kernel


def _bucket(n, sizes):
    for b in sizes:
        if b >= n:
            return b
    return None


class PortionGraph:
    def __init__(self, runner, T: int, S: int, R: int):
        from .batch import TILE_ROWS, WIDE_TILE_ROWS
        self.manager, self.T, self.S, self.R = runner.cache.manager, T, S, R
        cache, dev = runner.cache, runner.device
        self.layouts = cache.layouts
        self.vocab, self.max_positions = runner.spec.vocab, runner.spec.max_positions
        self.max_blocks = [(-(-runner.spec.max_positions // l.page_size) if l.kind == 0 else 0) for l in self.layouts]
        # (a request of n rows makes at most n / 16 + 1 tiles)
        self.n_tiles, self.n_wide = T // TILE_ROWS + S, T // WIDE_TILE_ROWS + S
        self.off, o = {}, 0
        for name, n in (("tokens", T), ("positions", T), ("logit_rows", R), ("state_slots", S), ("row_start", S + 1),
                        ("tiles", 4 * self.n_tiles), ("wide", 4 * self.n_wide)):
            self.off[name] = (o, n)
            o += n
        for g, l in enumerate(self.layouts):
            if l.kind == 0:
                self.off[f"bt{g}"] = (o, S * self.max_blocks[g])
                o += S * self.max_blocks[g]
                self.off[f"sm{g}"] = (o, T)
                o += T
        self.host = [torch.empty(o, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self.copied = [None, None]
        self.turn = 0
        self.dev = torch.zeros(o, dtype=torch.int32, device=dev)
        v = self._view
        tiles, wide = v("tiles").view(4, self.n_tiles), v("wide").view(4, self.n_wide)
        groups = []
        for g, l in enumerate(self.layouts):
            if l.kind != 0:
                groups.append(GroupStep(0, 0, None, None, None))
            else:
                groups.append(GroupStep(l.page_size, l.window, v(f"sm{g}"), v(f"bt{g}").view(S, self.max_blocks[g]),
                                        tiles, wide, False, 0))
        self.ctx = StepContext(T=T, S=S, R=R, tokens=v("tokens"), positions=v("positions"),
                               logit_rows=v("logit_rows"), state_slots=v("state_slots"), row_start=v("row_start"),
                               groups=groups, host_row_start=[0] * (S + 1), host_first_pos=[0] * S,
                               host_slots=[-1] * S, rids=[-1] * S)
        self._fill(self.host[0].numpy(), [], np.empty(0, np.int64), np.empty(0, np.int32), np.empty(0, np.int32),
                   np.empty(0, np.int32))
        self.dev.copy_(self.host[0])
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            runner.model.forward(self.ctx, cache)
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize(dev)
        self.graph = torch.cuda.CUDAGraph()
        collecting = gc.isenabled()       # (see DecodeGraph: no collection while the stream records)
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

    def _fill(self, hv, entries, rids, starts, counts, slots):
        """The step's tables into a host buffer; -> the number of wanted rows."""
        from .batch import plan_rows
        n = len(entries)
        tokens, positions, logit_rows, row_start, tiles, wide = plan_rows(entries, starts.tolist(), self.vocab,
                                                                          self.max_positions)
        rows = len(tokens)

        def put(name, vals, fill):
            b, ln = self.off[name]
            hv[b:b + ln] = fill
            hv[b:b + len(vals)] = vals
        put("tokens", tokens, 0), put("positions", positions, 0), put("logit_rows", logit_rows, 0)
        put("state_slots", slots, -1), put("row_start", row_start, rows)
        for name, table, width in (("tiles", tiles, self.n_tiles), ("wide", wide, self.n_wide)):
            b, ln = self.off[name]
            t = hv[b:b + ln].reshape(4, width)
            t[0, :], t[1, :], t[2, :], t[3, :] = -1, 0, 1, 0
            if table:
                t[:, :len(table)] = np.asarray(table, dtype=np.int32).T
        for g, l in enumerate(self.layouts):
            if l.kind != 0:
                continue
            (b0, n0), (b1, n1) = self.off[f"bt{g}"], self.off[f"sm{g}"]
            hv[b0:b0 + n0] = -1
            hv[b1:b1 + n1] = -1
            if n:
                bad = self.manager.step_tables(g, rids, starts, counts,
                                               hv[b0:b0 + n * self.max_blocks[g]].reshape(n, self.max_blocks[g]),
                                               hv[b1:b1 + rows])
                if bad >= 0:
                    raise BatchError(f"request {int(rids[bad])}: a token's page was given back already")
        return len(logit_rows)

    def run(self, entries, rids, starts, counts, slots):
        i = self.turn
        self.turn ^= 1
        if self.copied[i] is not None:
            self.copied[i].synchronize()      # the copy that last read this host buffer has ended
        wanted = self._fill(self.host[i].numpy(), entries, rids, starts, counts, slots)
        self.dev.copy_(self.host[i], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self.copied[i] = ev
        self.graph.replay()
        return self.logits, wanted


class DecodeGraphs:
    """The graphs of one runner, captured on demand."""

    def __init__(self, runner):
        self._runner = weakref.ref(runner)      # the runner owns these graphs; a reference back would be a cycle
        self.graphs: Dict[Tuple[int, int], DecodeGraph] = {}
        self.portions: Dict[Tuple[int, int, int], PortionGraph] = {}
        self.seen: Dict[Tuple[int, int, int], int] = {}      # bucket -> steps that fell into it so far

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
        # (contexts in buckets of 256, but no bucket beyond what a block table holds: whole pages up to the model's positions)
        held = min(-(-spec.max_positions // l.page_size) * l.page_size for l in runner.cache.layouts if l.kind == 0)
        ctx_bucket = min(-(-int(new_lens.max()) // DECODE_SPLIT) * DECODE_SPLIT, held)
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

    # -- steps that hold portions ---------------------------------------------------------------------
    def portion_bucket(self, entries: Sequence[StepEntry]):
        """(T, S, R) of the bucket that a step with portions falls into, or None if none takes it."""
        runner = self.runner
        if not runner.model.graph_safe or not runner.options.graph_portions:
            return None
        rows, wanted = sum(len(e.tokens) for e in entries), sum(len(e.want) for e in entries)
        T, S = _bucket(rows, PORTION_ROWS), _bucket(len(entries), PORTION_REQUESTS)
        if T is None or S is None or rows < 1:
            return None
        return (T, S, S if wanted <= S else T)

    def takes_portions(self, entries: Sequence[StepEntry]) -> bool:
        """Whether this step is replayed from a captured graph: its bucket has been met before (and is captured
        now if it was not), and there is room for another graph."""
        key = self.portion_bucket(entries)
        if key is None:
            return False
        self.seen[key] = self.seen.get(key, 0) + 1
        if key in self.portions:
            return True
        return self.seen[key] >= 2 and len(self.portions) < PORTION_GRAPHS_MAX

    def step_portions(self, entries: Sequence[StepEntry], borrow=False) -> torch.Tensor:
        """Runs a step of any mix from its bucket's graph; -> logits [R, vocab] at the wanted places (with `borrow`
        a view of the graph's own buffer, which holds them until the same graph is replayed)."""
        runner = self.runner
        mgr = runner.cache.manager
        key = self.portion_bucket(entries)
        rids = np.asarray([e.rid for e in entries], dtype=np.int64)
        counts = np.asarray([len(e.tokens) for e in entries], dtype=np.int32)
        starts = mgr.lengths(rids)
        # (what is wrong with the entries is found before pages are taken: plan_rows raises on them)
        from .batch import plan_rows
        plan_rows(entries, starts.tolist(), runner.spec.vocab, runner.spec.max_positions)
        slots = mgr.reserve_step(rids, starts + counts)
        g = self.portions.get(key)
        if g is None:
            g = self.portions[key] = PortionGraph(runner, *key)
        logits, wanted = g.run(entries, rids, starts, counts, slots)
        out = logits[:wanted] if borrow else logits[:wanted].clone()
        mgr.commit_step(rids, starts + counts)
        return out
