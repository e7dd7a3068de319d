"""One step's batch: which tokens of which requests run, where they stand, where their keys
and values go, and which rows' logits are wanted.

All index tables are built on the host as one int32 array and reach the device in one copy.
The reference's forward takes one request's tokens and its cache
(crates/denno-engine/src/model/mod.rs:58-59) and its batched form takes one decoded token per
session (:60-73); here a step takes any mix of both.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import numpy as np
import torch

TILE_ROWS = 16         # rows of one request that one workgroup of the plain attention kernel takes
WIDE_TILE_ROWS = 128   # the same for the MFMA attention kernel


@dataclass
class StepEntry:
    rid: int
    tokens: Sequence[int]          # the request's next tokens
    want: Sequence[int] = ()       # places among these tokens whose logits are wanted


@dataclass
class GroupStep:
    """What one cache group's mixers need for this step."""
    page_size: int
    window: int
    slot_map: Optional[torch.Tensor]       # int32 [T]: page * page_size + offset of each row's key
    block_tables: Optional[torch.Tensor]   # int32 [S, max_blocks], -1: page given back
    tiles: Optional[torch.Tensor]          # int32 [4, n_tiles]: request, first row, rows <= 16, first position
    tiles_wide: Optional[torch.Tensor] = None   # the same rows in tiles of up to 128
    single_rows: bool = False              # every request brings one row (a pure decode step)
    max_context: int = 0                   # the longest context after this step


@dataclass
class StepContext:
    T: int
    S: int
    R: int
    tokens: torch.Tensor           # int32 [T]
    positions: torch.Tensor        # int32 [T]
    logit_rows: torch.Tensor       # int32 [R]
    state_slots: torch.Tensor      # int32 [S]: each request's slot in the fixed-size state tensors
    row_start: torch.Tensor        # int32 [S + 1]: request s owns rows row_start[s] .. row_start[s+1]
    groups: List[Optional[GroupStep]]
    # the same on the host, for parts that loop over requests
    host_row_start: List[int] = field(default_factory=list)
    host_first_pos: List[int] = field(default_factory=list)
    host_slots: List[int] = field(default_factory=list)
    rids: List[int] = field(default_factory=list)


class BatchError(ValueError):
    pass


def plan_rows(entries: Sequence[StepEntry], starts: Sequence[int], vocab: int, max_positions: int):
    """Host arrays of the batch: tokens, positions, logit rows, row starts, tiles (narrow and wide)."""
    tokens, positions, logit_rows, row_start, tiles, wide = [], [], [], [0], [], []
    seen = set()
    rows = 0
    for s, (e, start) in enumerate(zip(entries, starts)):
        n = len(e.tokens)
        if n == 0:
            raise BatchError(f"request {e.rid}: an entry without tokens")
        if e.rid in seen:
            raise BatchError(f"request {e.rid} appears twice in one step")
        seen.add(e.rid)
        if start + n > max_positions:
            raise BatchError(f"request {e.rid}: {start} tokens in the cache + {n} exceed the model's "
                             f"{max_positions} positions")
        row0 = rows
        rows += n
        # (arrays, not loops over tokens: a prompt's portion is a thousand of them)
        ids = np.asarray(e.tokens, dtype=np.int64)
        bad = (ids < 0) | (ids >= vocab)
        if ids.ndim != 1 or bad.any():
            t = e.tokens[int(np.argmax(bad))] if ids.ndim == 1 else e.tokens
            raise BatchError(f"request {e.rid}: token id {t} is outside the vocabulary of {vocab}")
        tokens.append(ids)
        positions.append(np.arange(start, start + n, dtype=np.int64))
        for w in e.want:
            if not 0 <= w < n:
                raise BatchError(f"request {e.rid}: wanted place {w} is not among its {n} tokens")
            logit_rows.append(row0 + w)
        for i in range(0, n, TILE_ROWS):
            tiles.append((s, row0 + i, min(TILE_ROWS, n - i), start + i))
        for i in range(0, n, WIDE_TILE_ROWS):
            wide.append((s, row0 + i, min(WIDE_TILE_ROWS, n - i), start + i))
        row_start.append(row0 + n)
    # a tile's work grows with the keys before its last row: the kernel starts workgroups in this
    # order, the longest first (with the shortest last, the chip runs empty evenly)
    wide.sort(key=lambda t: -(t[3] + t[2]))
    none = np.empty(0, dtype=np.int64)
    return (np.concatenate(tokens) if tokens else none, np.concatenate(positions) if positions else none, logit_rows,
            row_start, tiles, wide)


def build_context(entries: Sequence[StepEntry], cache, vocab: int, max_positions: int, device) -> StepContext:
    """Reserves pages for the entries' tokens (raising cache.OutOfPages; pages taken for
    earlier entries stay with their requests) and builds the step's tables.  The cache manager is
    asked once per table for the whole step, not once per request."""
    mgr = cache.manager
    rids = np.asarray([e.rid for e in entries], dtype=np.int64)
    counts = np.asarray([len(e.tokens) for e in entries], dtype=np.int32)
    starts_a = mgr.lengths(rids)
    starts = starts_a.tolist()
    tokens, positions, logit_rows, row_start, tiles, wide = plan_rows(entries, starts, vocab, max_positions)
    slots_a = mgr.reserve_step(rids, starts_a + counts)
    T, S, R = len(tokens), len(entries), len(logit_rows)
    slots = slots_a.tolist()

    paged = [(g, layout, mgr.max_blocks(g, rids)) for g, layout in enumerate(cache.layouts) if layout.kind == 0]
    sizes = [("tokens", T), ("positions", T), ("logit_rows", R), ("state_slots", S), ("row_start", S + 1),
             ("tiles", 4 * len(tiles)), ("wide", 4 * len(wide))]
    for g, _, max_blocks in paged:
        sizes += [(f"bt{g}", S * max_blocks), (f"sm{g}", T)]
    offs, o = {}, 0
    for name, n in sizes:
        offs[name] = (o, n)
        o += n
    on_gpu = torch.device(device).type == "cuda"
    host = torch.empty(o, dtype=torch.int32, pin_memory=on_gpu)
    hv = host.numpy()

    def put(name, values):
        b, n = offs[name]
        hv[b:b + n] = values
    put("tokens", tokens), put("positions", positions), put("logit_rows", logit_rows)
    put("state_slots", slots_a), put("row_start", row_start)
    put("tiles", np.asarray(tiles, dtype=np.int32).T.reshape(-1))
    put("wide", np.asarray(wide, dtype=np.int32).T.reshape(-1))
    for g, layout, max_blocks in paged:
        (b0, n0), (b1, n1) = offs[f"bt{g}"], offs[f"sm{g}"]
        bad = mgr.step_tables(g, rids, starts_a, counts, hv[b0:b0 + n0].reshape(S, max_blocks), hv[b1:b1 + n1])
        if bad >= 0:
            raise BatchError(f"request {entries[bad].rid}: a token's page was given back already")
    dev = host.to(device, non_blocking=True) if on_gpu else host

    def view(name):
        b, n = offs[name]
        return dev[b:b + n]
    single = bool((counts == 1).all())
    max_context = int((starts_a + counts).max())
    tiles_dev = view("tiles").view(4, -1)
    wide_dev = view("wide").view(4, -1)
    groups = []
    max_blocks_of = {g: mb for g, _, mb in paged}
    for g, layout in enumerate(cache.layouts):
        if layout.kind != 0:
            groups.append(GroupStep(0, 0, None, None, None))
            continue
        groups.append(GroupStep(layout.page_size, layout.window, view(f"sm{g}"),
                                view(f"bt{g}").view(S, max_blocks_of[g]), tiles_dev, wide_dev, single, max_context))
    return StepContext(
        T=T, S=S, R=R, tokens=view("tokens"), positions=view("positions"), logit_rows=view("logit_rows"),
        state_slots=view("state_slots"), row_start=view("row_start"), groups=groups,
        host_row_start=row_start, host_first_pos=starts, host_slots=slots, rids=[e.rid for e in entries])
