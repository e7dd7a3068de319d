"""CacheManager: the Python face of the host core's page and slot bookkeeping
(csrc/host/cache_manager.h).  It owns no device memory."""
from __future__ import annotations

import ctypes
from ctypes import c_int, c_int64, c_void_p, POINTER
from dataclasses import dataclass
from typing import List, Sequence

import numpy as np

from ..build import load_library

PAGED, STATE = 0, 1

OK, NO_SLOT, DUPLICATE, UNKNOWN, OUT_OF_PAGES, BAD_ARGUMENT, CORRUPT = 0, -1, -2, -3, -4, -5, -6
_NAMES = {NO_SLOT: "no free request slot", DUPLICATE: "request id is live already",
          UNKNOWN: "no live request has this id", OUT_OF_PAGES: "out of pages",
          BAD_ARGUMENT: "bad argument", CORRUPT: "bookkeeping is corrupt"}


class CacheError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        super().__init__(f"{what}: {_NAMES.get(code, code)}")


class OutOfPages(CacheError):
    pass


@dataclass(frozen=True)
class SlotState:
    """A live request's record of fixed size (csrc/host/cache_manager.h): zero when its slot is given out."""
    num_computed: int     # tokens in the cache = the next token's position
    last_token: int       # the token sampled last, -1 before the first
    rng_seed: int
    rng_drawn: int        # numbers drawn from the request's generator so far


@dataclass(frozen=True)
class GroupLayout:
    kind: int            # PAGED or STATE
    n_pages: int = 0
    page_size: int = 1
    window: int = 0      # 0: all keys are kept


_host = None


def host_library():
    global _host
    if _host is None:
        lib = load_library("host")
        I, L, P = c_int, c_int64, c_void_p
        IP = POINTER(c_int)
        sig = {
            "dn_cache_create": (P, [I, IP, IP, IP, IP, I]), "dn_cache_destroy": (None, [P]),
            "dn_cache_add": (I, [P, L]), "dn_cache_release": (I, [P, L]), "dn_cache_reserve": (I, [P, L, I]),
            "dn_cache_commit": (I, [P, L, I]), "dn_cache_length": (I, [P, L]), "dn_cache_slot": (I, [P, L]),
            "dn_cache_state": (I, [P, L, c_void_p]), "dn_cache_set_rng": (I, [P, L, ctypes.c_uint64, ctypes.c_uint64]),
            "dn_cache_note_sampled": (I, [P, L, I]),
            "dn_cache_note_drawn_step": (None, [P, c_void_p, I]),
            "dn_cache_note_tokens_step": (None, [P, c_void_p, c_void_p, I]),
            "dn_sched_steps_done": (I, [P, c_void_p, c_void_p, I, IP]),
            "dn_sched_tokens_sampled": (I, [P, c_void_p, I, c_void_p, IP]),
            "dn_cache_rng_states": (I, [P, c_void_p, I, c_void_p, c_void_p, IP]),
            "dn_cache_generation": (L, [P, I]), "dn_cache_block_table": (I, [P, L, I, c_void_p, I]),
            "dn_cache_blocks": (I, [P, L, I]), "dn_cache_free_pages": (I, [P, I]),
            "dn_cache_pages_held": (I, [P, L, I]), "dn_cache_pages_needed": (I, [P, L, I, I, I]),
            "dn_cache_pages_peak": (I, [P, I, I, I]), "dn_cache_live": (I, [P]), "dn_cache_check": (I, [P]),
            "dn_cache_reuse_count": (L, [P, I]),
            "dn_cache_lengths": (I, [P, c_void_p, I, c_void_p, IP]),
            "dn_cache_reserve_step": (I, [P, c_void_p, c_void_p, I, c_void_p, IP]),
            "dn_cache_commit_step": (I, [P, c_void_p, c_void_p, I, IP]),
            "dn_cache_max_blocks": (I, [P, I, c_void_p, I]),
            "dn_cache_step_tables": (I, [P, I, c_void_p, c_void_p, c_void_p, I, I, I, c_void_p, c_void_p, I, IP]),
            "dn_sched_create": (P, [P, I, I, I, I, I]), "dn_sched_destroy": (None, [P]),
            "dn_sched_add": (I, [P, L, I, I]),
            "dn_sched_schedule": (I, [P, c_void_p, c_void_p, c_void_p, c_void_p, I, c_void_p, IP, I]),
            "dn_sched_step_done": (I, [P, L, I]), "dn_sched_token_sampled": (I, [P, L]),
            "dn_sched_finish": (I, [P, L]), "dn_sched_n_waiting": (I, [P]), "dn_sched_n_running": (I, [P]),
            "dn_sched_known": (I, [P, L]), "dn_sched_computed": (I, [P, L]), "dn_sched_generated": (I, [P, L]),
        }
        for name, (res, args) in sig.items():
            f = getattr(lib, name)
            f.restype, f.argtypes = res, args
        _host = lib
    return _host


class CacheManager:
    def __init__(self, groups: Sequence[GroupLayout], max_requests: int):
        self.groups = list(groups)
        self.max_requests = max_requests
        self._lib = host_library()
        n = len(self.groups)
        arr = lambda vals: (c_int * max(n, 1))(*vals)   # noqa: E731
        self._h = self._lib.dn_cache_create(
            n, arr([g.kind for g in self.groups]), arr([g.n_pages for g in self.groups]),
            arr([g.page_size for g in self.groups]), arr([g.window for g in self.groups]), max_requests)
        if not self._h:
            raise ValueError(f"cache manager: bad layout {self.groups} for {max_requests} requests")

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.dn_cache_destroy(self._h)
            self._h = None

    def _chk(self, rc, what):
        if rc < 0:
            raise (OutOfPages if rc == OUT_OF_PAGES else CacheError)(rc, what)
        return rc

    def add(self, rid: int) -> int:
        """-> the request's slot (index into per-request state tensors)."""
        return self._chk(self._lib.dn_cache_add(self._h, rid), f"add request {rid}")

    def release(self, rid: int) -> bool:
        """Gives back the request's pages and slot.  A stale release (unknown id) changes nothing
        and returns False, as a release with an old lease does in the reference
        (crates/denno-engine/src/engine.rs:751-754)."""
        rc = self._lib.dn_cache_release(self._h, rid)
        if rc == UNKNOWN:
            return False
        self._chk(rc, f"release request {rid}")
        return True

    def reserve(self, rid: int, new_len: int):
        """Pages for positions up to new_len in every paged group; raises OutOfPages and
        changes nothing if any pool is short."""
        self._chk(self._lib.dn_cache_reserve(self._h, rid, new_len), f"reserve {new_len} tokens for request {rid}")

    def try_reserve(self, rid: int, new_len: int) -> bool:
        rc = self._lib.dn_cache_reserve(self._h, rid, new_len)
        if rc == OUT_OF_PAGES:
            return False
        self._chk(rc, f"reserve {new_len} tokens for request {rid}")
        return True

    def commit(self, rid: int, new_len: int):
        self._chk(self._lib.dn_cache_commit(self._h, rid, new_len), f"commit {new_len} tokens of request {rid}")

    def length(self, rid: int) -> int:
        return self._chk(self._lib.dn_cache_length(self._h, rid), f"length of request {rid}")

    def has(self, rid: int) -> bool:
        return self._lib.dn_cache_length(self._h, rid) >= 0

    def slot(self, rid: int) -> int:
        return self._chk(self._lib.dn_cache_slot(self._h, rid), f"slot of request {rid}")

    # -- the request's slot record: position, generator, last token --------------------------
    def state(self, rid: int) -> "SlotState":
        out = np.empty(6, dtype=np.int64)
        self._chk(self._lib.dn_cache_state(self._h, rid, out.ctypes.data), f"state of request {rid}")
        v = out.tolist()
        return SlotState(v[0], v[1], v[2] | (v[3] << 32), v[4] | (v[5] << 32))

    def set_rng(self, rid: int, seed: int, drawn: int = 0):
        """The request's generator: its seed and how many numbers it has given (a request that comes
        back after preemption brings its count)."""
        self._chk(self._lib.dn_cache_set_rng(self._h, rid, seed & (2 ** 64 - 1), drawn), f"generator of request {rid}")

    def note_sampled(self, rid: int, token: int):
        """One number was drawn from the request's generator and gave `token`."""
        self._chk(self._lib.dn_cache_note_sampled(self._h, rid, token), f"sampled token of request {rid}")

    def note_drawn_step(self, rids: np.ndarray):
        """A number was drawn from the generator of each of these requests (ids that are no longer live are skipped)."""
        self._lib.dn_cache_note_drawn_step(self._h, rids.ctypes.data, len(rids))

    def note_tokens_step(self, rids: np.ndarray, tokens: np.ndarray):
        """The tokens that those draws gave (int32), once they are known."""
        self._lib.dn_cache_note_tokens_step(self._h, rids.ctypes.data, tokens.ctypes.data, len(rids))

    def rng_states(self, rids: np.ndarray):
        """-> (seeds, numbers drawn so far) of the requests, uint64 arrays."""
        seeds, drawn = np.empty(len(rids), dtype=np.uint64), np.empty(len(rids), dtype=np.uint64)
        failed = c_int(0)
        self._chk_step(self._lib.dn_cache_rng_states(self._h, rids.ctypes.data, len(rids), seeds.ctypes.data,
                                                     drawn.ctypes.data, failed), failed, rids, "generator")
        return seeds, drawn

    def generation(self, slot: int) -> int:
        return self._lib.dn_cache_generation(self._h, slot)

    def block_table(self, rid: int, group: int) -> np.ndarray:
        n = self._chk(self._lib.dn_cache_blocks(self._h, rid, group), f"block table of request {rid}")
        out = np.empty(max(n, 1), dtype=np.int32)
        self._chk(self._lib.dn_cache_block_table(self._h, rid, group, out.ctypes.data, n), "block table")
        return out[:n]

    # -- a whole step in one call each ----------------------------------------------------
    # rids: int64 array; lengths and counts: int32 arrays (numpy, contiguous)
    def _chk_step(self, rc, failed, rids, what):
        if rc < 0:
            raise (OutOfPages if rc == OUT_OF_PAGES else CacheError)(rc, f"{what} (request {int(rids[failed.value])})")

    def lengths(self, rids: np.ndarray) -> np.ndarray:
        out = np.empty(len(rids), dtype=np.int32)
        failed = c_int(0)
        self._chk_step(self._lib.dn_cache_lengths(self._h, rids.ctypes.data, len(rids), out.ctypes.data, failed),
                       failed, rids, "length")
        return out

    def reserve_step(self, rids: np.ndarray, new_lens: np.ndarray) -> np.ndarray:
        """Pages for every entry's tokens, entry after entry (entries before one that fails keep
        theirs); -> the requests' slots."""
        slots = np.empty(len(rids), dtype=np.int32)
        failed = c_int(0)
        self._chk_step(self._lib.dn_cache_reserve_step(self._h, rids.ctypes.data, new_lens.ctypes.data, len(rids),
                                                       slots.ctypes.data, failed), failed, rids, "reserve")
        return slots

    def commit_step(self, rids: np.ndarray, new_lens: np.ndarray):
        failed = c_int(0)
        self._chk_step(self._lib.dn_cache_commit_step(self._h, rids.ctypes.data, new_lens.ctypes.data, len(rids),
                                                      failed), failed, rids, "commit")

    def max_blocks(self, group: int, rids: np.ndarray) -> int:
        return self._chk(self._lib.dn_cache_max_blocks(self._h, group, rids.ctypes.data, len(rids)), "block tables")

    def step_tables(self, group: int, rids, starts, counts, block_tables: np.ndarray, slot_map: np.ndarray):
        """Fills block_tables [rows >= entries, max_blocks] and slot_map [>= tokens] (int32, contiguous,
        written in place: views of a pinned buffer will do) for the step's entries; -1 wherever
        there is nothing.  Returns the entry's index if one of its tokens has no page (given back,
        or never reserved), else -1."""
        failed = c_int(0)
        rc = self._lib.dn_cache_step_tables(self._h, group, rids.ctypes.data, starts.ctypes.data, counts.ctypes.data,
                                            len(rids), block_tables.shape[0], block_tables.shape[1],
                                            block_tables.ctypes.data, slot_map.ctypes.data, slot_map.shape[0], failed)
        if rc == BAD_ARGUMENT:
            return failed.value
        self._chk_step(rc, failed, rids, "step tables")
        return -1

    def free_pages(self, group: int) -> int:
        return self._chk(self._lib.dn_cache_free_pages(self._h, group), "free pages")

    def pages_held(self, rid: int, group: int) -> int:
        return self._chk(self._lib.dn_cache_pages_held(self._h, rid, group), "pages held")

    def pages_peak(self, group: int, total_len: int, chunk: int) -> int:
        return self._lib.dn_cache_pages_peak(self._h, group, total_len, chunk)

    def live(self) -> int:
        return self._lib.dn_cache_live(self._h)

    def reuse_count(self, group: int) -> int:
        """Pages handed out that some request had held before."""
        return self._lib.dn_cache_reuse_count(self._h, group)

    def check(self):
        """Raises if a page or slot is lost, held twice, or both free and held."""
        self._chk(self._lib.dn_cache_check(self._h), "cache check")
