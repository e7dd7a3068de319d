"""Trace replay: given token ids go through the model step by step; nothing is sampled.

A trace is a list of steps; a step is {"step": n, "entries": [{"id", "tokens", "want"}],
"end": [ids]}.  The replayer maps ids to requests of the runner's own cache (a request starts
when its id is first seen and gives its pages back when a step's `end` names it) and runs each
step through ModelRunner.step, the step function that generation uses.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .batch import StepEntry
from .runner import ModelRunner


class TraceReplayer:
    def __init__(self, runner: ModelRunner):
        self.runner = runner
        self._rid: Dict[str, int] = {}
        self._next = 0

    def run_step(self, record: dict) -> Optional[torch.Tensor]:
        """-> logits [wanted, vocab] on the device, or None if the step wants none."""
        entries, started = [], []
        try:
            for e in record.get("entries", []):
                name = str(e["id"])
                if not e["tokens"]:
                    # an entry that brings no tokens is a request left out of this step
                    if e.get("want"):
                        raise ValueError(f"step {record.get('step')}: request {name} wants logits of tokens it does not bring")
                    continue
                if name not in self._rid:
                    self.runner.start_request(self._next)
                    self._rid[name] = self._next
                    self._next += 1
                    started.append(name)
                entries.append(StepEntry(self._rid[name], e["tokens"], e.get("want", [])))
            logits = self.runner.step(entries)
        except Exception:
            # a step that cannot run leaves nothing of the requests it would have started
            for name in started:
                self.runner.end_request(self._rid.pop(name))
            raise
        for name in record.get("end", []):
            rid = self._rid.pop(str(name), None)
            if rid is not None:
                self.runner.end_request(rid)
        return logits if logits.shape[0] > 0 else None

    def live(self):
        return sorted(self._rid)
