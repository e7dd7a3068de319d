"""SamplingParams: the reference's generation parameters under their own names
(crates/denno-engine/src/engine.rs:40-77): max_tokens 256, temperature 1.0 when unset
(0 or less: greedy), top_k, top_p, stop_sequences, seed, and the four repetition controls."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple


# top-k / top-p work on the largest candidates only: the reference's own subset size for
# top-p (TOP_P_SUBSET, crates/denno-engine/src/sampler.rs:23)
TOP_CANDIDATES = 2048


@dataclass
class SamplingParams:
    max_tokens: int = 256
    temperature: Optional[float] = None      # None: 1.0 (sampler.rs:336); <= 0: greedy
    top_k: Optional[int] = None
    top_p: Optional[float] = None
    seed: Optional[int] = None               # None: the engine's default seed, else entropy
    repetition_penalty: Optional[float] = None     # None or 1.0: off
    frequency_penalty: Optional[float] = None      # None or 0: off
    presence_penalty: Optional[float] = None       # None or 0: off
    no_repeat_ngram_size: Optional[int] = None     # None or <= 1: off
    ignore_eos: bool = False                 # go on past an end-of-sequence token (benchmarks, random weights)
    # texts that end the generation where the first of them appears in the generated text, which is cut there
    # (engine.rs:44, 1241-1257); the engine needs a detokenizer for them
    stop_sequences: Tuple[str, ...] = ()

    def validate(self):
        if self.max_tokens < 0:
            raise ValueError("max_tokens must be >= 0")
        for name in ("frequency_penalty", "presence_penalty", "repetition_penalty", "temperature"):
            v = getattr(self, name)
            if v is not None and (v != v or v in (float("inf"), float("-inf"))):
                raise ValueError(f"{name} must be finite, got {v}")
        if self.repetition_penalty is not None and self.repetition_penalty <= 0:
            raise ValueError("repetition_penalty must be > 0")
        n = self.no_repeat_ngram_size
        if n is not None and not 2 <= n <= 1024:
            # the reference's bounds (crates/denno-cli/src/main.rs:665-668)
            raise ValueError(f"no_repeat_ngram_size must be between 2 and 1024, got {n}")
        if self.top_k is not None and not 1 <= self.top_k <= TOP_CANDIDATES:
            raise ValueError(f"top_k must be between 1 and {TOP_CANDIDATES}, got {self.top_k}")
        if self.top_p is not None and not 0.0 < self.top_p <= 1.0:
            raise ValueError("top_p must be in (0, 1]")
        if isinstance(self.stop_sequences, str) or not all(isinstance(x, str) for x in self.stop_sequences):
            raise ValueError("stop_sequences must be a list of strings")
        self.stop_sequences = tuple(self.stop_sequences)
        return self

    @property
    def effective_temperature(self) -> float:
        return 1.0 if self.temperature is None else float(self.temperature)

    @property
    def greedy(self) -> bool:
        return self.effective_temperature <= 0.0

    @property
    def has_penalties(self) -> bool:
        return ((self.repetition_penalty is not None and self.repetition_penalty != 1.0)
                or bool(self.frequency_penalty) or bool(self.presence_penalty)
                or (self.no_repeat_ngram_size is not None and self.no_repeat_ngram_size > 1))
