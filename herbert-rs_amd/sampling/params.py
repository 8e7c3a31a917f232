"""What a caller may ask of sampling and stopping.

Names, meanings and defaults follow the reference's command line
(crates/cli/src/main.rs:54-195): temperature 0.4 (0 = greedy), top_k 40
(0 = off), top_p 0.9 (1.0 = off), max_tokens 2048, ignore_eos, no_repeat_check,
think_budget 0 (no cap).
"""
from dataclasses import dataclass, field
from typing import Optional, Tuple

from ..errors import RequestError
from .think import ThinkTokens


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.4
    top_k: int = 40
    top_p: float = 0.9
    max_tokens: int = 2048
    stop_ids: Tuple[int, ...] = field(default=())   # further tokens that end a sequence
    ignore_eos: bool = False
    repeat_check: bool = True
    seed: Optional[int] = None                      # None: from the clock, as the reference does
    think_budget: int = 0                           # most tokens inside a think block, 0 = no cap
    think_tokens: Optional[ThinkTokens] = None      # the ids that cap needs (sampling.think.ThinkTokens)

    def validate(self):
        if self.temperature < 0:
            raise RequestError("temperature must be >= 0")
        if self.top_k < 0:
            raise RequestError("top_k must be >= 0")
        if not 0.0 < self.top_p:
            raise RequestError("top_p must be > 0")
        if self.max_tokens <= 0:
            raise RequestError("max_tokens must be > 0")
        if self.think_budget < 0:
            raise RequestError("think_budget must be >= 0")
        if self.think_budget > 0 and self.think_tokens is None:
            raise RequestError("think_budget needs think_tokens (the ids that open and close a think block "
                               "and of a line break)")

    @property
    def greedy(self):
        return self.temperature == 0.0
