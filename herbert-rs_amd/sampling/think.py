"""A cap on the tokens of a think block, as the reference's sampler has it
(crates/core/src/sampler.rs:154-232): between the token that opens a block and the one that
closes it the generated tokens are counted; where the count reaches the budget less one, a line
break is forced, from the budget on the closing token, by leaving only that token's logit finite
before the choice is made (sampler.rs:219-243). A budget of 0 caps nothing. The command line's
--nothink is a budget of 1 (crates/cli/src/main.rs:685-687): a block that the model opens is
closed at once."""
from dataclasses import dataclass
from typing import Optional


@dataclass(frozen=True)
class ThinkTokens:
    """The ids of the tokens that open and close a think block and of a line break
    (crates/cli/src/main.rs:671-684 looks them up in the tokenizer)."""
    open_id: int
    close_id: int
    newline_id: int


class ThinkBudget:
    """The state of one sequence."""

    def __init__(self, max_tokens, tokens):
        self.max_tokens = int(max_tokens)
        self.tokens = tokens
        self.in_think = False
        self.count = 0

    @property
    def active(self):
        return self.max_tokens > 0

    def set_in_think(self):
        """The block was opened by the prompt, not by a generated token (sampler.rs:181-186)."""
        self.in_think, self.count = True, 0

    def reset(self):
        """A new turn begins outside any block (sampler.rs:194-198)."""
        self.in_think, self.count = False, 0

    def track(self, token):
        """After every chosen token (sampler.rs:200-212)."""
        if token == self.tokens.open_id:
            self.in_think, self.count = True, 0
        elif token == self.tokens.close_id:
            self.in_think, self.count = False, 0
        elif self.in_think:
            self.count += 1

    def forced(self) -> Optional[int]:
        """The only token that may be chosen next, or None (sampler.rs:219-231)."""
        if not self.in_think or self.max_tokens == 0:
            return None
        if self.count + 1 == self.max_tokens:
            return self.tokens.newline_id
        if self.count + 1 > self.max_tokens:
            return self.tokens.close_id
        return None
