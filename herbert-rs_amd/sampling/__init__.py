"""Sampling parameters, the GPU sampler, and stop reasons."""
from .params import SamplingParams
from .think import ThinkBudget, ThinkTokens
from .stopping import (EOS, INTERRUPTED, LENGTH, MAX_TOKENS, REPETITION_LOOP, STOP_SEQUENCE,
                       STOP_TOKEN, detect_repetition_loop)

__all__ = ["EOS", "INTERRUPTED", "LENGTH", "MAX_TOKENS", "REPETITION_LOOP", "STOP_SEQUENCE",
           "STOP_TOKEN", "SamplingParams", "ThinkBudget", "ThinkTokens", "detect_repetition_loop"]
