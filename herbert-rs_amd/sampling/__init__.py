"""Sampling parameters, the GPU sampler, and stop reasons."""
from .params import SamplingParams
from .stopping import (EOS, LENGTH, MAX_TOKENS, REPETITION_LOOP, STOP_TOKEN,
                       detect_repetition_loop)

__all__ = ["EOS", "LENGTH", "MAX_TOKENS", "REPETITION_LOOP", "STOP_TOKEN", "SamplingParams",
           "detect_repetition_loop"]
