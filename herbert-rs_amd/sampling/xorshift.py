"""The reference's generator on the host: xorshift64 with shifts 13, 7, 17
(crates/core/src/sampler.rs:50-62); seed 0 becomes 0xdeadbeef (:30-34). The
GPU sampler steps the same recurrence; this copy seeds it and serves host code."""
import time

MASK64 = (1 << 64) - 1


def initial_state(seed):
    seed = int(seed) & MASK64
    return 0xDEADBEEF if seed == 0 else seed


def clock_seed():
    return time.time_ns() & MASK64


def step(state):
    x = state
    x ^= (x << 13) & MASK64
    x ^= x >> 7
    x ^= (x << 17) & MASK64
    return x


def to_unit(state):
    """The draw in [0, 1) that a state gives: its upper 24 bits over 2^24."""
    return (state >> 40) / float(1 << 24)


def sequence_seed(seed, index):
    """Seed of the index-th sequence of a call: every sequence has a stream of its own.
    The first sequence gets the seed itself, so one prompt behaves as the reference's one sampler."""
    if index == 0:
        return initial_state(seed)
    mixed = (int(seed) + index * 0x9E3779B97F4A7C15) & MASK64
    return step(initial_state(mixed))
