"""bin/trace_run against the plain implementation: the same requests whole, with the last 32
tokens one by one, and in batches of unequal lengths (slots used again), in float32 and bfloat16."""
import numpy as np
import pytest

from . import replay_util as ru
from .bounds import close
from .plain_cache import plain_logits
from .tiny import CONFIGS, make_folder, random_tokens

pytestmark = pytest.mark.gpu

# D has heads of 128: in bfloat16 its decoding runs the kernel that norms, rotates, writes the
# cache and attends in one, and its requests of more than a thousand tokens cross many pages
LENGTHS = {"A": [5, 11, 2, 70, 33, 127], "B": [1, 17, 33, 9, 140, 65], "C": [3, 200, 64, 129, 40, 75],
           "D": [3, 260, 64, 129, 1100, 77]}


def requests_for(name):
    vocab = CONFIGS[name][0]["vocab_size"]
    return {f"r{i}": random_tokens(vocab, n, 100 + 7 * i) for i, n in enumerate(LENGTHS[name])}


def check(name, folder, dtype, steps, tmp_path, label):
    vocab = CONFIGS[name][0]["vocab_size"]
    reqs = requests_for(name)
    out = ru.run_trace(folder, dtype, steps, str(tmp_path / label), ru.needed_tokens(steps), vocab)
    got = ru.collect(steps, out)
    assert len(got) == sum(len(t) for t in reqs.values())
    for (rid, pos), row in got.items():
        ref = plain_logits(folder, reqs[rid])[pos]
        ok, err = close(row, ref, dtype, name, label)
        assert ok, f"{label}: request {rid} position {pos}: error {err}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_whole_tail_and_batches(name, dtype, model_root, tmp_path):
    folder = make_folder(model_root, name, dtype)
    reqs = requests_for(name)
    check(name, folder, dtype, ru.trace_whole(reqs), tmp_path, "whole")
    check(name, folder, dtype, ru.trace_tail(reqs, 32), tmp_path, "tail")
    check(name, folder, dtype, ru.trace_batches(reqs, 4, 0.5), tmp_path, "batches")
