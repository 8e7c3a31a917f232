"""bin/trace_run against the plain implementation: the same requests whole, with the last 32
tokens one by one, and in batches of unequal lengths (slots used again), in float32 and bfloat16."""
import numpy as np
import pytest

from . import replay_util as ru
from .plain_cache import plain_logits
from .tiny import CONFIGS, make_folder, random_tokens

pytestmark = pytest.mark.gpu

# float32: the reference's own arithmetic, so rounding only. bfloat16: activations, cache and
# probabilities are rounded to 8 bits of mantissa (unit roundoff 2^-9) at about ten places a
# layer; the bound is on the error relative to the logits' root mean square.
F32_ABS = 1e-4
BF16_REL_RMS = 0.05

LENGTHS = {"A": [5, 11, 2, 70, 33, 127], "B": [1, 17, 33, 9, 140, 65], "C": [3, 200, 64, 129, 40, 75]}


def requests_for(name):
    vocab = CONFIGS[name][0]["vocab_size"]
    return {f"r{i}": random_tokens(vocab, n, 100 + 7 * i) for i, n in enumerate(LENGTHS[name])}


def check(name, folder, dtype, steps, tmp_path, label):
    vocab = CONFIGS[name][0]["vocab_size"]
    reqs = requests_for(name)
    out = ru.run_trace(folder, dtype, steps, str(tmp_path / label), ru.needed_tokens(steps), vocab)
    got = ru.collect(steps, out)
    assert len(got) == sum(len(t) for t in reqs.values())
    worst = 0.0
    for (rid, pos), row in got.items():
        ref = plain_logits(folder, reqs[rid])[pos]
        err = float(np.abs(row - ref).max())
        if dtype == "float32":
            assert err <= F32_ABS, f"{label}: request {rid} position {pos}: max abs err {err}"
        else:
            rms = float(np.sqrt((ref.astype(np.float64) ** 2).mean()))
            assert err <= BF16_REL_RMS * rms, \
                f"{label}: request {rid} position {pos}: err {err} vs rms {rms}"
        worst = max(worst, err)
    return worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_tail_and_batches(name, dtype, model_root, tmp_path):
    folder = make_folder(model_root, name, dtype)
    reqs = requests_for(name)
    check(name, folder, dtype, ru.trace_whole(reqs), tmp_path, "whole")
    check(name, folder, dtype, ru.trace_tail(reqs, 32), tmp_path, "tail")
    check(name, folder, dtype, ru.trace_batches(reqs, 4, 0.5), tmp_path, "batches")
