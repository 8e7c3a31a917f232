"""How close the engine's logits must be to the plain implementation's.

float32: the reference's own arithmetic in another order, so rounding only: an absolute bound.
bfloat16: activations, cache and probabilities are rounded to 8 bits of mantissa at about ten
places a layer; the error is measured against the root mean square of the plain logits of the
row, and the bound for a model is about twice the worst that its tests have been seen to give
(the worst of every run is printed after the tests). A fault that moves a few per cent of one
probability mass to a wrong key (a page's edge, a window's edge, a stale slot) shifts logits by
more than that.
"""
import numpy as np

from .conftest import observe

F32_ABS = 1e-4
# bfloat16, two measures of a row of logits against the plain row, both relative to the plain
# row's root mean square, both about twice the worst that the tests have been seen to give:
#  - the rms of the error: 0.005 to 0.010 for every configuration, the 8B widths included; a
#    fault that shifts a row coherently shows here first;
#  - the largest error: the maximum of V noisy values grows with V (about sqrt(2 ln V) times the
#    rms: 0.017 to 0.033 for vocabularies of 256 to 512, 0.043 to 0.051 for 151936).
# ("random": the drawn configurations of test_random_configs_gpu, worst seen 0.011 and 0.036, and
#  0.015 and 0.057 over one-off sweeps of 380 draws; a further sweep of 800 draws had one row of one
#  draw beyond the bound, 0.0188 and 0.065 (one head of 128, a window of 5 on both layers, width 128:
#  little to average over), the same to the last bit whether its sequence ran whole and alone or
#  in the draw's schedule, so rounding and no fault of cache or batch; the bound stays;
#  "long": contexts of 9,000 to 17,000 tokens with scores scaled up so that a few far keys hold a
#  query's weight, which also carries the rounding of those scores into the output: worst seen
#  0.0146 and 0.050; "deep": 1 to 36 layers at a quarter of the 8B width, vocabulary 4096: 0.0084 and
#  0.037 for one layer, 0.0114 and 0.050 for 36: the error hardly grows with depth, and in float32
#  it goes from 9e-6 for one layer to 1.1e-5 for 36)
BF16_REL_L2 = {"A": 0.012, "B": 0.018, "C": 0.018, "D": 0.02, "F": 0.02, "wide": 0.02, "odd": 0.02, "random": 0.02, "long": 0.025, "deep": 0.02}
BF16_REL_RMS = {"A": 0.04, "B": 0.05, "C": 0.05, "D": 0.05, "F": 0.05, "wide": 0.08, "odd": 0.04, "random": 0.06, "long": 0.08, "deep": 0.08}


def rel_rms_error(got, ref):
    """(largest absolute error, the same over the row's rms, rms of the error over the row's rms)."""
    diff = got.astype(np.float64) - ref.astype(np.float64)
    err = float(np.abs(diff).max())
    rms = max(float(np.sqrt((ref.astype(np.float64) ** 2).mean())), 1e-30)
    return err, err / rms, float(np.sqrt((diff ** 2).mean())) / rms


def close(got, ref, dtype, config, label=None):
    """(ok, error): the error is absolute in float32 and relative to the row's rms in bfloat16."""
    err, rel, rel_l2 = rel_rms_error(got, ref)
    if dtype == "float32":
        observe(f"float32 {config} {label or ''} abs", err)
        return err <= F32_ABS, err
    observe(f"bfloat16 {config} {label or ''} max / rms", rel)
    observe(f"bfloat16 {config} {label or ''} rms / rms", rel_l2)
    return rel <= BF16_REL_RMS[config] and rel_l2 <= BF16_REL_L2[config], max(rel, rel_l2)
