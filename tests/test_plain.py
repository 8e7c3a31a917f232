"""The plain implementation pinned by what fixes it beside the reference's text: vectors the
reference's own tests hold, special cases that reduce to a library routine, and invariants.
Each check is chosen so that a plausible mistake fails it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from .plain import model as pm
from .plain import ops
from .plain import sampler as ps


def rand(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


# ---- embedding
def test_embedding_rows_and_range():
    table = rand(7, 5)
    out = ops.embedding([0, 6, 3], table)
    assert torch.equal(out, F.embedding(torch.tensor([0, 6, 3]), table))
    with pytest.raises(ValueError):
        ops.embedding([7], table)


# ---- RMSNorm: eps inside the root and added to the mean, plain weight
def test_rms_norm_matches_library_and_eps_placement():
    x = rand(4, 24, seed=1)
    w = 1 + 0.1 * rand(24, seed=2)
    for eps in (1e-6, 1e-5):
        assert torch.allclose(ops.rms_norm(x, w, eps), F.rms_norm(x, (24,), w, eps), atol=1e-6)
    # with w = 1 the output's rms is sqrt(ms / (ms + eps)): eps outside the root, or times dim, fails
    small = rand(1, 16, seed=3) * 1e-3
    ms = float((small ** 2).mean())
    for eps in (1e-6, 1e-5):
        y = ops.rms_norm(small, torch.ones(16), eps)
        assert math.isclose(float(torch.sqrt((y ** 2).mean())), math.sqrt(ms / (ms + eps)), rel_tol=1e-4)
    assert not torch.allclose(ops.rms_norm(small, torch.ones(16), 1e-6),
                              ops.rms_norm(small, torch.ones(16), 1e-5), rtol=1e-2)
    assert torch.equal(ops.rms_norm(torch.zeros(1, 8), w[:8], 1e-6), torch.zeros(1, 8))
    # a "1 + w" norm would double the output for w = 1
    assert torch.allclose(ops.rms_norm(x, torch.ones(24), 1e-6), x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-6))


def test_linear_layout():
    x = rand(3, 6, seed=4)
    w = rand(10, 6, seed=5)          # [out, in], not square: a transposed read fails on shape
    assert torch.allclose(ops.linear(x, w), F.linear(x, w), atol=1e-6)


def test_head_norm_is_per_head():
    x = rand(5, 3, 8, seed=6)
    w = 1 + 0.1 * rand(8, seed=7)
    got = ops.head_rms_norm(x, w, 1e-6)
    assert torch.allclose(got, F.rms_norm(x, (8,), w, 1e-6), atol=1e-6)
    whole = F.rms_norm(x.reshape(5, 24), (24,), w.repeat(3), 1e-6).reshape(5, 3, 8)
    assert not torch.allclose(got, whole, atol=1e-3)


# ---- rotation
def test_rope_identity_norm_and_relative():
    hd = 16
    q = rand(6, 2, hd, seed=8)
    k = rand(6, 2, hd, seed=9)
    pos = list(range(6))
    rq = ops.apply_rope(q, pos, 10000.0)
    assert torch.allclose(rq[0], q[0])                                    # position 0 is the identity
    half = hd // 2
    pair_norm = lambda t: t[..., :half] ** 2 + t[..., half:] ** 2         # pairs are (j, j + hd/2)
    assert torch.allclose(pair_norm(rq), pair_norm(q), atol=1e-5)
    # scores depend on distances only: shifting all positions changes nothing
    rk = ops.apply_rope(k, pos, 10000.0)
    rq2 = ops.apply_rope(q, [p + 37 for p in pos], 10000.0)
    rk2 = ops.apply_rope(k, [p + 37 for p in pos], 10000.0)
    s1 = torch.einsum("ihd,jhd->hij", rq, rk)
    s2 = torch.einsum("ihd,jhd->hij", rq2, rk2)
    assert torch.allclose(s1, s2, atol=1e-4)


def test_rope_is_complex_multiplication_half_split():
    hd, theta = 8, 1e6
    x = rand(4, 1, hd, seed=10)
    pos = [0, 3, 17, 100]
    half = hd // 2
    inv = torch.tensor([1.0 / theta ** (2 * i / hd) for i in range(half)], dtype=torch.float64)
    z = torch.complex(x[..., :half].double(), x[..., half:].double())
    ang = torch.tensor(pos, dtype=torch.float64)[:, None] * inv[None, :]
    rot = z * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    want = torch.cat([rot.real, rot.imag], -1).float()
    got = ops.apply_rope(x, pos, theta)
    assert torch.allclose(got, want, atol=1e-5)
    # the interleaved pairing (2j, 2j+1) is a different function
    zi = torch.complex(x[..., 0::2].double(), x[..., 1::2].double()) * \
        torch.polar(torch.ones_like(ang), ang)[:, None, :]
    inter = torch.stack([zi.real, zi.imag], -1).reshape(4, 1, hd).float()
    assert not torch.allclose(got, inter, atol=1e-3)
    # theta matters
    assert not torch.allclose(got, ops.apply_rope(x, pos, 1e4), atol=1e-3)


def test_rope_inverse_frequencies():
    inv = ops.rope_inv_freq(8, 10000.0)
    assert torch.allclose(inv, torch.tensor([1.0, 0.1, 0.01, 0.001]), rtol=1e-5)


# ---- attention
@pytest.mark.parametrize("nq,nkv", [(4, 2), (6, 2), (3, 3), (5, 1)])
def test_attention_matches_library(nq, nkv):
    T, hd = 9, 8
    q, k, v = rand(T, nq, hd, seed=11), rand(T, nkv, hd, seed=12), rand(T, nkv, hd, seed=13)
    got = ops.causal_attention(q, k, v, list(range(T)))
    kk = k.repeat_interleave(nq // nkv, dim=1)       # consecutive query heads share a kv head
    vv = v.repeat_interleave(nq // nkv, dim=1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1),
                                          is_causal=True, scale=hd ** -0.5).transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-5)


def test_large_inputs_take_the_library_s_product_and_say_the_same(monkeypatch):
    """Beyond ops.WHOLE_FROM multiply-adds the product and the attention scores go through
    torch's matrix product on the CPU: the same sums as the loops that define them, a window and
    positions that do not start at zero included."""
    x, w = rand(7, 24, seed=31), rand(40, 24, seed=32)
    T, nq, nkv, hd = 37, 6, 2, 8
    q, k, v = rand(T, nq, hd, seed=33), rand(T, nkv, hd, seed=34), rand(T, nkv, hd, seed=35)
    positions = list(range(5, 5 + T))
    slow = (ops.linear(x, w), ops.causal_attention(q, k, v, positions),
            ops.causal_attention(q, k, v, positions, window=9))
    monkeypatch.setattr(ops, "WHOLE_FROM", 0)
    fast = (ops.linear(x, w), ops.causal_attention(q, k, v, positions),
            ops.causal_attention(q, k, v, positions, window=9))
    for a, b in zip(slow, fast):
        assert torch.allclose(a, b, atol=2e-6) and not torch.equal(a, torch.zeros_like(a))
    assert not torch.allclose(fast[1], fast[2], atol=1e-3)          # the window is not lost on the way


def test_attention_special_cases():
    hd = 4
    v = rand(5, 1, hd, seed=14)
    # one token: the output is its value
    one = ops.causal_attention(rand(1, 2, hd), rand(1, 1, hd), v[:1], [0])
    assert torch.allclose(one[0, 0], v[0, 0]) and torch.allclose(one[0, 1], v[0, 0])
    # equal scores: the mean of the visible values
    q = torch.zeros(5, 1, hd)
    out = ops.causal_attention(q, rand(5, 1, hd, seed=15), v, list(range(5)))
    for i in range(5):
        assert torch.allclose(out[i, 0], v[:i + 1, 0].mean(0), atol=1e-6)


def test_attention_window_counts_the_query_itself():
    T, hd = 8, 4
    q, k, v = rand(T, 1, hd, seed=16), rand(T, 1, hd, seed=17), rand(T, 1, hd, seed=18)
    out = ops.causal_attention(q, k, v, list(range(T)), window=3)
    # query 5 sees keys 3, 4, 5 only
    s = (k[3:6, 0] @ q[5, 0]) * hd ** -0.5
    want = (torch.softmax(s, 0)[:, None] * v[3:6, 0]).sum(0)
    assert torch.allclose(out[5, 0], want, atol=1e-6)
    full = ops.causal_attention(q, k, v, list(range(T)))
    assert torch.allclose(out[:3], full[:3], atol=1e-6) and not torch.allclose(out[5], full[5], atol=1e-4)


def test_silu_and_swiglu():
    g = torch.tensor([0.0, -100.0, 3.0, -1.5])
    assert torch.allclose(ops.silu(g), F.silu(g), atol=1e-6)
    assert ops.silu(torch.tensor([0.0]))[0] == 0 and torch.isfinite(ops.silu(g)).all()
    x, wg, wu, wd = rand(3, 6, seed=19), rand(10, 6, seed=20), rand(10, 6, seed=21), rand(6, 10, seed=22)
    want = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
    assert torch.allclose(ops.swiglu_mlp(x, wg, wu, wd), want, atol=1e-5)


def test_softmax_vectors_of_the_reference():
    # crates/backends/backend_common/src/speculative.rs:304-321
    p = ops.softmax(torch.tensor([1.0, 2.0, 3.0, 4.0]))
    assert abs(float(p.sum()) - 1.0) < 1e-6
    assert torch.allclose(ops.softmax(torch.zeros(4)), torch.full((4,), 0.25))


# ---- whole model
def tiny_weights(cfg, seed=0):
    H, nq, nkv, hd = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    I, V = cfg["intermediate_size"], cfg["vocab_size"]
    w = {"model.embed_tokens.weight": rand(V, H, seed=seed, scale=0.1),
         "model.norm.weight": 1 + 0.1 * rand(H, seed=seed + 1)}
    if not cfg.get("tie_word_embeddings", True):
        w["lm_head.weight"] = rand(V, H, seed=seed + 2, scale=0.1)
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        s = seed + 10 * (l + 1)
        w[p + "input_layernorm.weight"] = 1 + 0.1 * rand(H, seed=s)
        w[p + "post_attention_layernorm.weight"] = 1 + 0.1 * rand(H, seed=s + 1)
        w[p + "self_attn.q_proj.weight"] = rand(nq * hd, H, seed=s + 2, scale=0.1)
        w[p + "self_attn.k_proj.weight"] = rand(nkv * hd, H, seed=s + 3, scale=0.1)
        w[p + "self_attn.v_proj.weight"] = rand(nkv * hd, H, seed=s + 4, scale=0.1)
        w[p + "self_attn.o_proj.weight"] = rand(H, nq * hd, seed=s + 5, scale=0.1)
        w[p + "self_attn.q_norm.weight"] = 1 + 0.1 * rand(hd, seed=s + 6)
        w[p + "self_attn.k_norm.weight"] = 1 + 0.1 * rand(hd, seed=s + 7)
        w[p + "mlp.gate_proj.weight"] = rand(I, H, seed=s + 8, scale=0.1)
        w[p + "mlp.up_proj.weight"] = rand(I, H, seed=s + 9, scale=0.1)
        w[p + "mlp.down_proj.weight"] = rand(H, I, seed=s + 10, scale=0.1)
    return w


CFG = dict(num_hidden_layers=2, hidden_size=24, num_attention_heads=3, num_key_value_heads=1, head_dim=16,
           intermediate_size=40, vocab_size=50, rope_theta=1e4, rms_norm_eps=1e-6,
           tie_word_embeddings=False, max_position_embeddings=64)


def library_forward(cfg, w, tokens):
    """The same model from torch's own routines, vectorised: an independent second opinion."""
    nq, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps, T = cfg["rms_norm_eps"], len(tokens)
    x = F.embedding(torch.tensor(tokens), w["model.embed_tokens.weight"])
    half = hd // 2
    inv = 1.0 / cfg["rope_theta"] ** (torch.arange(half, dtype=torch.float32) * 2 / hd)
    ang = torch.arange(T, dtype=torch.float32)[:, None] * inv
    cos, sin = torch.cos(ang)[:, None], torch.sin(ang)[:, None]

    def rope(t):
        a, b = t[..., :half], t[..., half:]
        return torch.cat([a * cos - b * sin, a * sin + b * cos], -1)
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        y = F.rms_norm(x, (x.shape[-1],), w[p + "input_layernorm.weight"], eps)
        q = F.linear(y, w[p + "self_attn.q_proj.weight"]).view(T, nq, hd)
        k = F.linear(y, w[p + "self_attn.k_proj.weight"]).view(T, nkv, hd)
        v = F.linear(y, w[p + "self_attn.v_proj.weight"]).view(T, nkv, hd)
        q = rope(F.rms_norm(q, (hd,), w[p + "self_attn.q_norm.weight"], eps))
        k = rope(F.rms_norm(k, (hd,), w[p + "self_attn.k_norm.weight"], eps))
        k = k.repeat_interleave(nq // nkv, 1)
        v = v.repeat_interleave(nq // nkv, 1)
        a = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1),
                                           is_causal=True).transpose(0, 1).reshape(T, nq * hd)
        x = x + F.linear(a, w[p + "self_attn.o_proj.weight"])
        y = F.rms_norm(x, (x.shape[-1],), w[p + "post_attention_layernorm.weight"], eps)
        x = x + F.linear(F.silu(F.linear(y, w[p + "mlp.gate_proj.weight"])) *
                         F.linear(y, w[p + "mlp.up_proj.weight"]), w[p + "mlp.down_proj.weight"])
    x = F.rms_norm(x, (x.shape[-1],), w["model.norm.weight"], eps)
    head = w["lm_head.weight"] if not cfg.get("tie_word_embeddings", True) else w["model.embed_tokens.weight"]
    return F.linear(x, head)


def test_model_against_library_formulation():
    w = tiny_weights(CFG)
    tokens = [3, 14, 15, 9, 26, 5, 35]
    assert torch.allclose(pm.forward(CFG, w, tokens), library_forward(CFG, w, tokens), atol=2e-5)


def test_tied_head_and_separate_head():
    tied = dict(CFG, tie_word_embeddings=True)
    w = tiny_weights(tied)
    logits = pm.forward(tied, w, [1, 2, 3])
    w2 = dict(w, **{"lm_head.weight": rand(50, 24, seed=99)})
    assert torch.equal(pm.forward(tied, w2, [1, 2, 3]), logits)        # ignored when tied
    sep = tiny_weights(CFG)
    a = pm.forward(CFG, sep, [1, 2, 3])
    sep["lm_head.weight"] = sep["lm_head.weight"] * 2
    assert torch.allclose(pm.forward(CFG, sep, [1, 2, 3]), 2 * a, atol=1e-5)


def test_logits_at_chosen_rows_only():
    w = tiny_weights(CFG)
    tokens = [3, 9, 27, 1, 43, 5]
    whole = pm.forward(CFG, w, tokens)
    some = pm.forward(CFG, w, tokens, rows=[0, 4, 5])
    assert torch.equal(some, whole[[0, 4, 5]])


def test_causality_of_the_whole_model():
    w = tiny_weights(CFG)
    a = pm.forward(CFG, w, [4, 8, 15, 16, 23])
    b = pm.forward(CFG, w, [4, 8, 15, 42, 7])
    assert torch.allclose(a[:3], b[:3], atol=1e-6) and not torch.allclose(a[3], b[3], atol=1e-4)


def test_too_long_sequence_is_refused():
    w = tiny_weights(CFG)
    with pytest.raises(ValueError):
        pm.forward(dict(CFG, max_position_embeddings=4), w, [1, 2, 3, 4, 5])


# ---- sampler and helpers
def test_xorshift_vector_by_hand():
    x = 1
    x ^= (x << 13) & ps.MASK64
    x ^= x >> 7
    x ^= (x << 17) & ps.MASK64
    rng = ps.XorShift64(1)
    assert rng.next_u64() == x == 1082269761
    assert ps.XorShift64(0).state == 0xDEADBEEF
    r = ps.XorShift64(7).next_f32()
    assert 0.0 <= r < 1.0
    # The draw (crates/core/src/sampler.rs:58-62): the upper 24 bits of the new state over 2^24,
    # cut and not rounded. By hand, from the state 2^63 + 2^36 + 2^33:
    #   x ^= x << 13  (2^76 is lost)           -> 2^63 + 2^49 + 2^46 + 2^36 + 2^33
    #   x ^= x >> 7                            -> ... + 2^56 + 2^42 + 2^39 + 2^29 + 2^26
    #   x ^= x << 17  (2^80, 2^73, 2^66 lost; 2^63, 2^56, 2^46 meet their like and cancel)
    #      = 2^59 + 2^53 + 2^50 + 2^49 + 2^43 + 2^42 + 2^39 + 2^36 + 2^33 + 2^29 + 2^26
    #   x >> 40 = 2^19 + 2^13 + 2^10 + 2^9 + 2^3 + 2^2 = 534028
    # Bits 39 and 36 lie below the cut: a draw that kept 32 bits and let the conversion to
    # float32 round would give 534029 / 2^24.
    rng = ps.XorShift64((1 << 63) + (1 << 36) + (1 << 33))
    r = rng.next_f32()
    assert rng.state == 0x08260C9224000000
    assert r.dtype == np.float32 and float(r) == 534028.0 / 16777216.0
    assert float(r) != float(np.float32(rng.state >> 32) / np.float32(2.0 ** 32))
    # the engine's host copy of the generator, which seeds the GPU sampler, says the same
    from herbert_rs_amd.sampling import xorshift
    state = xorshift.step((1 << 63) + (1 << 36) + (1 << 33))
    assert state == 0x08260C9224000000 and xorshift.to_unit(state) == 534028.0 / 16777216.0


def test_sampler_reductions_to_argmax():
    logits = np.array([0.1, 2.5, -1.0, 2.5, 0.3], dtype=np.float32)
    assert ps.argmax(logits) == 1                                      # first of the equal maxima
    assert ps.sample(logits, 0.0, 40, 0.9, ps.XorShift64(3)) == 1
    for seed in range(5):
        assert ps.sample(logits, 0.7, 1, 1.0, ps.XorShift64(seed)) == 1       # top_k 1
        assert ps.sample(logits, 0.7, 0, 1e-6, ps.XorShift64(seed)) == 1      # top_p -> 0


def test_sampler_frequencies_follow_softmax():
    logits = np.array([1.0, 0.0, 2.0, -1.0], dtype=np.float32)
    t = 0.8
    rng = ps.XorShift64(11)
    n = 20000
    counts = np.bincount([ps.sample(logits, t, 0, 1.0, rng) for _ in range(n)], minlength=4)
    p = np.exp(logits / t) / np.exp(logits / t).sum()
    chi2 = float(((counts - n * p) ** 2 / (n * p)).sum())
    assert chi2 < 16.27        # 3 degrees of freedom, p = 0.001


def test_sampler_top_k_and_top_p_sets():
    logits = np.array([3.0, 1.0, 2.0, 0.0, 2.0], dtype=np.float32)
    work = ps.candidates(logits, 1.0, 3, 1.0)
    assert [i for i, _ in work] == [0, 2, 4]                           # value desc, index asc
    assert abs(sum(float(p) for _, p in work) - 1.0) < 1e-6
    work = ps.candidates(logits, 1.0, 0, 0.6)
    # probabilities 0.51, 0.19, 0.19, ...: the prefix reaching 0.6 is two tokens
    assert [i for i, _ in work] == [0, 2]
    assert abs(sum(float(p) for _, p in work) - 1.0) < 1e-6
    # the prefix ends where the running sum is >= top_p, not > (crates/core/src/sampler.rs:117-121):
    # logits ln 2, 0, 0 give exactly 0.5, 0.25, 0.25 in float32, and with top_p 0.75 the sum
    # meets top_p at the second token; a strict comparison would keep all three
    exact = np.log(np.array([2.0, 1.0, 1.0])).astype(np.float32)
    probs = ps.candidates(exact, 1.0, 0, 1.0)
    assert [float(p) for _, p in probs] == [0.5, 0.25, 0.25]
    work = ps.candidates(exact, 1.0, 0, 0.75)
    assert [i for i, _ in work] == [0, 1]
    assert [float(p) for _, p in work] == [np.float32(0.5) / np.float32(0.75), np.float32(0.25) / np.float32(0.75)]
    assert [i for i, _ in ps.candidates(exact, 1.0, 0, 0.7500001)] == [0, 1, 2]
    # the same edge where no exponential's rounding can blur it: four equal logits, top_p 0.5
    assert [(i, float(p)) for i, p in ps.candidates(np.full(4, 1.25, np.float32), 1.0, 0, 0.5)] == [(0, 0.5), (1, 0.5)]


def test_repetition_detector():
    # crates/core/src/decode_utils.rs:15-17: a pattern of 6 three times is found, of 5 is not
    assert ps.detect_repetition_loop([9, 9] + [1, 2, 3, 4, 5, 6] * 3) == 6
    assert ps.detect_repetition_loop([1, 2, 3, 4, 5] * 3) is None
    assert ps.detect_repetition_loop([1, 2, 3, 4, 5, 6] * 2) is None


def test_bf16_vectors_of_the_reference():
    # crates/backends/backend_common/src/bf16_convert.rs:75-101
    assert ps.f32_to_bf16_bits(1.0) == 0x3F80 and ps.f32_to_bf16_bits(0.0) == 0
    for i in range(128):
        v = (i - 64) * 0.1
        back = float(ps.bf16_bits_to_f32(ps.f32_to_bf16_bits(v)))
        assert abs(back - v) <= 0.01 * abs(v) + 1e-30
    # ties to even (crates/core/src/tensor.rs:46-56)
    half_up = np.uint32(0x3F808000).view(np.float32)      # exactly between 0x3F80 and 0x3F81
    assert ps.f32_to_bf16_bits(half_up) == 0x3F80
    half_up_odd = np.uint32(0x3F818000).view(np.float32)  # between 0x3F81 and 0x3F82
    assert ps.f32_to_bf16_bits(half_up_odd) == 0x3F82
    assert ps.f32_to_bf16_bits(np.uint32(0x3F808001).view(np.float32)) == 0x3F81


def test_scaled_rotation_frequencies():
    """Linear and yarn scaling pinned by what they reduce to: a factor of 1 is the plain rotation;
    linear scaling by f gives at position f p the angles of the plain rotation at p; yarn keeps the
    fast frequencies, divides the slow ones by the factor, and lies between in between."""
    R, theta = 32, 10000.0
    base = ops.rope_inv_freq(R, theta)
    assert torch.equal(ops.rope_inv_freq(R, theta, {"type": "linear", "factor": 1.0}), base)
    lin = ops.rope_inv_freq(R, theta, {"type": "linear", "factor": 4.0})
    assert torch.allclose(lin * 4.0, base, rtol=1e-6)
    c1, s1 = ops.rope_tables([12], R, theta, {"type": "linear", "factor": 4.0})
    c0, s0 = ops.rope_tables([3], R, theta)
    assert torch.allclose(c1, c0, atol=1e-6) and torch.allclose(s1, s0, atol=1e-6)
    y = {"type": "yarn", "factor": 1.0, "original_max_position_embeddings": 512, "beta_fast": 32.0, "beta_slow": 1.0}
    assert torch.allclose(ops.rope_inv_freq(R, theta, y), base, rtol=1e-6)
    y["factor"] = 8.0
    got = ops.rope_inv_freq(R, theta, y)
    wavelen = 2 * math.pi / base.double()
    fast, slow = wavelen < 512 / 32.0, wavelen > 512 / 1.0
    assert fast.any() and slow.any() and (~fast & ~slow).any()
    assert torch.equal(got[fast], base[fast]) and torch.allclose(got[slow] * 8.0, base[slow], rtol=1e-6)
    mid = ~fast & ~slow
    assert ((got[mid] < base[mid]) & (got[mid] > base[mid] / 8.0)).all()
    smooth = (512 / wavelen[mid] - 1.0) / 31.0
    assert torch.allclose(got[mid].double(), (1 - smooth) * base[mid].double() / 8.0 + smooth * base[mid].double(), rtol=1e-5)
