"""Plain, slow, whole-sequence formulas of the dense Qwen3 decoder.

One function for each part, written from the reference's text (paths are
relative to the reference's root; `bc/` = crates/backends/backend_common/src/).
No cache, no batching, no code shared with the engine. Everything runs on the
CPU in the dtype of its inputs (float32 by default, float64 to judge rounding).
"""
import math

import numpy as np
import torch


def embedding(ids, table):
    """x_t = E[id_t, :], no multiplier; an id >= vocab is an error.

    bc/generic_model.rs:104-111 (lookup), :165-171 (range check).
    """
    vocab = table.shape[0]
    rows = []
    for t in ids:
        t = int(t)
        if t < 0 or t >= vocab:
            raise ValueError(f"token id {t} out of range (vocab_size {vocab})")
        rows.append(table[t])
    return torch.stack(rows, 0)


def rms_norm(x, weight, eps):
    """y_i = x_i * 1/sqrt(sum(x^2)/dim + eps) * w_i over the last axis.

    bc/kernels.rs:54-64: eps is added to the mean inside the square root, the
    weight multiplies afterwards and is used as it is (not 1 + w).
    """
    dim = x.shape[-1]
    sum_sq = (x * x).sum(-1, keepdim=True)
    inv_rms = 1.0 / torch.sqrt(sum_sq / dim + eps)
    return x * inv_rms * weight


# Above this many multiply-adds (or query-key pairs) a formula is handed to torch's matrix
# product on the CPU instead of the loop that spells it out: the same sums, in the library's
# order. test_plain checks that both ways agree; the loops stay the definition.
WHOLE_FROM = 1 << 24


def linear(x, weight):
    """C[m, n] = sum_k A[m, k] * W[n, k]; weights are [out, in], no bias.

    crates/backends/backend_bf16/src/kernels.rs:154-164.
    """
    if x.shape[0] * weight.shape[0] * weight.shape[1] > WHOLE_FROM:
        return x @ weight.T
    out = torch.zeros(x.shape[0], weight.shape[0], dtype=x.dtype)
    for n in range(weight.shape[0]):
        out[:, n] = (x * weight[n]).sum(-1)
    return out


def split_heads(x, num_heads, head_dim):
    """Row layout [head0(hd) | head1(hd) | ...] -> [T, heads, hd].

    bc/generic_attention/mod.rs:63-65 (offset = h * head_dim).
    """
    assert x.shape[-1] == num_heads * head_dim
    return x.reshape(x.shape[0], num_heads, head_dim)


def head_rms_norm(x, weight, eps):
    """RMSNorm of each head vector alone, one weight [hd] for all heads.

    bc/generic_attention/mod.rs:62-76; x is [T, heads, hd].
    """
    out = torch.empty_like(x)
    for h in range(x.shape[1]):
        out[:, h] = rms_norm(x[:, h], weight, eps)
    return out


def rope_inv_freq(rotary_ndims, theta, scaling=None):
    """inv_freq_i = 1 / theta^(2i / R) in float32, i in [0, R/2), one frequency at a time.

    bc/loader_common.rs:185-188. scaling (a dict as config.json holds it, already reduced to
    type / factor / original_max_position_embeddings / beta_fast / beta_slow):
    linear, bc/loader_common.rs:212-215: 1 / (theta^(2i / R) * factor);
    yarn, bc/loader_common.rs:252-276: wavelen = 2 pi / freq; below original / beta_fast the
    frequency stays, above original / beta_slow it is divided by the factor, in between
    smooth = (original / wavelen - beta_slow) / (beta_fast - beta_slow) and
    (1 - smooth) * freq / factor + smooth * freq. All in float32.
    """
    f = np.float32
    theta32 = torch.tensor(theta, dtype=torch.float32)
    i2 = torch.arange(0, rotary_ndims // 2, dtype=torch.float32) * 2.0
    powers = torch.pow(theta32, i2 / float(rotary_ndims)).numpy()
    out = []
    for i in range(rotary_ndims // 2):
        power = f(powers[i])
        freq = f(1.0) / power
        if scaling and scaling["type"] == "linear":
            freq = f(1.0) / f(power * f(scaling["factor"]))
        elif scaling and scaling["type"] == "yarn":
            original = f(scaling["original_max_position_embeddings"])
            low, high = original / f(scaling["beta_fast"]), original / f(scaling["beta_slow"])
            wavelen = f(f(2.0) * f(np.pi)) / freq
            if wavelen < low:
                pass
            elif wavelen > high:
                freq = freq / f(scaling["factor"])
            else:
                smooth = f(original / wavelen - f(scaling["beta_slow"])) / f(f(scaling["beta_fast"]) - f(scaling["beta_slow"]))
                freq = f(f(f(1.0) - smooth) * f(freq / f(scaling["factor"]))) + f(smooth * freq)
        out.append(freq)
    return torch.tensor(np.array(out, dtype=np.float32))


def rope_tables(positions, rotary_ndims, theta, scaling=None):
    """cos/sin of ang = float32(pos) * inv_freq_i, the angle itself in float32.

    bc/loader_common.rs:193-199.
    """
    inv = rope_inv_freq(rotary_ndims, theta, scaling)
    pos = torch.as_tensor(positions, dtype=torch.float32)
    ang = pos[:, None] * inv[None, :]
    return torch.cos(ang), torch.sin(ang)


def apply_rope(x, positions, theta, rotary_ndims=None, scaling=None):
    """Half-split rotation: pairs (j, j + R/2); dims >= R stay.

    bc/kernels.rs:739-759: u_j = x0*c - x1*s ; u_{j+R/2} = x0*s + x1*c.
    x is [T, heads, hd]; positions are absolute indices in the sequence.
    """
    hd = x.shape[-1]
    rot = hd if rotary_ndims is None else rotary_ndims
    half = rot // 2
    cos, sin = rope_tables(positions, rot, theta, scaling)
    cos = cos.to(x.dtype)[:, None, :]
    sin = sin.to(x.dtype)[:, None, :]
    out = x.clone()
    x0 = x[..., :half]
    x1 = x[..., half:rot]
    out[..., :half] = x0 * cos - x1 * sin
    out[..., half:rot] = x0 * sin + x1 * cos
    return out


def causal_attention(q, k, v, positions, scale=None, window=None):
    """Scores, causal mask by count, softmax, PV; consecutive query heads share a kv head.

    q [T, nq, hd], k/v [T, nkv, hd] of ONE whole sequence whose token t sits at
    positions[t] (ascending). Query at position p sees the keys at positions <= p
    (bc/generic_attention/prefill/kernel_f32.rs:65-67), kv head = h / (nq / nkv)
    (bc/generic_attention/decode.rs:131-140), scale = 1/sqrt(hd)
    (bc/generic_attention/decode.rs:126), softmax with the maximum taken off
    (bc/kernels.rs:716-731), out = sum_j p_j v_j (bc/attention_common.rs:160-177).

    `window` is no part of the reference (it never reads a window); when given,
    a query at p sees only keys with p - window < position <= p.
    """
    T, nq, hd = q.shape
    nkv = k.shape[1]
    assert nq % nkv == 0
    group = nq // nkv
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    out = torch.zeros_like(q)
    if T * T * nq > WHOLE_FROM:
        # every query of a head at once: scores [T, T], keys out of sight at -inf
        pos = torch.as_tensor(list(positions))
        seen = pos[None, :] <= pos[:, None]
        if window is not None:
            seen &= pos[None, :] > pos[:, None] - window
        for h in range(nq):
            g = h // group
            s = (q[:, h] @ k[:, g].T) * scale
            s = s.masked_fill(~seen, float("-inf"))
            e = torch.exp(s - s.max(-1, keepdim=True).values)
            out[:, h] = (e / e.sum(-1, keepdim=True)) @ v[:, g]
        return out
    for h in range(nq):
        g = h // group
        for i in range(T):
            p = int(positions[i])
            keys = [j for j in range(T) if int(positions[j]) <= p
                    and (window is None or int(positions[j]) > p - window)]
            kk = k[keys, g]
            vv = v[keys, g]
            s = (kk * q[i, h]).sum(-1) * scale
            m = s.max()
            e = torch.exp(s - m)
            total = e.sum()
            prob = e / total if total > 0 else e
            out[i, h] = (prob[:, None] * vv).sum(0)
    return out


def silu(x):
    """x / (1 + exp(-x)); bc/kernels.rs:676-679."""
    return x / (1.0 + torch.exp(-x))


def swiglu_mlp(x, w_gate, w_up, w_down):
    """down(silu(gate(x)) * up(x)); bc/generic_mlp.rs:83-96, bc/kernels.rs:681-687."""
    g = linear(x, w_gate)
    u = linear(x, w_up)
    return linear(silu(g) * u, w_down)


def softmax(x):
    """bc/kernels.rs:716-731 (whole vector, guard sum > 0)."""
    m = x.max()
    e = torch.exp(x - m)
    s = e.sum()
    return e / s if s > 0 else e
