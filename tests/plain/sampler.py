"""Plain sampler: xorshift64, temperature, top-k, top-p, one value at a time.

Written from crates/core/src/sampler.rs of the reference. Arithmetic is done
in float32 step by step (numpy scalars) as the reference does in f32.
Where the reference leaves an order open (select_nth_unstable and
sort_unstable, sampler.rs:93,113) the candidates are ordered by value
descending and by index ascending among equals, which is one of the orders the
reference may produce.
"""
import numpy as np

MASK64 = (1 << 64) - 1


class XorShift64:
    """sampler.rs:30-34 (seed 0 becomes 0xdeadbeef), :50-62 (step and float)."""

    def __init__(self, seed):
        self.state = 0xDEADBEEF if seed == 0 else (seed & MASK64)

    def next_u64(self):
        x = self.state
        x ^= (x << 13) & MASK64
        x ^= x >> 7
        x ^= (x << 17) & MASK64
        self.state = x
        return x

    def next_f32(self):
        return np.float32(self.next_u64() >> 40) / np.float32(1 << 24)


def argmax(logits):
    """First maximal index, strict >; sampler.rs:244-254."""
    best, best_val = 0, -np.inf
    for i, v in enumerate(logits):
        if v > best_val:
            best, best_val = i, v
    return best


def candidates(logits, temperature, top_k, top_p):
    """The (index, probability) list that the CDF walk goes through, in its order.

    sampler.rs:84-131: divide by temperature; keep the top_k largest when
    0 < top_k < n; softmax with the maximum taken off; when top_p < 1 sort by
    probability descending, keep the shortest prefix whose running sum is
    >= top_p, renormalise.
    """
    logits = np.asarray(logits, dtype=np.float32)
    n = len(logits)
    t = np.float32(temperature)
    work = [(i, np.float32(v) / t) for i, v in enumerate(logits)]
    if 0 < top_k < n:
        work.sort(key=lambda iv: (-iv[1], iv[0]))
        work = work[:top_k]
    max_val = max(v for _, v in work)
    exps = [(i, np.exp(np.float32(v - max_val), dtype=np.float32)) for i, v in work]
    total = np.float32(0.0)
    for _, e in exps:
        total = np.float32(total + e)
    inv = np.float32(1.0) / total
    work = [(i, np.float32(e * inv)) for i, e in exps]
    if top_p < 1.0:
        work.sort(key=lambda iv: (-iv[1], iv[0]))
        cum = np.float32(0.0)
        cutoff = len(work)
        for pos, (_, p) in enumerate(work):
            cum = np.float32(cum + p)
            if cum >= np.float32(top_p):
                cutoff = pos + 1
                break
        work = work[:cutoff]
        total = np.float32(0.0)
        for _, p in work:
            total = np.float32(total + p)
        inv = np.float32(1.0) / total
        work = [(i, np.float32(p * inv)) for i, p in work]
    return work


def pick(work, r):
    """sampler.rs:134-144: first index whose running sum exceeds r, else the last."""
    cum = np.float32(0.0)
    for idx, p in work:
        cum = np.float32(cum + p)
        if r < cum:
            return idx
    return work[-1][0]


def sample(logits, temperature, top_k, top_p, rng):
    """sampler.rs:72-145. temperature 0 is argmax and draws nothing."""
    if len(logits) == 0:
        return 0
    if temperature == 0.0:
        return argmax(logits)
    work = candidates(logits, temperature, top_k, top_p)
    return pick(work, rng.next_f32())


def detect_repetition_loop(tokens):
    """crates/core/src/decode_utils.rs:14-33: a pattern of 6..100 tokens three times at the end."""
    n = len(tokens)
    for pat in range(6, 101):
        need = pat * 3
        if n < need:
            continue
        base = n - need
        pattern = tokens[base:base + pat]
        if all(tokens[base + r * pat:base + (r + 1) * pat] == pattern for r in (1, 2)):
            return pat
    return None


def f32_to_bf16_bits(value):
    """Round to nearest even on the upper 16 bits; crates/core/src/tensor.rs:46-56."""
    bits = int(np.float32(value).view(np.uint32))
    lsb = (bits >> 16) & 1
    round_bit = (bits >> 15) & 1
    sticky = bits & 0x7FFF
    result = bits >> 16
    if round_bit == 1 and (sticky != 0 or lsb == 1):
        result += 1
    return result & 0xFFFF


def bf16_bits_to_f32(bits):
    """Upper 16 bits of a float32; crates/core/src/tensor.rs:7-9."""
    return np.uint32((bits & 0xFFFF) << 16).view(np.float32)


def think_forced(history, budget, open_id, close_id, newline_id):
    """The token that the think budget forces after the generated tokens `history`, or None.

    crates/core/src/sampler.rs:200-231, from the whole history instead of a running state: a
    block is open if an opening token came after the last closing one; the count is the number
    of tokens since the last opening token (the opening token itself not counted; a forced
    line break counts like any token). count + 1 == budget forces the line break, count + 1 >
    budget the closing token; a budget of 0 forces nothing.
    """
    if budget == 0:
        return None
    last_open = max((i for i, t in enumerate(history) if t == open_id), default=-1)
    last_close = max((i for i, t in enumerate(history) if t == close_id), default=-1)
    if last_open < 0 or last_close > last_open:
        return None
    count = len(history) - 1 - last_open
    if count + 1 == budget:
        return newline_id
    if count + 1 > budget:
        return close_id
    return None
