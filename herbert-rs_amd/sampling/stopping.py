"""Why a sequence ends, and the reference's repetition check."""

EOS = "eos"
STOP_TOKEN = "stop_token"
MAX_TOKENS = "max_tokens"
REPETITION_LOOP = "repetition_loop"
LENGTH = "length"              # the model's max_position_embeddings is reached
STOP_SEQUENCE = "stop_sequence"  # the caller's own rule on the decoded text (crates/cli/src/main.rs:1328-1332,1360)
INTERRUPTED = "interrupted"    # the caller's interrupt flag was set (crates/cli/src/main.rs:1242-1245)


def detect_repetition_loop(tokens, min_pattern=6, max_pattern=100, repeats=3):
    """The pattern's length if the last tokens are one pattern of 6..100 tokens three times
    over (crates/core/src/decode_utils.rs:14-33), else None."""
    n = len(tokens)
    for pat in range(min_pattern, max_pattern + 1):
        need = pat * repeats
        if n < need:
            continue
        base = n - need
        first = tokens[base:base + pat]
        if all(tokens[base + r * pat:base + (r + 1) * pat] == first for r in range(1, repeats)):
            return pat
    return None
