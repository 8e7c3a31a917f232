"""Host side of every kernel: operand checks, then the launch.

Each function checks on the host that shapes, dtypes, devices and layouts are
what the kernel and its grid assume, and only then launches on the current
HIP stream. There is no fallback of any kind behind them.

The operations are those of the reference's op trait (crates/backends/backend_common/src/linear_ops.rs:68-437:
matmul, rms_norm, swiglu, rotation) and of its GPU command buffer
(crates/backends/backend_vulkan/src/backend.rs:182-281: embedding, norms, per-head norms, rotation, cache
append, attention, residual sums), several of them to a kernel here.
"""
import threading

import torch

from ..errors import BackendError
from . import lib

F32 = 0
BF16 = 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


def dtype_code(t):
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise BackendError(f"dtype {t.dtype} is not supported by the kernels") from None


_scoped = threading.local()      # .stream: the stream of the forward pass that this thread is in


class stream_scope:
    """While a forward pass runs, the launches go to the stream that was current when it began:
    looking the stream up costs as much as a launch does. A thread has its own."""

    def __enter__(self):
        self.outer = getattr(_scoped, "stream", None)
        _scoped.stream = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        _scoped.stream = self.outer
        return False


def _stream():
    s = getattr(_scoped, "stream", None)
    return s if s is not None else torch.cuda.current_stream().cuda_stream


def _check(t, name, dtype=None, shape=None):
    """Refuse what a kernel must not be given: not a contiguous GPU tensor, another dtype, another
    shape (None in `shape`: any size). Called for every operand of every launch, hence the short
    way through for what is right."""
    try:
        if t.is_cuda and t.is_contiguous() and (dtype is None or t.dtype == dtype):
            if shape is None or t.shape == shape:
                return
            got = t.shape
            if len(shape) == len(got) and all(s is None or s == d for s, d in zip(shape, got)):
                return
    except AttributeError:
        pass
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise BackendError(f"{name} must be a tensor on the GPU")
    if not t.is_contiguous():
        raise BackendError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise BackendError(f"{name} must be {dtype}, got {t.dtype}")
    raise BackendError(f"{name} must have shape {list(shape)}, got {list(t.shape)}")


def _ptr(t):
    return None if t is None else t.data_ptr()


def embed(ids, table, out, packed=False):
    """out[t, :] = table[ids[t], :] as float32. ids int32 [T], table [V, H], out f32 [T, H].
    packed: the table is stored in the MFMA kernels' order ([H / 32, V / 16, 64, 8])."""
    T = ids.shape[0]
    _check(ids, "ids", torch.int32, (T,))
    _check(table, "table", None, (None, None))
    H = table.shape[1]
    _check(out, "out", torch.float32, (T, H))
    lib.call("elementwise", "hb_embed", ids.data_ptr(), table.data_ptr(), dtype_code(table),
             out.data_ptr(), T, H, table.shape[0], 1 if packed else 0, _stream())


def rmsnorm(x, weight, out, eps, rows=None):
    """out[r] = rmsnorm(x[rows[r]] or x[r]) * weight. x f32 [T, H], weight f32 [H]."""
    _check(x, "x", torch.float32, (None, None))
    H = x.shape[1]
    _check(weight, "weight", torch.float32, (H,))
    if rows is not None:
        _check(rows, "rows", torch.int32, (None,))
        R = rows.shape[0]
    else:
        R = x.shape[0]
    _check(out, "out", None, (R, H))
    lib.call("elementwise", "hb_rmsnorm", x.data_ptr(), weight.data_ptr(), out.data_ptr(),
             dtype_code(out), _ptr(rows), R, H, float(eps), _stream())


def gemm_plain(a, w, c, accumulate=False):
    """c[M, N] (+)= a[M, K] @ w[N, K]^T in float32 arithmetic, any of f32 / bf16 storage."""
    _check(a, "a", None, (None, None))
    _check(w, "w", None, (None, None))
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K:
        raise BackendError(f"gemm: a is [{M}, {K}] but w is {list(w.shape)}")
    _check(c, "c", None, (M, N))
    if accumulate and c.dtype != torch.float32:
        raise BackendError("gemm: accumulation needs a float32 output")
    lib.call("gemm_plain", "hb_gemm_plain", a.data_ptr(), dtype_code(a), w.data_ptr(), dtype_code(w),
             c.data_ptr(), dtype_code(c), M, N, K, K, K, N, 1 if accumulate else 0, _stream())


def _check_paged(meta, cache, T):
    _check(meta.positions, "positions", torch.int32, (T,))
    _check(meta.seq_of, "seq_of", torch.int32, (T,))
    _check(meta.slots, "slots", torch.int32, (None,))
    _check(cache.page_table, "page_table", torch.int32, (None, None))
    _check(cache.k, "key pages", None, (None, None, cache.page_size, None))
    pages, nkv, page, hd = cache.k.shape
    _check(cache.v, "value pages", cache.k.dtype, (pages, nkv, hd, page))


ROPE_WRITE_SLICES = (2, 4, 8)


def rope_write_adds_slices(T, hd, rot_dims, dtype, write_kv, has_rotation):
    """True if qk_norm_rope_write can add up K slices of the projection itself for such a step: the
    kernel for bfloat16 prompts of 64 tokens or more does."""
    return (dtype == torch.bfloat16 and write_kv and T >= 64 and hd <= 128 and hd % 8 == 0
            and (not has_rotation or rot_dims == hd))


def qk_norm_rope_write(qkv, q_norm_w, k_norm_w, cos, sin, rot_dims, meta, cache, q_out, nq, nkv, hd, eps,
                       write_kv=True, qkv_slices=None):
    """Per-head norm (if weights given), rotation (if tables given), q to q_out, k / v to the pages.

    qkv f32 [T, (nq + 2 nkv) hd] (query heads only when write_kv is false); cos / sin f32 [max_pos, rot_dims / 2]; q_out [T, nq hd] in the
    cache's dtype; cache.k / cache.v [pages, nkv, page_size, hd].
    qkv_slices = (slices, pointer, floats between two), as kernels.mfma.gemm(..., defer_slices=True)
    returns it: the projection's sums still lie in that many slices (see rope_write_adds_slices),
    and qkv itself is not read.
    """
    T = qkv.shape[0]
    _check(qkv, "qkv", torch.float32, (T, (nq + (2 * nkv if write_kv else 0)) * hd))
    _check_paged(meta, cache, T)
    _check(q_out, "q_out", cache.k.dtype, (T, nq * hd))
    if tuple(cache.k.shape[1:]) != (nkv, cache.page_size, hd):
        raise BackendError(f"cache pages {list(cache.k.shape)} do not fit {nkv} kv heads of {hd}")
    for w, name in ((q_norm_w, "q_norm"), (k_norm_w, "k_norm")):
        if w is not None:
            _check(w, name, torch.float32, (hd,))
    if cos is not None:
        _check(cos, "cos", torch.float32, (None, rot_dims // 2))
        _check(sin, "sin", torch.float32, tuple(cos.shape))
        if meta.max_position >= cos.shape[0]:
            raise BackendError(f"position {meta.max_position} beyond the rotation table "
                               f"({cos.shape[0]} rows)")
    n_slices, src, stride = qkv_slices if qkv_slices is not None else (1, qkv.data_ptr(), 0)
    if n_slices > 1 and (n_slices not in ROPE_WRITE_SLICES or stride < qkv.numel() or not rope_write_adds_slices(
            T, hd, rot_dims, q_out.dtype, write_kv, cos is not None)):
        raise BackendError(f"qk_norm_rope_write does not add up {n_slices} slices of the projection here")
    lib.call("elementwise", "hb_qk_norm_rope_write", src, qkv.shape[1], _ptr(q_norm_w),
             _ptr(k_norm_w), _ptr(cos), _ptr(sin), rot_dims, meta.positions.data_ptr(),
             meta.seq_of.data_ptr(), meta.slots.data_ptr(), cache.page_table.data_ptr(),
             cache.page_table.shape[1], cache.page_size, q_out.data_ptr(), cache.k.data_ptr(),
             cache.v.data_ptr(), dtype_code(q_out), T, nq, nkv, hd, float(eps), 1 if write_kv else 0,
             n_slices, stride, _stream())


def attention_plain(q, meta, cache, out, nq, nkv, hd, scale, window):
    """Causal (and windowed) attention of every token over its slot's pages."""
    T = q.shape[0]
    _check(q, "q", cache.k.dtype, (T, nq * hd))
    _check(out, "out", cache.k.dtype, (T, nq * hd))
    _check_paged(meta, cache, T)
    if tuple(cache.k.shape[1:]) != (nkv, cache.page_size, hd):
        raise BackendError(f"cache pages {list(cache.k.shape)} do not fit {nkv} kv heads of {hd}")
    lib.call("attention_plain", "hb_attention_plain", q.data_ptr(), cache.k.data_ptr(),
             cache.v.data_ptr(), out.data_ptr(), dtype_code(q), meta.positions.data_ptr(),
             meta.seq_of.data_ptr(), meta.slots.data_ptr(), cache.page_table.data_ptr(),
             cache.page_table.shape[1], cache.page_size, T, nq, nkv, hd, float(scale),
             int(window or 0), _stream())


def swiglu(gu, out):
    """out[t, i] = silu(gu[t, i]) * gu[t, I + i]; gu f32 [T, 2I]."""
    _check(gu, "gate_up", torch.float32, (None, None))
    T, two_i = gu.shape
    if two_i % 2:
        raise BackendError("swiglu: the input's width must be even")
    _check(out, "out", None, (T, two_i // 2))
    lib.call("elementwise", "hb_swiglu", gu.data_ptr(), out.data_ptr(), dtype_code(out), T, two_i // 2,
             _stream())


def fill_u32(t, value):
    """Set every 32-bit word of a tensor (through a kernel, safe inside a captured graph)."""
    _check(t, "tensor")
    nbytes = t.numel() * t.element_size()
    if nbytes % 4:
        raise BackendError("fill: the tensor's size is no multiple of 4 bytes")
    lib.call("elementwise", "hb_fill_u32", t.data_ptr(), int(value), nbytes // 4, _stream())


ARGMAX_MAX_CHUNKS = 64


def argmax_scratch(rows, device):
    """The partial results of the first of argmax's two stages for up to `rows` rows, to be kept
    and handed to `argmax` again and again."""
    return (torch.empty((rows, ARGMAX_MAX_CHUNKS), dtype=torch.float32, device=device),
            torch.empty((rows, ARGMAX_MAX_CHUNKS), dtype=torch.int32, device=device))


def argmax(logits, out, scratch=None):
    """out[r] = first index of the largest value of logits[r]; logits f32 [R, V], out int32 [R].
    `scratch` as `argmax_scratch` makes it (for at least R rows), else it is allocated here."""
    _check(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    _check(out, "out", torch.int32, (R,))
    chunks = max(1, min(ARGMAX_MAX_CHUNKS, V // 8192, 1024 // R if R <= 1024 else 1))
    sv = si = None
    if chunks > 1 and scratch is not None:
        sv, si = scratch
        _check(sv, "argmax scratch values", torch.float32, (None, ARGMAX_MAX_CHUNKS))
        _check(si, "argmax scratch indices", torch.int32, tuple(sv.shape))
        if sv.shape[0] < R:
            raise BackendError("argmax: the scratch has fewer rows than the logits")
    elif chunks > 1:
        sv = torch.empty((R, chunks), dtype=torch.float32, device=logits.device)
        si = torch.empty((R, chunks), dtype=torch.int32, device=logits.device)
    lib.call("sampling", "hb_argmax", logits.data_ptr(), V, R, V, out.data_ptr(), _ptr(sv), _ptr(si),
             chunks, _stream())


SAMPLE_CHUNK = 8192


def sample(logits, temperature, top_k, top_p, rng_states, rng_index, out, scratch=None, sifted=None):
    """One token per row by temperature / top-k / top-p; rng_states int64 [n], advanced in place.

    `scratch` = (keys int32 [R, P2], idx int32 [R, P2]) with P2 the power of two >= V; needed
    unless 0 < top_k <= 1024 and top_k < V.
    `sifted` = (keys int32, idx int32), each of at least R * ceil(V / 8192) * top_k elements, optional:
    with them a long row is first sifted by a block for every 8192 logits (same result, sooner).
    """
    _check(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    _check(out, "out", torch.int32, (R,))
    _check(rng_states, "rng_states", torch.int64, (None,))
    if rng_index is not None:
        _check(rng_index, "rng_index", torch.int32, (R,))
    elif rng_states.shape[0] < R:
        raise BackendError("sample: fewer generator states than rows")
    keys = idx = None
    p2 = 0
    if scratch is not None:
        keys, idx = scratch
        p2 = keys.shape[1]
        _check(keys, "scratch keys", torch.int32, (None, p2))
        _check(idx, "scratch idx", torch.int32, tuple(keys.shape))
        if keys.shape[0] < R:
            raise BackendError("sample: scratch has fewer rows than the logits")
    pre_key = pre_idx = None
    if sifted is not None:
        pre_key, pre_idx = sifted
        need = R * (-(-V // SAMPLE_CHUNK)) * max(int(top_k), 1)
        _check(pre_key, "sifted keys", torch.int32, (None,))
        _check(pre_idx, "sifted idx", torch.int32, (None,))
        if pre_key.numel() < need or pre_idx.numel() < need:
            raise BackendError(f"sample: the buffers for sifted candidates hold fewer than {need} elements")
    lib.call("sampling", "hb_sample", logits.data_ptr(), V, R, V, float(temperature), int(top_k),
             float(top_p), rng_states.data_ptr(), _ptr(rng_index), out.data_ptr(), _ptr(keys),
             _ptr(idx), p2, _ptr(pre_key), _ptr(pre_idx), _stream())


NUCLEUS_CANDIDATES = 1024


def nucleus_buffers(rows, vocab, device):
    """(keys int32, idx int32, sums float32) that sample_nucleus needs for `rows` rows of `vocab` logits."""
    chunks = -(-vocab // SAMPLE_CHUNK)
    return (torch.empty(rows * chunks * NUCLEUS_CANDIDATES, dtype=torch.int32, device=device),
            torch.empty(rows * chunks * NUCLEUS_CANDIDATES, dtype=torch.int32, device=device),
            torch.empty(rows * chunks * 2, dtype=torch.float32, device=device))


def sample_nucleus(logits, temperature, top_p, rng_states, rng_index, out, buffers):
    """Top-p without top-k on rows of more than 1024 logits, the quick way: a row's prefix is looked
    for among its 1024 largest logits only (the softmax still runs over the whole row). A row whose
    prefix does not end among them gets out[r] = -1 and keeps its generator state: sample it with
    `sample`. `buffers` as `nucleus_buffers` makes them."""
    _check(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    _check(out, "out", torch.int32, (R,))
    _check(rng_states, "rng_states", torch.int64, (None,))
    if rng_index is not None:
        _check(rng_index, "rng_index", torch.int32, (R,))
    elif rng_states.shape[0] < R:
        raise BackendError("sample: fewer generator states than rows")
    keys, idx, sums = buffers
    chunks = -(-V // SAMPLE_CHUNK)
    _check(keys, "candidate keys", torch.int32, (None,))
    _check(idx, "candidate idx", torch.int32, (None,))
    _check(sums, "chunk sums", torch.float32, (None,))
    if min(keys.numel(), idx.numel()) < R * chunks * NUCLEUS_CANDIDATES or sums.numel() < R * chunks * 2:
        raise BackendError("sample: the buffers of the quick top-p are too small for these logits")
    lib.call("sampling", "hb_sample_nucleus", logits.data_ptr(), V, R, V, float(temperature), float(top_p),
             rng_states.data_ptr(), _ptr(rng_index), out.data_ptr(), keys.data_ptr(), idx.data_ptr(),
             sums.data_ptr(), _stream())


def sample_all(logits, temperature, rng_states, rng_index, out, sums):
    """Temperature sampling over whole rows (no top-k, no top-p): a block for every 8192 logits adds
    up its part of the softmax, a block a row takes the draw and walks the chunk it falls into.
    `sums`: float32 of at least R * ceil(V / 8192) * 2 elements."""
    _check(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    _check(out, "out", torch.int32, (R,))
    _check(rng_states, "rng_states", torch.int64, (None,))
    if rng_index is not None:
        _check(rng_index, "rng_index", torch.int32, (R,))
    elif rng_states.shape[0] < R:
        raise BackendError("sample: fewer generator states than rows")
    _check(sums, "chunk sums", torch.float32, (None,))
    if sums.numel() < R * (-(-V // SAMPLE_CHUNK)) * 2:
        raise BackendError("sample: the buffer of the chunks' sums is too small for these logits")
    lib.call("sampling", "hb_sample_all", logits.data_ptr(), V, R, V, float(temperature), rng_states.data_ptr(),
             _ptr(rng_index), out.data_ptr(), sums.data_ptr(), _stream())


def force_tokens(logits, rows, tokens):
    """Every logit of row rows[i] but that of tokens[i] becomes -inf, in place: the next choice in
    that row can only be that token. rows, tokens: lists of ints (checked here against the shape)."""
    _check(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    if len(rows) != len(tokens) or not rows:
        raise BackendError("force_tokens: needs as many tokens as rows, at least one")
    for r, t in zip(rows, tokens):
        if not (0 <= int(r) < R and 0 <= int(t) < V):
            raise BackendError(f"force_tokens: row {r} or token {t} outside logits of shape {R} x {V}")
    both = torch.tensor([list(map(int, rows)), list(map(int, tokens))], dtype=torch.int32, device=logits.device)
    lib.call("sampling", "hb_force_tokens", logits.data_ptr(), V, R, V, both[0].data_ptr(), both[1].data_ptr(),
             len(rows), _stream())
